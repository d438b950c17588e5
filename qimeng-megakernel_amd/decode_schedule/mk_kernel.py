"""Load and call the gfx950 decode megakernel through its C ABI.

Host-side counterpart of the reference's launcher module
(`…/A100/single_batch/decode_schedule/mk_kernel.py:40-111`): ``get_mk`` returns
the ``mk`` callable, ``call_mk(globs, mk)`` passes the 22 tensors and 3 scalars
in the reference's positional order, ``run_instructions`` executes an arbitrary
instruction list.  Instead of a pybind module the callable wraps
``libqmk_hip.so`` (``include/qmk.h``) with ctypes: tensors cross the boundary as
raw device pointers and sizes, the launch goes onto torch's current stream.

There is no fallback: a missing library is an ``ImportError``, a non-GPU tensor
a ``ValueError`` and a device-side error a ``RuntimeError``.
"""
from __future__ import annotations

import ctypes
import math
from pathlib import Path
from typing import Any, Sequence

import torch

from ..instruction import Instruction
from .globs import Globals
from .instructions import scheduler as _scheduler
from .instructions.instruction_defs import REFERENCE_GEOMETRY, TileGeometry
from .model_config import LlamaConfig

_LIBRARY_NAME = "libqmk_hip.so"

QMK_FLAG_KEEP_BARRIERS = 1
QMK_FLAG_XCD_COUNTERS = 2
QMK_FLAG_TAGGED = 4
QMK_XCD_COUNTER_ROWS = 54
QMK_MODEL_LLAMA_3_2_1B = 0
QMK_MODEL_QWEN3_1_7B = 1
QMK_QUERY_ABI_VERSION, QMK_QUERY_CU_COUNT, QMK_QUERY_THREADS, QMK_QUERY_LDS_BYTES = 0, 1, 2, 3
QMK_QUERY_MAX_QUEUES, QMK_QUERY_INSTRUCTION_WORDS, QMK_QUERY_MAX_PARTIALS = 4, 5, 6

_P = ctypes.c_void_p
_I = ctypes.c_int32


class QmkArgs(ctypes.Structure):
    """Mirror of ``struct QmkArgs`` in include/qmk.h (field order is the ABI)."""

    _fields_ = [
        ("struct_size", ctypes.c_uint32), ("model", ctypes.c_uint32),
        ("flags", ctypes.c_uint32), ("spin_limit", ctypes.c_uint32),
        ("instructions", _P), ("hidden_states", _P), ("q_post_rope", _P), ("k_cache", _P), ("v_cache", _P),
        ("attn_out", _P), ("attn_lse_intermediates", _P), ("attn_out_intermediates", _P), ("silu_out", _P),
        ("logits", _P), ("attn_norm_weights", _P), ("qkv_weights", _P), ("rope_cos", _P), ("rope_sin", _P),
        ("o_proj_weights", _P), ("mlp_norm_weights", _P), ("up_proj_weights", _P), ("gate_proj_weights", _P),
        ("down_proj_weights", _P), ("lm_head_norm_weights", _P), ("lm_head_weights", _P), ("barriers", _P),
        ("num_queues", _I), ("num_insts", _I), ("num_layers", _I), ("num_layer_barriers", _I),
        ("barrier_slots", _I), ("max_seq_len", _I), ("max_splits", _I), ("vocab_size", _I), ("rope_rows", _I),
        ("pos_id", _I), ("attn_scale", ctypes.c_float), ("rms_norm_eps", ctypes.c_float),
        ("qkv_blocks_per_head", _I), ("oproj_blocks", _I), ("upgate_blocks_per_bucket", _I), ("down_arrivals", _I),
        ("timeline", _P), ("stream", _P), ("workspace", _P), ("workspace_bytes", ctypes.c_uint64),
        ("embed_tokens", _P), ("token_out", _P),
        ("qkv_raw", _P), ("q_norm_weights", _P), ("k_norm_weights", _P),
    ]


_EXPORTS = ("qmk_decode_step", "qmk_decode_step_static", "qmk_query", "qmk_status_fetch", "qmk_error_string", "qmk_workspace_bytes")

# (name, dtype, ndim) of the 22 tensors, in the positional order of mk(...).
_TENSOR_ARGS: tuple[tuple[str, torch.dtype, int], ...] = (
    ("instructions", torch.int32, 3),
    ("hidden_states", torch.bfloat16, 1),
    ("q_post_rope", torch.bfloat16, 1),
    ("k_cache", torch.bfloat16, 5),
    ("v_cache", torch.bfloat16, 5),
    ("attn_out", torch.bfloat16, 1),
    ("attn_lse_intermediates", torch.float32, 2),
    ("attn_out_intermediates", torch.float32, 3),
    ("silu_out", torch.bfloat16, 1),
    ("logits", torch.bfloat16, 1),
    ("attn_norm_weights", torch.bfloat16, 2),
    ("qkv_weights", torch.bfloat16, 3),
    ("rope_cos", torch.float32, 2),
    ("rope_sin", torch.float32, 2),
    ("o_proj_weights", torch.bfloat16, 3),
    ("mlp_norm_weights", torch.bfloat16, 2),
    ("up_proj_weights", torch.bfloat16, 3),
    ("gate_proj_weights", torch.bfloat16, 3),
    ("down_proj_weights", torch.bfloat16, 3),
    ("lm_head_norm_weights", torch.bfloat16, 1),
    ("lm_head_weights", torch.bfloat16, 2),
    ("barriers", torch.int32, 3),
)


# The Qwen3 op set's mk(...) takes three tensors more, in the reference's positional order
# (`…/qwen/qwen3__0_6b/A100/single_batch/decode_schedule/mk_kernel.py:84-110`): qkv_raw after
# hidden_states, the two per-head norm weights after qkv_weights.
_QWEN3_TENSOR_ARGS: tuple[tuple[str, torch.dtype, int], ...] = (
    _TENSOR_ARGS[:2] + (("qkv_raw", torch.bfloat16, 1),) + _TENSOR_ARGS[2:12]
    + (("q_norm_weights", torch.bfloat16, 2), ("k_norm_weights", torch.bfloat16, 2)) + _TENSOR_ARGS[12:]
)


def _model_id(shape: Any) -> int:
    """The compiled kernel instantiation for ``shape`` (layer count and vocabulary are run-time values)."""
    key = (shape.hidden_size, shape.intermediate_size, shape.head_dim, shape.num_attention_heads,
           shape.num_key_value_heads, bool(getattr(shape, "qk_norm", False)))
    table = {
        (2048, 8192, 64, 32, 8, False): QMK_MODEL_LLAMA_3_2_1B,
        (2048, 6144, 128, 16, 8, True): QMK_MODEL_QWEN3_1_7B,
    }
    if key not in table:
        raise ValueError(f"no kernel was compiled for the layer geometry {key}")
    return table[key]


def _default_mk_dir() -> Path:
    """Directory that holds the built library: the package root, next to ``csrc/``."""
    return Path(__file__).resolve().parent.parent


def load_library(mk_dir: Path | None = None) -> ctypes.CDLL:
    root = (_default_mk_dir() if mk_dir is None else Path(mk_dir)).resolve()
    dso = root / _LIBRARY_NAME
    if not dso.is_file():
        raise ImportError(f"missing prebuilt kernel {dso}; build it first (python -c 'import __graft_entry__ as g; g.build()')")
    try:
        lib = ctypes.CDLL(str(dso))
    except OSError as exc:
        raise ImportError(f"cannot load prebuilt kernel {dso}: {exc}") from exc
    for name in _EXPORTS:
        if not hasattr(lib, name):
            raise ImportError(f"{dso} does not export {name}")
    lib.qmk_decode_step.argtypes = [ctypes.POINTER(QmkArgs)]
    lib.qmk_decode_step.restype = ctypes.c_int
    lib.qmk_decode_step_static.argtypes = [ctypes.POINTER(QmkArgs)]
    lib.qmk_decode_step_static.restype = ctypes.c_int
    lib.qmk_query.argtypes = [ctypes.c_int]
    lib.qmk_query.restype = ctypes.c_int
    lib.qmk_status_fetch.argtypes = [_P, ctypes.POINTER(_I * 4)]
    lib.qmk_status_fetch.restype = ctypes.c_int
    lib.qmk_error_string.argtypes = [ctypes.c_int]
    lib.qmk_error_string.restype = ctypes.c_char_p
    lib.qmk_workspace_bytes.argtypes = [ctypes.c_int]
    lib.qmk_workspace_bytes.restype = ctypes.c_uint64
    return lib


def _tensor_for_mk(t: torch.Tensor | None) -> torch.Tensor | None:
    if t is None:
        return t
    return t.data if isinstance(t, torch.nn.Parameter) else t


class MegaKernel:
    """The ``mk`` callable.

    ``geometry`` is the tile geometry the instruction tensor was scheduled with
    (it fixes the final counter values the kernel waits for); ``reset_barriers``
    selects whether the kernel clears the counters when it retires (default) or
    leaves their final values in place like the reference kernel.  ``tagged``
    lets the small activation vectors travel between workgroups as
    self-announcing tagged units (``QMK_FLAG_TAGGED``) whenever the schedule
    allows it: the kernel clears its counters itself, the down projection is
    not split along K and there are at most 63 layers.  The workspace that mode
    needs belongs to this object — or, with ``static_scratch``, to the library:
    the call then goes through ``qmk_decode_step_static``, which allocates
    nothing and takes no workspace (one array per GPU, shared by every such
    call: do not overlap them on two streams).

    ``greedy_into(embed_tokens, tokens, index)`` arms device-side step chaining
    for the next call: the kernel itself writes the greedy token to
    ``tokens.view(-1)[index]`` and copies its embedding row into
    ``hidden_states`` (the reference does both on the host between launches,
    `models/LLM/decode.py:1386-1397`).
    """

    def __init__(self, lib: ctypes.CDLL, geometry: TileGeometry | None = None, *, reset_barriers: bool = True,
                 spin_limit: int = 0, xcd_counters: bool = True, tagged: bool = True, static_scratch: bool = False):
        self._lib = lib
        self.static_scratch = static_scratch
        self.geometry = geometry
        self.reset_barriers = reset_barriers
        self.spin_limit = int(spin_limit)
        self.xcd_counters = xcd_counters   # use per-XCD sub-counters when `barriers` has room for them
        self._xcd_counters = False
        self.tagged = tagged
        self._tagged = False
        self._workspace: torch.Tensor | None = None
        self._barriers: torch.Tensor | None = None   # the counters of the bound launch: cleared by check() after an error
        self._greedy: tuple[torch.Tensor, torch.Tensor, int] | None = None
        self.timeline: torch.Tensor | None = None
        self._args = QmkArgs()
        self._args.struct_size = ctypes.sizeof(QmkArgs)
        self._args.model = QMK_MODEL_LLAMA_3_2_1B
        self._bound_key: tuple | None = None

    # -- library passthroughs ------------------------------------------------
    def query(self, what: int) -> int:
        return int(self._lib.qmk_query(int(what)))

    def error_string(self, code: int) -> str:
        return self._lib.qmk_error_string(int(code)).decode()

    def check(self, stream: torch.cuda.Stream | None = None) -> None:
        """Synchronise and raise if a kernel reported a device-side error."""
        detail = (_I * 4)()
        handle = (stream or torch.cuda.current_stream()).cuda_stream
        code = int(self._lib.qmk_status_fetch(_P(handle), ctypes.byref(detail)))
        if code != 0:
            # A workgroup that gives up does not retire: the counters, the arrival word and the tagged units are
            # those of a step that never finished, and the next launch would take them for its own.
            if self._workspace is not None:
                self._workspace.zero_()
            if self._barriers is not None:
                self._barriers.zero_()
            raise RuntimeError(
                f"megakernel device error {code} ({self.error_string(code)}): workgroup={detail[0]} "
                f"instruction={detail[1]} opcode={detail[2]} operand={detail[3]}; "
                "the counters (and the workspace) of the aborted step have been cleared"
            )

    def with_options(self, **kw: Any) -> "MegaKernel":
        other = MegaKernel(self._lib, kw.pop("geometry", self.geometry),
                           reset_barriers=kw.pop("reset_barriers", self.reset_barriers),
                           spin_limit=kw.pop("spin_limit", self.spin_limit),
                           xcd_counters=kw.pop("xcd_counters", self.xcd_counters),
                           tagged=kw.pop("tagged", self.tagged),
                           static_scratch=kw.pop("static_scratch", self.static_scratch))
        if kw:
            raise TypeError(f"unknown options {sorted(kw)}")
        return other

    def greedy_into(self, embed_tokens: torch.Tensor, tokens: torch.Tensor, index: int) -> None:
        """The next call also samples: ``tokens.view(-1)[index] = argmax(logits)``, ``hidden_states = embed_tokens[that]``."""
        if not self.reset_barriers:
            raise ValueError("device-side sampling needs the self-clearing counters (reset_barriers=True)")
        if embed_tokens.dtype != torch.bfloat16 or embed_tokens.dim() != 2 or not embed_tokens.is_contiguous():
            raise TypeError("embed_tokens must be a contiguous bf16 [vocab, hidden] tensor")
        if tokens.dtype != torch.int64 or not tokens.is_contiguous():
            raise TypeError("tokens must be a contiguous int64 tensor")
        if embed_tokens.device.type != "cuda" or tokens.device != embed_tokens.device:
            raise ValueError("embed_tokens and tokens must live on the same GPU")
        if not 0 <= index < tokens.numel():
            raise IndexError(f"token index {index} outside a buffer of {tokens.numel()}")
        self._greedy = (embed_tokens, tokens, int(index))

    # -- the call -------------------------------------------------------------
    def _bind(self, tensors: Sequence[torch.Tensor]) -> None:
        a = self._args
        device = tensors[1].device
        shape = LlamaConfig.shape()
        a.model = _model_id(shape)
        qwen = a.model == QMK_MODEL_QWEN3_1_7B
        if len(tensors) != (25 if qwen else 22):
            raise TypeError(f"mk for this model takes {25 if qwen else 22} tensors, got {len(tensors)}")
        spec = _QWEN3_TENSOR_ARGS if qwen else _TENSOR_ARGS
        for (name, dtype, ndim), t in zip(spec, tensors):
            if not isinstance(t, torch.Tensor):
                raise TypeError(f"{name} must be a torch.Tensor, got {type(t).__name__}")
            if t.device.type != "cuda":
                raise ValueError(f"{name} must live on the GPU, got {t.device}")
            if t.device != device:
                raise ValueError(f"{name} is on {t.device}, hidden_states on {device}")
            if t.dtype != dtype:
                raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
            if t.dim() != ndim:
                raise ValueError(f"{name} must have {ndim} dims, got shape {tuple(t.shape)}")
            if not t.is_contiguous():
                raise ValueError(f"{name} must be contiguous")
            setattr(a, name, t.data_ptr())
        if qwen:
            expect_raw, expect_qn, expect_kn = tensors[2], tensors[13], tensors[14]
            tensors = tuple(tensors[:2]) + tuple(tensors[3:13]) + tuple(tensors[15:])
        else:
            a.qkv_raw = a.q_norm_weights = a.k_norm_weights = None
        (instructions, hidden, _q, k_cache, v_cache, _ao, lse, part, silu, logits, attn_norm, qkv, cos, sin, o_w,
         mlp_norm, up, gate, down, lm_norm, lm_w, barriers) = tensors
        L = int(barriers.shape[0])
        self._barriers = barriers
        H, F = shape.hidden_size, shape.intermediate_size

        def expect(name: str, t: torch.Tensor, want: tuple[int, ...]) -> None:
            if tuple(t.shape) != want:
                raise ValueError(f"{name} has shape {tuple(t.shape)}, the kernel needs {want}")

        if instructions.shape[2] != 32:
            raise ValueError("instructions must be [queues, length, 32]")
        expect("hidden_states", hidden, (H,))
        if qwen:
            expect("qkv_raw", expect_raw, (shape.qkv_out_dim,))
            expect("q_norm_weights", expect_qn, (L, shape.head_dim))
            expect("k_norm_weights", expect_kn, (L, shape.head_dim))
        expect("q_post_rope", tensors[2], (shape.num_attention_heads * shape.head_dim,))
        expect("attn_out", tensors[5], (shape.num_attention_heads * shape.head_dim,))
        expect("silu_out", silu, (F,))
        S = int(k_cache.shape[2])
        expect("k_cache", k_cache, (L, 1, S, shape.num_key_value_heads, shape.head_dim))
        expect("v_cache", v_cache, (L, 1, S, shape.num_key_value_heads, shape.head_dim))
        P = int(lse.shape[1])
        expect("attn_lse_intermediates", lse, (shape.num_attention_heads, P))
        expect("attn_out_intermediates", part, (shape.num_attention_heads, P, shape.head_dim))
        V = int(logits.shape[0])
        expect("lm_head_weights", lm_w, (V, H))
        expect("lm_head_norm_weights", lm_norm, (H,))
        expect("attn_norm_weights", attn_norm, (L, H))
        expect("mlp_norm_weights", mlp_norm, (L, H))
        expect("qkv_weights", qkv, (L, shape.qkv_out_dim, H))
        expect("o_proj_weights", o_w, (L, H, H))
        expect("up_proj_weights", up, (L, F, H))
        expect("gate_proj_weights", gate, (L, F, H))
        expect("down_proj_weights", down, (L, H, F))
        if cos.shape != sin.shape or cos.shape[1] != shape.head_dim:
            raise ValueError("rope_cos/rope_sin must both be [positions, head_dim]")
        a.num_queues, a.num_insts = int(instructions.shape[0]), int(instructions.shape[1])
        a.num_layers, a.num_layer_barriers, a.barrier_slots = L, int(barriers.shape[1]), int(barriers.shape[2])
        a.max_seq_len, a.max_splits, a.vocab_size, a.rope_rows = S, P, V, int(cos.shape[0])
        geometry = self.geometry or REFERENCE_GEOMETRY
        (a.qkv_blocks_per_head, a.oproj_blocks, a.upgate_blocks_per_bucket, a.down_arrivals) = geometry.expected_counts(shape)
        # Per-XCD sub-counters for the all-to-all edges need room in `barriers` (rows 10..25 of
        # every layer) and a schedule with a single down-projection K slice.
        self._xcd_counters = (
            self.xcd_counters
            and int(barriers.shape[1]) >= QMK_XCD_COUNTER_ROWS
            and int(barriers.shape[2]) == 48
            and barriers.data_ptr() % 128 == 0
            and geometry.num_split_k(shape) == 1
        )
        self._tagged = self.tagged and self.reset_barriers and geometry.num_split_k(shape) == 1 and L <= 63
        if self.static_scratch:
            self._workspace = None
            a.workspace, a.workspace_bytes = None, 0
        elif self._tagged or self.reset_barriers:   # the workspace also carries the greedy candidates
            nbytes = int(self._lib.qmk_workspace_bytes(int(a.model)))
            if self._workspace is None or self._workspace.device != device:
                self._workspace = torch.zeros(nbytes, dtype=torch.uint8, device=device)
            else:
                self._workspace.zero_()
            if self._workspace.data_ptr() % 128 != 0:
                raise RuntimeError("torch returned a workspace that is not 128-byte aligned")
            a.workspace, a.workspace_bytes = self._workspace.data_ptr(), nbytes
        else:
            a.workspace, a.workspace_bytes = None, 0

    def __call__(self, *args: Any) -> None:
        if len(args) not in (25, 28):
            raise TypeError(f"mk takes 22 (Qwen3 op set: 25) tensors and 3 scalars, got {len(args)} positional arguments")
        tensors, (pos_id, attn_scale, rms_norm_eps) = args[:-3], args[-3:]
        if isinstance(tensors[0], torch.Tensor) and tensors[0].numel() == 0:
            return  # empty queues: nothing to launch
        key = tuple((t.data_ptr(), tuple(t.shape)) if isinstance(t, torch.Tensor) else None for t in tensors) + (
            self.geometry, LlamaConfig.shape(), self.tagged, self.reset_barriers, self.xcd_counters, self.static_scratch)
        if key != self._bound_key:
            self._bind(tensors)
            self._bound_key = key
        a = self._args
        a.pos_id = int(pos_id)
        a.attn_scale = float(attn_scale)
        a.rms_norm_eps = float(rms_norm_eps)
        a.flags = ((0 if self.reset_barriers else QMK_FLAG_KEEP_BARRIERS) | (QMK_FLAG_XCD_COUNTERS if self._xcd_counters else 0)
                   | (QMK_FLAG_TAGGED if self._tagged else 0))
        a.spin_limit = self.spin_limit
        a.timeline = self.timeline.data_ptr() if self.timeline is not None else None
        if self._greedy is not None:
            embed, tokens, index = self._greedy
            self._greedy = None
            if tuple(embed.shape) != (a.vocab_size, LlamaConfig.shape().hidden_size) or embed.device != tensors[1].device:
                raise ValueError(f"embed_tokens has shape {tuple(embed.shape)} on {embed.device}; the kernel needs "
                                 f"({a.vocab_size}, {LlamaConfig.shape().hidden_size}) on {tensors[1].device}")
            a.embed_tokens, a.token_out = embed.data_ptr(), tokens.data_ptr() + 8 * index
        else:
            a.embed_tokens, a.token_out = None, None
        a.stream = torch.cuda.current_stream(tensors[1].device).cuda_stream
        step = self._lib.qmk_decode_step_static if self.static_scratch else self._lib.qmk_decode_step
        rc = int(step(ctypes.byref(a)))
        if rc != 0:
            raise RuntimeError(f"{step.__name__} failed with {rc}: {self.error_string(rc)}")


_LIB_CACHE: dict[Path, ctypes.CDLL] = {}


def get_mk(mk_dir: Path | None = None, *, geometry: TileGeometry | None = None, reset_barriers: bool = True,
           spin_limit: int = 0, xcd_counters: bool = True, tagged: bool = True, static_scratch: bool = False) -> MegaKernel:
    """Return the ``mk`` callable bound to the prebuilt library in ``mk_dir``.

    ``geometry`` defaults to the MI355X schedule of this package; pass
    ``REFERENCE_GEOMETRY`` to run instruction tensors built by the A100 scheduler.
    """
    root = (_default_mk_dir() if mk_dir is None else Path(mk_dir)).resolve()
    lib = _LIB_CACHE.get(root)
    if lib is None:
        lib = load_library(root)
        _LIB_CACHE[root] = lib
    if geometry is None:
        geometry = _scheduler.mi355x_scheduler(num_partials=1).geometry
    return MegaKernel(lib, geometry, reset_barriers=reset_barriers, spin_limit=spin_limit, xcd_counters=xcd_counters,
                      tagged=tagged, static_scratch=static_scratch)


def call_mk(globs: Globals, mk: Any) -> None:
    """One decode step with the current ``Globals`` (builds the instruction tensor on first use)."""
    shape = LlamaConfig.shape()
    if globs.instructions is None:
        _scheduler.build(globs)
    qwen = bool(getattr(shape, "qk_norm", False))
    instructions = globs.instructions
    plan = getattr(globs, "instruction_plan", None)
    if plan is not None and plan[0] is instructions:   # streams with a wider split-KV fan-out for the request's later positions
        position = globs.position_id if globs.position_id is not None else 0
        for first, tensor in plan[1]:
            if position >= first:
                instructions = tensor
    mk(
        instructions,
        globs.hidden_states,
        *((globs.qkv_raw,) if qwen else ()),
        globs.q_post_rope,
        _tensor_for_mk(globs.k_cache),
        _tensor_for_mk(globs.v_cache),
        globs.attn_out,
        globs.attn_lse_intermediates,
        globs.attn_out_intermediates,
        globs.silu_out,
        globs.logits,
        globs.attn_norm_weights,
        globs.qkv_weights,
        *((_tensor_for_mk(globs.q_norm_weights), _tensor_for_mk(globs.k_norm_weights)) if qwen else ()),
        globs.rope_cos,
        globs.rope_sin,
        globs.o_proj_weights,
        globs.mlp_norm_weights,
        globs.up_proj_weights,
        globs.gate_proj_weights,
        globs.down_proj_weights,
        globs.lm_head_norm_weights,
        globs.lm_head_weights,
        globs.barriers,
        globs.position_id if globs.position_id is not None else 0,
        1.0 / math.sqrt(shape.head_dim),
        shape.rms_norm_eps,
    )


def run_instructions(globs: Globals, instructions: list[Instruction], *, mk: Any = None,
                     sm_count: int | None = None) -> None:
    """Deal ``instructions`` round-robin onto the workgroup queues and execute them once.

    The counters keep their final values (nothing is cleared), so a caller can
    compare them with a sequential VM run, as the reference's kernel-vs-VM tests do.
    """
    mk_call = get_mk() if mk is None else mk
    if isinstance(mk_call, MegaKernel) and mk_call.reset_barriers:
        mk_call = mk_call.with_options(reset_barriers=False)
    if sm_count is None:
        sm_count = _scheduler._get_sm_count(globs.hidden_states.device)
    queues = _scheduler._round_robin_assign_to_sms(instructions, sm_count)
    _scheduler.tensorize_instructions(globs, queues)
    call_mk(globs, mk_call)
