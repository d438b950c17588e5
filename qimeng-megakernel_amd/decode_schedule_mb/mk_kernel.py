"""Load and call the gfx950 batch decode kernel through its C ABI.

Host-side counterpart of the reference's launcher of the batch route
(`…/A100/multi_batch/decode_schedule/mk_kernel.py:41-111`): ``get_mk`` returns the ``mk``
callable, ``call_mk(globs, mk)`` passes the 22 tensors, ``pos_id, batch_size, attn_scale,
rms_norm_eps``, the three control tensors and the three RMSNorm scratch tensors in the
reference's positional order, ``run_instructions`` executes an arbitrary instruction list.  The
callable wraps ``qmk_decode_step_batch`` of ``libqmk_hip.so`` (``include/qmk.h``) with ctypes.

A shape with the Qwen3 op set (``qk_norm``: Qwen3-1.7B) has no batch route in the reference; its
``mk`` takes three more tensors behind the 32 arguments — ``qkv_raw [B, QKV]``, ``q_norm_weights``,
``k_norm_weights`` — the ones the reference's Qwen3 launcher adds to the batch-1 call
(`…/qwen/qwen3__0_6b/A100/single_batch/decode_schedule/mk_kernel.py`).

There is no fallback: a missing library is an ``ImportError``, a non-GPU tensor a
``ValueError`` and a device-side error a ``RuntimeError``.
"""
from __future__ import annotations

import ctypes
import math
from pathlib import Path
from typing import Any, Sequence

import torch

from ..decode_schedule import mk_kernel as _single
from ..decode_schedule.instructions.scheduler import tensorize_instructions
from ..decode_schedule.model_config import LlamaConfig
from ..instruction import Instruction
from .row_state import rows_of as _batch_size
from .globs import Globals
from .instructions import scheduler as _scheduler

_P = ctypes.c_void_p
_I = ctypes.c_int32
MAX_BATCH = 16


class QmkBatchArgs(ctypes.Structure):
    """Mirror of ``struct QmkBatchArgs`` in include/qmk.h (field order is the ABI)."""

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
        ("pos_id", _I), ("batch_size", _I), ("kv_block_size", _I), ("oproj_blocks", _I), ("down_blocks", _I),
        ("attn_scale", ctypes.c_float), ("rms_norm_eps", ctypes.c_float),
        ("position_ids", _P), ("active_mask", _P), ("attn_partial_valid", _P),
        ("attn_rms_out", _P), ("mlp_rms_out", _P), ("lm_head_rms_out", _P),
        ("timeline", _P), ("stream", _P),
        ("qkv_raw", _P), ("q_norm_weights", _P), ("k_norm_weights", _P),
        ("first_inst", _I), ("inst_count", _I),
    ]


# (name, dtype, ndim) of the 22 tensors, in the positional order of mk(...).
_TENSOR_ARGS: tuple[tuple[str, torch.dtype, int], ...] = (
    ("instructions", torch.int32, 3),
    ("hidden_states", torch.bfloat16, 2),
    ("q_post_rope", torch.bfloat16, 2),
    ("k_cache", torch.bfloat16, 5),
    ("v_cache", torch.bfloat16, 5),
    ("attn_out", torch.bfloat16, 2),
    ("attn_lse_intermediates", torch.float32, 3),
    ("attn_out_intermediates", torch.float32, 4),
    ("silu_out", torch.bfloat16, 2),
    ("logits", torch.bfloat16, 2),
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


def _check(name: str, t: Any, device: torch.device, dtypes: tuple[torch.dtype, ...], shape: tuple[int, ...] | None, ndim: int) -> None:
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor, got {type(t).__name__}")
    if t.device.type != "cuda" or t.device != device:
        raise ValueError(f"{name} must live on {device}, got {t.device}")
    if t.dtype not in dtypes:
        raise TypeError(f"{name} must be {' or '.join(map(str, dtypes))}, got {t.dtype}")
    if t.dim() != ndim:
        raise ValueError(f"{name} must have {ndim} dims, got shape {tuple(t.shape)}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    if shape is not None and tuple(t.shape) != shape:
        raise ValueError(f"{name} has shape {tuple(t.shape)}, the kernel needs {shape}")


class BatchMegaKernel:
    """The ``mk`` callable of the batch route.

    ``reset_barriers``: the kernel clears the counters when it retires (default) or leaves their
    final values in place like the reference kernel, whose host loop zeroes them before every step.
    ``xcd_counters``: the blocks of the O-projection, the up/gate and the down projection are counted on eight
    sub-counters (words 0, 32, .. 224 of their counter row, one 128-byte line per XCD) instead of all on word 0, where
    hundreds of arrivals from eight XCDs queue on one line.  Taken when the kernel clears the counters itself and
    a row has the 256 words (Llama shape: 6 rows and more, Qwen3-1.7B shape: 8 and more); a launch that keeps the counters
    leaves the reference's words.
    """

    XCD_COUNTER_WORDS = 32 * 8

    def __init__(self, lib: ctypes.CDLL, *, reset_barriers: bool = True, spin_limit: int = 0, xcd_counters: bool = True):
        self._lib = lib
        self.reset_barriers = reset_barriers
        self.xcd_counters = xcd_counters
        self.spin_limit = int(spin_limit)
        self.residual_tiles = (16, 16)   # rows per O-proj / down-projection block of the stream (set per call by call_mk)
        self.timeline: torch.Tensor | None = None
        self._args = QmkBatchArgs()
        self._args.struct_size = ctypes.sizeof(QmkBatchArgs)
        self._bound_key: tuple | None = None
        self._barriers: torch.Tensor | None = None   # the counters of the bound launch: cleared by check() after an error
        self._window = (0, 0)            # (first column, columns) of the launch; (0, 0): the whole tensor

    def error_string(self, code: int) -> str:
        return self._lib.qmk_error_string(int(code)).decode()

    def check(self, stream: torch.cuda.Stream | None = None) -> None:
        """Synchronise and raise if a kernel reported a device-side error."""
        detail = (_I * 4)()
        handle = (stream or torch.cuda.current_stream()).cuda_stream
        code = int(self._lib.qmk_status_fetch(_P(handle), ctypes.byref(detail)))
        if code != 0:
            if self._barriers is not None:   # a workgroup that gives up does not retire: the counters are those of an unfinished step
                self._barriers.zero_()
            raise RuntimeError(
                f"megakernel device error {code} ({self.error_string(code)}): workgroup={detail[0]} "
                f"instruction={detail[1]} opcode={detail[2]} operand={detail[3]}; "
                "the counters of the aborted step have been cleared"
            )

    def with_options(self, **kw: Any) -> "BatchMegaKernel":
        other = BatchMegaKernel(self._lib, reset_barriers=kw.pop("reset_barriers", self.reset_barriers),
                                spin_limit=kw.pop("spin_limit", self.spin_limit),
                                xcd_counters=kw.pop("xcd_counters", self.xcd_counters))
        if kw:
            raise TypeError(f"unknown options {sorted(kw)}")
        return other

    def _bind(self, tensors: Sequence[torch.Tensor], B: int, position_ids: Any, active_mask: Any, partial_valid: Any,
              rms: Sequence[Any], qwen3: Sequence[Any] = ()) -> None:
        a = self._args
        shape = LlamaConfig.shape()
        a.model = _single._model_id(shape)
        if a.model not in (_single.QMK_MODEL_LLAMA_3_2_1B, _single.QMK_MODEL_QWEN3_1_7B):
            raise ValueError("the batch route is compiled for the Llama-3.2-1B and Qwen3-1.7B layer geometries only")
        if not 1 <= B <= MAX_BATCH:
            raise ValueError(f"batch_size must be in [1, {MAX_BATCH}], got {B}")
        device = tensors[1].device if isinstance(tensors[1], torch.Tensor) else None
        for (name, dtype, ndim), t in zip(_TENSOR_ARGS, tensors):
            _check(name, t, device, (dtype,), None, ndim)
            setattr(a, name, t.data_ptr())
        (instructions, hidden, q, k_cache, v_cache, ao, lse, part, silu, logits, attn_norm, qkv, cos, sin, o_w,
         mlp_norm, up, gate, down, lm_norm, lm_w, barriers) = tensors
        L = int(barriers.shape[0])
        self._barriers = barriers
        H, F = shape.hidden_size, shape.intermediate_size
        nq, nkv, d = shape.num_attention_heads, shape.num_key_value_heads, shape.head_dim

        def expect(name: str, t: torch.Tensor, want: tuple[int, ...]) -> None:
            if tuple(t.shape) != want:
                raise ValueError(f"{name} has shape {tuple(t.shape)}, the kernel needs {want}")

        if instructions.shape[2] != 32:
            raise ValueError("instructions must be [queues, length, 32]")
        expect("hidden_states", hidden, (B, H))
        expect("q_post_rope", q, (B, nq * d))
        expect("attn_out", ao, (B, nq * d))
        expect("silu_out", silu, (B, F))
        S = int(k_cache.shape[2])
        expect("k_cache", k_cache, (L, B, S, nkv, d))
        expect("v_cache", v_cache, (L, B, S, nkv, d))
        P = int(lse.shape[2])
        expect("attn_lse_intermediates", lse, (B, nq, P))
        expect("attn_out_intermediates", part, (B, nq, P, d))
        V = int(logits.shape[1])
        expect("logits", logits, (B, V))
        expect("lm_head_weights", lm_w, (V, H))
        expect("lm_head_norm_weights", lm_norm, (H,))
        expect("attn_norm_weights", attn_norm, (L, H))
        expect("mlp_norm_weights", mlp_norm, (L, H))
        expect("qkv_weights", qkv, (L, shape.qkv_out_dim, H))
        expect("o_proj_weights", o_w, (L, H, H))
        expect("up_proj_weights", up, (L, F, H))
        expect("gate_proj_weights", gate, (L, F, H))
        expect("down_proj_weights", down, (L, H, F))
        if cos.shape != sin.shape or cos.shape[1] != d:
            raise ValueError("rope_cos/rope_sin must both be [positions, head_dim]")
        if barriers.shape[1] < 10 or barriers.shape[2] < B * (nq + 2 * nkv):
            raise ValueError(f"barriers must be [layers, >= 10, >= {B * (nq + 2 * nkv)}], got {tuple(barriers.shape)}")
        # The control tensors (`…/multi_batch/decode_kernel/mk.cu:112-151`) and the RMSNorm scratch (`:199-216`).
        if position_ids is not None:
            _check("position_ids", position_ids, device, (torch.int32,), (B,), 1)
        if active_mask is not None:
            _check("active_mask", active_mask, device, (torch.uint8, torch.bool), (B,), 1)
        if partial_valid is not None:
            _check("attn_partial_valid", partial_valid, device, (torch.uint8, torch.bool), (B, nq, P), 3)
        for name, t in zip(("attn_rms_out", "mlp_rms_out", "lm_head_rms_out"), rms):
            if t is None:
                raise ValueError(f"{name} must be provided")
            _check(name, t, device, (torch.bfloat16,), (B, H), 2)
            setattr(a, name, t.data_ptr())
        a.qkv_raw = a.q_norm_weights = a.k_norm_weights = None
        if shape.qk_norm:
            if len(qwen3) != 3 or any(t is None for t in qwen3):
                raise ValueError("the Qwen3 op set needs qkv_raw, q_norm_weights and k_norm_weights behind the 32 arguments")
            _check("qkv_raw", qwen3[0], device, (torch.bfloat16,), (B, shape.qkv_out_dim), 2)
            _check("q_norm_weights", qwen3[1], device, (torch.bfloat16,), (L, d), 2)
            _check("k_norm_weights", qwen3[2], device, (torch.bfloat16,), (L, d), 2)
            a.qkv_raw, a.q_norm_weights, a.k_norm_weights = (t.data_ptr() for t in qwen3)
        elif qwen3:
            raise TypeError("qkv_raw / q_norm_weights / k_norm_weights belong to the Qwen3 op set only")
        a.position_ids = position_ids.data_ptr() if position_ids is not None else None
        a.active_mask = active_mask.data_ptr() if active_mask is not None else None
        a.attn_partial_valid = partial_valid.data_ptr() if partial_valid is not None else None
        a.num_queues, a.num_insts = int(instructions.shape[0]), int(instructions.shape[1])
        a.num_layers, a.num_layer_barriers, a.barrier_slots = L, int(barriers.shape[1]), int(barriers.shape[2])
        a.max_seq_len, a.max_splits, a.vocab_size, a.rope_rows = S, P, V, int(cos.shape[0])
        a.batch_size = B
        a.kv_block_size = int(shape.attn_kv_block_size)

    def __call__(self, *args: Any) -> None:
        want = 35 if LlamaConfig.shape().qk_norm else 32
        if len(args) != want:
            raise TypeError(f"mk of the batch route takes 22 tensors, 4 scalars and {want - 26} tensors for this shape, "
                            f"got {len(args)} positional arguments")
        tensors = args[:22]
        pos_id, B, attn_scale, rms_norm_eps = args[22:26]
        position_ids, active_mask, partial_valid = args[26:29]
        rms = args[29:32]
        if isinstance(tensors[0], torch.Tensor) and tensors[0].numel() == 0:
            return
        key = tuple((t.data_ptr(), tuple(t.shape)) if isinstance(t, torch.Tensor) else None for t in (*tensors, *args[26:])) + (
            int(B), LlamaConfig.shape())
        if key != self._bound_key:
            self._bind(tensors, int(B), position_ids, active_mask, partial_valid, rms, args[32:])
            self._bound_key = key
        a = self._args
        a.pos_id = int(pos_id)
        a.attn_scale = float(attn_scale)
        a.rms_norm_eps = float(rms_norm_eps)
        a.flags = 0 if self.reset_barriers else _single.QMK_FLAG_KEEP_BARRIERS
        if self.xcd_counters and self.reset_barriers and a.barrier_slots >= self.XCD_COUNTER_WORDS:
            a.flags |= _single.QMK_FLAG_XCD_COUNTERS
        a.spin_limit = self.spin_limit
        hidden = LlamaConfig.shape().hidden_size
        a.oproj_blocks, a.down_blocks = hidden // self.residual_tiles[0], hidden // self.residual_tiles[1]
        a.timeline = self.timeline.data_ptr() if self.timeline is not None else None
        a.stream = torch.cuda.current_stream(tensors[1].device).cuda_stream
        a.first_inst, a.inst_count = self._window
        self._launch(tensors[1].device)

    # ---- one instruction column per launch (`…/multi_batch/decode_kernel/mk.h:44-115`) ----
    def mk_step(self, *args: Any) -> None:
        """The reference's ``mk_step``: the 22 tensors, then ``inst_idx``, then the arguments of ``mk`` from ``pos_id``
        on; runs column ``inst_idx`` of the instruction tensor.  The counters carry the step from one column to the
        next, so this object must have been made with ``reset_barriers=False`` and the caller zeroes them before
        column 0, as the reference's callers do."""
        if self.reset_barriers:
            raise ValueError("mk_step needs counters that outlive a launch: get_mk(reset_barriers=False)")
        inst_idx = int(args[22])
        if not 0 <= inst_idx < int(args[0].shape[1]):
            raise ValueError("mk_step: inst_idx out of range")
        self._window = (inst_idx, 1)
        try:
            self(*args[:22], *args[23:])
        finally:
            self._window = (0, 0)

    def mk_step_loop(self, *args: Any) -> None:
        """The reference's ``mk_step_loop``: the arguments of ``mk``; every column in its own launch, one after the other."""
        for inst_idx in range(int(args[0].shape[1])):
            self.mk_step(*args[:22], inst_idx, *args[22:])

    def _launch(self, device: torch.device) -> None:
        rc = int(self._lib.qmk_decode_step_batch(ctypes.byref(self._args)))
        if rc != 0:
            raise RuntimeError(f"qmk_decode_step_batch failed with {rc}: {self.error_string(rc)}")


def get_mk(mk_dir: Path | None = None, *, reset_barriers: bool = True, spin_limit: int = 0, xcd_counters: bool = True) -> BatchMegaKernel:
    """Return the ``mk`` callable of the batch route bound to the prebuilt library in ``mk_dir``."""
    root = (_single._default_mk_dir() if mk_dir is None else Path(mk_dir)).resolve()
    lib = _single._LIB_CACHE.get(root)
    if lib is None:
        lib = _single.load_library(root)
        _single._LIB_CACHE[root] = lib
    if not hasattr(lib, "qmk_decode_step_batch"):
        raise ImportError(f"{root / 'libqmk_hip.so'} does not export qmk_decode_step_batch")
    lib.qmk_decode_step_batch.argtypes = [ctypes.POINTER(QmkBatchArgs)]
    lib.qmk_decode_step_batch.restype = ctypes.c_int
    return BatchMegaKernel(lib, reset_barriers=reset_barriers, spin_limit=spin_limit, xcd_counters=xcd_counters)


def _mask_for_mk(t: torch.Tensor | None, device: torch.device) -> torch.Tensor | None:
    """`…/multi_batch/decode_schedule/mk_launch_tensors.py:19-26`: on the device, u8 or bool, contiguous."""
    if t is None:
        return None
    if t.device != device:
        t = t.to(device)
    if t.dtype not in (torch.uint8, torch.bool):
        t = t.to(torch.uint8)
    return t if t.is_contiguous() else t.contiguous()


def call_mk(globs: Globals, mk: Any, *, column_by_column: bool = False) -> None:
    """One decode step with the current ``Globals`` (builds the request's instruction tensor on first use).
    ``column_by_column``: through ``mk.mk_step_loop`` — one launch per instruction column, for bisecting a step; the
    caller zeroes ``globs.barriers`` first and ``mk`` keeps the counters (``reset_barriers=False``)."""
    shape = LlamaConfig.shape()
    B = _batch_size(globs)
    device = globs.hidden_states.device
    if globs.instructions is None:
        build(globs)
    position_ids = globs.position_ids
    if position_ids is not None and position_ids.numel() == B:
        if position_ids.device != device or position_ids.dtype != torch.int32:
            position_ids = position_ids.to(device=device, dtype=torch.int32)
        position_ids = position_ids.contiguous()
    else:
        position_ids = None
    active = _mask_for_mk(globs.active_mask, device) if globs.active_mask is not None and globs.active_mask.numel() == B else None
    if isinstance(mk, BatchMegaKernel):
        mk.residual_tiles = tuple(getattr(globs, "residual_tiles", (16, 16)))
    launch = mk.mk_step_loop if column_by_column else mk
    launch(
        globs.instructions,
        globs.hidden_states,
        globs.q_post_rope,
        _single._tensor_for_mk(globs.k_cache),
        _single._tensor_for_mk(globs.v_cache),
        globs.attn_out,
        globs.attn_lse_intermediates,
        globs.attn_out_intermediates,
        globs.silu_out,
        globs.logits,
        globs.attn_norm_weights,
        globs.qkv_weights,
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
        B,
        1.0 / math.sqrt(shape.head_dim),
        shape.rms_norm_eps,
        position_ids,
        active,
        _mask_for_mk(globs.attn_partial_valid, device),
        globs.attn_rms_out,
        globs.mlp_rms_out,
        globs.lm_head_rms_out,
        *((globs.qkv_raw, globs.q_norm_weights, globs.k_norm_weights) if shape.qk_norm else ()),
    )


def build(globs: Globals, kv_capacity: int | None = None) -> torch.Tensor:
    """The request's instruction tensor: the run-time template of the MI355X scheduler (256 queues),
    valid for every step of the request."""
    sched = _scheduler.mi355x_scheduler(_batch_size(globs))
    capacity = int(globs.k_cache.shape[2]) if kv_capacity is None else kv_capacity
    if sched.partials_for_capacity(capacity) > int(globs.attn_lse_intermediates.shape[-1]):
        raise ValueError("attn_lse_intermediates has fewer partial slots than the schedule's split-KV fan-out")
    globs.residual_tiles = (sched.oproj_tile, sched.down_tile)
    return tensorize_instructions(globs, sched.runtime_queues(capacity))


def run_instructions(globs: Globals, instructions: list[Instruction], *, mk: Any = None, workers: int | None = None) -> None:
    """Deal ``instructions`` round-robin onto the queues and execute them once.  The counters keep
    their final values, so a caller can compare them with a sequential VM run."""
    mk_call = get_mk() if mk is None else mk
    if isinstance(mk_call, BatchMegaKernel) and mk_call.reset_barriers:
        mk_call = mk_call.with_options(reset_barriers=False)
    queues = _scheduler.deal(instructions, workers or _scheduler.MI355X_WORKERS)
    # rows per O-proj / down block: what the stream's own instructions say, else what the caller was built with
    tiles = list(getattr(globs, "residual_tiles", (16, 16)))
    for ins in instructions:
        if ins.opcode() in (5, 8):
            tiles[0 if ins.opcode() == 5 else 1] = ins.tile_N_granularity
    globs.residual_tiles = tuple(tiles)
    tensorize_instructions(globs, queues)
    call_mk(globs, mk_call)
