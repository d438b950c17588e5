"""Load and call the gfx950 MoE decode kernels through their C ABI.

Host-side counterpart of the reference's launcher of the MoE route
(`…/qwen/qwen1_5_moe_a2_7b/A100/single_batch/decode_schedule/mk_kernel.py:63-205`): ``get_mk`` returns
the ``mk`` callable, ``call_mk(globs, mk)`` passes the 39 tensors and 3 scalars in the reference's
positional order (its three unused dense-MLP positions included), ``run_instructions`` executes an
arbitrary instruction list.  The callable wraps ``qmk_decode_step_moe`` of ``libqmk_hip.so``
(``include/qmk.h``) with ctypes.  There is no fallback: a missing library is an ``ImportError``, a
non-GPU tensor a ``ValueError`` and a device-side error a ``RuntimeError``.

Two layer geometries are compiled: Qwen1.5-MoE-A2.7B (the reference's route) and Qwen3-30B-A3B, for which the
reference has no route: its ``mk`` here takes the same positional list with ``None`` in the places of the
tensors the model does not have (QKV bias, the six shared-expert tensors) and the three tensors of the Qwen3
op set (``qkv_raw``, ``q_norm_weights``, ``k_norm_weights``) appended behind ``barriers``.
"""
from __future__ import annotations

import ctypes
import math
from pathlib import Path
from typing import Any

import torch

from ..decode_schedule import mk_kernel as _single
from ..decode_schedule.instructions.scheduler import tensorize_instructions
from ..instruction import Instruction
from .globs import Globals
from .instructions import scheduler as _scheduler
from .model_config import QwenMoeConfig

_P = ctypes.c_void_p
_I = ctypes.c_int32
QMK_MODEL_QWEN1_5_MOE_A2_7B = 2
QMK_MODEL_QWEN3_30B_A3B = 3
MI355X_QUEUES = 256
# (hidden, head_dim, query heads, KV heads, QK norm) -> compiled kernel
_MODELS = {(2048, 128, 16, 16, False): QMK_MODEL_QWEN1_5_MOE_A2_7B, (2048, 128, 32, 4, True): QMK_MODEL_QWEN3_30B_A3B}
_QWEN3_EXTRA = ("qkv_raw", "q_norm_weights", "k_norm_weights")
_SHARED = ("shared_expert_gate_proj_weights", "shared_expert_up_proj_weights", "shared_expert_down_proj_weights",
           "shared_expert_silu_out", "shared_out", "shared_expert_gate_weights")

# The positional order of mk(...): name in QmkMoeArgs, or None for the three unused dense-MLP positions.
_TENSOR_ORDER = (
    "instructions", "hidden_states", "normed_hidden_states", "q_post_rope", "k_cache", "v_cache", "attn_out",
    "attn_lse_intermediates", "attn_out_intermediates", "silu_out", "logits", "attn_norm_weights", "qkv_weights", "qkv_bias",
    "rope_cos", "rope_sin", "o_proj_weights", "mlp_norm_weights", None, None, None, "lm_head_norm_weights", "lm_head_weights",
    "router_weights", "router_logits_buf", "expert_indices", "expert_weights", "shared_expert_gate_proj_weights",
    "shared_expert_up_proj_weights", "shared_expert_down_proj_weights", "shared_expert_silu_out", "shared_out",
    "shared_expert_gate_weights", "expert_gate_up_proj_weights", "expert_down_proj_weights", "routed_silu_buffer",
    "routed_out_f32", "routed_out", "barriers",
)
_DTYPES = {"instructions": torch.int32, "attn_lse_intermediates": torch.float32, "attn_out_intermediates": torch.float32,
           "rope_cos": torch.float32, "rope_sin": torch.float32, "router_logits_buf": torch.float32, "expert_indices": torch.int64,
           "expert_weights": torch.float32, "routed_out_f32": torch.float32, "barriers": torch.int32}


class QmkMoeArgs(ctypes.Structure):
    """Mirror of ``struct QmkMoeArgs`` in include/qmk.h (field order is the ABI)."""

    _fields_ = (
        [("struct_size", ctypes.c_uint32), ("model", ctypes.c_uint32), ("flags", ctypes.c_uint32), ("spin_limit", ctypes.c_uint32)]
        + [(name, _P) for name in _TENSOR_ORDER if name is not None]
        + [(name, _I) for name in ("num_queues", "num_insts", "num_layers", "num_layer_barriers", "barrier_slots", "max_seq_len",
                                   "max_splits", "vocab_size", "rope_rows", "pos_id", "num_experts", "top_k", "shared_ffn", "moe_ffn",
                                   "shared_k_slices")]
        + [("attn_scale", ctypes.c_float), ("rms_norm_eps", ctypes.c_float), ("timeline", _P), ("stream", _P), ("workspace", _P),
           ("workspace_bytes", ctypes.c_uint64)]
        + [(name, _P) for name in _QWEN3_EXTRA] + [("norm_topk_prob", _I), ("routed_upgate_tile", _I), ("oproj_tile", _I), ("local_routing", _I),
           ("qkv_tile", _I), ("reserved0", _I)]
    )


class MoeMegaKernel:
    """The ``mk`` callable of the MoE route.  ``reset_barriers``: the kernel clears the counters when it
    retires (default), or leaves their final values like the reference kernel.  ``tagged``: the residual stream
    (combine -> QKV / O-projection / LM head, O-projection -> router / up-gate ops / combine) and q, k, v travel
    as self-announcing tagged units instead of through counters, as on the dense route; whole steps only, so it
    applies when the kernel also clears its counters.  Same values bit for bit, 705 against 603 tok/s."""

    def __init__(self, lib: ctypes.CDLL, *, reset_barriers: bool = True, spin_limit: int = 0, tagged: bool = True,
                 local_routing: bool | None = None):
        self._lib = lib
        #: tagged launches: the routed ops take the routing decision themselves (None: where the model has no shared expert,
        #: i.e. where nothing runs beside the router and the top-k)
        self.local_routing = local_routing
        self.reset_barriers = reset_barriers
        self.tagged = tagged
        self.spin_limit = int(spin_limit)
        self.timeline: torch.Tensor | None = None
        self._workspace: torch.Tensor | None = None
        self._barriers: torch.Tensor | None = None   # the counters of the bound launch: cleared by check() after an error
        self._args = QmkMoeArgs()
        self._args.struct_size = ctypes.sizeof(QmkMoeArgs)
        self._args.model = QMK_MODEL_QWEN1_5_MOE_A2_7B   # rebound per call from the shape
        self._bound_key: tuple | None = None
        self._tagged = False

    def error_string(self, code: int) -> str:
        return self._lib.qmk_error_string(int(code)).decode()

    def check(self, stream: torch.cuda.Stream | None = None) -> None:
        detail = (_I * 4)()
        handle = (stream or torch.cuda.current_stream()).cuda_stream
        code = int(self._lib.qmk_status_fetch(_P(handle), ctypes.byref(detail)))
        if code != 0:
            # A workgroup that gives up does not retire: counters and tagged units are those of an unfinished step.
            if self._workspace is not None:
                self._workspace.zero_()
            if self._barriers is not None:
                self._barriers.zero_()
            raise RuntimeError(
                f"megakernel device error {code} ({self.error_string(code)}): workgroup={detail[0]} "
                f"instruction={detail[1]} opcode={detail[2]} operand={detail[3]}; "
                "the counters (and the workspace) of the aborted step have been cleared"
            )

    def with_options(self, **kw: Any) -> "MoeMegaKernel":
        other = MoeMegaKernel(self._lib, reset_barriers=kw.pop("reset_barriers", self.reset_barriers),
                              spin_limit=kw.pop("spin_limit", self.spin_limit), tagged=kw.pop("tagged", self.tagged),
                              local_routing=kw.pop("local_routing", self.local_routing))
        if kw:
            raise TypeError(f"unknown options {sorted(kw)}")
        return other

    def _bind(self, tensors: dict[str, torch.Tensor | None]) -> None:
        a, s = self._args, QwenMoeConfig.shape()
        key = (s.hidden_size, s.head_dim, s.num_attention_heads, s.num_key_value_heads, bool(s.qk_norm))
        if key not in _MODELS:
            raise ValueError(f"no MoE kernel was compiled for the attention geometry {key} (hidden, head_dim, query heads, KV heads, QK norm)")
        a.model = _MODELS[key]
        absent = set() if s.has_shared_expert else set(_SHARED)
        if not s.qkv_bias:
            absent.add("qkv_bias")
        if not s.qk_norm:
            absent.update(_QWEN3_EXTRA)
        device = tensors["hidden_states"].device
        for name, t in tensors.items():
            if name in absent:
                if t is not None:
                    raise ValueError(f"{name} must be None for this model")
                setattr(a, name, None)
                continue
            if not isinstance(t, torch.Tensor):
                raise TypeError(f"{name} must be a torch.Tensor, got {type(t).__name__}")
            if t.device.type != "cuda" or t.device != device:
                raise ValueError(f"{name} must live on the GPU of hidden_states, got {t.device}")
            want = _DTYPES.get(name, torch.bfloat16)
            if t.dtype != want:
                raise TypeError(f"{name} must be {want}, got {t.dtype}")
            if not t.is_contiguous():
                raise ValueError(f"{name} must be contiguous")
            setattr(a, name, t.data_ptr())
        L, H = int(tensors["barriers"].shape[0]), s.hidden_size
        nq, nkv, d = s.num_attention_heads, s.num_key_value_heads, s.head_dim
        AW, QKV = nq * d, (nq + 2 * nkv) * d
        E, k = int(tensors["router_weights"].shape[1]), int(tensors["expert_indices"].numel())
        Fs = int(tensors["shared_expert_gate_proj_weights"].shape[1]) if s.has_shared_expert else 0
        Fm = int(tensors["routed_silu_buffer"].shape[-1])
        V = int(tensors["logits"].numel())

        def numel(name: str, want: int) -> None:
            if tensors[name].numel() != want:
                raise ValueError(f"{name} has {tensors[name].numel()} elements ({tuple(tensors[name].shape)}), the kernel needs {want}")

        if tensors["instructions"].dim() != 3 or tensors["instructions"].shape[2] != 32:
            raise ValueError("instructions must be [queues, length, 32]")
        S = int(tensors["k_cache"].shape[2])
        P = int(tensors["attn_lse_intermediates"].shape[-1])
        sizes = [("hidden_states", H), ("normed_hidden_states", H), ("q_post_rope", AW), ("attn_out", AW), ("silu_out", Fm),
                 ("k_cache", L * S * nkv * d), ("v_cache", L * S * nkv * d), ("attn_lse_intermediates", nq * P),
                 ("attn_out_intermediates", nq * P * d), ("attn_norm_weights", L * H), ("mlp_norm_weights", L * H),
                 ("qkv_weights", L * QKV * H), ("o_proj_weights", L * H * AW),
                 ("lm_head_norm_weights", H), ("lm_head_weights", V * H), ("router_weights", L * E * H),
                 ("router_logits_buf", E), ("expert_weights", k),
                 ("expert_gate_up_proj_weights", L * E * 2 * Fm * H), ("expert_down_proj_weights", L * E * H * Fm),
                 ("routed_silu_buffer", k * Fm), ("routed_out_f32", H), ("routed_out", H)]
        if s.qkv_bias:
            sizes.append(("qkv_bias", L * QKV))
        if s.has_shared_expert:
            sizes += [("shared_expert_gate_proj_weights", L * Fs * H), ("shared_expert_up_proj_weights", L * Fs * H),
                      ("shared_expert_down_proj_weights", L * H * Fs), ("shared_expert_silu_out", Fs), ("shared_out", H),
                      ("shared_expert_gate_weights", L * H)]
        if s.qk_norm:
            sizes += [("qkv_raw", QKV), ("q_norm_weights", L * d), ("k_norm_weights", L * d)]
        for name, want in sizes:
            numel(name, want)
        if tensors["rope_cos"].shape != tensors["rope_sin"].shape or tensors["rope_cos"].shape[-1] != d:
            raise ValueError("rope_cos/rope_sin must both be [positions, head_dim]")
        bar = tensors["barriers"]
        self._barriers = bar
        if bar.dim() != 3 or bar.shape[1] < 15 or bar.shape[2] < 128:
            raise ValueError(f"barriers must be [layers, >= 15, >= 128], got {tuple(bar.shape)}")
        a.num_queues, a.num_insts = int(tensors["instructions"].shape[0]), int(tensors["instructions"].shape[1])
        a.num_layers, a.num_layer_barriers, a.barrier_slots = L, int(bar.shape[1]), int(bar.shape[2])
        a.max_seq_len, a.max_splits, a.vocab_size, a.rope_rows = S, P, V, int(tensors["rope_cos"].shape[0])
        a.num_experts, a.top_k, a.shared_ffn, a.moe_ffn = E, k, Fs, Fm
        a.shared_k_slices = int(s.num_downproj_split_k_shared) if s.has_shared_expert else 0
        a.norm_topk_prob, a.routed_upgate_tile, a.oproj_tile = int(bool(s.norm_topk_prob)), int(s.routed_upgate_tile), int(s.oproj_tile)
        a.local_routing = int(self.local_routing if self.local_routing is not None else not s.has_shared_expert)
        a.qkv_tile = int(s.qkv_tile)
        nbytes = int(self._lib.qmk_moe_workspace_bytes(k, a.shared_k_slices))
        if nbytes == 0:
            raise ValueError(f"top_k {k} / {a.shared_k_slices} K slices are outside what the kernel supports")
        if self._workspace is None or self._workspace.device != device or self._workspace.numel() < nbytes:
            self._workspace = torch.zeros(nbytes, dtype=torch.uint8, device=device)
        a.workspace, a.workspace_bytes = self._workspace.data_ptr(), nbytes

    def __call__(self, *args: Any) -> None:
        order = _TENSOR_ORDER + (_QWEN3_EXTRA if len(args) == len(_TENSOR_ORDER) + 3 + len(_QWEN3_EXTRA) else ())
        if len(args) != len(order) + 3:
            raise TypeError(f"mk of the MoE route takes {len(_TENSOR_ORDER)} tensors (with the Qwen3 op set's attention "
                            f"{len(_TENSOR_ORDER) + len(_QWEN3_EXTRA)}) and 3 scalars, got {len(args)} positional arguments")
        tensors = {name: t for name, t in zip(order, args) if name is not None}
        for name in _QWEN3_EXTRA:
            tensors.setdefault(name, None)
        pos_id, attn_scale, rms_norm_eps = args[len(order):]
        if isinstance(tensors["instructions"], torch.Tensor) and tensors["instructions"].numel() == 0:
            return
        key = tuple((t.data_ptr(), tuple(t.shape)) if isinstance(t, torch.Tensor) else None for t in tensors.values()) + (QwenMoeConfig.shape(),)
        if key != self._bound_key:
            self._bind(tensors)
            self._bound_key = key
        a = self._args
        a.pos_id, a.attn_scale, a.rms_norm_eps = int(pos_id), float(attn_scale), float(rms_norm_eps)
        self._tagged = self.tagged and self.reset_barriers and a.num_layers <= 63
        a.flags = (0 if self.reset_barriers else _single.QMK_FLAG_KEEP_BARRIERS) | (_single.QMK_FLAG_TAGGED if self._tagged else 0)
        a.spin_limit = self.spin_limit
        a.timeline = self.timeline.data_ptr() if self.timeline is not None else None
        a.stream = torch.cuda.current_stream(tensors["hidden_states"].device).cuda_stream
        rc = int(self._lib.qmk_decode_step_moe(ctypes.byref(a)))
        if rc != 0:
            raise RuntimeError(f"qmk_decode_step_moe failed with {rc}: {self.error_string(rc)}")


def get_mk(mk_dir: Path | None = None, *, reset_barriers: bool = True, spin_limit: int = 0, tagged: bool = True,
           local_routing: bool | None = None) -> MoeMegaKernel:
    """Return the ``mk`` callable of the MoE route bound to the prebuilt library in ``mk_dir``."""
    root = (_single._default_mk_dir() if mk_dir is None else Path(mk_dir)).resolve()
    lib = _single._LIB_CACHE.get(root)
    if lib is None:
        lib = _single.load_library(root)
        _single._LIB_CACHE[root] = lib
    for name in ("qmk_decode_step_moe", "qmk_moe_workspace_bytes"):
        if not hasattr(lib, name):
            raise ImportError(f"{root / 'libqmk_hip.so'} does not export {name}")
    lib.qmk_decode_step_moe.argtypes = [ctypes.POINTER(QmkMoeArgs)]
    lib.qmk_decode_step_moe.restype = ctypes.c_int
    lib.qmk_moe_workspace_bytes.argtypes = [ctypes.c_int, ctypes.c_int]
    lib.qmk_moe_workspace_bytes.restype = ctypes.c_uint64
    return MoeMegaKernel(lib, reset_barriers=reset_barriers, spin_limit=spin_limit, tagged=tagged, local_routing=local_routing)


def call_mk(globs: Globals, mk: Any) -> None:
    """One decode step with the current ``Globals`` (builds the instruction tensor on first use)."""
    s = QwenMoeConfig.shape()
    if globs.instructions is None:
        build(globs, mk)
    unused = globs.hidden_states          # the three dense-MLP positions of the reference's argument list
    g = globs
    mk(g.instructions, g.hidden_states, g.normed_hidden_states, g.q_post_rope, g.k_cache, g.v_cache, g.attn_out,
       g.attn_lse_intermediates, g.attn_out_intermediates, g.silu_out, g.logits, g.attn_norm_weights, g.qkv_weights, g.qkv_bias,
       g.rope_cos, g.rope_sin, g.o_proj_weights, g.mlp_norm_weights, unused, unused, unused, g.lm_head_norm_weights, g.lm_head_weights,
       g.router_weights, g.router_logits_buf, g.expert_indices, g.expert_weights, g.shared_expert_gate_proj_weights,
       g.shared_expert_up_proj_weights, g.shared_expert_down_proj_weights, g.shared_expert_silu_out, g.shared_out,
       g.shared_expert_gate_weights, g.expert_gate_up_proj_weights, g.expert_down_proj_weights, g.routed_silu_buffer,
       g.routed_out_f32, g.routed_out, g.barriers,
       *((g.qkv_raw, g.q_norm_weights, g.k_norm_weights) if s.qk_norm else ()),
       g.position_id if g.position_id is not None else 0, 1.0 / math.sqrt(s.head_dim), float(s.rms_norm_eps))


def mi355x_scheduler(shape: Any = None, *, tagged: bool = True, kv_capacity: int | None = None) -> _scheduler.MoeScheduler:
    """One queue per CU; both up/gate phases ahead of both down projections; the instructions of a layer placed
    by role (the queues of the router and the top-k take no shared up/gate rows); eight experts per router
    instruction; few split-KV partials per KV head, merged by the O-projection workgroups themselves
    (Qwen1.5 shape, contexts up to 263: 753 tok/s with 8 partials, against 728 with 16 and 719 with the merge by the
    last split-KV arrival; Qwen3-30B-A3B shape, 4 KV heads: 2 partials, 4 when the request's cache holds more than 256
    tokens — a 512-token request: 492 against 487 tok/s, 3 % at its long end; 6 and 8 cost the O-projection a second
    round of partial reads); a routed down projection
    waits for its own slot only.  ``tagged``: the stream is for launches with QMK_FLAG_TAGGED, where the consumers of
    the routing decision take it themselves, the top-k instruction (a report for the caller) runs in the next layer's
    attention phase, and — without a shared expert — one routed down-projection instruction takes all expert slots of
    its 8 rows and commits them, so the stream has no combine instructions; a launch on counters needs the stream
    built with ``tagged=False``: top-k in front of its consumers, down projections per slot, combine instructions."""
    from .model_config import num_partials_for

    shape = shape or QwenMoeConfig.shape()
    few = 2 if kv_capacity is None or kv_capacity <= 256 else 4
    partials = min(8 if shape.num_key_value_heads > 4 else few, num_partials_for(MI355X_QUEUES, shape))
    return _scheduler.MoeScheduler(shape, MI355X_QUEUES, partials, interleave_experts=True, merge_in_oproj=True, router_span=8,
                                   placed=True, down_per_slot=True, topk_late=tagged and not shape.has_shared_expert,
                                   commit_in_down=tagged and not shape.has_shared_expert)


def build(globs: Globals, mk: Any = None) -> torch.Tensor:
    """The instruction tensor of a request; ``mk``: the callable it is built for (a launch on counters gets a stream
    whose top-k instruction precedes its consumers)."""
    tagged = True
    if isinstance(mk, MoeMegaKernel):
        tagged = mk.tagged and mk.reset_barriers and QwenMoeConfig.shape().num_hidden_layers <= 63 and mk.local_routing is not False
    sched = mi355x_scheduler(tagged=tagged, kv_capacity=int(globs.k_cache.shape[2]))
    if sched.num_partials > int(globs.attn_lse_intermediates.shape[-1]):
        raise ValueError("attn_lse_intermediates has fewer partial slots than the schedule's split-KV fan-out")
    return tensorize_instructions(globs, sched.queues())


def run_instructions(globs: Globals, instructions: list[Instruction], *, mk: Any = None, queues: int | None = None) -> None:
    """Deal ``instructions`` round-robin onto the queues and execute them once, counters kept."""
    mk_call = get_mk() if mk is None else mk
    if isinstance(mk_call, MoeMegaKernel) and mk_call.reset_barriers:
        mk_call = mk_call.with_options(reset_barriers=False)
    tensorize_instructions(globs, _scheduler.deal(instructions, queues or MI355X_QUEUES))
    call_mk(globs, mk_call)
