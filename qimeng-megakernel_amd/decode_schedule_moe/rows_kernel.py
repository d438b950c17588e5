"""Several MoE requests ("rows") in ONE launch per step: buffers, launcher and schedule.

The reference has no MoE route for batch sizes above one; its batch route is dense
(`…/llama3_2__1b/A100/multi_batch/decode_schedule/mk_kernel.py:56-111`).  Here a step of B requests is the
batch-1 MoE route (`…/qwen1_5_moe_a2_7b/A100/single_batch/decode_schedule/mk_kernel.py:63-205`) run for every
row on that row's own buffers — same tokens, logits and caches as the row decoded alone, bit for bit — but in one
launch (``qmk_decode_step_moe_rows`` of ``libqmk_hip.so``), which reads the attention weights, the router and the LM
head once per step and each expert once for all the rows that picked it.

Every per-request buffer of the batch-1 ``Globals`` gets a leading row dimension (``hidden_states [B, H]``,
``k_cache [B, L, 1, S, Hkv, D]``, ``logits [B, V]`` …); ``row_view(globs, r)`` is row r's slice as a batch-1
``Globals`` over the same memory, which is what the tests run the batch-1 kernel and the oracle on.
"""
from __future__ import annotations

import ctypes
import math
from pathlib import Path
from typing import Any

import torch

from ..decode_schedule import mk_kernel as _single
from ..decode_schedule.instructions.scheduler import tensorize_instructions
from . import mk_kernel as _moe
from .globs import Globals
from .instructions import scheduler as _scheduler
from .model_config import QwenMoeConfig

_P = ctypes.c_void_p
_I = ctypes.c_int32
MAX_ROWS = 4

#: the buffers of ``Globals`` that belong to a request (leading row dimension); everything else exists once
ROW_BUFFERS = ("hidden_states", "normed_hidden_states", "q_post_rope", "k_cache", "v_cache", "attn_out", "attn_lse_intermediates",
               "attn_out_intermediates", "silu_out", "logits", "qkv_raw", "router_logits_buf", "expert_indices", "expert_weights",
               "routed_silu_buffer", "routed_out_f32", "routed_out")


class QmkMoeRowsArgs(ctypes.Structure):
    """Mirror of ``struct QmkMoeRowsArgs`` in include/qmk.h."""

    _fields_ = [("struct_size", ctypes.c_uint32), ("batch_size", _I), ("position_ids", _P), ("distinct_experts", _P),
                ("step", _moe.QmkMoeArgs)]


def build_rows_globals(weights: dict[str, torch.Tensor], shape: Any, kv_capacity: int, rows: int, device: torch.device | str, *,
                       max_partials: int = 8) -> Globals:
    """Buffers for ``rows`` requests over one copy of ``weights``: the batch-1 buffers with a leading row dimension,
    plus ``position_ids`` (int32 [rows]) and ``distinct_experts`` (int32 [L]: what the last launch streamed)."""
    from .. import synthetic

    if not 1 <= rows <= MAX_ROWS:
        raise ValueError(f"1..{MAX_ROWS} rows")
    g = synthetic.build_moe_globals(weights, shape, kv_capacity, device, max_partials=max_partials)
    for name in ROW_BUFFERS:
        t = getattr(g, name, None)
        if t is not None:
            setattr(g, name, torch.zeros((rows,) + tuple(t.shape), dtype=t.dtype, device=t.device))
    g.position_ids = torch.zeros(rows, dtype=torch.int32, device=g.hidden_states.device)
    g.distinct_experts = torch.zeros(shape.num_hidden_layers, dtype=torch.int32, device=g.hidden_states.device)
    return g


def row_view(globs: Globals, row: int) -> Globals:
    """Row ``row`` of a rows ``Globals`` as a batch-1 ``Globals`` over the same memory (its own counters: the batch-1
    kernel and the oracle that run on a view must not touch the rows launch's)."""
    import dataclasses

    view = dataclasses.replace(globs)
    for name in ROW_BUFFERS:
        t = getattr(globs, name, None)
        if t is not None:
            setattr(view, name, t[row])
    view.barriers = torch.zeros_like(globs.barriers)
    view.instructions = None
    view.embed_tokens = globs.embed_tokens
    view.position_id = 0
    return view


class MoeRowsMegaKernel:
    """The callable of the rows route: ``mk(globs)`` launches one step for all rows of ``globs`` at ``globs.position_ids``.
    Tagged hand-over and self-clearing counters always; the workspace (one set of tagged units per row) belongs to
    this object.  A missing library is an ``ImportError``, a device-side error a ``RuntimeError`` from ``check()``."""

    def __init__(self, lib: ctypes.CDLL, *, spin_limit: int = 0):
        self._lib = lib
        self.spin_limit = int(spin_limit)
        self.timeline: torch.Tensor | None = None
        self._workspace: torch.Tensor | None = None
        self._barriers: torch.Tensor | None = None
        self._args = QmkMoeRowsArgs()
        self._args.struct_size = ctypes.sizeof(QmkMoeRowsArgs)
        self._args.step.struct_size = ctypes.sizeof(_moe.QmkMoeArgs)
        self._bound_key: tuple | None = None

    def error_string(self, code: int) -> str:
        return self._lib.qmk_error_string(int(code)).decode()

    def check(self, stream: torch.cuda.Stream | None = None) -> None:
        detail = (_I * 4)()
        handle = (stream or torch.cuda.current_stream()).cuda_stream
        code = int(self._lib.qmk_status_fetch(_P(handle), ctypes.byref(detail)))
        if code != 0:
            if self._workspace is not None:
                self._workspace.zero_()
            if self._barriers is not None:
                self._barriers.zero_()
            raise RuntimeError(
                f"megakernel device error {code} ({self.error_string(code)}): workgroup={detail[0]} "
                f"instruction={detail[1]} opcode={detail[2]} operand={detail[3]}; "
                "the counters and the workspace of the aborted step have been cleared"
            )

    def _bind(self, g: Globals) -> None:
        r, a, s = self._args, self._args.step, QwenMoeConfig.shape()
        key = (s.hidden_size, s.head_dim, s.num_attention_heads, s.num_key_value_heads, bool(s.qk_norm))
        if key not in _moe._MODELS or s.has_shared_expert:
            raise ValueError(f"no rows kernel was compiled for the geometry {key} (models without a shared expert only)")
        a.model = _moe._MODELS[key]
        B = int(g.hidden_states.shape[0])
        device = g.hidden_states.device
        L, H = int(g.barriers.shape[0]), s.hidden_size
        nq, nkv, d = s.num_attention_heads, s.num_key_value_heads, s.head_dim
        AW, QKV = nq * d, (nq + 2 * nkv) * d
        E, k = int(g.router_weights.shape[1]), int(g.expert_indices.shape[-1])
        Fm, V = int(g.routed_silu_buffer.shape[-1]), int(g.logits.shape[-1])
        S, P = int(g.k_cache.shape[3]), int(g.attn_lse_intermediates.shape[-1])
        absent = set(_moe._SHARED) | ({"qkv_bias"} if not s.qkv_bias else set()) | (set(_moe._QWEN3_EXTRA) if not s.qk_norm else set())
        sizes = {"hidden_states": B * H, "normed_hidden_states": B * H, "q_post_rope": B * AW, "attn_out": B * AW, "silu_out": B * Fm,
                 "k_cache": B * L * S * nkv * d, "v_cache": B * L * S * nkv * d, "attn_lse_intermediates": B * nq * P,
                 "attn_out_intermediates": B * nq * P * d, "logits": B * V, "router_logits_buf": B * E, "expert_indices": B * k,
                 "expert_weights": B * k, "routed_silu_buffer": B * k * Fm, "routed_out_f32": B * H, "routed_out": B * H,
                 "qkv_raw": B * QKV, "attn_norm_weights": L * H, "mlp_norm_weights": L * H, "qkv_weights": L * QKV * H,
                 "o_proj_weights": L * H * AW, "lm_head_norm_weights": H, "lm_head_weights": V * H, "router_weights": L * E * H,
                 "expert_gate_up_proj_weights": L * E * 2 * Fm * H, "expert_down_proj_weights": L * E * H * Fm,
                 "q_norm_weights": L * d, "k_norm_weights": L * d}
        for name in [n for n in _moe._TENSOR_ORDER if n is not None] + list(_moe._QWEN3_EXTRA):
            t = getattr(g, name, None)
            if name in absent:
                if t is not None:
                    raise ValueError(f"{name} must be None for this model")
                setattr(a, name, None)
                continue
            if not isinstance(t, torch.Tensor):
                raise TypeError(f"{name} must be a torch.Tensor, got {type(t).__name__}")
            if t.device != device or t.device.type != "cuda":
                raise ValueError(f"{name} must live on the GPU of hidden_states, got {t.device}")
            want = _moe._DTYPES.get(name, torch.bfloat16)
            if t.dtype != want:
                raise TypeError(f"{name} must be {want}, got {t.dtype}")
            if not t.is_contiguous():
                raise ValueError(f"{name} must be contiguous")
            if name in sizes and t.numel() != sizes[name]:
                raise ValueError(f"{name} has {t.numel()} elements ({tuple(t.shape)}), the kernel needs {sizes[name]}")
            setattr(a, name, t.data_ptr())
        if g.instructions.dim() != 3 or g.instructions.shape[2] != 32:
            raise ValueError("instructions must be [queues, length, 32]")
        if g.position_ids.dtype != torch.int32 or g.position_ids.numel() != B or g.position_ids.device != device:
            raise ValueError("position_ids must be int32 [rows] on the GPU")
        if g.distinct_experts is not None and (g.distinct_experts.dtype != torch.int32 or g.distinct_experts.numel() < L):
            raise ValueError("distinct_experts must be int32 [layers]")
        if g.rope_cos.shape != g.rope_sin.shape or g.rope_cos.shape[-1] != d:
            raise ValueError("rope_cos/rope_sin must both be [positions, head_dim]")
        bar = g.barriers
        if bar.dim() != 3 or bar.shape[1] < 15 or bar.shape[2] < B * nq:
            raise ValueError(f"barriers must be [layers, >= 15, >= rows x query heads = {B * nq}], got {tuple(bar.shape)}")
        self._barriers = bar
        a.num_queues, a.num_insts = int(g.instructions.shape[0]), int(g.instructions.shape[1])
        a.num_layers, a.num_layer_barriers, a.barrier_slots = L, int(bar.shape[1]), int(bar.shape[2])
        a.max_seq_len, a.max_splits, a.vocab_size, a.rope_rows = S, P, V, int(g.rope_cos.shape[0])
        a.num_experts, a.top_k, a.shared_ffn, a.moe_ffn, a.shared_k_slices = E, k, 0, Fm, 0
        a.norm_topk_prob, a.routed_upgate_tile, a.oproj_tile, a.local_routing = int(bool(s.norm_topk_prob)), 0, int(s.oproj_tile), 1
        a.qkv_tile = int(s.qkv_tile)
        a.flags = _single.QMK_FLAG_TAGGED
        nbytes = int(self._lib.qmk_moe_rows_workspace_bytes(B))
        if nbytes == 0:
            raise ValueError(f"{B} rows are outside what the kernel supports")
        if self._workspace is None or self._workspace.device != device or self._workspace.numel() < nbytes:
            self._workspace = torch.zeros(nbytes, dtype=torch.uint8, device=device)
        a.workspace, a.workspace_bytes = self._workspace.data_ptr(), nbytes
        r.batch_size = B
        r.position_ids = g.position_ids.data_ptr()
        r.distinct_experts = g.distinct_experts.data_ptr() if g.distinct_experts is not None else None

    def __call__(self, g: Globals) -> None:
        if g.instructions is None:
            build(g)
        if g.instructions.numel() == 0:
            return
        names = [n for n in _moe._TENSOR_ORDER if n is not None] + list(_moe._QWEN3_EXTRA) + ["position_ids", "distinct_experts"]
        key = tuple((t.data_ptr(), tuple(t.shape)) if isinstance(t, torch.Tensor) else None for t in (getattr(g, n, None) for n in names))
        key += (QwenMoeConfig.shape(),)
        if key != self._bound_key:
            self._bind(g)
            self._bound_key = key
        a, s = self._args.step, QwenMoeConfig.shape()
        a.attn_scale, a.rms_norm_eps = 1.0 / math.sqrt(s.head_dim), float(s.rms_norm_eps)
        a.spin_limit = self.spin_limit
        a.timeline = self.timeline.data_ptr() if self.timeline is not None else None
        a.stream = torch.cuda.current_stream(g.hidden_states.device).cuda_stream
        rc = int(self._lib.qmk_decode_step_moe_rows(ctypes.byref(self._args)))
        if rc != 0:
            raise RuntimeError(f"qmk_decode_step_moe_rows failed with {rc}: {self.error_string(rc)}")


def get_mk(mk_dir: Path | None = None, *, spin_limit: int = 0) -> MoeRowsMegaKernel:
    root = (_single._default_mk_dir() if mk_dir is None else Path(mk_dir)).resolve()
    lib = _single._LIB_CACHE.get(root)
    if lib is None:
        lib = _single.load_library(root)
        _single._LIB_CACHE[root] = lib
    for name in ("qmk_decode_step_moe_rows", "qmk_moe_rows_workspace_bytes"):
        if not hasattr(lib, name):
            raise ImportError(f"{root / 'libqmk_hip.so'} does not export {name}")
    lib.qmk_decode_step_moe_rows.argtypes = [ctypes.POINTER(QmkMoeRowsArgs)]
    lib.qmk_decode_step_moe_rows.restype = ctypes.c_int
    lib.qmk_moe_rows_workspace_bytes.argtypes = [ctypes.c_int]
    lib.qmk_moe_rows_workspace_bytes.restype = ctypes.c_uint64
    return MoeRowsMegaKernel(lib, spin_limit=spin_limit)


def mi355x_scheduler(rows: int, shape: Any = None, *, kv_capacity: int | None = None, queues: int = _moe.MI355X_QUEUES,
                     num_partials: int | None = None, merge_in_oproj: bool = False) -> _scheduler.MoeRowsScheduler:
    """One queue per CU.  Split-KV fan-out: the batch-1 stream's (2 slices per KV head, 4 when the request's cache holds
    more than 256 tokens) as long as rows x KV heads x slices stays within a quarter of the queues.  The partials of a
    (row, KV head) are merged by the group's last arrival (``merge_in_oproj=True``: by every O-projection workgroup, as
    in the batch-1 stream — with several rows that is four trips to memory per workgroup instead of one)."""
    shape = shape or QwenMoeConfig.shape()
    if num_partials is None:
        few = 2 if kv_capacity is None or kv_capacity <= 256 else 4
        num_partials = max(1, min(few, queues // (4 * rows * shape.num_key_value_heads)))
    return _scheduler.MoeRowsScheduler(shape, queues, num_partials, rows, merge_in_oproj=merge_in_oproj)


def build(globs: Globals, *, queues: int = _moe.MI355X_QUEUES, num_partials: int | None = None, merge_in_oproj: bool = False) -> torch.Tensor:
    """The instruction tensor of a batch of requests."""
    rows = int(globs.hidden_states.shape[0])
    sched = mi355x_scheduler(rows, kv_capacity=int(globs.k_cache.shape[3]), queues=queues, num_partials=num_partials,
                             merge_in_oproj=merge_in_oproj)
    if sched.num_partials > int(globs.attn_lse_intermediates.shape[-1]):
        raise ValueError("attn_lse_intermediates has fewer partial slots than the schedule's split-KV fan-out")
    return tensorize_instructions(globs, sched.queues())
