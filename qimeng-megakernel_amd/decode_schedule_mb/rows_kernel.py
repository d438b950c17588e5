"""The batch route at 1..4 rows on the batch-1 kernel's row-streaming engine (``qmk_decode_step_rows``).

At these batch sizes the 16-column matrix-core tiles of the batch kernel are mostly empty and its hand-overs cost more
than its arithmetic; here every weight row is streamed once, as in the batch-1 kernel, and multiplied with every row's
activation vector.  Same ``Globals`` as the batch route (`…/llama3_2__1b/A100/multi_batch/decode_schedule/globs.py`,
``position_ids`` / ``active_mask`` included), but the instruction stream is the batch-1 route's
(`…/single_batch/decode_schedule/instructions/scheduler.py:138-358`) with one split-KV instruction per (row, KV head,
slice).  The reference has no counterpart of this stream: a step is its batch-1 route run for every active row, and the
kernel reproduces that row's results bit for bit.  A missing library is an ``ImportError``; there is no fallback.
"""
from __future__ import annotations

import ctypes
import dataclasses
from dataclasses import dataclass
from pathlib import Path
from typing import Any

import torch

from ..decode_schedule import mk_kernel as _single
from ..decode_schedule.instructions import scheduler as _dense
from ..decode_schedule.instructions.instruction_defs import DecodeAttentionSplitKV
from ..decode_schedule.model_config import LlamaConfig
from ..instruction import Instruction
from . import mk_kernel as _mb
from .globs import Globals

_P = ctypes.c_void_p
MAX_ROWS = 4


class QmkRowsArgs(ctypes.Structure):
    """Mirror of ``struct QmkRowsArgs`` in include/qmk.h."""

    _fields_ = [("struct_size", ctypes.c_uint32), ("qkv_blocks_per_head", ctypes.c_int32), ("workspace", _P),
                ("workspace_bytes", ctypes.c_uint64), ("step", _mb.QmkBatchArgs)]


@dataclass
class DecodeAttentionSplitKVRow(DecodeAttentionSplitKV):
    """Opcode 2 for one row of the batch: the batch-1 instruction on that row's buffers at that row's position."""

    batch_row: int = 0


@dataclass(frozen=True)
class RowsScheduler:
    """One step of ``rows`` requests: the batch-1 MI355X stream (QKV tiles, O-projection, up/gate blocks, down
    projection, LM head: each instruction for all rows) with one split-KV instruction per (row, KV head, slice).
    ``merge_in_oproj``: every O-projection workgroup merges every row's partials itself (the batch-1 default: one trip
    to memory per row and workgroup); otherwise the last split-KV arrival of a (row, KV head) merges its group."""

    dense: _dense.DecodeScheduler
    rows: int
    merge_in_oproj: bool = False

    @property
    def num_partials(self) -> int:
        return self.dense.num_partials

    def layer(self, layer: int) -> list[Instruction]:
        d = self.dense
        mode = _dense.ATTENTION_MERGE_MODES["oproj" if self.merge_in_oproj else "last"]
        attention = [DecodeAttentionSplitKVRow(layer, h, d.num_partials, part, mode, batch_row=r)
                     for r in range(self.rows) for h in range(d.shape.num_key_value_heads) for part in range(d.num_partials)]
        return [*d.qkvproj(layer), *attention, *d.oproj(layer), *d.upgate(layer), *d.downproj(layer)]

    def instruction_list(self, num_layers: int | None = None) -> list[Instruction]:
        layers = self.dense.shape.num_hidden_layers if num_layers is None else num_layers
        out: list[Instruction] = []
        for layer in range(layers):
            out += self.layer(layer)
        if layers == self.dense.shape.num_hidden_layers:
            out += self.dense.lmhead()
        return out

    def queues(self, num_layers: int | None = None) -> list[list[Instruction]]:
        return _dense._round_robin_assign_to_sms(self.instruction_list(num_layers), self.dense.sm_count)


def mi355x_scheduler(rows: int, shape: Any = None, *, kv_capacity: int | None = None, queues: int = _dense.MI355X_CU_COUNT,
                     num_partials: int | None = None, merge_in_oproj: bool = False) -> RowsScheduler:
    """One queue per CU; the split-KV fan-out of the batch-1 stream as long as rows x KV heads x slices stays within half
    of the queues (Llama shape, 4 rows, context 900: a layer takes 44.0 us with 4 slices per KV head, 45.6 with 2, 47.9 with 1)."""
    if not 1 <= rows <= MAX_ROWS:
        raise ValueError(f"1..{MAX_ROWS} rows")
    shape = shape or LlamaConfig.shape()
    if num_partials is None:
        num_partials = _dense.pick_num_partials(queues, kv_capacity, shape=shape)
        num_partials = max(1, min(num_partials, queues // (2 * rows * shape.num_key_value_heads)))
    dense = _dense.mi355x_scheduler(shape, sm_count=queues, num_partials=num_partials,
                                    attention_merge="oproj" if merge_in_oproj else "last", oproj_spares_attention=False)
    return RowsScheduler(dense, rows, merge_in_oproj)


class RowsMegaKernel(_mb.BatchMegaKernel):
    """The ``mk`` callable of the rows engine: the batch route's argument list (its three RMSNorm row buffers and
    ``attn_partial_valid`` are taken and not used), launched through ``qmk_decode_step_rows``.  Tagged hand-over and
    self-clearing counters always; the workspace (one set of tagged units per row) belongs to this object."""

    def __init__(self, lib: ctypes.CDLL, *, spin_limit: int = 0):
        super().__init__(lib, reset_barriers=True, spin_limit=spin_limit)
        self._rows = QmkRowsArgs()
        self._rows.struct_size = ctypes.sizeof(QmkRowsArgs)
        self._args = self._rows.step                      # the batch route's binder fills the nested struct in place
        self._args.struct_size = ctypes.sizeof(_mb.QmkBatchArgs)
        self._workspace: torch.Tensor | None = None
        self.qkv_blocks_per_head = 0

    def with_options(self, **kw: Any) -> "RowsMegaKernel":
        other = RowsMegaKernel(self._lib, spin_limit=kw.pop("spin_limit", self.spin_limit))
        if kw:
            raise TypeError(f"unknown options {sorted(kw)}")
        return other

    def check(self, stream: torch.cuda.Stream | None = None) -> None:
        try:
            super().check(stream)
        except RuntimeError:
            if self._workspace is not None:      # the tagged units of a step that never finished
                self._workspace.zero_()
            raise

    def _launch(self, device: torch.device) -> None:
        B = int(self._args.batch_size)
        nbytes = int(self._lib.qmk_rows_workspace_bytes(B))
        if nbytes == 0:
            raise ValueError(f"the rows engine takes 1..{MAX_ROWS} rows, got {B}")
        if self._workspace is None or self._workspace.device != device or self._workspace.numel() < nbytes:
            self._workspace = torch.zeros(nbytes, dtype=torch.uint8, device=device)
        self._rows.workspace, self._rows.workspace_bytes = self._workspace.data_ptr(), nbytes
        self._rows.qkv_blocks_per_head = int(self.qkv_blocks_per_head)
        rc = int(self._lib.qmk_decode_step_rows(ctypes.byref(self._rows)))
        if rc != 0:
            raise RuntimeError(f"qmk_decode_step_rows failed with {rc}: {self.error_string(rc)}")


def get_mk(mk_dir: Path | None = None, *, spin_limit: int = 0) -> RowsMegaKernel:
    root = (_single._default_mk_dir() if mk_dir is None else Path(mk_dir)).resolve()
    lib = _single._LIB_CACHE.get(root)
    if lib is None:
        lib = _single.load_library(root)
        _single._LIB_CACHE[root] = lib
    for name in ("qmk_decode_step_rows", "qmk_rows_workspace_bytes"):
        if not hasattr(lib, name):
            raise ImportError(f"{root / 'libqmk_hip.so'} does not export {name}")
    lib.qmk_decode_step_rows.argtypes = [ctypes.POINTER(QmkRowsArgs)]
    lib.qmk_decode_step_rows.restype = ctypes.c_int
    lib.qmk_rows_workspace_bytes.argtypes = [ctypes.c_int]
    lib.qmk_rows_workspace_bytes.restype = ctypes.c_uint64
    return RowsMegaKernel(lib, spin_limit=spin_limit)


def build(globs: Globals, *, queues: int = _dense.MI355X_CU_COUNT, num_partials: int | None = None, merge_in_oproj: bool = False,
          num_layers: int | None = None) -> torch.Tensor:
    """The request's instruction tensor for the rows engine (valid for every step of the request)."""
    rows = _mb._batch_size(globs)
    sched = mi355x_scheduler(rows, kv_capacity=int(globs.k_cache.shape[2]), queues=queues, num_partials=num_partials,
                             merge_in_oproj=merge_in_oproj)
    if sched.num_partials > int(globs.attn_lse_intermediates.shape[-1]):
        raise ValueError("attn_lse_intermediates has fewer partial slots than the schedule's split-KV fan-out")
    globs.rows_geometry = sched.dense.geometry
    return _dense.tensorize_instructions(globs, sched.queues(num_layers))


def call_mk(globs: Globals, mk: RowsMegaKernel) -> None:
    """One decode step of all rows of ``globs`` (builds the request's instruction tensor on first use)."""
    if globs.instructions is None:
        build(globs)
    geometry = getattr(globs, "rows_geometry", None) or mi355x_scheduler(_mb._batch_size(globs)).dense.geometry
    mk.qkv_blocks_per_head = geometry.expected_counts(LlamaConfig.shape())[0]
    _mb.call_mk(globs, mk)
