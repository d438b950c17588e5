"""Scheduler of the batch route (B <= 16: one M tile).

Two layouts, both the reference's (`…/A100/multi_batch/decode_schedule/instructions/scheduler.py`):

* ``instruction_list`` / ``queues``: the instructions of a step in dependency order, dealt
  round-robin (`:399-440`); the split-KV instructions carry the context length and activity the
  request has when the list is built.
* ``runtime_queues``: a template built once per request (`:443-537`): every op starts on a fresh
  round of the workers (short ops are padded with no-ops, the RMSNorm rows occupy the first B
  workers of a round), and the attention instructions leave length and activity to the
  ``position_ids`` / ``active_mask`` of the launch.

``workers`` is the number of instruction queues: 2 per SM on the reference's A100 (216), one per
CU on MI355X (256).
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass
from typing import Any, Sequence

from ...decode_schedule.model_config import DecodeShape, LlamaConfig
from ...instruction import INTS_PER_INSTRUCTION, Instruction
from ..row_state import RowState
from .instruction_defs import (
    MAX_BATCH,
    TILE_N_GRANULARITY,
    AttnRMS,
    DecodeAttentionReduction,
    DecodeAttentionSplitKV,
    DecodeAttentionSplitKVMerge,
    DownProj_GEMM_Residual,
    LMHeadProj_GEMM,
    LMHeadRMS,
    MlpRMS,
    NoOp,
    OProj_GEMM_Residual,
    QKVProj_GEMM_RoPE,
    UpGateProj_GEMM_SiLU,
)

MAX_TILE_BLOCKS_PER_INSTRUCTION = INTS_PER_INSTRUCTION - 6
MAX_REDUCTION_LIST = INTS_PER_INSTRUCTION - 5
A100_WORKERS = 108 * 2
MI355X_WORKERS = 256


def _ceil_div(a: int, b: int) -> int:
    return -(-a // b)


def _spans(n: int, parts: int) -> list[tuple[int, int]]:
    """Contiguous, as-even-as-possible cut of n blocks into at most ``parts`` spans."""
    if n <= 0:
        return []
    groups = min(n, parts)
    small, extra = divmod(n, groups)
    out, lo = [], 0
    for g in range(groups):
        hi = lo + small + (1 if g < extra else 0)
        out.append((lo, hi))
        lo = hi
    return out


def partials_for_blocks(active_rows: int, max_blocks: int, workers: int, kv_heads: int) -> int:
    """Split-KV fan-out: about one split-KV instruction per worker, never more slices than 16-token
    blocks, never more than a reduction instruction can list (`scheduler.py:351-376`)."""
    if active_rows <= 0:
        return 1
    max_blocks = max(1, max_blocks)
    target = min(workers, active_rows * kv_heads * max_blocks)
    p = _ceil_div(target, active_rows * kv_heads)
    return min(MAX_REDUCTION_LIST, max(1, min(p, max_blocks)))


@dataclass
class BatchScheduler:
    shape: DecodeShape
    workers: int
    batch_size: int
    merge_in_last: bool = False   # the last split-KV arrival of a head group merges: no reduction instructions
    oproj_tile: int = TILE_N_GRANULARITY   # rows per O-proj block: 16 (the reference's), or 8
    down_tile: int = TILE_N_GRANULARITY    # rows per down-projection block
    skew_upgate: bool = False     # run-time template: no up/gate blocks for the down projection's workers, O-proj blocks beside the attention's
    split_kv_per_worker: float = 1.0   # split-KV instructions of a step per worker that the fan-out aims at (the reference: one)
    split_kv_cap: int = MAX_REDUCTION_LIST   # ... and never more slices per KV head than this
    lone_slice_tokens: int = 0         # where the rule gives two or three slices and the slices' tokens are at most this many: one slice
                                       # (the only slice of its heads writes attn_out itself: no counted arrival, no merge)

    def __post_init__(self) -> None:
        if not 1 <= self.batch_size <= MAX_BATCH:
            raise ValueError(f"batch size must be in [1, {MAX_BATCH}], got {self.batch_size}")
        if self.workers < 1:
            raise ValueError("workers must be positive")

    # ---- per-op emitters ---------------------------------------------------
    def attn_rms(self, layer: int) -> list[Instruction]:
        return [AttnRMS(layer, self.batch_size, batch_row=r) for r in range(self.batch_size)]

    def mlp_rms(self, layer: int) -> list[Instruction]:
        return [MlpRMS(layer, self.batch_size, batch_row=r) for r in range(self.batch_size)]

    def lmhead_rms(self) -> list[Instruction]:
        return [LMHeadRMS(self.batch_size, batch_row=r) for r in range(self.batch_size)]

    def qkvproj(self, layer: int) -> list[Instruction]:
        blocks = _ceil_div(self.shape.qkv_out_dim, TILE_N_GRANULARITY)
        return [QKVProj_GEMM_RoPE(layer, self.batch_size, 0, lo, hi) for lo, hi in _spans(blocks, self.workers)]

    def oproj(self, layer: int) -> list[Instruction]:
        blocks = _ceil_div(self.shape.hidden_size, self.oproj_tile)
        return [OProj_GEMM_Residual(layer, self.batch_size, 0, lo, hi, 0, tile_N_granularity=self.oproj_tile)
                for lo, hi in _spans(blocks, self.workers)]

    def upgate(self, layer: int) -> list[Instruction]:
        blocks = _ceil_div(self.shape.intermediate_size, TILE_N_GRANULARITY)
        out: list[Instruction] = []
        for lo, hi in _spans(blocks, self.workers):
            mine = list(range(lo, hi))
            for at in range(0, len(mine), MAX_TILE_BLOCKS_PER_INSTRUCTION):
                out.append(UpGateProj_GEMM_SiLU(layer, self.batch_size, 0, mine[at : at + MAX_TILE_BLOCKS_PER_INSTRUCTION]))
        return out

    def upgate_skewed(self, layer: int) -> list[Instruction]:
        """One instruction (or no-op) per worker, in worker order.  The workers of the down projection's round (the
        first H/16) get no up/gate block: they ask for their whole down-projection block while the others, whose first
        blocks have been waiting in registers since the attention phase, run the up/gate projection, so that the down
        projection starts from weights that have arrived (Llama shape, 8 rows: 8 470 -> 8 700 tok/s, with the arrivals
        counted per XCD; one block each as before: the down projection waits 2-7 us for its weights)."""
        blocks = _ceil_div(self.shape.intermediate_size, TILE_N_GRANULARITY)
        busy = min(self.workers, len(self.downproj(layer)))
        idle = self.workers - busy
        if idle <= 0 or blocks > idle * MAX_TILE_BLOCKS_PER_INSTRUCTION:
            return self.upgate(layer)
        heavy, extra = divmod(blocks, idle)
        out: list[Instruction] = []
        at = 0
        for worker in range(self.workers):
            n = 0 if worker < busy else heavy + (1 if worker - busy < extra else 0)
            out.append(UpGateProj_GEMM_SiLU(layer, self.batch_size, 0, list(range(at, at + n))) if n else NoOp())
            at += n
        assert at == blocks
        return out

    def qkv_round(self, layer: int, num_partials: int) -> list[Instruction]:
        """The QKV projection's round(s) of the run-time template.  With ``skew_upgate`` its blocks start behind the
        workers of the split-KV round where all of them fit there — an attention worker then starts its slice without
        a QKV block of its own in front, and the norm rows' workers (the first B) run no QKV block behind their row
        (Llama shape, 8 rows: 49.0 -> 46.7 us per layer) — otherwise behind the norm rows' workers, otherwise at 0."""
        plain = self.qkvproj(layer)
        if not self.skew_upgate or len(plain) > self.workers:
            return plain + [NoOp()] * (-len(plain) % self.workers)
        slices = len(self.attention_split_kv(layer, num_partials))
        start = next((at for at in (slices, self.batch_size) if at + len(plain) <= self.workers), 0)
        others = self.workers - self.batch_size
        blocks = _ceil_div(self.shape.qkv_out_dim, TILE_N_GRANULARITY)
        if start == 0 and 0 < others and blocks <= 2 * others:
            # A block for every worker (Qwen3-1.7B shape: 256): the norm rows' workers still get none, a few of the others
            # two — a second block costs 1 us, a block behind a norm row ends the phase 2.7 us late.
            start = self.batch_size
            plain = [QKVProj_GEMM_RoPE(layer, self.batch_size, 0, lo, hi) for lo, hi in _spans(blocks, others)]
        return [NoOp()] * start + plain + [NoOp()] * (self.workers - start - len(plain))

    def oproj_round(self, layer: int, num_partials: int) -> list[Instruction]:
        """The O-projection's round of the run-time template.  With ``skew_upgate`` its blocks go, two to a worker, to
        the down-projection workers that the split-KV round left free, where there are enough of them: a worker that
        has just run an attention slice could not ask for its O-projection block ahead and ends the phase 2 us late
        (Llama shape, 8 rows: 52.4 -> 50.5 us per layer)."""
        plain = self.oproj(layer)
        first = len(self.attention_split_kv(layer, num_partials))
        last = min(self.workers, len(self.downproj(layer)))
        free = last - first
        blocks = _ceil_div(self.shape.hidden_size, self.oproj_tile)
        if not self.skew_upgate or free <= 0 or 2 * free < len(plain) or len(plain) > self.workers:
            return plain + [NoOp()] * (-len(plain) % self.workers)
        placed = [OProj_GEMM_Residual(layer, self.batch_size, 0, lo, hi, 0, tile_N_granularity=self.oproj_tile)
                  for lo, hi in _spans(blocks, free)]
        return [NoOp()] * first + placed + [NoOp()] * (self.workers - first - len(placed))

    def downproj(self, layer: int) -> list[Instruction]:
        blocks = _ceil_div(self.shape.hidden_size, self.down_tile)
        return [DownProj_GEMM_Residual(layer, self.batch_size, 0, lo, hi, tile_N_granularity=self.down_tile)
                for lo, hi in _spans(blocks, self.workers)]

    def lmhead(self) -> list[Instruction]:
        blocks = _ceil_div(self.shape.vocab_size, TILE_N_GRANULARITY)
        return [LMHeadProj_GEMM(self.batch_size, lo, hi) for lo, hi in _spans(blocks, self.workers)]

    def attention_split_kv(self, layer: int, num_partials: int, globs: Any = None) -> list[Instruction]:
        """With ``globs``: length and activity fixed from the request's present state; without: left
        to the launch (seq_len = is_active = -1)."""
        kvb = self.shape.attn_kv_block_size
        make = DecodeAttentionSplitKVMerge if self.merge_in_last else DecodeAttentionSplitKV
        out: list[Instruction] = []
        for b in range(self.batch_size):
            if globs is not None:
                state = RowState.of(globs)
                on, seq_len = state.is_active(b), state.position(b) + 1
                total = max(1, _ceil_div(seq_len, kvb)) if on else 0
                per = max(1, _ceil_div(total, num_partials)) if on else 1
            for kvh in range(self.shape.num_key_value_heads):
                for part in range(num_partials):
                    if globs is None:
                        out.append(make(layer, b, kvh, num_partials, part))
                        continue
                    t0 = part * per * kvb
                    t1 = min(min(part * per + per, total) * kvb, seq_len)
                    work = on and t0 < t1 and t1 > 0
                    out.append(make(layer, b, kvh, num_partials, part, seq_len, 1 if work else 0))
        return out

    def attention_reduction(self, layer: int, num_partials: int, globs: Any = None) -> list[Instruction]:
        out: list[Instruction] = []
        if self.merge_in_last:
            return out
        for b in range(self.batch_size):
            for head0 in range(0, self.shape.num_attention_heads, self.shape.attn_reduction_size):
                if globs is None:
                    out.append(DecodeAttentionReduction(layer, b, head0, num_partials, list(range(num_partials))))
                else:
                    out.append(DecodeAttentionReduction(layer, b, head0, num_partials, list(range(num_partials)),
                                                        valid_partials=num_partials, is_active=1 if RowState.of(globs).is_active(b) else 0))
        return out

    # ---- fan-out -------------------------------------------------------------
    def partials_for_request(self, globs: Any) -> int:
        kvb = self.shape.attn_kv_block_size
        state = RowState.of(globs)
        rows = [b for b in range(self.batch_size) if state.is_active(b)]
        blocks = max([1] + [_ceil_div(state.position(b) + 1, kvb) for b in rows])
        return self._fan_out(len(rows), blocks)

    def _split_kv_workers(self) -> int:
        return max(1, int(self.workers * self.split_kv_per_worker))

    def _fan_out(self, rows: int, blocks: int) -> int:
        p = min(self.split_kv_cap, partials_for_blocks(rows, blocks, self._split_kv_workers(), self.shape.num_key_value_heads))
        if p in (2, 3) and self.merge_in_last and blocks * self.shape.attn_kv_block_size <= self.lone_slice_tokens:
            return 1   # (three slices: 6 and 7 rows with heads of 64 — 45.5 -> 40.5 us per layer at context 300, 47 -> 45.5 at 900)
        if self.merge_in_last:
            # The rule rounds up: 12 rows of 8 KV heads get 3 slices, 288 instructions for 256 workers — a second round of
            # 32 behind the first (Qwen3-1.7B shape, 12 rows: 1.83 ms per step against 1.64 at 16 rows).  Never more
            # instructions than workers.
            while p > 1 and p * max(rows, 1) * self.shape.num_key_value_heads > self.workers:
                p -= 1
        return p

    def partials_for_capacity(self, kv_capacity: int) -> int:
        blocks = max(1, _ceil_div(kv_capacity, self.shape.attn_kv_block_size))
        return self._fan_out(self.batch_size, blocks)

    # ---- whole step: dependency order, dealt round-robin ---------------------
    def instruction_list(self, globs: Any, num_layers: int | None = None) -> list[Instruction]:
        layers = self.shape.num_hidden_layers if num_layers is None else num_layers
        p = self.partials_for_request(globs)
        out: list[Instruction] = []
        for layer in range(layers):
            out += self.attn_rms(layer) + self.qkvproj(layer)
            out += self.attention_split_kv(layer, p, globs) + self.attention_reduction(layer, p, globs)
            out += self.oproj(layer) + self.mlp_rms(layer) + self.upgate(layer) + self.downproj(layer)
        if layers == self.shape.num_hidden_layers:
            out += self.lmhead_rms() + self.lmhead()
        return out

    def queues(self, globs: Any, num_layers: int | None = None) -> list[list[Instruction]]:
        return deal(self.instruction_list(globs, num_layers), self.workers)

    # ---- whole step: a template for every step of a request ------------------
    def runtime_instruction_list(self, kv_capacity: int, num_layers: int | None = None) -> list[Instruction]:
        layers = self.shape.num_hidden_layers if num_layers is None else num_layers
        p = self.partials_for_capacity(kv_capacity)
        out: list[Instruction] = []

        def rows_round(rows: Sequence[Instruction]) -> None:   # one instruction slot per worker
            out.extend(list(rows) + [NoOp()] * (self.workers - len(rows)))

        def rounds(segment: Sequence[Instruction]) -> None:    # whole rounds, the last one padded
            for at in range(0, len(segment), self.workers):
                chunk = list(segment[at : at + self.workers])
                out.extend(chunk + [NoOp()] * (self.workers - len(chunk)))

        for layer in range(layers):
            rows_round(self.attn_rms(layer))
            out.extend(self.qkv_round(layer, p))
            rounds(self.attention_split_kv(layer, p))
            rounds(self.attention_reduction(layer, p))
            out.extend(self.oproj_round(layer, p))
            rows_round(self.mlp_rms(layer))
            rounds(self.upgate_skewed(layer) if self.skew_upgate else self.upgate(layer))
            rounds(self.downproj(layer))
        if layers == self.shape.num_hidden_layers:
            rows_round(self.lmhead_rms())
            rounds(self.lmhead())
        return out

    def runtime_queues(self, kv_capacity: int, num_layers: int | None = None) -> list[list[Instruction]]:
        return deal(self.runtime_instruction_list(kv_capacity, num_layers), self.workers)


def deal(instructions: Sequence[Instruction], workers: int) -> list[list[Instruction]]:
    queues: list[list[Instruction]] = [[] for _ in range(workers)]
    for i, ins in enumerate(instructions):
        queues[i % workers].append(ins)
    return queues


def reference_scheduler(batch_size: int, shape: DecodeShape | None = None) -> BatchScheduler:
    """The A100 route's worker count: two queues per SM."""
    return BatchScheduler(shape or LlamaConfig.shape(), A100_WORKERS, batch_size)


def mi355x_scheduler(batch_size: int, shape: DecodeShape | None = None, *, merge_in_last: bool = True,
                     residual_tile: int = 16, skew_upgate: bool = True) -> BatchScheduler:
    """One queue per CU; the split-KV partials are merged by the last arrival of each head group.
    ``residual_tile`` 8 gives the two projections that add to the residual stream one 8-row block per
    workgroup instead of 16-row blocks on half the CUs; measured slower at batch 8 (every workgroup
    reads all activations, so twice the workgroups read them twice: 7478 against 8015 tok/s).
    Split-KV fan-out: with heads of 64 half as many slices as the reference's one-instruction-per-worker rule gives —
    what a slice saves in scores the merge by the last arrival (a counted arrival, a second read of the partials,
    a second hand-over) costs again: Llama shape, contexts 500 / 1000, step time with the reference's fan-out against
    half of it: B=2 938/947 -> 853/856 us, B=4 938/947 -> 881/905, B=8 1021/1048 -> 972/1009, B=16 1187/1233 ->
    1108/1176.  With heads of 128 (Qwen3-1.7B shape, B=8: 1566/1636 us with 4 slices, 1591/1721 with 2) the rule stays.
    Never more than 4 slices (mean step time at contexts 250 / 500 / 1000 with 4 against 8 slices: Llama shape B=2
    843 against 856 us; Qwen3 shape B=2 1345 against 1362, B=4 1432 against 1433).  With heads of 64 and a cache of at
    most 2048 tokens one slice where the rule gives two: the only slice of its heads writes attn_out itself (Llama
    shape B=8: 963 against 980 us; the second slice halves a loop of 0.9 us per 128 tokens and costs a merge of 4 us)."""
    if residual_tile not in (8, 16):
        raise ValueError("blocks of the residual projections have 8 or 16 rows")
    shape = shape or LlamaConfig.shape()
    return BatchScheduler(shape, MI355X_WORKERS, batch_size, merge_in_last=merge_in_last, oproj_tile=residual_tile,
                          down_tile=residual_tile, skew_upgate=skew_upgate, split_kv_per_worker=0.5 if shape.head_dim <= 64 else 1.0,
                          split_kv_cap=4, lone_slice_tokens=2048 if shape.head_dim <= 64 else 0)
