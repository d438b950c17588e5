"""Scheduler of the MoE decode route: one step's instructions in dependency order, dealt round-robin
(the reference's way) or placed queue by queue (``placed=True``: the MI355X stream).

Emission order per layer 1 -> 2 -> 3 -> 4 -> 8 -> 9 -> 10 -> 11 -> 12 -> 13 -> 14, then 7
(`…/qwen1_5_moe_a2_7b/A100/single_batch/decode_schedule/instructions/scheduler.py:139-370`).
``sm_count`` is the number of instruction queues: 108 in the reference.
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass
from typing import Sequence

from ...instruction import Instruction
from ..model_config import A100_SM_COUNT, MoeShape, QwenMoeConfig, num_partials_for
from .instruction_defs import (
    TILE_N_GRANULARITY,
    DecodeAttentionReduction,
    DecodeAttentionSplitKV,
    DecodeAttentionSplitKVMerge,
    DecodeAttentionSplitKVRow,
    MoE_Combine_Commit,
    OProj_GEMV_Residual,
    RMS_LMHead_GEMV,
    RMS_QKVProj_GEMV_RoPE,
    RoutedExpert_DownProj,
    RoutedExpert_UpGate_SiLU,
    RoutedExperts_DownCommit_Rows,
    RoutedExperts_UpGate_Rows,
    Router_GEMV,
    Router_SoftmaxTopK,
    Router_SoftmaxTopKRow,
    SharedExpert_DownProj,
    SharedExpert_UpGate_SiLU,
)


def _ceil_div(a: int, b: int) -> int:
    return -(-a // b)


def _spans(n: int, parts: int) -> list[tuple[int, int]]:
    """Contiguous, as-even-as-possible cut of n tiles into at most ``parts`` spans."""
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


@dataclass
class MoeScheduler:
    shape: MoeShape
    sm_count: int
    num_partials: int
    interleave_experts: bool = False   # both up/gate phases before both down projections (the reference: 10, 11, 12, 13)
    merge_in_last: bool = False        # the last split-KV arrival of a KV head merges: no reduction instructions
    merge_in_oproj: bool = False       # every O-projection instruction merges all partials itself: no reduction instructions
    router_span: int = 1               # experts per router instruction
    placed: bool = False               # queues() places the instructions of a layer by role instead of dealing them
    down_per_slot: bool = False        # a routed down projection waits for its own slot's up/gate tiles only (tile_M_idx = 1)
    commit_in_down: bool = False       # tagged launches without a shared expert: opcode 13 with tile_M_idx = 2 takes all expert slots
                                       # of 8 rows and commits them (the combine step's arithmetic): no opcode 14 in the stream
    topk_late: bool = False            # placed streams for tagged launches: the consumers take the routing decision themselves,
                                       # the top-k instruction runs last in its layer on a queue without a combine instruction (it only reports the routing)

    def qkvproj(self, layer: int) -> list[Instruction]:
        tile = self.shape.qkv_tile
        tiles = _ceil_div(self.shape.qkv_out_dim, tile)
        return [RMS_QKVProj_GEMV_RoPE(layer, 0, lo, hi, tile_N_granularity=tile) for lo, hi in _spans(tiles, self.sm_count)]

    def attention_split_kv(self, layer: int) -> list[Instruction]:
        if self.merge_in_oproj:
            make = lambda *a: DecodeAttentionSplitKVMerge(*a, merge_in_last=2)
        else:
            make = DecodeAttentionSplitKVMerge if self.merge_in_last else DecodeAttentionSplitKV
        return [make(layer, kvh, self.num_partials, part)
                for kvh in range(self.shape.num_key_value_heads) for part in range(self.num_partials)]

    def attention_reduction(self, layer: int) -> list[Instruction]:
        if self.merge_in_last or self.merge_in_oproj:
            return []
        return [DecodeAttentionReduction(layer, h0, self.num_partials, list(range(self.num_partials)))
                for h0 in range(0, self.shape.num_attention_heads, self.shape.attn_reduction_size)]

    def oproj(self, layer: int) -> list[Instruction]:
        merges = self.num_partials if self.merge_in_oproj else 0
        return [OProj_GEMV_Residual(layer, 0, lo, hi, merges, tile_N_granularity=self.shape.oproj_tile)
                for lo, hi in _spans(self.shape.num_oproj_blocks, self.sm_count)]

    def router_gemv(self, layer: int) -> list[Instruction]:
        """One instruction per expert: the top-k waits for all of them."""
        e = self.shape.num_experts
        return [Router_GEMV(layer, lo, hi, 1 if lo == 0 else 0) for lo, hi in _spans(e, _ceil_div(e, max(1, self.router_span)))]

    def router_softmax_topk(self, layer: int) -> list[Instruction]:
        return [Router_SoftmaxTopK(layer)]

    def shared_upgate(self, layer: int) -> list[Instruction]:
        if not self.shape.has_shared_expert:
            return []
        if self.placed:
            return [ins for _, ins in self._placed_shared_upgate(layer)]
        tiles = _ceil_div(self.shape.intermediate_size, TILE_N_GRANULARITY)
        return [SharedExpert_UpGate_SiLU(layer, 0, lo, hi, 1 if lo == 0 else 0) for lo, hi in _spans(tiles, self.sm_count)]

    def shared_downproj(self, layer: int) -> list[Instruction]:
        """K split into ``num_downproj_split_k_shared`` slices, each with its own share of the queues."""
        k = self.shape.num_downproj_split_k_shared
        if not self.shape.has_shared_expert or k < 1:
            return []
        per_group = max(1, self.sm_count // k)
        out: list[Instruction] = []
        for slice_idx in range(k):
            first = slice_idx * per_group
            last = min((slice_idx + 1) * per_group, self.sm_count) if slice_idx < k - 1 else self.sm_count
            for lo, hi in _spans(self.shape.num_hidden_blocks, max(1, last - first)):
                out.append(SharedExpert_DownProj(layer, 0, lo, hi, slice_idx, split_K_granularity=self.shape.split_k_granularity_shared))
        return out

    def routed_upgate(self, layer: int) -> list[Instruction]:
        if self.placed:
            return [ins for _, ins in self._placed_routed_upgate(layer)]
        per_expert = max(1, self.sm_count // self.shape.num_experts_per_tok)
        tile = self.shape.routed_upgate_tile
        return [RoutedExpert_UpGate_SiLU(layer, slot, lo, hi, tile_N_granularity=tile)
                for slot in range(self.shape.num_experts_per_tok)
                for lo, hi in _spans(self.shape.num_routed_upgate_blocks, per_expert)]

    def routed_downproj(self, layer: int) -> list[Instruction]:
        if self.commit_in_down:
            rows = TILE_N_GRANULARITY // 2
            tiles = self.shape.hidden_size // rows
            # an instruction commits at most 16 rows: with fewer than tiles / 2 queues a queue gets several
            return [RoutedExpert_DownProj(layer, 0, 2, lo, hi, tile_N_granularity=rows)
                    for lo, hi in _spans(tiles, max(self.sm_count, _ceil_div(tiles, 2)))]
        per_expert = max(1, self.sm_count // self.shape.num_experts_per_tok)
        return [RoutedExpert_DownProj(layer, slot, 1 if self.down_per_slot else 0, lo, hi)
                for slot in range(self.shape.num_experts_per_tok)
                for lo, hi in _spans(self.shape.num_hidden_blocks, per_expert)]

    def combine_commit(self, layer: int) -> list[Instruction]:
        if self.commit_in_down:
            return []
        return [MoE_Combine_Commit(layer, lo, hi) for lo, hi in _spans(self.shape.num_hidden_blocks, self.sm_count)]

    def lmhead(self) -> list[Instruction]:
        tiles = _ceil_div(self.shape.vocab_size, TILE_N_GRANULARITY)
        return [RMS_LMHead_GEMV(lo, hi) for lo, hi in _spans(tiles, self.sm_count)]

    def layer(self, layer: int) -> list[Instruction]:
        head = (self.qkvproj(layer) + self.attention_split_kv(layer) + self.attention_reduction(layer) + self.oproj(layer)
                + self.router_gemv(layer) + self.router_softmax_topk(layer))
        if self.interleave_experts:
            # the shared down projection's wait for all shared up/gate rows passes while the routed rows stream
            experts = self.shared_upgate(layer) + self.routed_upgate(layer) + self.shared_downproj(layer) + self.routed_downproj(layer)
        else:
            experts = self.shared_upgate(layer) + self.shared_downproj(layer) + self.routed_upgate(layer) + self.routed_downproj(layer)
        return head + experts + self.combine_commit(layer)

    # ---- placement by role (``placed=True``) -------------------------------------------------------------
    # With the stream dealt round-robin, the queues that run the router and the top-k of a layer start that
    # layer's expert phases one or two hand-overs after everybody else, with the same amount of work ahead of
    # them, and the down projections wait for the slowest queue.  Placed: the last queues of the device take the
    # router and the top-k and no shared up/gate rows; the O-projection queues take one shared up/gate tile and
    # the queues that only wait during the O-projection two; the routed up/gate tiles go where the shared ones
    # left room (three tiles of the two phases per queue at most), filling the queues up to one level of weight
    # rows streamed between the attention and the down projections (`_room_for_routed_rows`).

    def _roles(self) -> tuple[list[int], list[int], int]:
        """(queues of the O-projection and the expert phases, queues of the router and the top-k, O-proj count)."""
        n = self.sm_count
        side = len(self.router_gemv(0)) + 1
        if side * 4 > n:                       # a device too small to set queues aside
            return list(range(n)), list(range(n)), min(n, self.shape.num_oproj_blocks)
        return list(range(n - side)), list(range(n - side, n)), min(n - side, self.shape.num_oproj_blocks)

    def _late_topk_queue(self) -> int:
        """A queue in the middle: the first ones run the split-KV slices, the last ones the router."""
        return max(self.sm_count // 2 - 1, 0)

    @staticmethod
    def _weighted_sizes(tiles: int, weights: Sequence[int]) -> list[int]:
        """``tiles`` cut in proportion to ``weights`` (largest remainders first, earlier entries on ties)."""
        total = sum(weights)
        raw = [tiles * w / total for w in weights]
        sizes = [int(r) for r in raw]
        order = sorted(range(len(weights)), key=lambda i: (-(raw[i] - sizes[i]), i))
        for i in order[: tiles - sum(sizes)]:
            sizes[i] += 1
        return sizes

    def _shared_sizes(self) -> dict[int, int]:
        main, _, oproj_queues = self._roles()
        if not self.shape.has_shared_expert:
            return {q: 0 for q in main}
        tiles = _ceil_div(self.shape.intermediate_size, TILE_N_GRANULARITY)
        weights = [1 if i < oproj_queues else 2 for i in range(len(main))]
        return dict(zip(main, self._weighted_sizes(tiles, weights)))

    def _placed_shared_upgate(self, layer: int) -> list[tuple[int, Instruction]]:
        out, lo = [], 0
        for queue, size in self._shared_sizes().items():
            if size:
                out.append((queue, SharedExpert_UpGate_SiLU(layer, 0, lo, lo + size, 1 if lo == 0 else 0)))
                lo += size
        return out

    def _room_for_routed_rows(self, shared: dict[int, int], routed_rows: int) -> list[float]:
        """Per queue, the weight rows of the routed up/gate phase that bring every queue to the same number of rows
        streamed between the attention and the down projections (O-projection rows, two per shared up/gate output, two
        per routed one): the level that ``routed_rows`` fill up.  The queues of the router and the top-k count as the
        least loaded of the others: their routed rows cannot start before everybody's."""
        main, _, _ = self._roles()
        load = {q: 2.0 * TILE_N_GRANULARITY * shared.get(q, 0) for q in main}
        wide = self.shape.num_attention_heads * self.shape.head_dim / self.shape.hidden_size     # an O-projection row in rows of H
        for i, ins in enumerate(self.oproj(0)):
            load[main[i % len(main)]] += (ins.tile_N_end_idx - ins.tile_N_start_idx) * ins.tile_N_granularity * wide
        least = min(load.values())
        loads = [load.get(q, least) for q in range(self.sm_count)]
        lo, hi = least, max(loads) + routed_rows
        for _ in range(60):                      # the level T with sum(max(0, T - load)) = routed_rows
            mid = (lo + hi) / 2
            lo, hi = (mid, hi) if sum(max(0.0, mid - x) for x in loads) < routed_rows else (lo, mid)
        return [max(0.0, hi - x) for x in loads]

    def _placed_routed_upgate(self, layer: int) -> list[tuple[int, Instruction]]:
        shared = self._shared_sizes()
        blocks, slots, tile = self.shape.num_routed_upgate_blocks, self.shape.num_experts_per_tok, self.shape.routed_upgate_tile
        queues = list(range(self.sm_count))
        if self.shape.has_shared_expert:
            weights = self._room_for_routed_rows(shared, 2 * tile * blocks * slots)
        else:                                    # nothing else in the phase: the tiles evenly on all queues
            weights = [1] * len(queues)
        sizes = self._weighted_sizes(blocks * slots, weights)
        out, slot, lo = [], 0, 0
        for queue, size in zip(queues, sizes):
            while size:                          # a span ends with its expert slot: the rest goes to the next slot
                take = min(size, blocks - lo)
                out.append((queue, RoutedExpert_UpGate_SiLU(layer, slot, lo, lo + take, tile_N_granularity=tile)))
                size, lo = size - take, lo + take
                if lo == blocks:
                    slot, lo = slot + 1, 0
        return out

    def _place_layer(self, out: list[list[Instruction]], layer: int) -> None:
        n = self.sm_count
        main, side, _ = self._roles()

        def spread(instructions: Sequence[Instruction], queues: Sequence[int]) -> None:
            for i, ins in enumerate(instructions):
                out[queues[i % len(queues)]].append(ins)

        everyone = list(range(n))
        spread(self.qkvproj(layer), everyone)
        spread(self.attention_split_kv(layer), everyone)
        spread(self.attention_reduction(layer), everyone)
        if self.topk_late and layer > 0:
            # The previous layer's reporting top-k: nobody inside the launch waits for it, and this is where a queue
            # has time — between its QKV rows and its O-projection rows, while the few split-KV workgroups work.
            # (The router that overwrites the logits it reads cannot start before this queue's O-projection rows.)
            out[self._late_topk_queue()] += self.router_softmax_topk(layer - 1)
        # without a shared expert nothing runs beside the router: its queues take O-projection rows like everybody else
        spread(self.oproj(layer), main if self.shape.has_shared_expert else everyone)
        router = self.router_gemv(layer)
        spread(router, side)
        topk_queue = side[len(router) % len(side)]
        if not self.topk_late:
            out[topk_queue] += self.router_softmax_topk(layer)
        for queue, ins in self._placed_shared_upgate(layer):
            out[queue].append(ins)
        if not self.interleave_experts:
            spread(self.shared_downproj(layer), everyone)
        for queue, ins in self._placed_routed_upgate(layer):
            out[queue].append(ins)
        if self.interleave_experts:
            spread(self.shared_downproj(layer), everyone)
        spread(self.routed_downproj(layer), everyone)
        spread(self.combine_commit(layer), everyone[::-1])   # not on the O-projection's queues

    def instruction_list(self, num_layers: int | None = None) -> list[Instruction]:
        layers = self.shape.num_hidden_layers if num_layers is None else num_layers
        out: list[Instruction] = []
        for layer in range(layers):
            out += self.layer(layer)
        if layers == self.shape.num_hidden_layers:
            out += self.lmhead()
        return out

    def queues(self, num_layers: int | None = None) -> list[list[Instruction]]:
        if not self.placed:
            return deal(self.instruction_list(num_layers), self.sm_count)
        layers = self.shape.num_hidden_layers if num_layers is None else num_layers
        out: list[list[Instruction]] = [[] for _ in range(self.sm_count)]
        for layer in range(layers):
            self._place_layer(out, layer)
        if layers == self.shape.num_hidden_layers:
            for i, ins in enumerate(self.lmhead()):
                out[i % self.sm_count].append(ins)
        if self.topk_late and layers > 0:      # the last layer's report: the last instruction of its queue
            out[self._late_topk_queue()] += self.router_softmax_topk(layers - 1)
        return out


@dataclass
class MoeRowsScheduler:
    """One step of ``rows`` requests in one launch (a model without a shared expert, tagged hand-over): per layer the QKV
    rows, one split-KV instruction per (row, KV head, slice), the O-projection tiles (each merges every row's partials
    itself), the router (``router_span`` experts per instruction), one part of the distinct experts' gate/up rows per
    queue, the committing down-projection tiles; the rows' reporting top-k instructions of layer l run behind layer
    l + 1's QKV rows, where their queue waits for the attention anyway; then the LM head."""

    shape: MoeShape
    sm_count: int
    num_partials: int
    rows: int
    router_span: int = 8
    commit_tile: int = 8
    merge_in_oproj: bool = False     # True: every O-projection workgroup merges every row's split-KV partials itself (the
                                     # batch-1 stream's way); False: the last split-KV arrival of a (row, KV head) merges its
                                     # group, and the O-projection reads the rows' finished attention outputs in one trip

    def __post_init__(self) -> None:
        if self.shape.has_shared_expert:
            raise ValueError("the rows stream is built for models without a shared expert")
        if not 1 <= self.rows <= 4:
            raise ValueError("1..4 rows")
        self._one = MoeScheduler(self.shape, self.sm_count, self.num_partials, merge_in_oproj=self.merge_in_oproj,
                                 merge_in_last=not self.merge_in_oproj, router_span=self.router_span)

    def attention_split_kv(self, layer: int) -> list[Instruction]:
        return [DecodeAttentionSplitKVRow(layer, kvh, self.num_partials, part, merge_in_last=2 if self.merge_in_oproj else 1, batch_row=row)
                for row in range(self.rows) for kvh in range(self.shape.num_key_value_heads) for part in range(self.num_partials)]

    def topk_reports(self, layer: int) -> list[Instruction]:
        return [Router_SoftmaxTopKRow(layer, batch_row=row) for row in range(self.rows)]

    def routed_upgate(self, layer: int) -> list[Instruction]:
        return [RoutedExperts_UpGate_Rows(layer, part, self.sm_count) for part in range(self.sm_count)]

    def routed_down_commit(self, layer: int) -> list[Instruction]:
        tiles = self.shape.hidden_size // self.commit_tile
        per = max(1, 16 // self.commit_tile)       # an instruction commits at most 16 rows
        return [RoutedExperts_DownCommit_Rows(layer, lo, hi, self.commit_tile)
                for lo, hi in _spans(tiles, max(self.sm_count, _ceil_div(tiles, per)))]

    def _report_queues(self) -> list[int]:
        """Queues in the middle of the device: the first ones run the split-KV slices, the last ones the router."""
        mid = max(self.sm_count // 2 - 1, 0)
        return [(mid + i) % self.sm_count for i in range(self.rows)]

    def queues(self, num_layers: int | None = None) -> list[list[Instruction]]:
        layers = self.shape.num_hidden_layers if num_layers is None else num_layers
        n = self.sm_count
        out: list[list[Instruction]] = [[] for _ in range(n)]

        def spread(instructions: Sequence[Instruction], queues: Sequence[int]) -> None:
            for i, ins in enumerate(instructions):
                out[queues[i % len(queues)]].append(ins)

        everyone = list(range(n))
        for layer in range(layers):
            spread(self._one.qkvproj(layer), everyone)
            spread(self.attention_split_kv(layer), everyone)
            if layer > 0:
                for queue, ins in zip(self._report_queues(), self.topk_reports(layer - 1)):
                    out[queue].append(ins)
            spread(self._one.oproj(layer), everyone)
            spread(self._one.router_gemv(layer), everyone[::-1])    # the last queues: the first ones ran the attention
            spread(self.routed_upgate(layer), everyone)
            spread(self.routed_down_commit(layer), everyone)
        if layers == self.shape.num_hidden_layers:
            spread(self._one.lmhead(), everyone)
        if layers > 0:
            for queue, ins in zip(self._report_queues(), self.topk_reports(layers - 1)):
                out[queue].append(ins)
        return out

    def instruction_list(self, num_layers: int | None = None) -> list[Instruction]:
        return [ins for q in self.queues(num_layers) for ins in q]


def deal(instructions: Sequence[Instruction], queues: int) -> list[list[Instruction]]:
    out: list[list[Instruction]] = [[] for _ in range(queues)]
    for i, ins in enumerate(instructions):
        out[i % queues].append(ins)
    return out


def reference_scheduler(shape: MoeShape | None = None, sm_count: int = A100_SM_COUNT) -> MoeScheduler:
    """The reference's stream for ``shape``: its queue count, its split-KV fan-out and its QKV tiles of 16 rows (a launch
    of this stream takes ``.shape`` of the result, whose ``qkv_tile`` says so)."""
    shape = dataclasses.replace(shape or QwenMoeConfig.shape(), qkv_tile=TILE_N_GRANULARITY)
    return MoeScheduler(shape, sm_count, num_partials_for(sm_count, shape))
