"""The twelve opcodes of the MoE decode route and their counter protocol.

Opcodes, operand order and defaults are the reference's
(`…/qwen1_5_moe_a2_7b/A100/single_batch/decode_schedule/instructions/instruction_defs.py:24-262`).
Opcodes 1-4 and 7 are the dense route's attention and LM head (QKV with bias); 5 and 6 are unused;
8-14 replace the dense MLP.

Counters ``barriers[layer, opcode - 1, slot]`` (`…/instructions/python_vm.py:109-560`):

=====  =============================  ==========================  ================================
row    producer                       slot                        final count
=====  =============================  ==========================  ================================
0      1 RMS + QKV + bias + RoPE      q/k/v head index            head_dim / 16
1      2 split-KV attention           query head                  num_partials
2      3 attention reduction          0                           Hq
3      4 O-proj + residual            0                           hidden / 16
7      8 RMS + router logits          0: experts, 1: normed row   E, 1
8      9 softmax + top-k              0                           1 (set, not added)
9      10 shared up/gate + SiLU       0                           shared_intermediate / 16
10     11 shared down (split K)       hidden block                num_downproj_split_k_shared
11     12 routed up/gate + SiLU       0                           top_k * moe_intermediate / 16
12     13 routed down                 hidden block                top_k
13     14 combine + commit            0                           hidden / 16
14     12 routed up/gate (this build)  expert slot                 moe_intermediate / tile
=====  =============================  ==========================  ================================

Row 14 is this build's: the reference counts the routed up/gate tiles of all slots on one word (row 11), and a routed
down projection whose ``tile_M_idx`` is 1 (0 in the reference's streams) waits for the row-14 word of its own slot
instead.  The last word of layer 0's row 14 is the kernel's retirement count.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import ClassVar

from ...instruction import Instruction

TILE_M_GRANULARITY = 1
TILE_N_GRANULARITY = 16
ROUTER_TILE_N_GRANULARITY = 1
SPLIT_K_GRANULARITY_SHARED = 5632 // 4   # default operand of opcode 11; schedulers pass the shape's


@dataclass
class NoOp(Instruction):
    OPCODE: ClassVar[int] = 0


@dataclass
class RMS_QKVProj_GEMV_RoPE(Instruction):
    OPCODE: ClassVar[int] = 1
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (14,)
    layer_idx: int
    tile_M_idx: int
    tile_N_start_idx: int
    tile_N_end_idx: int
    tile_M_granularity: int = TILE_M_GRANULARITY
    tile_N_granularity: int = TILE_N_GRANULARITY


@dataclass
class DecodeAttentionSplitKV(Instruction):
    OPCODE: ClassVar[int] = 2
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (1,)
    layer_idx: int
    kv_head_idx: int
    num_partials: int
    partial_idx: int


@dataclass
class DecodeAttentionSplitKVMerge(DecodeAttentionSplitKV):
    """Extension of this build (same opcode, one more word), for streams without reduction instructions.
    1: the instruction whose arrival completes its KV head's counters also merges that head group's partials
    into ``attn_out`` and counts the heads on the reduction row.  2: the instruction counts one arrival on the
    reduction row and nothing else; the O-projection instructions, whose ``reduction_block_idx`` then carries
    the fan-out, merge the partials of all heads themselves."""

    merge_in_last: int = 1


@dataclass
class DecodeAttentionReduction(Instruction):
    OPCODE: ClassVar[int] = 3
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (2,)
    layer_idx: int
    head_start_idx: int
    num_partials: int
    reduction_list: list[int]
    is_terminal: int = 1
    output_partial_idx: int = 0


@dataclass
class OProj_GEMV_Residual(Instruction):
    OPCODE: ClassVar[int] = 4
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (3,)
    layer_idx: int
    tile_M_idx: int
    tile_N_start_idx: int
    tile_N_end_idx: int
    reduction_block_idx: int
    tile_M_granularity: int = TILE_M_GRANULARITY
    tile_N_granularity: int = TILE_N_GRANULARITY


@dataclass
class RMS_LMHead_GEMV(Instruction):
    OPCODE: ClassVar[int] = 7
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (14,)
    start_output_block_idx: int
    end_output_block_idx: int
    tile_M_granularity: int = TILE_M_GRANULARITY
    tile_N_granularity: int = TILE_N_GRANULARITY


@dataclass
class Router_GEMV(Instruction):
    """RMSNorm + router logits of experts [start, end); one instruction also publishes the normalised row."""

    OPCODE: ClassVar[int] = 8
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (4,)
    layer_idx: int
    tile_N_start_idx: int
    tile_N_end_idx: int
    write_normed_hidden: int = 0
    tile_N_granularity: int = ROUTER_TILE_N_GRANULARITY


@dataclass
class Router_SoftmaxTopK(Instruction):
    """softmax over all router logits, top-k: expert_indices / expert_weights."""

    OPCODE: ClassVar[int] = 9
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (8,)
    layer_idx: int


@dataclass
class SharedExpert_UpGate_SiLU(Instruction):
    OPCODE: ClassVar[int] = 10
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (8,)
    layer_idx: int
    tile_M_idx: int
    tile_N_start_idx: int
    tile_N_end_idx: int
    init_shared_out: int = 0
    tile_M_granularity: int = TILE_M_GRANULARITY
    tile_N_granularity: int = TILE_N_GRANULARITY


@dataclass
class SharedExpert_DownProj(Instruction):
    OPCODE: ClassVar[int] = 11
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (10,)
    layer_idx: int
    tile_M_idx: int
    tile_N_start_idx: int
    tile_N_end_idx: int
    split_K_idx: int
    tile_M_granularity: int = TILE_M_GRANULARITY
    tile_N_granularity: int = TILE_N_GRANULARITY
    split_K_granularity: int = SPLIT_K_GRANULARITY_SHARED


@dataclass
class RoutedExpert_UpGate_SiLU(Instruction):
    """``expert_idx`` is the slot 0..top_k-1; the physical expert is expert_indices[slot] at run time."""

    OPCODE: ClassVar[int] = 12
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (9,)
    layer_idx: int
    expert_idx: int
    tile_N_start_idx: int
    tile_N_end_idx: int
    tile_M_granularity: int = TILE_M_GRANULARITY
    tile_N_granularity: int = TILE_N_GRANULARITY


@dataclass
class RoutedExpert_DownProj(Instruction):
    OPCODE: ClassVar[int] = 13
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (12,)
    layer_idx: int
    expert_idx: int
    tile_M_idx: int
    tile_N_start_idx: int
    tile_N_end_idx: int
    tile_M_granularity: int = TILE_M_GRANULARITY
    tile_N_granularity: int = TILE_N_GRANULARITY


@dataclass
class MoE_Combine_Commit(Instruction):
    OPCODE: ClassVar[int] = 14
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (11, 13)
    layer_idx: int
    tile_N_start_idx: int
    tile_N_end_idx: int
    tile_N_granularity: int = TILE_N_GRANULARITY


# ---- several requests ("rows") in one launch: this build's stream, the reference has no MoE route for batch sizes
# above one.  Opcodes 1, 4, 7, 8 keep their words and act on all rows; 2 and 9 name their row in the word behind the
# batch-1 operands; 15 and 16 take the place of 12, 13 and 14.

@dataclass
class DecodeAttentionSplitKVRow(DecodeAttentionSplitKVMerge):
    """Opcode 2 for one row of the batch: the batch-1 instruction on that row's buffers at that row's position."""

    batch_row: int = 0


@dataclass
class Router_SoftmaxTopKRow(Router_SoftmaxTopK):
    """Opcode 9 for one row of the batch (the report of that row's routing for the caller)."""

    batch_row: int = 0


@dataclass
class RoutedExperts_UpGate_Rows(Instruction):
    """Gate/up rows of the layer's distinct experts (the rows' picks merged on the device, ascending expert index):
    item g = (list entry g // (Fm/2), output pair g % (Fm/2)); wave w of part ``part_idx`` takes the items
    ``part_idx*8 + w + k * num_parts*8``.  The parts of a layer must cover 0..num_parts-1 exactly once."""

    OPCODE: ClassVar[int] = 15
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (8,)
    layer_idx: int
    part_idx: int
    num_parts: int
    tile_N_granularity: int = 2


@dataclass
class RoutedExperts_DownCommit_Rows(Instruction):
    """Down-projection rows [start*tile, end*tile) of every distinct expert against the silu vectors of the rows that
    picked it, the rows' terms added per request in slot order, and the commit of those rows for every request."""

    OPCODE: ClassVar[int] = 16
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (15,)
    layer_idx: int
    tile_N_start_idx: int
    tile_N_end_idx: int
    tile_N_granularity: int = 8


ROWS_INSTRUCTION_BY_OPCODE = {
    cls.OPCODE: cls
    for cls in (NoOp, RMS_QKVProj_GEMV_RoPE, DecodeAttentionSplitKVRow, OProj_GEMV_Residual, RMS_LMHead_GEMV, Router_GEMV,
                Router_SoftmaxTopKRow, RoutedExperts_UpGate_Rows, RoutedExperts_DownCommit_Rows)
}

INSTRUCTION_BY_OPCODE = {
    cls.OPCODE: cls
    for cls in (NoOp, RMS_QKVProj_GEMV_RoPE, DecodeAttentionSplitKV, DecodeAttentionReduction, OProj_GEMV_Residual, RMS_LMHead_GEMV,
                Router_GEMV, Router_SoftmaxTopK, SharedExpert_UpGate_SiLU, SharedExpert_DownProj, RoutedExpert_UpGate_SiLU,
                RoutedExpert_DownProj, MoE_Combine_Commit)
}
