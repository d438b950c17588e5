"""The ten opcodes of the batch route and their counter protocol.

Opcodes, operand order and defaults are the reference's
(`…/A100/multi_batch/decode_schedule/instructions/instruction_defs.py:11-211`), so a stream
built by either scheduler serialises to the same words.  Compared with the batch-1 route the
three RMSNorms are instructions of their own — one per batch row, writing ``attn_rms_out`` /
``mlp_rms_out`` / ``lm_head_rms_out`` — the projections are GEMMs over all B rows, and the two
attention instructions carry the batch row they work on.

Counters ``barriers[layer, opcode - 1, slot]`` (`…/instructions/python_vm.py:139-730`):

=====  ===========================  ==========================================  =====================
row    producer                     slot                                        final count
=====  ===========================  ==========================================  =====================
0      1 attention RMSNorm row      0                                           B
1      2 QKV GEMM + RoPE            q/k/v head index                            head_dim / 16
2      3 split-KV attention         batch_row * (Hq + 2 Hkv) + query head       num_partials
3      4 attention reduction        batch_row                                   Hq
4      5 O-proj GEMM + residual     0                                           hidden / 16
5      6 MLP RMSNorm row            0                                           B
6      7 up/gate GEMM + SiLU        0                                           intermediate / 16
7      8 down GEMM + residual       0                                           hidden / 16
8      9 LM-head RMSNorm row        0  (of the last layer)                      B
=====  ===========================  ==========================================  =====================
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import ClassVar

from ...instruction import Instruction

TILE_M_GRANULARITY = 16   # batch rows per GEMM tile: one tile covers the whole batch (B <= 16)
TILE_N_GRANULARITY = 16   # output rows per GEMM block
MAX_BATCH = TILE_M_GRANULARITY


@dataclass
class NoOp(Instruction):
    OPCODE: ClassVar[int] = 0


@dataclass
class AttnRMS(Instruction):
    """attn_rms_out[batch_row] = RMSNorm(hidden_states[batch_row]); words 3..5 are reserved."""

    OPCODE: ClassVar[int] = 1
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (8,)
    layer_idx: int
    batch_size: int
    res0: int = 0
    res1: int = 0
    res2: int = 0
    batch_row: int = 0


@dataclass
class QKVProj_GEMM_RoPE(Instruction):
    """QKV rows of blocks [start, end) for all batch rows from attn_rms_out; RoPE at each row's
    position; q -> q_post_rope, k/v -> the row's cache line."""

    OPCODE: ClassVar[int] = 2
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (1,)
    layer_idx: int
    batch_size: int
    tile_M_idx: int
    tile_N_start_idx: int
    tile_N_end_idx: int
    tile_M_granularity: int = TILE_M_GRANULARITY
    tile_N_granularity: int = TILE_N_GRANULARITY


@dataclass
class DecodeAttentionSplitKV(Instruction):
    """One context slice of one (batch row, KV head).  ``seq_len`` -1: the row's position + 1 at run
    time; ``is_active`` 0: only counts, 1: always works, -1: follows the row's active flag."""

    OPCODE: ClassVar[int] = 3
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (2,)
    layer_idx: int
    batch_idx: int
    kv_head_idx: int
    num_partials: int
    partial_idx: int
    seq_len: int = -1
    is_active: int = -1


@dataclass
class DecodeAttentionSplitKVMerge(DecodeAttentionSplitKV):
    """Extension of this build (same opcode, one more word): with ``merge_in_last`` set, the instruction
    whose arrival completes the head group's counters also merges the group's partials into ``attn_out``
    and counts on the reduction row; such a stream carries no reduction instructions."""

    merge_in_last: int = 1


@dataclass
class DecodeAttentionReduction(Instruction):
    """Log-sum-exp merge of the listed partials for four query heads of one batch row."""

    OPCODE: ClassVar[int] = 4
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (3,)
    layer_idx: int
    batch_idx: int
    head_start_idx: int
    num_partials: int
    reduction_list: list[int]
    is_terminal: bool = True
    output_partial_idx: int = 0
    valid_partials: int = -1
    is_active: int = -1


@dataclass
class OProj_GEMM_Residual(Instruction):
    OPCODE: ClassVar[int] = 5
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (4,)
    layer_idx: int
    batch_size: int
    tile_M_idx: int
    tile_N_start_idx: int
    tile_N_end_idx: int
    reduction_block_idx: int
    tile_M_granularity: int = TILE_M_GRANULARITY
    tile_N_granularity: int = TILE_N_GRANULARITY


@dataclass
class MlpRMS(Instruction):
    OPCODE: ClassVar[int] = 6
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (5,)
    layer_idx: int
    batch_size: int
    res0: int = 0
    res1: int = 0
    res2: int = 0
    batch_row: int = 0


@dataclass
class UpGateProj_GEMM_SiLU(Instruction):
    OPCODE: ClassVar[int] = 7
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (6,)
    layer_idx: int
    batch_size: int
    tile_M_idx: int
    tile_N_block_idxs: list[int]
    tile_M_granularity: int = TILE_M_GRANULARITY
    tile_N_granularity: int = TILE_N_GRANULARITY


@dataclass
class DownProj_GEMM_Residual(Instruction):
    """Full K per instruction: one rounding of the whole product, as the fused route."""

    OPCODE: ClassVar[int] = 8
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (7,)
    layer_idx: int
    batch_size: int
    tile_M_idx: int
    tile_N_start_idx: int
    tile_N_end_idx: int
    tile_M_granularity: int = TILE_M_GRANULARITY
    tile_N_granularity: int = TILE_N_GRANULARITY


@dataclass
class LMHeadRMS(Instruction):
    """lm_head_rms_out[batch_row]; words 2..5 are reserved, the row is word 6 as for the other two."""

    OPCODE: ClassVar[int] = 9
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (8,)
    batch_size: int
    res0: int = 0
    res1: int = 0
    res2: int = 0
    res3: int = 0
    batch_row: int = 0


@dataclass
class LMHeadProj_GEMM(Instruction):
    OPCODE: ClassVar[int] = 10
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (9,)
    batch_size: int
    start_output_block_idx: int
    end_output_block_idx: int
    tile_M_granularity: int = TILE_M_GRANULARITY
    tile_N_granularity: int = TILE_N_GRANULARITY


OPCODE_TO_CLASS = {
    cls.OPCODE: cls
    for cls in (NoOp, AttnRMS, QKVProj_GEMM_RoPE, DecodeAttentionSplitKV, DecodeAttentionReduction, OProj_GEMM_Residual,
                MlpRMS, UpGateProj_GEMM_SiLU, DownProj_GEMM_Residual, LMHeadRMS, LMHeadProj_GEMM)
}
