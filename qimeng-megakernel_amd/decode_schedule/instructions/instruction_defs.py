"""The seven decode opcodes and the counter protocol that orders them.

Opcodes, operand order and barrier rows are those of the reference route
(`…/A100/single_batch/decode_schedule/instructions/instruction_defs.py:24-177`),
so an instruction tensor from either scheduler runs on the gfx950 kernel.
What differs is that the tile geometry is not baked into module constants: it
is a ``TileGeometry`` record, because the MI355X schedule cuts the output rows
finer (256 workgroups instead of 108) and does not split the down projection
along K.  ``REFERENCE_GEOMETRY`` reproduces the reference's numbers.

Counter protocol (``barriers[layer, opcode-1, slot]``, monotone within a step):

=====  ==========================  =====================================  ======================
row    producer                    slot                                   final count
=====  ==========================  =====================================  ======================
0      1 RMS+QKV+RoPE              q/k/v head index                       head_dim / qkv_tile_n
1      2 split-KV attention        query head                             num_partials
2      3 attention reduction       0                                      num_attention_heads
3      4 O-proj + residual         0                                      hidden / oproj_tile_n
4      5 RMS+up/gate+SiLU          block // (split_k / upgate_tile_n)     split_k / upgate_tile_n
5      6 down-proj + residual      0                                      (hidden / down_tile_n) * (inter / split_k)
=====  ==========================  =====================================  ======================
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass
from typing import ClassVar

from ...instruction import Instruction
from ..model_config import DecodeShape, LLAMA_3_2_1B

FIRST_OPCODE = 1
LAST_OPCODE = 7
TILE_M_GRANULARITY = 1


def BARRIER_ROW(opcode: int) -> int:
    """Counter row written by ``opcode`` (padding opcode 0 owns none)."""
    if type(opcode) is not int:
        raise TypeError(f"opcode must be int, got {type(opcode).__name__}")
    if opcode < FIRST_OPCODE or opcode > LAST_OPCODE:
        raise ValueError(f"opcode must be in [{FIRST_OPCODE}, {LAST_OPCODE}], got {opcode}")
    return opcode - FIRST_OPCODE


@dataclass(frozen=True)
class TileGeometry:
    """Output-row tile sizes per GEMV opcode and the down-projection K split."""

    qkv_tile_n: int = 16
    oproj_tile_n: int = 16
    upgate_tile_n: int = 16
    down_tile_n: int = 16
    lmhead_tile_n: int = 16
    split_k: int = 2048

    def validate(self, shape: DecodeShape) -> None:
        def need(cond: bool, msg: str) -> None:
            if not cond:
                raise ValueError(f"tile geometry does not fit the model shape: {msg}")

        need(self.qkv_tile_n % 2 == 0, "RoPE pairs must stay inside one QKV tile")
        need(shape.head_dim % self.qkv_tile_n == 0, "QKV tiles must not straddle heads")
        need(shape.hidden_size % self.oproj_tile_n == 0, "hidden % oproj_tile_n")
        need(shape.hidden_size % self.down_tile_n == 0, "hidden % down_tile_n")
        need(shape.intermediate_size % self.split_k == 0, "intermediate % split_k")
        need(self.split_k % self.upgate_tile_n == 0, "split_k % upgate_tile_n")

    # ---- final counter values (what a consumer waits for) ----
    def qkv_blocks_per_head(self, shape: DecodeShape) -> int:
        return shape.head_dim // self.qkv_tile_n

    def oproj_blocks(self, shape: DecodeShape) -> int:
        return shape.hidden_size // self.oproj_tile_n

    def upgate_blocks_per_bucket(self, shape: DecodeShape) -> int:
        return self.split_k // self.upgate_tile_n

    def num_split_k(self, shape: DecodeShape) -> int:
        return shape.intermediate_size // self.split_k

    def down_arrivals(self, shape: DecodeShape) -> int:
        return (shape.hidden_size // self.down_tile_n) * self.num_split_k(shape)

    def expected_counts(self, shape: DecodeShape) -> tuple[int, int, int, int]:
        """The four numbers the device needs besides the instruction words."""
        return (
            self.qkv_blocks_per_head(shape),
            self.oproj_blocks(shape),
            self.upgate_blocks_per_bucket(shape),
            self.down_arrivals(shape),
        )


#: The reference's geometry: every tile 16 rows, down projection in 4 K-slices.
REFERENCE_GEOMETRY = TileGeometry()

#: MI355X: 256 workgroups.  QKV in 4-row tiles (3 per workgroup), O-proj and
#: down-proj in 8-row tiles (one per workgroup), full-K down projection so the
#: residual update is a single deterministic bf16 add, as in the fused form.
MI355X_GEOMETRY = TileGeometry(
    qkv_tile_n=4,
    oproj_tile_n=8,
    upgate_tile_n=16,
    down_tile_n=8,
    lmhead_tile_n=16,
    split_k=LLAMA_3_2_1B.intermediate_size,
)

# Module-level names the reference exposes, bound to the reference geometry.
TILE_N_GRANULARITY = REFERENCE_GEOMETRY.qkv_tile_n
SPLIT_K_GRANULARITY = REFERENCE_GEOMETRY.split_k
NUM_DOWNPROJ_SPLIT_K = REFERENCE_GEOMETRY.num_split_k(LLAMA_3_2_1B)
DOWNPROJ_BARRIER_COUNT = REFERENCE_GEOMETRY.down_arrivals(LLAMA_3_2_1B)
UPGATE_BLOCKS_PER_SIGNAL_BUCKET = REFERENCE_GEOMETRY.upgate_blocks_per_bucket(LLAMA_3_2_1B)


@dataclass
class NoOp(Instruction):
    """Queue padding; the device skips it."""

    OPCODE: ClassVar[int] = 0


@dataclass
class RMS_QKVProj_GEMV_RoPE(Instruction):
    """RMSNorm -> rows [start, end) * tile of W_qkv -> RoPE on q,k -> q_post_rope / KV append."""

    OPCODE: ClassVar[int] = 1
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (6,)
    layer_idx: int
    tile_M_idx: int
    tile_N_start_idx: int
    tile_N_end_idx: int
    tile_M_granularity: int = TILE_M_GRANULARITY
    tile_N_granularity: int = TILE_N_GRANULARITY


@dataclass
class DecodeAttentionSplitKV(Instruction):
    """One KV head, one contiguous slice of the context, all query heads of the group.

    ``merge_in_last`` extends the reference's four operands (its word is 0 in any
    stream the reference scheduler builds).  1: the workgroup whose arrival
    completes the head group's split-KV counter also performs the log-sum-exp
    merge of all partials and publishes on the reduction row.  2: the partial only
    arrives on the reduction row (slot 0, one arrival per instruction) and every
    O-proj instruction merges the partials itself (its ``reduction_block_idx``
    then carries ``num_partials``).  Either way the schedule carries no separate
    reduction instructions.
    """

    OPCODE: ClassVar[int] = 2
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (1,)
    layer_idx: int
    kv_head_idx: int
    num_partials: int
    partial_idx: int
    merge_in_last: int = 0


@dataclass
class DecodeAttentionReduction(Instruction):
    """Log-sum-exp merge of the listed partials for ``attn_reduction_size`` query heads."""

    OPCODE: ClassVar[int] = 3
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (2,)
    layer_idx: int
    head_start_idx: int
    num_partials: int
    reduction_list: list[int]
    is_terminal: bool = True
    output_partial_idx: int = 0


@dataclass
class OProj_GEMV_Residual(Instruction):
    """hidden[rows] += W_o[rows] . attn_out

    ``reduction_block_idx`` is 0 in the reference's streams.  A positive value P
    means: wait for the ``num_kv_heads * P`` split-KV arrivals on the reduction
    row and merge the P partials of every head before the GEMV.
    """

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
class RMS_UpGateProj_GEMV_SiLU(Instruction):
    """RMSNorm -> up and gate rows of the listed blocks -> silu(gate) * up -> silu_out"""

    OPCODE: ClassVar[int] = 5
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (4,)
    layer_idx: int
    tile_M_idx: int
    tile_N_block_idxs: list[int]
    tile_M_granularity: int = TILE_M_GRANULARITY
    tile_N_granularity: int = TILE_N_GRANULARITY


@dataclass
class DownProj_GEMV_Residual(Instruction):
    """hidden[rows] += W_d[rows, split] . silu_out[split]; split b waits only on up/gate bucket b."""

    OPCODE: ClassVar[int] = 6
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (5,)
    layer_idx: int
    tile_M_idx: int
    tile_N_start_idx: int
    tile_N_end_idx: int
    split_K_idx: int
    tile_M_granularity: int = TILE_M_GRANULARITY
    tile_N_granularity: int = TILE_N_GRANULARITY
    split_K_granularity: int = SPLIT_K_GRANULARITY


@dataclass
class RMS_LMHead_GEMV(Instruction):
    """Final RMSNorm -> logits rows of blocks [start, end)."""

    OPCODE: ClassVar[int] = 7
    PREV_OPCODES: ClassVar[tuple[int, ...]] = (6,)
    start_output_block_idx: int
    end_output_block_idx: int
    tile_M_granularity: int = TILE_M_GRANULARITY
    tile_N_granularity: int = TILE_N_GRANULARITY


OPCODE_TO_CLASS: dict[int, type] = {
    cls.OPCODE: cls
    for cls in (
        NoOp,
        RMS_QKVProj_GEMV_RoPE,
        DecodeAttentionSplitKV,
        DecodeAttentionReduction,
        OProj_GEMV_Residual,
        RMS_UpGateProj_GEMV_SiLU,
        DownProj_GEMV_Residual,
        RMS_LMHead_GEMV,
    )
}

__all__ = [name for name in dir() if not name.startswith("_") and name not in ("dataclasses", "dataclass", "ClassVar")]
