"""Host-side instruction scheduler: one decode step -> per-workgroup queues -> int32 tensor.

Follows the structure of the reference scheduler
(`…/A100/single_batch/decode_schedule/instructions/scheduler.py:138-358`): a flat
dependency-ordered instruction list per layer (QKV, split-KV, reduction, O-proj,
up/gate, down) plus the LM head, dealt round-robin onto the workgroup queues and
padded with NoOps to a rectangular ``int32[queues, length, 32]`` tensor.

The numbers are MI355X's: 256 workgroups (one per CU), the tile geometry of
``MI355X_GEOMETRY`` and a KV-length-aware split-KV fan-out.  ``DecodeScheduler``
takes all of them as arguments; ``reference_scheduler()`` plugs in the A100
numbers (108 queues, 16-row tiles, 4 K-slices, 13 partials) and reproduces the
reference's instruction stream word for word, which is what the known-answer
tests check.
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass
from typing import Any, Iterable, Sequence

import torch

from ...instruction import INTS_PER_INSTRUCTION, Instruction
from ..model_config import DecodeShape, LlamaConfig
from .instruction_defs import (
    MI355X_GEOMETRY,
    REFERENCE_GEOMETRY,
    DecodeAttentionReduction,
    DecodeAttentionSplitKV,
    DownProj_GEMV_Residual,
    NoOp,
    OProj_GEMV_Residual,
    RMS_LMHead_GEMV,
    RMS_QKVProj_GEMV_RoPE,
    RMS_UpGateProj_GEMV_SiLU,
    TileGeometry,
)

A100_SM_COUNT = 108
MI355X_CU_COUNT = 256

# Up/gate instruction: [opcode, layer, tile_M, len, blocks..., tile_M_g, tile_N_g]
MAX_TILE_BLOCKS_PER_INSTRUCTION = INTS_PER_INSTRUCTION - 6
# Reduction instruction: [opcode, layer, head, count, len, list..., terminal, output]
ATTENTION_REDUCTION_LIST_CAPACITY = INTS_PER_INSTRUCTION - 7
MAX_REDUCTION_LIST = ATTENTION_REDUCTION_LIST_CAPACITY
#: The reference's CUDA kernel keeps a 16-entry merge workspace; the gfx950
#: kernel merges from registers and is bounded only by the instruction slot.
REFERENCE_MAX_ATTENTION_PARTIALS = 16
MAX_ATTENTION_PARTIALS = ATTENTION_REDUCTION_LIST_CAPACITY
#: with the merge done by the O-proj workgroups no instruction lists the partials
MAX_SELF_MERGE_PARTIALS = 64
#: value of the split-KV instruction's ``merge_in_last`` word per merge mode
ATTENTION_MERGE_MODES = {"separate": 0, "last": 1, "oproj": 2}
#: KV tokens per split-KV partial the fan-out aims for: five passes of a workgroup (8 waves x 8
#: tokens per pass).  Finer splits cost more in merging than they save in streaming (measured:
#: at a 1032-token capacity 4 partials per KV head beat 5 by 3 % and 3 by 2 %).
KV_TOKENS_PER_PASS = 320


def _ceil_div(a: int, b: int) -> int:
    return -(-a // b)


def _split_n_tiles(num_n_tiles: int, sm_count: int) -> list[tuple[int, int]]:
    """Contiguous, as-even-as-possible cut of ``num_n_tiles`` into at most ``sm_count`` spans."""
    if num_n_tiles <= 0:
        return []
    groups = min(num_n_tiles, sm_count)
    small, extra = divmod(num_n_tiles, groups)
    spans: list[tuple[int, int]] = []
    lo = 0
    for g in range(groups):
        hi = lo + small + (1 if g < extra else 0)
        spans.append((lo, hi))
        lo = hi
    return spans


def _chunk_list(items: Sequence[int], chunk_size: int) -> list[list[int]]:
    if chunk_size <= 0:
        raise ValueError("chunk_size must be positive")
    return [list(items[i : i + chunk_size]) for i in range(0, len(items), chunk_size)]


def _round_robin_assign_to_sms(instructions: Iterable[Instruction], sm_count: int) -> list[list[Instruction]]:
    queues: list[list[Instruction]] = [[] for _ in range(sm_count)]
    for i, ins in enumerate(instructions):
        queues[i % sm_count].append(ins)
    return queues


def _get_device(globs: Any) -> torch.device:
    for f in dataclasses.fields(globs):
        value = getattr(globs, f.name)
        if isinstance(value, torch.Tensor):
            return value.device
    return torch.device("cpu")


def _get_sm_count(device: torch.device) -> int:
    """Workgroup count of the schedule: the CU count, capped at 256; 1 off-GPU.

    Mirrors the reference's device probe (`scheduler.py:69-82`), which returns 1
    on a CPU device so that the Python VM runs a single queue.
    """
    device = torch.device(device)
    if device.type != "cuda":
        return 1
    cu_count = torch.cuda.get_device_properties(device).multi_processor_count
    return min(int(cu_count), MI355X_CU_COUNT)


def pick_num_partials(
    sm_count: int,
    kv_capacity: int | None = None,
    *,
    shape: DecodeShape | None = None,
    max_partials: int = MAX_ATTENTION_PARTIALS,
) -> int:
    """Split-KV fan-out per KV head.

    Never more than one wave of workgroups (``sm_count // num_kv_heads``, the
    reference's rule, `scheduler.py:85-94`) nor more than the instruction slot
    can list; and, when the KV capacity of the request is known, no more than
    one partial per ``KV_TOKENS_PER_PASS`` tokens, so short contexts do not pay
    for empty partials and the merge.
    """
    shape = shape or LlamaConfig.shape()
    cap = max(1, sm_count // shape.num_key_value_heads)
    p = min(max_partials, cap)
    if kv_capacity is not None:
        p = min(p, max(1, _ceil_div(int(kv_capacity), KV_TOKENS_PER_PASS)))
    return p


def _validate_num_partials(num_partials: int, max_partials: int = MAX_ATTENTION_PARTIALS) -> None:
    if not 1 <= num_partials <= max_partials:
        raise ValueError(f"num_partials must be in [1, {max_partials}], got {num_partials}")


@dataclass(frozen=True)
class DecodeScheduler:
    """Everything that determines the instruction stream of one decode step."""

    shape: DecodeShape
    geometry: TileGeometry
    sm_count: int
    num_partials: int
    #: who merges the split-KV partials: "separate" reduction instructions (the reference), the
    #: "last" split-KV arrival of a head group, or every "oproj" workgroup for itself
    attention_merge: str = "separate"
    #: give the queues that have just run a split-KV instruction no O-proj rows (their turn in the
    #: round is a no-op): they start late and would otherwise finish the MLP behind everybody else
    oproj_spares_attention: bool = False

    def __post_init__(self) -> None:
        self.geometry.validate(self.shape)
        if self.sm_count < 1:
            raise ValueError("sm_count must be positive")
        _validate_num_partials(self.num_partials, MAX_SELF_MERGE_PARTIALS if self.attention_merge == "oproj" else MAX_ATTENTION_PARTIALS)
        if self.attention_merge not in ATTENTION_MERGE_MODES:
            raise ValueError(f"attention_merge must be one of {sorted(ATTENTION_MERGE_MODES)}")

    # ---- per-op emitters -------------------------------------------------
    def qkvproj(self, layer_idx: int) -> list[Instruction]:
        g = self.geometry.qkv_tile_n
        blocks = _ceil_div(self.shape.qkv_out_dim, g)
        return [
            RMS_QKVProj_GEMV_RoPE(layer_idx, 0, lo, hi, tile_N_granularity=g)
            for lo, hi in _split_n_tiles(blocks, self.sm_count)
        ]

    def attention_split_kv(self, layer_idx: int) -> list[Instruction]:
        return [
            DecodeAttentionSplitKV(layer_idx, kv_head, self.num_partials, p, ATTENTION_MERGE_MODES[self.attention_merge])
            for kv_head in range(self.shape.num_key_value_heads)
            for p in range(self.num_partials)
        ]

    def attention_reduction(self, layer_idx: int) -> list[Instruction]:
        if self.attention_merge != "separate":
            return []
        step = self.shape.attn_reduction_size
        return [
            DecodeAttentionReduction(
                layer_idx, head0, self.num_partials, list(range(self.num_partials))
            )
            for head0 in range(0, self.shape.num_attention_heads, step)
        ]

    def oproj(self, layer_idx: int, first_queue: int = 0) -> list[Instruction]:
        """``first_queue``: the queue the first instruction of this round is dealt to."""
        g = self.geometry.oproj_tile_n
        blocks = _ceil_div(self.shape.hidden_size, g)
        merges = self.num_partials if self.attention_merge == "oproj" else 0
        n_attn = self.shape.num_key_value_heads * self.num_partials
        if self.oproj_spares_attention and self.attention_merge == "oproj" and 0 < n_attn < self.sm_count:
            # The split-KV instructions directly precede this round: they went to the n_attn queues
            # before first_queue.
            sm = self.sm_count
            attention = {(first_queue - 1 - k) % sm for k in range(n_attn)}
            works = [((first_queue + j) % sm) not in attention for j in range(sm)]
            if sum(works) <= blocks:
                spans = iter(_split_n_tiles(blocks, sum(works)))
                out: list[Instruction] = []
                for w in works:
                    if w:
                        lo, hi = next(spans)
                        out.append(OProj_GEMV_Residual(layer_idx, 0, lo, hi, merges, tile_N_granularity=g))
                    else:
                        out.append(NoOp())
                return out
        return [
            OProj_GEMV_Residual(layer_idx, 0, lo, hi, merges, tile_N_granularity=g)
            for lo, hi in _split_n_tiles(blocks, self.sm_count)
        ]

    def upgate(self, layer_idx: int) -> list[Instruction]:
        """Strided block lists, so every down-proj bucket fills at the same pace."""
        g = self.geometry.upgate_tile_n
        blocks = _ceil_div(self.shape.intermediate_size, g)
        groups = min(blocks, self.sm_count)
        out: list[Instruction] = []
        for first in range(groups):
            mine = list(range(first, blocks, groups))
            for chunk in _chunk_list(mine, MAX_TILE_BLOCKS_PER_INSTRUCTION):
                out.append(RMS_UpGateProj_GEMV_SiLU(layer_idx, 0, chunk, tile_N_granularity=g))
        return out

    def downproj(self, layer_idx: int) -> list[Instruction]:
        """One workgroup group per K-slice; the output tiles are spread inside each group."""
        g = self.geometry.down_tile_n
        splits = self.geometry.num_split_k(self.shape)
        blocks = _ceil_div(self.shape.hidden_size, g)
        per_group = max(1, self.sm_count // splits)
        out: list[Instruction] = []
        for split in range(splits):
            first = split * per_group
            last = self.sm_count if split == splits - 1 else min((split + 1) * per_group, self.sm_count)
            for lo, hi in _split_n_tiles(blocks, max(1, last - first)):
                out.append(
                    DownProj_GEMV_Residual(
                        layer_idx, 0, lo, hi, split,
                        tile_N_granularity=g,
                        split_K_granularity=self.geometry.split_k,
                    )
                )
        return out

    def lmhead(self) -> list[Instruction]:
        g = self.geometry.lmhead_tile_n
        blocks = _ceil_div(self.shape.vocab_size, g)
        return [
            RMS_LMHead_GEMV(lo, hi, tile_N_granularity=g)
            for lo, hi in _split_n_tiles(blocks, self.sm_count)
        ]

    # ---- whole step ------------------------------------------------------
    def layer(self, layer_idx: int, start: int = 0) -> list[Instruction]:
        """``start``: instructions dealt before this layer's (the round-robin carries on from there)."""
        head = [
            *self.qkvproj(layer_idx),
            *self.attention_split_kv(layer_idx),
            *self.attention_reduction(layer_idx),
        ]
        return [
            *head,
            *self.oproj(layer_idx, (start + len(head)) % self.sm_count),
            *self.upgate(layer_idx),
            *self.downproj(layer_idx),
        ]

    def instruction_list(self, num_layers: int | None = None) -> list[Instruction]:
        layers = self.shape.num_hidden_layers if num_layers is None else num_layers
        out: list[Instruction] = []
        for layer_idx in range(layers):
            out.extend(self.layer(layer_idx, len(out)))
        if layers == self.shape.num_hidden_layers:
            out.extend(self.lmhead())
        return out

    def queues(self, num_layers: int | None = None) -> list[list[Instruction]]:
        return _round_robin_assign_to_sms(self.instruction_list(num_layers), self.sm_count)

    def expected_counts(self) -> tuple[int, int, int, int]:
        return self.geometry.expected_counts(self.shape)


def reference_scheduler(shape: DecodeShape | None = None, sm_count: int = A100_SM_COUNT) -> DecodeScheduler:
    """The A100 route's numbers: 16-row tiles, split_k 2048, P = min(16, sm // kv_heads)."""
    shape = shape or LlamaConfig.shape()
    p = pick_num_partials(sm_count, shape=shape, max_partials=REFERENCE_MAX_ATTENTION_PARTIALS)
    return DecodeScheduler(shape, REFERENCE_GEOMETRY, sm_count, p)


def mi355x_scheduler(
    shape: DecodeShape | None = None,
    sm_count: int = MI355X_CU_COUNT,
    kv_capacity: int | None = None,
    num_partials: int | None = None,
    attention_merge: str = "oproj",
    oproj_spares_attention: bool = True,
) -> DecodeScheduler:
    shape = shape or LlamaConfig.shape()
    geometry = dataclasses.replace(MI355X_GEOMETRY, split_k=shape.intermediate_size)
    # Up/gate blocks are dealt round-robin: halve the block when that is what makes every
    # workgroup get the same number of them (intermediate 6144: 384 blocks of 16, 768 of 8).
    blocks = shape.intermediate_size // geometry.upgate_tile_n
    if blocks % sm_count != 0 and (2 * blocks) % sm_count == 0:
        geometry = dataclasses.replace(geometry, upgate_tile_n=geometry.upgate_tile_n // 2)
    p = num_partials or pick_num_partials(sm_count, kv_capacity, shape=shape)
    return DecodeScheduler(shape, geometry, sm_count, p, attention_merge, oproj_spares_attention=oproj_spares_attention)


def scheduler_for(globs: Any) -> DecodeScheduler:
    """Scheduler for the device and KV capacity of ``globs`` (cached on the object)."""
    cached = getattr(globs, "_decode_scheduler", None)
    device = _get_device(globs)
    sm_count = _get_sm_count(device)
    kv_capacity = int(globs.k_cache.shape[2]) if getattr(globs, "k_cache", None) is not None else None
    max_p = MAX_SELF_MERGE_PARTIALS
    lse = getattr(globs, "attn_lse_intermediates", None)
    if lse is not None:
        max_p = min(max_p, int(lse.shape[-1]))
    p = pick_num_partials(sm_count, kv_capacity, max_partials=max_p)
    sched = mi355x_scheduler(sm_count=sm_count, num_partials=p)
    if cached == sched:
        return cached
    try:
        globs._decode_scheduler = sched
    except AttributeError:
        pass
    return sched


# ---- reference-named module functions (MI355X numbers) ---------------------
def schedule_qkvproj_gemv(layer_idx: int, sm_count: int) -> list[Instruction]:
    return mi355x_scheduler(sm_count=sm_count, num_partials=1).qkvproj(layer_idx)


def schedule_attention_split_kv(layer_idx: int, num_partials: int) -> list[Instruction]:
    _validate_num_partials(num_partials)
    return mi355x_scheduler(num_partials=num_partials).attention_split_kv(layer_idx)


def schedule_attention_reduction(layer_idx: int, num_partials: int) -> list[Instruction]:
    _validate_num_partials(num_partials)
    return mi355x_scheduler(num_partials=num_partials).attention_reduction(layer_idx)


def schedule_oproj_gemv(layer_idx: int, sm_count: int) -> list[Instruction]:
    return mi355x_scheduler(sm_count=sm_count, num_partials=1).oproj(layer_idx)


def schedule_upgate(layer_idx: int, sm_count: int) -> list[Instruction]:
    return mi355x_scheduler(sm_count=sm_count, num_partials=1).upgate(layer_idx)


def schedule_downproj(layer_idx: int, sm_count: int) -> list[Instruction]:
    return mi355x_scheduler(sm_count=sm_count, num_partials=1).downproj(layer_idx)


def schedule_lmhead_gemv(sm_count: int) -> list[Instruction]:
    return mi355x_scheduler(sm_count=sm_count, num_partials=1).lmhead()


def build_instruction_list(globs: Any, num_layers: int | None = None) -> list[Instruction]:
    """Flat dependency-ordered list (what a sequential VM executes)."""
    return scheduler_for(globs).instruction_list(num_layers)


def build_instruction_queues(globs: Any, num_layers: int | None = None) -> list[list[Instruction]]:
    return scheduler_for(globs).queues(num_layers)


def tensorize_instructions(globs: Any, instruction_queues: list[list[Instruction]]) -> torch.Tensor:
    """Pad queues to equal length with NoOps and store ``int32[queues, length, 32]`` on ``globs``."""
    length = max((len(q) for q in instruction_queues), default=0)
    rows: list[list[int]] = []
    for q in instruction_queues:
        q.extend(NoOp() for _ in range(length - len(q)))
        rows.extend(ins.padded() for ins in q)
    tensor = torch.tensor(rows, dtype=torch.int32).view(len(instruction_queues), length, INTS_PER_INSTRUCTION)
    tensor = tensor.to(_get_device(globs))
    globs.instructions = tensor
    return tensor


#: Heads of 128: tokens of context per split-KV slice beyond which a request's later steps get a wider fan-out
#: (Qwen3-1.7B shape, step time at contexts ~64 / ~512 / ~1000 with 4, 8, 12 slices per KV head: 838/853/932,
#: 854/856/903, 869/870/882 us).  Heads of 64 keep one stream per request: there the attention phase hides behind
#: the rows the O-proj workgroups fetch for the up/gate GEMV, and the one fan-out of the capacity rule is the best one.
LONG_CONTEXT_TOKENS_PER_SLICE = 80
LONG_CONTEXT_FAN_OUT_STEP = 4


def fan_out_plan(sm_count: int, kv_capacity: int | None, *, shape: DecodeShape | None = None,
                 max_partials: int = MAX_ATTENTION_PARTIALS) -> list[tuple[int, int]]:
    """``[(first position, fan-out), ...]``: the split-KV fan-out of a request's decode steps by position.
    The first entry (position 0) is the fan-out ``pick_num_partials`` gives; the fan-out only ever grows."""
    shape = shape or LlamaConfig.shape()
    base = pick_num_partials(sm_count, kv_capacity, shape=shape, max_partials=max_partials)
    plan = [(0, base)]
    if shape.head_dim <= 64 or kv_capacity is None:
        return plan
    cap = min(max_partials, max(1, sm_count // shape.num_key_value_heads))
    p = base
    while True:
        p += LONG_CONTEXT_FAN_OUT_STEP
        first = (p - LONG_CONTEXT_FAN_OUT_STEP // 2) * LONG_CONTEXT_TOKENS_PER_SLICE   # 8 slices from context 480 on, 12 from 800 on
        if p > cap or first >= int(kv_capacity):
            return plan
        plan.append((first, p))


def build(globs: Any, num_layers: int | None = None) -> torch.Tensor:
    """The request's instruction tensor on ``globs.instructions``; where the fan-out plan has later entries, their
    tensors wait in ``globs.instruction_plan`` (``call_mk`` picks by ``position_id``)."""
    base = tensorize_instructions(globs, build_instruction_queues(globs, num_layers))
    globs.instruction_plan = None
    sched = scheduler_for(globs)
    kv_capacity = int(globs.k_cache.shape[2]) if getattr(globs, "k_cache", None) is not None else None
    lse = getattr(globs, "attn_lse_intermediates", None)
    max_p = MAX_SELF_MERGE_PARTIALS if lse is None else min(MAX_SELF_MERGE_PARTIALS, int(lse.shape[-1]))
    plan = fan_out_plan(sched.sm_count, kv_capacity, shape=sched.shape, max_partials=max_p)
    if len(plan) > 1 and plan[0][1] == sched.num_partials:
        later = []
        for first, p in plan[1:]:
            tensorize_instructions(globs, dataclasses.replace(sched, num_partials=p).queues(num_layers))
            later.append((first, globs.instructions))
        globs.instructions = base
        globs.instruction_plan = (base, later)
    return base
