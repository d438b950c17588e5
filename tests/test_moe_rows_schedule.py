"""The instruction stream of several MoE requests in one launch (no GPU): every piece of work of a step is scheduled
exactly once, the words are what the kernel decodes, and the byte accounting of a batch step adds up.

The reference has no MoE route for batch sizes above one; the stream is this build's.  A step is defined as the
batch-1 route (…/qwen1_5_moe_a2_7b/A100/single_batch/decode_schedule/instructions/scheduler.py:139-370) for every row.
"""
import dataclasses

import pytest

from qimeng_megakernel_amd.decode_schedule_moe import rows_kernel
from qimeng_megakernel_amd.decode_schedule_moe.instructions import instruction_defs as D
from qimeng_megakernel_amd.decode_schedule_moe.instructions import scheduler as S
from qimeng_megakernel_amd.decode_schedule_moe.model_config import QWEN1_5_MOE_A2_7B, QWEN3_30B_A3B
from qimeng_megakernel_amd.instruction import decode_words


@pytest.mark.parametrize("rows, queues, partials, merge_in_oproj", [(4, 256, 4, False), (2, 256, 2, True), (1, 64, 2, False), (3, 108, 1, True)])
def test_every_piece_of_a_step_is_scheduled_once(rows, queues, partials, merge_in_oproj):
    shape = dataclasses.replace(QWEN3_30B_A3B, num_hidden_layers=3)
    sched = S.MoeRowsScheduler(shape, queues, partials, rows, merge_in_oproj=merge_in_oproj)
    qs = sched.queues()
    assert len(qs) == queues
    flat = [ins for q in qs for ins in q]
    for layer in range(3):
        of = lambda op: [i for i in flat if i.opcode() == op and getattr(i, "layer_idx", None) == layer]
        # QKV rows, O-projection rows, committed rows: each output row once
        for op, total, tile_of in ((1, shape.qkv_out_dim, lambda i: i.tile_N_granularity), (4, shape.hidden_size, lambda i: i.tile_N_granularity),
                                   (16, shape.hidden_size, lambda i: i.tile_N_granularity)):
            covered = sorted((i.tile_N_start_idx * tile_of(i), i.tile_N_end_idx * tile_of(i)) for i in of(op))
            assert covered[0][0] == 0 and covered[-1][1] == total
            assert all(a[1] == b[0] for a, b in zip(covered, covered[1:]))
        assert all((i.tile_N_end_idx - i.tile_N_start_idx) * i.tile_N_granularity <= 16 for i in of(16))
        # who merges the split-KV partials: every O-projection workgroup (its word carries the fan-out), or the last arrival
        assert all(i.reduction_block_idx == (partials if merge_in_oproj else 0) for i in of(4))
        # one split-KV instruction per (row, KV head, slice), merged by the O-projection workgroups
        assert sorted((i.batch_row, i.kv_head_idx, i.partial_idx) for i in of(2)) == [
            (r, h, p) for r in range(rows) for h in range(shape.num_key_value_heads) for p in range(partials)]
        assert all(i.merge_in_last == (2 if merge_in_oproj else 1) and i.num_partials == partials for i in of(2))
        # the router's experts once; one report per row
        experts = sorted((i.tile_N_start_idx, i.tile_N_end_idx) for i in of(8))
        assert experts[0][0] == 0 and experts[-1][1] == shape.num_experts and all(a[1] == b[0] for a, b in zip(experts, experts[1:]))
        assert sum(i.write_normed_hidden for i in of(8)) == 1
        assert sorted(i.batch_row for i in of(9)) == list(range(rows))
        # the parts of the distinct experts' gate/up rows: 0..n-1 once, all naming the same n
        parts = of(15)
        assert sorted(i.part_idx for i in parts) == list(range(queues)) and {i.num_parts for i in parts} == {queues}
    # within a queue: a layer's gate/up part precedes its committing tile (which reads what the part's looks have seen),
    # and the report of layer l stands behind layer l + 1's attention
    for q in qs:
        order = [(i.opcode(), getattr(i, "layer_idx", -1)) for i in q]
        for layer in range(3):
            if (16, layer) in order:
                assert (15, layer) in order and order.index((15, layer)) < order.index((16, layer))
            if (9, layer) in order and layer + 1 < 3:
                assert order.index((9, layer)) > order.index((1, layer + 1))
    assert sum(1 for i in flat if i.opcode() == 7) >= 1
    assert sorted({i.opcode() for i in flat}) == [1, 2, 4, 7, 8, 9, 15, 16]


def test_instruction_words():
    assert D.DecodeAttentionSplitKVRow(5, 3, 4, 1, merge_in_last=2, batch_row=2).serialize() == [2, 5, 3, 4, 1, 2, 2]
    assert D.Router_SoftmaxTopKRow(7, batch_row=3).serialize() == [9, 7, 3]
    assert D.RoutedExperts_UpGate_Rows(1, 17, 256).serialize() == [15, 1, 17, 256, 2]
    assert D.RoutedExperts_DownCommit_Rows(2, 10, 11).serialize() == [16, 2, 10, 11, 8]
    for ins in (D.DecodeAttentionSplitKVRow(5, 3, 4, 1, merge_in_last=2, batch_row=2), D.RoutedExperts_UpGate_Rows(1, 17, 256),
                D.RoutedExperts_DownCommit_Rows(2, 10, 11), D.Router_SoftmaxTopKRow(7, batch_row=3)):
        assert decode_words(ins.padded(), D.ROWS_INSTRUCTION_BY_OPCODE) == ins


def test_models_with_a_shared_expert_have_no_rows_stream():
    with pytest.raises(ValueError, match="shared expert"):
        S.MoeRowsScheduler(QWEN1_5_MOE_A2_7B, 256, 2, 2)
    with pytest.raises(ValueError, match="rows"):
        S.MoeRowsScheduler(QWEN3_30B_A3B, 256, 2, 5)


def test_fan_out_of_the_default_schedule():
    assert rows_kernel.mi355x_scheduler(4, QWEN3_30B_A3B, kv_capacity=520).num_partials == 4    # 64 split-KV instructions
    assert rows_kernel.mi355x_scheduler(4, QWEN3_30B_A3B, kv_capacity=128).num_partials == 2
    assert rows_kernel.mi355x_scheduler(4, QWEN3_30B_A3B, kv_capacity=520, queues=64).num_partials == 1
