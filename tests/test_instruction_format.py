"""Instruction wire format and the scheduler's known answers (pure integer work).

Known answers are hand-derived from the reference scheduler's arithmetic
(`…/decode_schedule/instructions/scheduler.py:138-358`) and, for the full
stream, pinned by a digest written from the imported reference
(tests/golden/reference_schedule_sm108.json).
"""
import hashlib
import json

import numpy as np
import pytest

from conftest import GOLDEN
from qimeng_megakernel_amd.instruction import INTS_PER_INSTRUCTION, Instruction, decode_words, run_pyvm_sequence
from qimeng_megakernel_amd.decode_schedule.instructions import instruction_defs as D
from qimeng_megakernel_amd.decode_schedule.instructions import scheduler as S
from qimeng_megakernel_amd.decode_schedule.model_config import LLAMA_3_2_1B


def test_serialize_known_words():
    assert D.RMS_QKVProj_GEMV_RoPE(3, 0, 10, 12).serialize() == [1, 3, 0, 10, 12, 1, 16]
    assert D.DecodeAttentionSplitKV(2, 5, 13, 7).serialize() == [2, 2, 5, 13, 7, 0]
    assert D.DecodeAttentionSplitKV(2, 5, 13, 7, 2).padded()[:7] == [2, 2, 5, 13, 7, 2, 0]
    assert D.DecodeAttentionReduction(1, 8, 3, [0, 1, 2]).serialize() == [3, 1, 8, 3, 3, 0, 1, 2, 1, 0]
    assert D.OProj_GEMV_Residual(0, 0, 4, 6, 0).serialize() == [4, 0, 0, 4, 6, 0, 1, 16]
    assert D.RMS_UpGateProj_GEMV_SiLU(0, 0, [7, 115, 223]).serialize() == [5, 0, 0, 3, 7, 115, 223, 1, 16]
    assert D.DownProj_GEMV_Residual(9, 0, 0, 5, 2).serialize() == [6, 9, 0, 0, 5, 2, 1, 16, 2048]
    assert D.RMS_LMHead_GEMV(75, 150).serialize() == [7, 75, 150, 1, 16]
    assert D.NoOp().serialize() == [0]


def test_padding_and_overflow():
    words = D.RMS_LMHead_GEMV(0, 1).padded()
    assert len(words) == INTS_PER_INSTRUCTION and words[5:] == [0] * 27
    full = D.RMS_UpGateProj_GEMV_SiLU(0, 0, list(range(26)))
    assert len(full.serialize()) == 32
    with pytest.raises(ValueError):
        D.RMS_UpGateProj_GEMV_SiLU(0, 0, list(range(27))).padded()


def test_none_tuple_and_bad_field():
    import dataclasses

    @dataclasses.dataclass
    class Odd(Instruction):
        OPCODE = 9
        a: object = None
        b: tuple = (4, 5)

    assert Odd().serialize() == [9, 0, 2, 4, 5]
    with pytest.raises(ValueError):
        Odd(a=1.5).serialize()


def test_decode_words_roundtrip():
    for ins in S.mi355x_scheduler(num_partials=5).layer(3)[::37]:
        back = decode_words(ins.padded(), D.OPCODE_TO_CLASS)
        assert back == ins


def test_barrier_row():
    assert [D.BARRIER_ROW(op) for op in range(1, 8)] == list(range(7))
    with pytest.raises(ValueError):
        D.BARRIER_ROW(0)
    with pytest.raises(TypeError):
        D.BARRIER_ROW(True)


def test_run_pyvm_sequence_missing_handler():
    with pytest.raises(KeyError):
        run_pyvm_sequence(None, [D.NoOp()], {})


# ---------------------------------------------------------------- scheduler ----
def test_split_n_tiles_known_answers():
    def sizes(n, sm):
        out = {}
        for lo, hi in S._split_n_tiles(n, sm):
            out[hi - lo] = out.get(hi - lo, 0) + 1
        return out

    assert sizes(192, 108) == {2: 84, 1: 24}          # QKV blocks on 108 SMs
    assert sizes(128, 108) == {2: 20, 1: 88}          # O-proj
    assert sizes(128, 27) == {5: 20, 4: 7}            # down-proj inside one K-slice group
    assert sizes(8016, 108) == {75: 24, 74: 84}       # LM head
    assert S._split_n_tiles(0, 4) == [] and S._split_n_tiles(3, 8) == [(0, 1), (1, 2), (2, 3)]


def test_reference_schedule_known_answers():
    r = S.reference_scheduler()
    assert r.num_partials == 13
    per_layer = [len(x) for x in (r.qkvproj(0), r.attention_split_kv(0), r.attention_reduction(0), r.oproj(0), r.upgate(0), r.downproj(0))]
    assert per_layer == [108, 104, 8, 108, 108, 108]
    assert len(r.lmhead()) == 108
    flat = r.instruction_list()
    assert len(flat) == 8812
    assert max(len(q) for q in r.queues()) == 82
    # strided up/gate: 512 blocks over 108 groups -> 80 groups of 5, 28 of 4
    lens = [len(i.tile_N_block_idxs) for i in r.upgate(0)]
    assert lens.count(5) == 80 and lens.count(4) == 28
    assert r.upgate(0)[7].tile_N_block_idxs == [7, 115, 223, 331, 439]
    # down-proj: 4 K-slice groups of 27 SMs
    assert [i.split_K_idx for i in r.downproj(0)] == [s for s in range(4) for _ in range(27)]
    assert r.expected_counts() == (4, 128, 128, 512)


def test_reference_schedule_digest_from_imported_reference():
    fix = json.loads((GOLDEN / "reference_schedule_sm108.json").read_text())
    r = S.reference_scheduler()
    arr = np.asarray([i.padded() for i in r.instruction_list()], dtype=np.int32)
    assert arr.shape[0] == fix["total"]
    for idx, words in fix["samples"].items():
        assert arr[int(idx)].tolist() == words
    assert hashlib.sha256(arr.tobytes()).hexdigest() == fix["sha256_flat_int32"]


def _coverage(ins_list, shape):
    """rows written per output tensor by a layer's instructions."""
    import collections

    rows = collections.defaultdict(collections.Counter)
    for i in ins_list:
        op = i.opcode()
        if op in (1, 4, 6):
            t = i.tile_N_granularity
            key = (op, getattr(i, "split_K_idx", 0))
            for r in range(i.tile_N_start_idx * t, i.tile_N_end_idx * t):
                rows[key][r] += 1
        elif op == 5:
            t = i.tile_N_granularity
            for b in i.tile_N_block_idxs:
                for r in range(b * t, (b + 1) * t):
                    rows[(5, 0)][r] += 1
        elif op == 7:
            t = i.tile_N_granularity
            for r in range(i.start_output_block_idx * t, i.end_output_block_idx * t):
                rows[(7, 0)][r] += 1
    return rows


@pytest.mark.parametrize("make", [S.reference_scheduler, lambda: S.mi355x_scheduler(num_partials=16)])
def test_every_output_row_exactly_once(make):
    sched = make()
    shape = sched.shape
    rows = _coverage(sched.layer(0) + sched.lmhead(), shape)
    assert sorted(rows[(1, 0)]) == list(range(shape.qkv_out_dim)) and set(rows[(1, 0)].values()) == {1}
    assert sorted(rows[(4, 0)]) == list(range(shape.hidden_size)) and set(rows[(4, 0)].values()) == {1}
    assert sorted(rows[(5, 0)]) == list(range(shape.intermediate_size)) and set(rows[(5, 0)].values()) == {1}
    for split in range(sched.geometry.num_split_k(shape)):
        assert sorted(rows[(6, split)]) == list(range(shape.hidden_size))
    assert sorted(rows[(7, 0)]) == list(range(shape.vocab_size)) and set(rows[(7, 0)].values()) == {1}


def _simulate(sched, num_layers):
    """In-order execution of the round-robin queues against the counter protocol (integers only).

    Returns the final counters; raises if the queues deadlock.
    """
    shape, geo = sched.shape, sched.geometry
    bph, opb, ubk, dwn = sched.expected_counts()
    ctr = np.zeros((num_layers, 10, shape.num_heads), dtype=np.int64)
    nq, nkv, ratio = shape.num_attention_heads, shape.num_key_value_heads, shape.gqa_ratio

    def ready(i):
        op = i.opcode()
        if op == 1:
            return i.layer_idx == 0 or ctr[i.layer_idx - 1, 5, 0] == dwn
        if op == 2:
            r = ctr[i.layer_idx, 0]
            return all(r[i.kv_head_idx * ratio + j] == bph for j in range(ratio)) and r[nq + i.kv_head_idx] == bph and r[nq + nkv + i.kv_head_idx] == bph
        if op == 3:
            return all(ctr[i.layer_idx, 1, i.head_start_idx + j] == i.num_partials for j in range(ratio))
        if op == 4:
            return ctr[i.layer_idx, 2, 0] == (nkv * i.reduction_block_idx if i.reduction_block_idx else nq)
        if op == 5:
            return ctr[i.layer_idx, 3, 0] == opb
        if op == 6:
            return ctr[i.layer_idx, 4, i.split_K_idx] == ubk
        if op == 7:
            return ctr[num_layers - 1, 5, 0] == dwn
        return True

    def retire(i):
        op = i.opcode()
        if op == 1:
            for b in range(i.tile_N_start_idx, i.tile_N_end_idx):
                ctr[i.layer_idx, 0, b // bph] += 1
        elif op == 2:
            if i.merge_in_last == 2:
                ctr[i.layer_idx, 2, 0] += 1
                return
            ctr[i.layer_idx, 1, i.kv_head_idx * ratio : (i.kv_head_idx + 1) * ratio] += 1
            if i.merge_in_last == 1 and ctr[i.layer_idx, 1, i.kv_head_idx * ratio] == i.num_partials:
                ctr[i.layer_idx, 2, 0] += ratio
        elif op == 3:
            ctr[i.layer_idx, 2, 0] += ratio
        elif op == 4:
            ctr[i.layer_idx, 3, 0] += i.tile_N_end_idx - i.tile_N_start_idx
        elif op == 5:
            for b in i.tile_N_block_idxs:
                ctr[i.layer_idx, 4, b // ubk] += 1
        elif op == 6:
            ctr[i.layer_idx, 5, 0] += i.tile_N_end_idx - i.tile_N_start_idx

    queues = sched.queues(num_layers)
    heads = [0] * len(queues)
    remaining = sum(len(q) for q in queues)
    while remaining:
        progressed = False
        for qi, q in enumerate(queues):
            while heads[qi] < len(q) and ready(q[heads[qi]]):
                retire(q[heads[qi]])
                heads[qi] += 1
                remaining -= 1
                progressed = True
        if not progressed:
            raise AssertionError("instruction queues deadlock")
    return ctr


@pytest.mark.parametrize("which", ["reference", "mi355x", "mi355x_last", "mi355x_97"])
def test_queues_drain_and_counters_end_state(which):
    import dataclasses

    shape = dataclasses.replace(LLAMA_3_2_1B, num_hidden_layers=3)
    if which == "reference":
        sched = S.reference_scheduler(shape)
    elif which == "mi355x":
        sched = S.mi355x_scheduler(shape, num_partials=16)
    elif which == "mi355x_last":
        sched = S.mi355x_scheduler(shape, num_partials=5, attention_merge="last")
    else:  # an awkward workgroup count must still be a valid schedule
        sched = S.mi355x_scheduler(shape, sm_count=97, num_partials=7)
    ctr = _simulate(sched, 3)
    bph, opb, ubk, dwn = sched.expected_counts()
    for layer in range(3):
        assert (ctr[layer, 0, : shape.num_heads] == bph).all()
        if sched.attention_merge == "oproj":
            assert ctr[layer, 1].sum() == 0
            assert ctr[layer, 2, 0] == shape.num_key_value_heads * sched.num_partials
        else:
            assert (ctr[layer, 1, : shape.num_attention_heads] == sched.num_partials).all()
            assert ctr[layer, 2, 0] == shape.num_attention_heads
        assert ctr[layer, 3, 0] == opb
        assert (ctr[layer, 4, : sched.geometry.num_split_k(shape)] == ubk).all()
        assert ctr[layer, 5, 0] == dwn
    assert ctr[:, 6:].sum() == 0


def test_pick_num_partials():
    assert S.pick_num_partials(108, max_partials=16) == 13            # the reference's A100 answer
    assert S.pick_num_partials(256) == S.MAX_ATTENTION_PARTIALS == 25
    assert S.pick_num_partials(256, kv_capacity=40) == 1
    assert S.pick_num_partials(256, kv_capacity=300) == 1
    assert S.pick_num_partials(256, kv_capacity=400) == 2
    assert S.pick_num_partials(256, kv_capacity=1032) == 4
    assert S.pick_num_partials(4) == 1
    with pytest.raises(ValueError):
        S.schedule_attention_split_kv(0, 26)


def test_fan_out_plan_by_position():
    """One stream per request for heads of 64; heads of 128 get 4 more slices per KV head every 320 tokens of context
    (8 from position 480 on, 12 from 800 on, ...), never beyond one workgroup per slice or the partial slots."""
    from qimeng_megakernel_amd.decode_schedule.model_config import QWEN3_1_7B
    assert S.fan_out_plan(256, 1040, shape=LLAMA_3_2_1B, max_partials=32) == [(0, 4)]
    assert S.fan_out_plan(256, None, shape=QWEN3_1_7B, max_partials=32) == [(0, 32)]
    assert S.fan_out_plan(256, 1040, shape=QWEN3_1_7B, max_partials=32) == [(0, 4), (480, 8), (800, 12)]
    assert S.fan_out_plan(256, 1040, shape=QWEN3_1_7B, max_partials=8) == [(0, 4), (480, 8)]
    assert S.fan_out_plan(256, 200, shape=QWEN3_1_7B, max_partials=32) == [(0, 1)]
    assert S.fan_out_plan(256, 600, shape=QWEN3_1_7B, max_partials=32) == [(0, 2), (320, 6)]
    plan = S.fan_out_plan(256, 4096, shape=QWEN3_1_7B, max_partials=32)
    assert plan[0] == (0, 13) and plan[-1] == (2160, 29) and all(b[1] - a[1] == 4 for a, b in zip(plan, plan[1:]))


def test_geometry_validation():
    with pytest.raises(ValueError):
        D.TileGeometry(qkv_tile_n=3).validate(LLAMA_3_2_1B)
    with pytest.raises(ValueError):
        D.TileGeometry(qkv_tile_n=48).validate(LLAMA_3_2_1B)
    with pytest.raises(ValueError):
        D.TileGeometry(split_k=3000).validate(LLAMA_3_2_1B)
    assert D.MI355X_GEOMETRY.expected_counts(LLAMA_3_2_1B) == (16, 256, 512, 256)


def test_tensorize_pads_with_noops():
    import torch

    class G:  # minimal stand-in with one tensor field
        pass

    import dataclasses

    @dataclasses.dataclass
    class Holder:
        instructions: object = None
        hidden_states: object = None

    g = Holder(hidden_states=torch.zeros(4))
    queues = [[D.RMS_LMHead_GEMV(0, 1), D.RMS_LMHead_GEMV(1, 2)], [D.RMS_LMHead_GEMV(2, 3)]]
    t = S.tensorize_instructions(g, queues)
    assert t.shape == (2, 2, 32) and t.dtype == torch.int32 and g.instructions is t
    assert t[1, 1].tolist() == [0] * 32 and t[0, 1, :5].tolist() == [7, 1, 2, 1, 16]


@pytest.mark.parametrize("shape_name,partials", [("llama", 4), ("llama", 32), ("qwen", 4)])
def test_oproj_round_spares_the_queues_that_ran_attention(shape_name, partials):
    """MI355X schedule: in every layer the queues that were dealt a split-KV instruction get a no-op
    in the O-proj round; the O-proj rows are still covered exactly once, and nobody gets more than
    two 8-row tiles."""
    from qimeng_megakernel_amd.decode_schedule.model_config import QWEN3_1_7B

    shape = LLAMA_3_2_1B if shape_name == "llama" else QWEN3_1_7B
    sched = S.mi355x_scheduler(shape, num_partials=partials)
    queues = sched.queues(num_layers=10)          # the round-robin origin moves by 32 queues per layer
    sm = sched.sm_count
    for layer in range(10):
        attention = {q for q in range(sm) if any(i.opcode() == 2 and i.layer_idx == layer for i in queues[q])}
        assert len(attention) == shape.num_key_value_heads * partials
        rows = []
        for q in range(sm):
            mine = [i for i in queues[q] if i.opcode() == 4 and i.layer_idx == layer]
            if q in attention and len(attention) < sm:   # all queues in attention: nobody to spare
                assert mine == []
                # its slot in the round is a no-op right behind its split-KV instruction
                at = next(k for k, i in enumerate(queues[q]) if i.opcode() == 2 and i.layer_idx == layer)
                assert queues[q][at + 1].opcode() == 0
            else:
                assert len(mine) == 1 and 1 <= mine[0].tile_N_end_idx - mine[0].tile_N_start_idx <= 2
                t = mine[0].tile_N_granularity
                rows += range(mine[0].tile_N_start_idx * t, mine[0].tile_N_end_idx * t)
        assert sorted(rows) == list(range(shape.hidden_size))
    # switched off, every queue has O-proj rows again
    plain = dataclasses_replace(sched, oproj_spares_attention=False)
    assert all(i.opcode() == 4 for i in plain.oproj(0))


def dataclasses_replace(obj, **kw):
    import dataclasses

    return dataclasses.replace(obj, **kw)
