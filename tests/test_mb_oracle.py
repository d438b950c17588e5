"""Batch decode route (2..16 rows): instruction set, scheduler, per-row state and the two CPU oracles.

What is pinned here is everything the gfx950 kernel of this route is checked against (its own
parity tests need a GPU).  Three independent anchors:

* ``tests/golden/mb_reduced_seed0.json`` — written by ``make_fixtures_mb.py`` from the imported
  reference while this repository's scheduler, VM and fused oracle ran in lock-step with the
  reference's (bit-identical instruction words, buffers, counters and row state for six steps of a
  ragged three-row request in which one row retires);
* the batch-1 oracle (itself pinned elsewhere): the reference's arithmetic is row-wise, so every
  row of a batch must reproduce what that row gives alone, bit for bit;
* integer properties of the instruction streams (coverage, counters, round structure).
"""
import dataclasses
import hashlib
import json
import sys

import numpy as np
import pytest
import torch

from conftest import GOLDEN, ROOT

sys.path.insert(0, str(ROOT / "oracle"))
from fused_mb_oracle import FusedBatchOracle  # noqa: E402
from fused_oracle import FusedOracle  # noqa: E402
from pyvm_mb_oracle import BatchInstructionVM  # noqa: E402
from qimeng_megakernel_amd import synthetic  # noqa: E402
from qimeng_megakernel_amd.decode_schedule.model_config import LLAMA_3_2_1B, LlamaConfig  # noqa: E402
from qimeng_megakernel_amd.decode_schedule_mb import mk_kernel  # noqa: E402
from qimeng_megakernel_amd.decode_schedule_mb.row_state import RowState, rows_of  # noqa: E402
from qimeng_megakernel_amd.decode_schedule_mb.globs import Globals  # noqa: E402
from qimeng_megakernel_amd.decode_schedule_mb.instructions import instruction_defs as D  # noqa: E402
from qimeng_megakernel_amd.decode_schedule_mb.instructions import scheduler as S  # noqa: E402

FIX = json.loads((GOLDEN / "mb_reduced_seed0.json").read_text())
MB_FULL = dataclasses.replace(LLAMA_3_2_1B, attn_kv_block_size=FIX["kv_block"])
MB_SMALL = dataclasses.replace(MB_FULL, num_hidden_layers=FIX["layers"], vocab_size=FIX["vocab"])


@pytest.fixture(autouse=True)
def _no_grad_and_shape():
    LlamaConfig.set_shape(MB_SMALL)
    with torch.no_grad():
        yield
    LlamaConfig.set_shape(LLAMA_3_2_1B)


def _words(instructions) -> np.ndarray:
    return np.asarray([i.padded() for i in instructions], dtype=np.int32)


def _bits(t: torch.Tensor) -> list:
    return t.contiguous().view(torch.int16).to(torch.int32).bitwise_and(0xFFFF).tolist()


def _request(weights):
    g = synthetic.build_batch_globals(weights, MB_SMALL, FIX["kv_capacity"], FIX["rows"], "cpu")
    gen = torch.Generator().manual_seed(FIX["seed"] + 1)
    g.k_cache.copy_(torch.randn(g.k_cache.shape, generator=gen).bfloat16())
    g.v_cache.copy_(torch.randn(g.v_cache.shape, generator=gen).bfloat16())
    g.position_ids.copy_(torch.tensor(FIX["start_positions"], dtype=torch.int32))
    RowState.of(g)
    return g


@pytest.fixture(scope="module")
def weights():
    return synthetic.random_weights(MB_SMALL, FIX["seed"], max_positions=FIX["kv_capacity"])


# ---------------------------------------------------------------- wire format --
def test_wire_format_known_words():
    """Operand order and defaults of `…/multi_batch/…/instruction_defs.py:11-211`."""
    assert D.AttnRMS(3, 5, batch_row=4).serialize() == [1, 3, 5, 0, 0, 0, 4]
    assert D.QKVProj_GEMM_RoPE(2, 8, 0, 10, 12).serialize() == [2, 2, 8, 0, 10, 12, 16, 16]
    assert D.DecodeAttentionSplitKV(1, 2, 7, 4, 3).serialize() == [3, 1, 2, 7, 4, 3, -1, -1]
    assert D.DecodeAttentionSplitKV(1, 2, 7, 4, 3, 130, 1).serialize() == [3, 1, 2, 7, 4, 3, 130, 1]
    assert D.DecodeAttentionReduction(1, 2, 4, 3, [0, 1, 2]).serialize() == [4, 1, 2, 4, 3, 3, 0, 1, 2, 1, 0, -1, -1]
    assert D.OProj_GEMM_Residual(0, 8, 0, 4, 6, 0).serialize() == [5, 0, 8, 0, 4, 6, 0, 16, 16]
    assert D.MlpRMS(9, 8, batch_row=7).serialize() == [6, 9, 8, 0, 0, 0, 7]
    assert D.UpGateProj_GEMM_SiLU(0, 8, 0, [7, 8, 9]).serialize() == [7, 0, 8, 0, 3, 7, 8, 9, 16, 16]
    assert D.DownProj_GEMM_Residual(9, 8, 0, 0, 5).serialize() == [8, 9, 8, 0, 0, 5, 16, 16]
    assert D.LMHeadRMS(8, batch_row=2).serialize() == [9, 8, 0, 0, 0, 0, 2]
    assert D.LMHeadProj_GEMM(8, 75, 150).serialize() == [10, 8, 75, 150, 16, 16]
    assert sorted(D.OPCODE_TO_CLASS) == list(range(11))


# ------------------------------------------------------------------ scheduler --
def test_full_size_runtime_template_matches_the_reference_digest():
    meta = FIX["full_size_runtime_template"]
    LlamaConfig.set_shape(MB_FULL)
    queues = S.reference_scheduler(meta["rows"], MB_FULL).runtime_queues(meta["kv_capacity"])
    arr = np.stack([_words(q) for q in queues])
    assert list(arr.shape) == meta["shape"]
    assert hashlib.sha256(arr.tobytes()).hexdigest() == meta["sha256"]


def test_runtime_template_is_made_of_whole_rounds():
    sched = S.mi355x_scheduler(8, MB_FULL)
    flat = sched.runtime_instruction_list(1024, num_layers=2)
    assert len(flat) % sched.workers == 0
    rounds = [flat[i : i + sched.workers] for i in range(0, len(flat), sched.workers)]
    for r in rounds:   # a round holds one kind of instruction (and padding)
        assert len({i.opcode() for i in r} - {0}) == 1
    first = rounds[0]   # the RMSNorm rows sit in the first B slots of their round
    assert [i.opcode() for i in first[:8]] == [1] * 8 and [i.batch_row for i in first[:8]] == list(range(8))
    assert all(i.opcode() == 0 for i in first[8:])
    # attention instructions leave length and activity to the launch
    assert all(i.seq_len == -1 and i.is_active == -1 for i in flat if i.opcode() == 3)
    assert all(i.valid_partials == -1 and i.is_active == -1 for i in flat if i.opcode() == 4)


def test_up_gate_blocks_stay_off_the_down_projection_workers():
    """MI355X template: the workers of the down projection's round get no up/gate block, the others share all of
    them; the reference's deal stays even."""
    sched = S.mi355x_scheduler(8, MB_FULL)
    mine = sched.upgate_skewed(0)
    counts = [len(i.tile_N_block_idxs) if i.opcode() == 7 else 0 for i in mine]
    busy = len(sched.downproj(0))
    assert len(mine) == sched.workers and busy == 128
    assert set(counts[:busy]) == {0} and set(counts[busy:]) == {4} and sum(counts) == MB_FULL.intermediate_size // 16
    flat = [b for i in mine if i.opcode() == 7 for b in i.tile_N_block_idxs]
    assert flat == list(range(MB_FULL.intermediate_size // 16))
    even = [len(i.tile_N_block_idxs) for i in S.reference_scheduler(8, MB_FULL).upgate(0)]
    assert max(even) - min(even) <= 1
    assert not S.mi355x_scheduler(8, MB_FULL, skew_upgate=False).skew_upgate
    # 8-row blocks put a down-projection block on every worker: nobody is left to take the up/gate blocks alone
    assert [i.opcode() for i in S.mi355x_scheduler(8, MB_FULL, residual_tile=8).upgate_skewed(0)] == [7] * 256


def test_o_proj_blocks_go_beside_the_attention_workers():
    """MI355X template: where the split-KV round leaves at least half of the down-projection workers free, the
    O-projection's blocks go to those, two to a worker; otherwise (and in the reference's template) one block per
    worker from worker 0 on."""
    sched = S.mi355x_scheduler(8, MB_FULL)
    p = sched.partials_for_capacity(1024)
    slices = len(sched.attention_split_kv(0, p))
    assert slices == 64
    placed = sched.oproj_round(0, p)
    assert len(placed) == sched.workers
    assert all(i.opcode() == 0 for i in placed[:slices] + placed[128:])
    spans = [(i.tile_N_start_idx, i.tile_N_end_idx) for i in placed[slices:128]]
    assert spans == [(2 * k, 2 * k + 2) for k in range(64)]
    full = S.mi355x_scheduler(16, MB_FULL)   # 128 slices: no down-projection worker is free
    plain = full.oproj_round(0, full.partials_for_capacity(1024))
    assert [i.opcode() for i in plain] == [5] * 128 + [0] * 128
    assert [(i.tile_N_start_idx, i.tile_N_end_idx) for i in plain[:128]] == [(k, k + 1) for k in range(128)]
    ref = S.reference_scheduler(8, MB_FULL)
    assert ref.oproj_round(0, 4)[: len(ref.oproj(0))] == ref.oproj(0)


def test_qkv_blocks_go_behind_the_attention_workers():
    """MI355X template: the QKV round starts behind the split-KV round's workers where both fit side by side, else behind
    the norm rows' workers, else (and in the reference's template) at worker 0."""
    def first(sched):
        r = sched.qkv_round(0, sched.partials_for_capacity(1024))
        assert len(r) % sched.workers == 0 and [i for i in r if i.opcode() == 2] == sched.qkvproj(0)
        return next(k for k, i in enumerate(r) if i.opcode() == 2)
    assert first(S.mi355x_scheduler(8, MB_FULL)) == 64       # 64 slices + 192 blocks = 256 workers
    assert first(S.mi355x_scheduler(16, MB_FULL)) == 16      # 128 slices: behind the 16 norm rows
    assert first(S.mi355x_scheduler(8, MB_FULL, skew_upgate=False)) == 0
    assert first(S.reference_scheduler(8, MB_FULL)) == 0


@pytest.mark.parametrize("make,rows", [(S.reference_scheduler, 3), (S.mi355x_scheduler, 8), (S.mi355x_scheduler, 16)])
def test_every_output_once_and_final_counters(make, rows):
    shape = MB_SMALL
    sched = make(rows, shape)
    flat = sched.runtime_instruction_list(256)
    p = sched.partials_for_capacity(256)
    out = {op: [] for op in (2, 5, 7, 8, 10)}
    for i in flat:
        if i.opcode() in (2, 5, 8):
            out[i.opcode()] += range(i.tile_N_start_idx * i.tile_N_granularity, i.tile_N_end_idx * i.tile_N_granularity)
            assert i.tile_N_granularity == (16 if i.opcode() == 2 else sched.oproj_tile if i.opcode() == 5 else sched.down_tile)
        elif i.opcode() == 7:
            for b in i.tile_N_block_idxs:
                out[7] += range(b * 16, b * 16 + 16)
        elif i.opcode() == 10:
            out[10] += range(i.start_output_block_idx * 16, i.end_output_block_idx * 16)
    L = shape.num_hidden_layers
    assert sorted(out[2]) == sorted(list(range(shape.qkv_out_dim)) * L)
    assert sorted(out[5]) == sorted(list(range(shape.hidden_size)) * L) == sorted(out[8])
    assert sorted(out[7]) == sorted(list(range(shape.intermediate_size)) * L)
    assert sorted(out[10]) == list(range(shape.vocab_size))
    attn = [(i.layer_idx, i.batch_idx, i.kv_head_idx, i.partial_idx) for i in flat if i.opcode() == 3]
    assert len(attn) == len(set(attn)) == L * rows * shape.num_key_value_heads * p
    red = [(i.layer_idx, i.batch_idx, i.head_start_idx) for i in flat if i.opcode() == 4]
    # the MI355X stream has no reduction instructions: the last split-KV arrival of a head group merges
    assert len(red) == len(set(red)) == (0 if sched.merge_in_last else L * rows * shape.num_attention_heads // 4)
    assert all(i.padded()[8] == int(sched.merge_in_last) for i in flat if i.opcode() == 3)
    with pytest.raises(ValueError):
        make(17, shape)


def test_fan_out_policy():
    """`scheduler.py:351-376`: about one split-KV instruction per worker, at most one per KV block,
    at most what a reduction instruction lists."""
    assert S.partials_for_blocks(8, 16, 216, 8) == 4        # ceil(216 / 64)
    assert S.partials_for_blocks(1, 2, 216, 8) == 2         # two blocks: two slices
    assert S.partials_for_blocks(2, 100, 216, 8) == 14      # ceil(216 / 16)
    assert S.partials_for_blocks(1, 1000, 256, 8) == S.MAX_REDUCTION_LIST
    assert S.partials_for_blocks(0, 5, 216, 8) == 1
    # this build's stream: half that fan-out for heads of 64 (the merge by the last arrival costs what a slice saves), the rule
    # itself for heads of 128; never more than 4 slices; with heads of 64 one slice instead of two while the cache is small
    from qimeng_megakernel_amd.decode_schedule.model_config import QWEN3_1_7B
    llama = dataclasses.replace(LLAMA_3_2_1B, attn_kv_block_size=64)
    assert [S.mi355x_scheduler(b, llama).partials_for_capacity(1040) for b in (2, 4, 8, 16)] == [4, 4, 1, 1]
    assert [S.mi355x_scheduler(b, llama).partials_for_capacity(4096) for b in (2, 4, 8, 16)] == [4, 4, 2, 1]
    assert [S.mi355x_scheduler(b, QWEN3_1_7B).partials_for_capacity(1040) for b in (2, 4, 8, 16)] == [4, 4, 4, 2]
    # streams with a reduction instruction keep both slices
    assert S.mi355x_scheduler(8, llama, merge_in_last=False).partials_for_capacity(1040) == 2


# -------------------------------------------------------------------- oracles --
def test_request_of_the_reference_fixture(weights):
    """Both oracles reproduce the six recorded steps: instruction words, tokens, top-4 logits, row state."""
    vm_g, fu_g = _request(weights), _request(weights)
    vm, fused = BatchInstructionVM(MB_SMALL), FusedBatchOracle(MB_SMALL)
    sched = S.reference_scheduler(FIX["rows"], MB_SMALL)
    toks = {"my_vm": list(FIX["start_tokens"]), "my_fused": list(FIX["start_tokens"])}
    for step, want in enumerate(FIX["steps"]):
        for name, g in (("my_vm", vm_g), ("my_fused", fu_g)):
            for b in range(FIX["rows"]):
                g.hidden_states[b].copy_(g.embed_tokens[toks[name][b]])
            assert g.position_ids.tolist() == want["positions"] and g.active_mask.tolist() == want["active"]
        vm_g.barriers.zero_()
        flat = sched.instruction_list(vm_g)
        assert hashlib.sha256(_words(flat).tobytes()).hexdigest() == FIX["instruction_list_sha256"][step]
        vm.run(vm_g, flat)
        fused.decode_step(fu_g)
        assert _bits(vm_g.hidden_states[:, ::128]) == want["hidden_bits_sampled"]
        for name, g in (("my_vm", vm_g), ("my_fused", fu_g)):
            ids = torch.tensor(want[name]["top_ids"])
            assert _bits(g.logits.gather(1, ids)) == want[name]["top_bits"], (step, name)
            nxt = g.logits.float().argmax(dim=-1)
            assert nxt.tolist() == want[name]["tokens"]
            RowState.of(g).advance(nxt, [FIX["eos_token"]] if step >= 1 else [])
            toks[name] = nxt.tolist()
    assert vm_g.active_mask.tolist() == [True, False, True] and RowState.of(vm_g).finished.tolist() == [False, True, False]


def test_every_row_of_a_batch_equals_that_row_alone(weights):
    """The fused batch oracle against the batch-1 oracle: bit for bit, at ragged positions."""
    g = _request(weights)
    tokens = (5, 900, 1234)
    for b, t in enumerate(tokens):
        g.hidden_states[b].copy_(g.embed_tokens[t])
    before_k, before_v = g.k_cache.clone(), g.v_cache.clone()
    FusedBatchOracle(MB_SMALL).decode_step(g)
    one = FusedOracle(MB_SMALL)
    for b, t in enumerate(tokens):
        g1 = synthetic.build_globals(weights, MB_SMALL, FIX["kv_capacity"], "cpu")
        g1.k_cache[:, 0].copy_(before_k[:, b]); g1.v_cache[:, 0].copy_(before_v[:, b])
        g1.hidden_states.copy_(g1.embed_tokens[t]); g1.position_id = FIX["start_positions"][b]
        one.decode_step(g1)
        for name in ("hidden_states", "q_post_rope", "attn_out", "silu_out", "logits"):
            assert torch.equal(getattr(g1, name), getattr(g, name)[b]), (b, name)
        assert torch.equal(g1.k_cache[:, 0], g.k_cache[:, b]) and torch.equal(g1.v_cache[:, 0], g.v_cache[:, b])


def test_inactive_row_is_frozen_and_forced(weights):
    g = _request(weights)
    g.active_mask[1] = False
    for b in range(3):
        g.hidden_states[b].copy_(g.embed_tokens[10 + b])
    frozen = (g.hidden_states[1].clone(), g.k_cache[:, 1].clone(), g.q_post_rope[1].clone())
    v = _request(weights); v.active_mask[1] = False
    v.hidden_states.copy_(g.hidden_states)
    FusedBatchOracle(MB_SMALL).decode_step(g)
    BatchInstructionVM(MB_SMALL, 8, 8).run(v, S.mi355x_scheduler(3, MB_SMALL, residual_tile=8).instruction_list(v))
    for x in (g, v):
        assert torch.equal(x.hidden_states[1], frozen[0]) and torch.equal(x.k_cache[:, 1], frozen[1])
        assert torch.equal(x.q_post_rope[1], frozen[2])
        assert float(x.attn_out[1].abs().max()) == 0 and float(x.silu_out[1].abs().max()) == 0
        assert bool((x.logits[1].float() == torch.tensor(-1e9).bfloat16().float()).all())
    assert float(v.attn_rms_out[1].abs().max()) == 0 and not bool(v.attn_partial_valid[1].any())
    assert bool(torch.isinf(v.attn_lse_intermediates[1, :, : S.mi355x_scheduler(3, MB_SMALL).partials_for_request(v)]).all())


def test_vm_agrees_with_fused_and_counters_complete(weights):
    f, v = _request(weights), _request(weights)
    for b in range(3):
        for g in (f, v):
            g.hidden_states[b].copy_(g.embed_tokens[20 + b])
    FusedBatchOracle(MB_SMALL).decode_step(f)
    sched = S.mi355x_scheduler(3, MB_SMALL, residual_tile=8)
    assert (sched.oproj_tile, sched.down_tile) == (8, 8) and S.mi355x_scheduler(3, MB_SMALL).down_tile == 16
    BatchInstructionVM(MB_SMALL, sched.oproj_tile, sched.down_tile).run(v, sched.runtime_instruction_list(FIX["kv_capacity"]))
    for name in ("q_post_rope", "attn_out", "silu_out", "hidden_states", "logits"):
        a, b_ = getattr(f, name).float(), getattr(v, name).float()
        assert float((a - b_).abs().max()) <= 2.0 ** -5 * max(1.0, float(a.abs().max())), name
    assert v.logits.float().argmax(-1).tolist() == f.logits.float().argmax(-1).tolist()
    s, p = MB_SMALL, sched.partials_for_capacity(FIX["kv_capacity"])
    stride = s.num_attention_heads + 2 * s.num_key_value_heads
    for layer in range(s.num_hidden_layers):
        bar = v.barriers[layer]
        assert int(bar[0, 0]) == 3 and int(bar[5, 0]) == 3
        assert bar[1, :stride].tolist() == [s.head_dim // 16] * stride
        for b in range(3):
            assert bar[2, b * stride : b * stride + s.num_attention_heads].tolist() == [p] * s.num_attention_heads
            assert int(bar[3, b]) == s.num_attention_heads
        assert int(bar[4, 0]) == s.hidden_size // 8 == int(bar[7, 0]) and int(bar[6, 0]) == s.intermediate_size // 16
    assert int(v.barriers[s.num_hidden_layers - 1, 8, 0]) == 3


# ---------------------------------------------------------------- row state ----
def test_row_state_advances_and_retires_rows():
    g = Globals(hidden_states=torch.zeros(3, 4), position_ids=torch.tensor([5, 0, 9], dtype=torch.int32))
    state = RowState.of(g)
    assert RowState.of(g) is state and g.active_mask is state.active_mask and g.position_ids is state.position_ids
    assert state.kv_lengths().tolist() == [6, 1, 10] and g.active_mask.tolist() == [True] * 3
    state.advance(torch.tensor([7, 2, 8]), [2])
    assert g.position_ids.tolist() == [6, 0, 10] and g.active_mask.tolist() == [True, False, True]
    assert state.finished.tolist() == [False, True, False] and state.kv_lengths().tolist() == [7, 1, 11]
    state.advance(torch.tensor([2, 2, 3]), torch.tensor([2]))      # a retired row stays retired
    assert g.position_ids.tolist() == [6, 0, 11] and g.active_mask.tolist() == [False, False, True]
    assert state.finished.tolist() == [True, True, False] and state.last_tokens.tolist() == [2, 2, 3]
    state.advance(torch.tensor([4, 4, 4]))                         # no end-of-sequence tokens: only the live row moves
    assert g.position_ids.tolist() == [6, 0, 12]
    assert state.follows(0, 2) is False and state.follows(1, 0) is True
    assert state.follows(-1, 2) is True and state.follows(-1, 0) is False
    assert rows_of(g) == 3 and state.rows == 3 and state.position(2) == 12
    state.restart(4)
    assert g.position_ids.tolist() == [4, 4, 4] and g.active_mask.tolist() == [True] * 3 and not state.finished.any()
    # a caller that replaces one of the two boundary tensors gets a fresh state bound to the new one
    g.active_mask = torch.tensor([True, False, True])
    assert RowState.of(g) is not state and RowState.of(g).active_mask is g.active_mask


def test_mk_of_the_batch_route_checks_its_arguments(weights):
    """The launcher refuses what the reference's host checks refuse (`…/multi_batch/decode_kernel/mk.cu:52-216`)
    before anything reaches a device; a missing library is an ImportError."""
    with pytest.raises(ImportError, match="missing prebuilt kernel"):
        mk_kernel.get_mk(ROOT / "tests")
    mk = mk_kernel.get_mk()
    g = _request(weights)
    g.instructions = torch.zeros(4, 1, 32, dtype=torch.int32)
    with pytest.raises(ValueError, match="must live on"):
        mk_kernel.call_mk(g, mk)
    with pytest.raises(TypeError, match="positional arguments"):
        mk(g.instructions, g.hidden_states)


def test_two_stage_argmax_is_the_first_maximum():
    """The graph-safe argmax of the host loop returns what `argmax` does, ties included (first index wins)."""
    from qimeng_megakernel_amd.decode_batch import argmax_rows

    gen = torch.Generator().manual_seed(11)
    for vocab in (128256, 2048, 96, 1000):
        logits = torch.randn(5, vocab, generator=gen).to(torch.bfloat16).float()
        logits[1, 7] = logits[1, vocab - 3] = 9.0          # a tie across runs
        logits[2, vocab // 2] = logits[2, vocab // 2 + 1] = 9.0   # a tie inside a run
        want = torch.stack([torch.nonzero(r == r.max())[0, 0] for r in logits])
        assert torch.equal(argmax_rows(logits), want)
