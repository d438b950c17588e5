"""Batch route on the Qwen3-1.7B layer geometry (Qwen3 op set): the two CPU oracles the GPU kernel is checked against.

The reference has no batch route for this op set; its Qwen3 fused operations take one row.  Anchors:

* ``tests/golden/qwen3_mb_reduced_seed0.json`` — written by ``make_fixtures_qwen3_mb.py`` while the imported
  functions of the reference's Qwen3 route ran row by row in lock-step with ``FusedBatchOracle`` (bit-identical
  buffers after every layer for six steps of a ragged three-row request in which one row retires);
* closed forms for what the op set adds: a per-head RMSNorm that a dropped norm, a norm over the wrong axis or a
  weight applied before the rounding would fail, at a position whose rotation is a known permutation;
* the instruction VM against the fused oracle on the same inputs, through both schedulers' lists.
"""
import dataclasses
import json
import sys

import pytest
import torch

from conftest import GOLDEN, ROOT

sys.path.insert(0, str(ROOT / "oracle"))
from fused_mb_oracle import FusedBatchOracle, RowView  # noqa: E402
from fused_oracle import FusedOracle  # noqa: E402
from pyvm_mb_oracle import BatchInstructionVM  # noqa: E402
from qimeng_megakernel_amd import synthetic  # noqa: E402
from qimeng_megakernel_amd.decode_schedule.model_config import QWEN3_1_7B, LlamaConfig  # noqa: E402
from qimeng_megakernel_amd.decode_schedule_mb.instructions import scheduler as S  # noqa: E402
from qimeng_megakernel_amd.decode_schedule_mb.row_state import RowState  # noqa: E402

FIX = json.loads((GOLDEN / "qwen3_mb_reduced_seed0.json").read_text())
SMALL = dataclasses.replace(QWEN3_1_7B, num_hidden_layers=FIX["layers"], vocab_size=FIX["vocab"])


@pytest.fixture(autouse=True)
def _shape():
    LlamaConfig.set_shape(SMALL)
    with torch.no_grad():
        yield


@pytest.fixture(scope="module")
def weights():
    return synthetic.random_weights(SMALL, FIX["seed"], max_positions=FIX["kv_capacity"])


def _bits(t: torch.Tensor) -> list:
    return t.contiguous().view(torch.int16).to(torch.int32).bitwise_and(0xFFFF).tolist()


def _request(weights, partials):
    g = synthetic.build_batch_globals(weights, SMALL, FIX["kv_capacity"], FIX["rows"], "cpu", max_partials=partials)
    gen = torch.Generator().manual_seed(FIX["seed"] + 1)
    g.k_cache.copy_(torch.randn(g.k_cache.shape, generator=gen).bfloat16())
    g.v_cache.copy_(torch.randn(g.v_cache.shape, generator=gen).bfloat16())
    g.position_ids.copy_(torch.tensor(FIX["start_positions"], dtype=torch.int32))
    RowState.of(g)
    return g


@pytest.mark.parametrize("route", ["fused", "vm"])
def test_request_of_the_reference_fixture(weights, route):
    """Six steps: greedy tokens, row state, top-4 logits bit for bit and samples of the hidden state."""
    g = _request(weights, FIX["max_partials"] if route == "fused" else 27)
    # the stream the fixture's VM leg was recorded with: this build's placement, the reference's split-KV fan-out rule
    sched = dataclasses.replace(S.mi355x_scheduler(FIX["rows"], SMALL), split_kv_per_worker=1.0, split_kv_cap=S.MAX_REDUCTION_LIST, lone_slice_tokens=0)
    fused, vm = FusedBatchOracle(SMALL), BatchInstructionVM(SMALL)
    tokens = list(FIX["start_tokens"])
    for step, want in enumerate(FIX["steps"]):
        assert g.position_ids.tolist() == want["positions"] and g.active_mask.tolist() == want["active"]
        for b in range(FIX["rows"]):
            g.hidden_states[b].copy_(g.embed_tokens[tokens[b]])
        if route == "fused":
            fused.decode_step(g)
            assert [_bits(g.hidden_states[b, ::128]) for b in range(FIX["rows"])] == want["hidden_bits_sampled"]
        else:
            g.barriers.zero_()
            vm.run(g, sched.instruction_list(g))
        ids = torch.tensor(want[route]["top_ids"])
        assert [_bits(g.logits[b][ids[b]]) for b in range(FIX["rows"])] == want[route]["top_bits"], step
        nxt = g.logits.float().argmax(dim=-1)
        assert nxt.tolist() == want[route]["tokens"], step
        RowState.of(g).advance(nxt, [FIX["eos_token"]] if step >= 1 else [])
        tokens = nxt.tolist()
    assert g.active_mask.tolist() == [True, False, True]


def test_per_head_norm_closed_form(weights):
    """Position 0 rotates nothing (cos 1, sin 0).  With an attention norm of ones, a hidden row e_j scaled by c and
    QKV rows chosen by hand, q of head h is a known vector: its per-head norm has a closed form that differs
    from no norm, from a norm over all heads, and from a weight applied before the division."""
    w = {k: v.clone() for k, v in weights.items()}
    d, nq, nkv, H = SMALL.head_dim, SMALL.num_attention_heads, SMALL.num_key_value_heads, SMALL.hidden_size
    w["qkv_weights"][0].zero_()
    # every head's q (and k) row block reads column 0 of the normed hidden state with a head-specific pattern
    pattern = torch.arange(1, d + 1, dtype=torch.float32) / d                    # 1/d .. 1
    for h in range(nq + nkv):
        w["qkv_weights"][0, h * d : (h + 1) * d, 0] = (pattern * (h + 1) / 8).bfloat16()
    w["q_norm_weights"][0] = (torch.arange(d) % 3 + 1).bfloat16()                # 1, 2, 3, 1, ...
    w["k_norm_weights"][0] = torch.full((d,), 0.5).bfloat16()
    g = synthetic.build_batch_globals(w, SMALL, 8, 2, "cpu", max_partials=2)
    g.position_ids.zero_()
    g.hidden_states.zero_()
    g.hidden_states[:, 0] = 3.0                                                   # RMSNorm of c*e_0 is sqrt(H)*e_0 (eps aside)
    FusedBatchOracle(SMALL).qkv_rope(g, 0)
    y0 = float((torch.tensor(3.0) * torch.rsqrt(torch.tensor(9.0 / H) + SMALL.rms_norm_eps)).bfloat16())
    for b in range(2):
        for h in range(nq):
            raw = (w["qkv_weights"][0, h * d : (h + 1) * d, 0].float() * y0).bfloat16()   # one GEMV term, rounded
            assert torch.equal(g.qkv_raw[b, h * d : (h + 1) * d], raw)
            x = raw.float()
            want = (w["q_norm_weights"][0].float() * (x * torch.rsqrt(x.pow(2).mean() + SMALL.rms_norm_eps))).bfloat16()
            got = g.q_post_rope[b, h * d : (h + 1) * d]
            assert torch.equal(got, want), (b, h)
            assert not torch.equal(got, raw)                                                      # a dropped norm
            assert float(got.float().pow(2).mean()) > 1.0                                          # weights 1..3 on a unit-RMS vector
        k = g.k_cache[0, b, 0]
        assert k.shape == (nkv, d)
        for h in range(nkv):
            # unit RMS times 0.5: the scale of the head's pattern has gone
            assert abs(float(k[h].float().pow(2).mean()) - 0.25) < 2e-3, h
        raw_v = (w["qkv_weights"][0, (nq + nkv) * d :, 0].float() * y0).bfloat16().view(nkv, d)
        assert torch.equal(g.v_cache[0, b, 0], raw_v)                                              # v: no norm, no rotation


def test_rows_do_not_see_each_other(weights):
    """Row b of a batch gives what the batch-1 oracle of the Qwen3 route gives for that row alone, bit for bit;
    a retired row leaves hidden state, caches and raw vector untouched."""
    g = _request(weights, 8)
    g.active_mask[1] = False
    gen = torch.Generator().manual_seed(3)
    g.hidden_states.copy_((torch.randn(g.hidden_states.shape, generator=gen) * 0.5).bfloat16())
    alone = []
    for b in range(FIX["rows"]):
        one = synthetic.build_globals(weights, SMALL, FIX["kv_capacity"], "cpu", max_partials=8)
        one.k_cache.copy_(g.k_cache[:, b : b + 1]); one.v_cache.copy_(g.v_cache[:, b : b + 1])
        one.hidden_states.copy_(g.hidden_states[b]); one.position_id = int(g.position_ids[b])
        alone.append(one)
    before = {n: getattr(g, n)[1].clone() for n in ("hidden_states", "qkv_raw", "q_post_rope")}
    cache_before = g.k_cache[:, 1].clone()
    FusedBatchOracle(SMALL).decode_step(g)
    single = FusedOracle(SMALL)
    for b in (0, 2):
        single.decode_step(alone[b])
        for name in ("hidden_states", "logits", "attn_out", "silu_out", "qkv_raw", "q_post_rope"):
            assert torch.equal(getattr(g, name)[b], getattr(alone[b], name)), (b, name)
        assert torch.equal(g.k_cache[:, b], alone[b].k_cache[:, 0])
    for n, t in before.items():
        assert torch.equal(getattr(g, n)[1], t), n
    assert torch.equal(g.k_cache[:, 1], cache_before)
    assert float(g.attn_out[1].abs().max()) == 0 and float(g.silu_out[1].abs().max()) == 0
    assert bool((g.logits[1].float() == torch.tensor(-1e9).bfloat16().float()).all())


def test_row_view_is_a_window_not_a_copy(weights):
    g = _request(weights, 8)
    v = RowView(g, 2)
    assert v.position_id == FIX["start_positions"][2] and v.k_cache.shape[1] == 1
    v.hidden_states.fill_(1.0)
    v.k_cache[0, 0, 5].fill_(2.0)
    assert float(g.hidden_states[2].min()) == 1.0 and float(g.k_cache[0, 2, 5].min()) == 2.0
    assert v.qkv_weights is g.qkv_weights
    with pytest.raises(AttributeError):
        v.position_id = 3


@pytest.mark.parametrize("make", [S.mi355x_scheduler, S.reference_scheduler], ids=["mi355x", "a100"])
def test_vm_against_the_fused_oracle(weights, make):
    """Same inputs through the instruction list of either scheduler: the tiled arithmetic gives the row-by-row
    result within one bf16 step of the hidden state's scale, and the same greedy tokens."""
    a, b = _request(weights, 27), _request(weights, 27)
    b.active_mask[1] = a.active_mask[1] = False
    for r in range(FIX["rows"]):
        for g in (a, b):
            g.hidden_states[r].copy_(g.embed_tokens[FIX["start_tokens"][r]])
    FusedBatchOracle(SMALL).decode_step(a)
    sched = make(FIX["rows"], SMALL)
    BatchInstructionVM(SMALL, sched.oproj_tile, sched.down_tile).run(b, sched.instruction_list(b))
    live = [0, 2]
    scale = float(a.hidden_states[live].float().abs().max())
    assert float((a.hidden_states[live].float() - b.hidden_states[live].float()).abs().max()) <= scale * 2.0 ** -7
    assert a.logits.float().argmax(-1).tolist() == b.logits.float().argmax(-1).tolist()
    assert torch.equal(a.hidden_states[1], b.hidden_states[1])
    # the reduction instructions of this shape merge its GQA pair of heads
    if not sched.merge_in_last:
        assert all(i.padded()[3] % SMALL.attn_reduction_size == 0 for i in sched.attention_reduction(0, 2))
        assert len(sched.attention_reduction(0, 2)) == FIX["rows"] * SMALL.num_attention_heads // SMALL.attn_reduction_size
