"""CPU checks of the oracles for the Qwen3-30B-A3B geometry of the MoE route (no GPU).

The reference has no route for this shape: the oracle is its Qwen3 route's attention half in front of its MoE
route's block with two switches, ``norm_topk_prob`` (…/qwen1_5_moe_a2_7b/…/fused/operations.py:405) and no shared
expert.  The halves are pinned where the reference has them (tests/test_qwen3_oracle.py, tests/test_moe_oracle.py and
their fixtures); here the two switches are pinned by what the mathematics fixes — experts that are all the same
expert make the block's output that expert's output exactly when the weights sum to one; a shared expert with
all-zero weights is no shared expert — and the composed step by the fixture tests/golden/qwen3_moe_reduced_seed0.json,
written from the imported reference's functions in lock-step.
"""
import copy
import dataclasses
import json

import pytest
import torch
import torch.nn.functional as F

from conftest import GOLDEN
from fused_moe_oracle import FusedMoeOracle
from fused_oracle import rms_norm
from pyvm_moe_oracle import MoeInstructionVM
from qimeng_megakernel_amd import synthetic
from qimeng_megakernel_amd.decode_schedule_moe import mk_kernel
from qimeng_megakernel_amd.decode_schedule_moe.instructions import scheduler as S
from qimeng_megakernel_amd.decode_schedule_moe.model_config import QWEN1_5_MOE_A2_7B, QWEN3_30B_A3B, QwenMoeConfig

SMALL = dataclasses.replace(QWEN3_30B_A3B, num_hidden_layers=2, vocab_size=2048, num_experts=16, num_experts_per_tok=4,
                            moe_intermediate_size=256)


@pytest.fixture(autouse=True)
def _shape():
    QwenMoeConfig.set_shape(SMALL)
    with torch.no_grad():
        yield
    QwenMoeConfig.set_shape(QWEN1_5_MOE_A2_7B)


@pytest.fixture(scope="module")
def weights():
    return synthetic.random_moe_weights(SMALL, 0, 96)


def _globs(weights, shape=SMALL, position=41, token=99):
    g = synthetic.build_moe_globals(weights, shape, 96, "cpu")
    gen = torch.Generator().manual_seed(5)
    g.k_cache.copy_(torch.randn(g.k_cache.shape, generator=gen).bfloat16())
    g.v_cache.copy_(torch.randn(g.v_cache.shape, generator=gen).bfloat16())
    g.hidden_states.copy_(g.embed_tokens[token])
    g.position_id = position
    return g


def test_shape_and_byte_accounting():
    s = QWEN3_30B_A3B
    assert (s.num_hidden_layers, s.num_attention_heads, s.num_key_value_heads, s.head_dim) == (48, 32, 4, 128)
    assert s.qkv_out_dim == 5120 and not s.has_shared_expert and s.norm_topk_prob and s.qk_norm and not s.qkv_bias
    attn = (5120 * 2048 + 4096 * 2048) * 2
    per_layer = attn + 128 * 2048 * 2 + 8 * 3 * 768 * 2048 * 2
    assert attn == 37_748_736 and per_layer == 113_770_496                      # the figures the roofline is priced with
    assert s.weight_bytes_per_token() == 48 * (per_layer + 2 * 2048 * 2 + 2 * 128 * 2) + 151936 * 2048 * 2 + 2048 * 2
    assert 6.08e9 < s.weight_bytes_per_token() < 6.09e9
    assert s.kv_bytes_per_context_token() == 48 * 2 * 4 * 128 * 2


def test_renormalised_weights_closed_form(weights):
    """The top-k weights are the picks' softmax probabilities over their own sum; without the switch they are the raw ones."""
    g = _globs(weights)
    oracle = FusedMoeOracle(SMALL)
    oracle.qkv_rope(g, 0); oracle.attention(g, 0); oracle.oproj_residual(g, 0)
    normed = rms_norm(g.hidden_states, g.mlp_norm_weights[0], SMALL.rms_norm_eps)
    oracle.router(g, 0, normed)
    probs = torch.softmax(F.linear(normed.float().unsqueeze(0), g.router_weights[0].float()).squeeze(0).double(), dim=-1)
    top = probs.topk(SMALL.num_experts_per_tok)
    assert g.expert_indices.tolist() == top.indices.tolist()
    assert torch.allclose(g.expert_weights.double(), top.values / top.values.sum(), rtol=1e-6)
    assert abs(float(g.expert_weights.sum()) - 1.0) < 1e-6
    raw = FusedMoeOracle(dataclasses.replace(SMALL, norm_topk_prob=False))
    raw.router(g, 0, normed)
    assert torch.allclose(g.expert_weights.double(), top.values, rtol=1e-6) and float(g.expert_weights.sum()) < 0.9


@pytest.mark.parametrize("which", ["fused", "vm"])
def test_identical_experts_make_the_block_one_expert(weights, which):
    """Every expert the same expert: the routed sum is (sum of the weights) x that expert's output, i.e. the expert's
    output itself exactly when the weights are renormalised — dropping the renormalisation, an expert or the
    residual fails this."""
    w = dict(weights)
    w["expert_gate_up_proj_weights"] = weights["expert_gate_up_proj_weights"][:, :1].expand(-1, SMALL.num_experts, -1, -1).contiguous()
    w["expert_down_proj_weights"] = weights["expert_down_proj_weights"][:, :1].expand(-1, SMALL.num_experts, -1, -1).contiguous()
    g = _globs(w)
    fused, vm = FusedMoeOracle(SMALL), MoeInstructionVM(SMALL)
    sched = S.reference_scheduler(SMALL)
    if which == "fused":
        fused.qkv_rope(g, 0); fused.attention(g, 0); fused.oproj_residual(g, 0)
    else:
        vm.run(g, sched.qkvproj(0) + sched.attention_split_kv(0) + sched.attention_reduction(0) + sched.oproj(0))
    before = g.hidden_states.clone()
    normed = rms_norm(before, g.mlp_norm_weights[0], SMALL.rms_norm_eps)
    gate_up = F.linear(normed.unsqueeze(0), w["expert_gate_up_proj_weights"][0, 0]).squeeze(0)
    mid = SMALL.moe_intermediate_size
    silu = (F.silu(gate_up[:mid].float()) * gate_up[mid:].float()).to(torch.bfloat16)
    expert = F.linear(silu.unsqueeze(0), w["expert_down_proj_weights"][0, 0]).squeeze(0).float()     # bf16 values
    if which == "fused":
        fused.moe_block(g, 0)
    else:
        vm.run(g, sched.router_gemv(0) + sched.router_softmax_topk(0) + sched.routed_upgate(0) + sched.routed_downproj(0) + sched.combine_commit(0))
    want = before.float() + expert
    got = g.hidden_states.float()
    # weights that sum to 1 within fp32 rounding: the routed sum is the expert's output to ~1e-6, then one bf16 rounding (two in the fused form)
    assert float((got - want).abs().max()) <= 2.0 ** -7 * float(want.abs().max())
    unnormalised = before.float() + 0.5 * expert
    assert float((got - unnormalised).abs().max()) > 10 * float((got - want).abs().max())


def test_no_shared_expert_equals_a_shared_expert_of_zeros(weights):
    """The shared-expert-free block against the reference's block shape with an all-zero shared expert: the same bits."""
    with_shared = dataclasses.replace(SMALL, intermediate_size=512, num_downproj_split_k_shared=4)
    w = dict(weights)
    L, H = SMALL.num_hidden_layers, SMALL.hidden_size
    w["shared_expert_gate_proj_weights"] = torch.zeros(L, 512, H, dtype=torch.bfloat16)
    w["shared_expert_up_proj_weights"] = torch.zeros(L, 512, H, dtype=torch.bfloat16)
    w["shared_expert_down_proj_weights"] = torch.zeros(L, H, 512, dtype=torch.bfloat16)
    w["shared_expert_gate_weights"] = (torch.randn(L, 1, H) * 0.02).bfloat16()
    a, b = _globs(weights), _globs(w, shape=with_shared)
    FusedMoeOracle(SMALL).decode_step(a)
    FusedMoeOracle(with_shared).decode_step(b)
    assert torch.equal(a.hidden_states, b.hidden_states) and torch.equal(a.logits, b.logits)
    a, b = _globs(weights), _globs(w, shape=with_shared)
    MoeInstructionVM(SMALL).run(a, S.reference_scheduler(SMALL).instruction_list())
    MoeInstructionVM(with_shared).run(b, S.reference_scheduler(with_shared).instruction_list())
    assert torch.equal(a.hidden_states, b.hidden_states) and torch.equal(a.logits, b.logits)
    assert torch.equal(a.expert_indices, b.expert_indices) and torch.equal(a.expert_weights, b.expert_weights)


@pytest.mark.parametrize("stream", ["reference", "mi355x"])
def test_vm_against_fused_and_final_counters(weights, stream):
    f, v = _globs(weights), _globs(weights)
    FusedMoeOracle(SMALL).decode_step(f)
    sched = S.reference_scheduler(SMALL) if stream == "reference" else mk_kernel.mi355x_scheduler(SMALL, tagged=False)
    flat = sched.instruction_list()
    assert {i.opcode() for i in flat} == ({1, 2, 3, 4, 7, 8, 9, 12, 13, 14} if stream == "reference" else {1, 2, 4, 7, 8, 9, 12, 13, 14})
    MoeInstructionVM(SMALL).run(v, copy.deepcopy(flat))
    for name in ("q_post_rope", "attn_out", "hidden_states", "logits"):
        a, b = getattr(f, name).float(), getattr(v, name).float()
        assert float((a - b).abs().max()) <= 2.0 ** -5 * max(1.0, float(a.abs().max())), name
    assert f.logits.float().argmax().item() == v.logits.float().argmax().item()
    assert f.expert_indices.tolist() == v.expert_indices.tolist()
    s = SMALL
    for layer in range(s.num_hidden_layers):
        bar = v.barriers[layer]
        assert bar[0, : s.num_heads].tolist() == [s.head_dim // sched.shape.qkv_tile] * s.num_heads      # 16 rows in the reference's stream, 4 in this one's
        assert int(bar[3, 0]) == s.num_oproj_blocks and int(bar[13, 0]) == s.num_hidden_blocks
        assert bar[7, :2].tolist() == [s.num_experts, 1] and int(bar[8, 0]) == 1
        assert int(bar[9].abs().sum()) == 0 == int(bar[10].abs().sum())             # no shared expert: its rows stay clear
        assert int(bar[11, 0]) == s.num_experts_per_tok * s.num_routed_upgate_blocks
        assert bar[14, : s.num_experts_per_tok].tolist() == [s.num_routed_upgate_blocks] * s.num_experts_per_tok   # this build's per-slot counts
        assert bar[12, : s.num_hidden_blocks].tolist() == [s.num_experts_per_tok] * s.num_hidden_blocks
    assert float(v.routed_out_f32.abs().max()) == 0.0


def test_committing_down_projection_equals_down_projections_plus_combine(weights):
    """The stream for tagged launches (opcode 13 with tile_M_idx = 2: all expert slots of 8 rows and the commit, no
    opcode 14; the reporting top-k one layer late) through the VM: every buffer bit for bit what the stream on
    counters (down projection per slot, combine instructions) leaves, and the rows committed are counted."""
    a, b = _globs(weights), _globs(weights)
    classic, fused = mk_kernel.mi355x_scheduler(SMALL, tagged=False), mk_kernel.mi355x_scheduler(SMALL)
    assert fused.commit_in_down and fused.topk_late and not classic.commit_in_down
    flat = fused.instruction_list()
    assert 14 not in {i.opcode() for i in flat} and all(i.tile_M_idx == 2 for i in flat if i.opcode() == 13)
    MoeInstructionVM(SMALL).run(a, copy.deepcopy(classic.instruction_list()))
    MoeInstructionVM(SMALL).run(b, copy.deepcopy(flat))
    for name in ("hidden_states", "logits", "k_cache", "v_cache", "expert_indices", "expert_weights", "routed_out_f32", "attn_out"):
        assert torch.equal(getattr(a, name), getattr(b, name)), name
    for layer in range(SMALL.num_hidden_layers):
        assert int(b.barriers[layer, 13, 0]) == 0 and int(b.barriers[layer, 13, 1]) == SMALL.hidden_size // 8
    assert sum(1 for q in fused.queues() for i in q if i.opcode() == 9) == SMALL.num_hidden_layers


def test_full_size_stream():
    """The stream a request of the full shape runs: 48 layers on 256 queues, 768 routed up/gate tiles of 8 outputs per
    layer dealt three to a queue, one O-projection tile of 8 rows per queue, five QKV tiles of 4 rows per queue, every
    queue in dependency order."""
    sched = mk_kernel.mi355x_scheduler(QWEN3_30B_A3B, tagged=False)
    queues = sched.queues(2)
    assert len(queues) == 256 and sched.num_partials == 2
    phase = {1: 0, 2: 1, 4: 3, 8: 4, 9: 5, 12: 7, 13: 9, 14: 10}
    for q in queues:
        order = [(i.padded()[1], phase[i.opcode()]) for i in q]
        assert order == sorted(order)
        layer0 = [i for i in q if i.padded()[1] == 0]
        assert sum(i.padded()[4] - i.padded()[3] for i in layer0 if i.opcode() == 12) == 3
        assert sum(i.padded()[4] - i.padded()[3] for i in layer0 if i.opcode() == 4) == 1
        assert [(i.padded()[4] - i.padded()[3], i.padded()[6]) for i in layer0 if i.opcode() == 1] == [(5, 4)]
        assert all(i.padded()[3] == 1 for i in layer0 if i.opcode() == 13)           # a down projection waits for its own slot
    flat = [i for q in queues for i in q]
    assert sum(1 for i in flat if i.opcode() == 9) == 2 and sum(1 for i in flat if i.opcode() == 8) == 2 * 16


FIXTURE = GOLDEN / "qwen3_moe_reduced_seed0.json"


@pytest.mark.skipif(not FIXTURE.is_file(), reason="fixture not written yet")
def test_fixture_written_from_the_imported_reference():
    """The composed step as the reference's own functions compute it (tests/golden/make_fixtures_qwen3_moe.py: its Qwen3
    route's attention ops, its MoE route's block ops with the renormalisation of its line 405 and an all-zero shared
    expert, in lock-step with this oracle): tokens, routing and top-4 logits of every step."""
    fix = json.loads(FIXTURE.read_text())
    shape = dataclasses.replace(QWEN3_30B_A3B, **fix["shape"])
    QwenMoeConfig.set_shape(shape)
    w = synthetic.random_moe_weights(shape, fix["seed"], fix["kv_capacity"])
    g = synthetic.build_moe_globals(w, shape, fix["kv_capacity"], "cpu", max_partials=fix["max_partials"])
    gen = torch.Generator().manual_seed(fix["seed"] + 1)
    g.k_cache.copy_(torch.randn(g.k_cache.shape, generator=gen).bfloat16())
    g.v_cache.copy_(torch.randn(g.v_cache.shape, generator=gen).bfloat16())
    oracle, tok = FusedMoeOracle(shape), fix["start_token"]
    for step, want in enumerate(fix["steps"]):
        g.hidden_states.copy_(g.embed_tokens[tok]); g.position_id = fix["start_position"] + step
        routing = []
        for layer in range(shape.num_hidden_layers):
            oracle.decode_layer(g, layer)
            routing.append(g.expert_indices.tolist())
        oracle.lm_head(g)
        assert routing == want["experts_per_layer"], step
        ids = torch.tensor(want["top_ids"])
        assert g.logits[ids].view(torch.int16).to(torch.int32).bitwise_and(0xFFFF).tolist() == want["top_bits"], step
        tok = int(g.logits.float().argmax())
        assert tok == want["token"], step
