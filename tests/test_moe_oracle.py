"""MoE decode route at batch 1: instruction set, scheduler and the two CPU oracles.

What is pinned here is everything the gfx950 kernel of this route is checked against (its own parity
tests need a GPU).  Anchors:

* ``tests/golden/moe_reduced_seed0.json`` — written by ``make_fixtures_moe.py`` from the imported
  reference while this repository's scheduler, VM and fused oracle ran in lock-step with the
  reference's (bit-identical instruction words — also of the full-size stream —, buffers and counters
  for six greedy steps);
* closed forms of the MoE block that a dropped term, a wrong expert index or a forgotten gate would
  break (a router with prescribed logits, identical experts, a shared gate at zero);
* integer properties of the instruction stream.
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
from fused_moe_oracle import FusedMoeOracle  # noqa: E402
from pyvm_moe_oracle import MoeInstructionVM  # noqa: E402
from qimeng_megakernel_amd import synthetic  # noqa: E402
from qimeng_megakernel_amd.decode_schedule_moe import mk_kernel  # noqa: E402
from qimeng_megakernel_amd.decode_schedule_moe.instructions import instruction_defs as D  # noqa: E402
from qimeng_megakernel_amd.decode_schedule_moe.instructions import scheduler as S  # noqa: E402
from qimeng_megakernel_amd.decode_schedule_moe.model_config import QWEN1_5_MOE_A2_7B, num_partials_for  # noqa: E402

FIX = json.loads((GOLDEN / "moe_reduced_seed0.json").read_text())
SMALL = dataclasses.replace(QWEN1_5_MOE_A2_7B, **FIX["shape"])


@pytest.fixture(autouse=True)
def _no_grad():
    with torch.no_grad():
        yield


@pytest.fixture(scope="module")
def weights():
    return synthetic.random_moe_weights(SMALL, FIX["seed"], FIX["kv_capacity"])


def _words(instructions) -> np.ndarray:
    return np.asarray([i.padded() for i in instructions], dtype=np.int32)


def _bits(t: torch.Tensor) -> list:
    return t.contiguous().view(torch.int16).to(torch.int32).bitwise_and(0xFFFF).tolist()


def _request(weights, shape=SMALL):
    g = synthetic.build_moe_globals(weights, shape, FIX["kv_capacity"], "cpu")
    gen = torch.Generator().manual_seed(FIX["seed"] + 1)
    g.k_cache.copy_(torch.randn(g.k_cache.shape, generator=gen).bfloat16())
    g.v_cache.copy_(torch.randn(g.v_cache.shape, generator=gen).bfloat16())
    return g


# ---------------------------------------------------------------- wire format --
def test_wire_format_known_words():
    """Operand order and defaults of `…/qwen1_5_moe_a2_7b/…/instruction_defs.py:24-262`."""
    assert D.Router_GEMV(3, 5, 6, 1).serialize() == [8, 3, 5, 6, 1, 1]
    assert D.Router_SoftmaxTopK(2).serialize() == [9, 2]
    assert D.SharedExpert_UpGate_SiLU(1, 0, 4, 8, 1).serialize() == [10, 1, 0, 4, 8, 1, 1, 16]
    assert D.SharedExpert_DownProj(1, 0, 4, 8, 3).serialize() == [11, 1, 0, 4, 8, 3, 1, 16, 1408]
    assert D.RoutedExpert_UpGate_SiLU(1, 2, 0, 4).serialize() == [12, 1, 2, 0, 4, 1, 16]
    assert D.RoutedExpert_DownProj(1, 2, 0, 0, 5).serialize() == [13, 1, 2, 0, 0, 5, 1, 16]
    assert D.MoE_Combine_Commit(1, 0, 2).serialize() == [14, 1, 0, 2, 16]
    assert D.RMS_QKVProj_GEMV_RoPE(0, 0, 3, 7).serialize() == [1, 0, 0, 3, 7, 1, 16]
    assert D.DecodeAttentionReduction(0, 4, 3, [0, 1, 2]).serialize() == [3, 0, 4, 3, 3, 0, 1, 2, 1, 0]
    assert D.RMS_LMHead_GEMV(10, 20).serialize() == [7, 10, 20, 1, 16]
    assert sorted(D.INSTRUCTION_BY_OPCODE) == [0, 1, 2, 3, 4, 7, 8, 9, 10, 11, 12, 13, 14]


# ------------------------------------------------------------------ scheduler --
def test_instruction_streams_match_the_reference_digests():
    full = S.reference_scheduler(QWEN1_5_MOE_A2_7B).instruction_list()
    meta = FIX["full_size_instruction_list"]
    assert len(full) == meta["instructions"] and hashlib.sha256(_words(full).tobytes()).hexdigest() == meta["sha256"]
    small = S.reference_scheduler(SMALL)
    assert (small.sm_count, small.num_partials) == (FIX["queues"], FIX["num_partials"]) == (108, num_partials_for(108, SMALL))
    flat = small.instruction_list()
    assert len(flat) == FIX["instructions_per_step"] and hashlib.sha256(_words(flat).tobytes()).hexdigest() == FIX["instruction_list_sha256"]


@pytest.mark.parametrize("queues", [108, 256])
def test_every_tile_once(queues):
    s = QWEN1_5_MOE_A2_7B
    sched = S.MoeScheduler(s, queues, num_partials_for(queues, s))
    layer = sched.layer(3)
    spans = {op: [] for op in (1, 4, 10, 14)}
    for i in layer:
        if i.opcode() in spans:
            spans[i.opcode()] += range(i.tile_N_start_idx, i.tile_N_end_idx)
    assert spans[1] == list(range(s.qkv_out_dim // s.qkv_tile)) and spans[4] == spans[14] == list(range(s.num_hidden_blocks))
    assert all(i.tile_N_granularity == s.qkv_tile for i in layer if i.opcode() == 1)
    if queues == 256:    # the tile of the shape deals the QKV rows evenly; the reference's tile of 16 does not
        assert {i.tile_N_end_idx - i.tile_N_start_idx for i in layer if i.opcode() == 1} == {3} and s.qkv_tile == 8
        sixteen = S.reference_scheduler(s, 256).qkvproj(3)
        assert {i.tile_N_end_idx - i.tile_N_start_idx for i in sixteen} == {1, 2} and all(i.tile_N_granularity == 16 for i in sixteen)
    assert spans[10] == list(range(s.intermediate_size // 16))
    assert sum(i.init_shared_out for i in layer if i.opcode() == 10) == 1
    routers = [i for i in layer if i.opcode() == 8]
    assert [(i.tile_N_start_idx, i.tile_N_end_idx) for i in routers] == [(e, e + 1) for e in range(s.num_experts)]
    assert sum(i.write_normed_hidden for i in routers) == 1 and len([i for i in layer if i.opcode() == 9]) == 1
    shared_down = sorted((i.split_K_idx, b) for i in layer if i.opcode() == 11 for b in range(i.tile_N_start_idx, i.tile_N_end_idx))
    assert shared_down == [(k, b) for k in range(s.num_downproj_split_k_shared) for b in range(s.num_hidden_blocks)]
    assert all(i.split_K_granularity == s.intermediate_size // 4 for i in layer if i.opcode() == 11)
    for op, blocks in ((12, s.num_moe_intermediate_blocks), (13, s.num_hidden_blocks)):
        got = sorted((i.expert_idx, b) for i in layer if i.opcode() == op for b in range(i.tile_N_start_idx, i.tile_N_end_idx))
        assert got == [(slot, b) for slot in range(s.num_experts_per_tok) for b in range(blocks)]
    order = [i.opcode() for i in layer]
    assert order == sorted(order, key=[1, 2, 3, 4, 8, 9, 10, 11, 12, 13, 14].index)


# -------------------------------------------------------------------- oracles --
def test_request_of_the_reference_fixture(weights):
    vm_g, fu_g = _request(weights), _request(weights)
    vm, fused, sched = MoeInstructionVM(SMALL), FusedMoeOracle(SMALL), S.reference_scheduler(SMALL)
    tok = {"my_vm": FIX["start_token"], "my_fused": FIX["start_token"]}
    for step, want in enumerate(FIX["steps"]):
        for name, g in (("my_vm", vm_g), ("my_fused", fu_g)):
            g.position_id = want["position"]
            g.hidden_states.copy_(g.embed_tokens[tok[name]])
        vm_g.barriers.zero_()
        vm.run(vm_g, sched.instruction_list())
        for layer in range(SMALL.num_hidden_layers):
            fused.decode_layer(fu_g, layer)
            rec = want["my_fused"]["experts_per_layer"][layer]
            assert fu_g.expert_indices.tolist() == rec["indices"] and fu_g.expert_weights.tolist() == rec["weights"]
        fused.lm_head(fu_g)
        assert vm_g.expert_indices.tolist() == want["my_vm"]["last_layer_experts"]["indices"]
        assert vm_g.expert_weights.tolist() == want["my_vm"]["last_layer_experts"]["weights"]
        for name, g in (("my_vm", vm_g), ("my_fused", fu_g)):
            ids = torch.tensor(want[name]["top_ids"])
            assert _bits(g.logits[ids]) == want[name]["top_bits"], (step, name)
            assert _bits(g.hidden_states[::128]) == want[name]["hidden_bits_sampled"], (step, name)
            tok[name] = int(g.logits.float().argmax())
            assert tok[name] == want[name]["token"]


@pytest.mark.parametrize("merge", ["oproj", "last"])
def test_vm_agrees_with_fused_and_counters_complete(weights, merge):
    f, v = _request(weights), _request(weights)
    for g in (f, v):
        g.position_id = 41
        g.hidden_states.copy_(g.embed_tokens[99])
    FusedMoeOracle(SMALL).decode_step(f)
    from qimeng_megakernel_amd.decode_schedule_moe.mk_kernel import mi355x_scheduler

    sched = mi355x_scheduler(SMALL)          # 256 queues placed by role, expert phases interleaved, the O-projection merges
    assert sched.merge_in_oproj and sched.placed
    if merge == "last":                      # the other stream without reduction instructions
        sched = dataclasses.replace(sched, merge_in_oproj=False, merge_in_last=True, num_partials=16)
    assert not any(i.opcode() == 3 for i in sched.instruction_list())
    MoeInstructionVM(SMALL).run(v, sched.instruction_list())
    for name in ("q_post_rope", "attn_out", "hidden_states", "logits"):
        a, b = getattr(f, name).float(), getattr(v, name).float()
        assert float((a - b).abs().max()) <= 2.0 ** -5 * max(1.0, float(a.abs().max())), name
    assert f.logits.float().argmax().item() == v.logits.float().argmax().item()
    s = SMALL
    for layer in range(s.num_hidden_layers):
        bar = v.barriers[layer]
        assert bar[0, : s.num_heads].tolist() == [s.head_dim // s.qkv_tile] * s.num_heads
        if merge == "last":
            assert bar[1, : s.num_attention_heads].tolist() == [sched.num_partials] * s.num_attention_heads
        else:                                # split-KV instructions count on the reduction row only
            assert int(bar[1].abs().sum()) == 0
        assert int(bar[2, 0]) == (s.num_attention_heads if merge == "last" else s.num_key_value_heads * sched.num_partials)
        assert int(bar[3, 0]) == s.num_hidden_blocks == int(bar[13, 0])
        assert bar[7, :2].tolist() == [s.num_experts, 1] and int(bar[8, 0]) == 1
        assert int(bar[9, 0]) == s.intermediate_size // 16 and int(bar[11, 0]) == s.num_experts_per_tok * s.num_moe_intermediate_blocks
        assert bar[10, : s.num_hidden_blocks].tolist() == [s.num_downproj_split_k_shared] * s.num_hidden_blocks
        assert bar[12, : s.num_hidden_blocks].tolist() == [s.num_experts_per_tok] * s.num_hidden_blocks
    assert float(v.routed_out_f32.abs().max()) == 0.0      # the combine step hands the accumulator back cleared


def test_placed_stream_is_the_same_instructions_by_role():
    """The MI355X stream at full size: the queues hold exactly the instruction list, every queue runs its layer's
    phases in dependency order, the queues of the router and the top-k take no shared up/gate rows, and no queue
    takes more than three up/gate tiles of a layer."""
    from collections import Counter

    from qimeng_megakernel_amd.decode_schedule_moe.mk_kernel import mi355x_scheduler
    from qimeng_megakernel_amd.decode_schedule_moe.model_config import QWEN1_5_MOE_A2_7B as FULL

    sched = mi355x_scheduler(FULL, tagged=False)    # the stream for launches on counters: every queue in dependency order
    queues = sched.queues()
    assert len(queues) == 256 and sched.placed
    # The stream for tagged launches of a shape without a shared expert differs in two things: the top-k instruction,
    # which nobody inside such a launch waits for, runs in the NEXT layer's attention phase (between its queue's QKV rows
    # and O-projection rows; the last layer's is the queue's last instruction), and one routed down-projection
    # instruction per 8 rows takes all expert slots and commits them, so there are no combine instructions.
    from qimeng_megakernel_amd.decode_schedule_moe.model_config import QWEN3_30B_A3B
    assert [tuple(i.padded()) for q in mi355x_scheduler(FULL).queues() for i in q] == [tuple(i.padded()) for q in queues for i in q]   # a shared expert: neither
    counters, tagged_stream = mi355x_scheduler(QWEN3_30B_A3B, tagged=False).queues(2), mi355x_scheduler(QWEN3_30B_A3B).queues(2)
    same = lambda qs: Counter(tuple(i.padded()) for q in qs for i in q if i.opcode() not in (13, 14))
    assert same(counters) == same(tagged_stream)
    assert not any(i.opcode() == 14 for q in tagged_stream for i in q) and sum(i.opcode() == 14 for q in counters for i in q) == 2 * 128
    down = [i for q in tagged_stream for i in q if i.opcode() == 13]
    assert len(down) == 2 * 256 and all(i.tile_M_idx == 2 and i.expert_idx == 0 and i.tile_N_granularity == 8 for i in down)
    assert sorted((i.layer_idx, r) for i in down for r in range(i.tile_N_start_idx * 8, i.tile_N_end_idx * 8)) == \
        [(layer, r) for layer in range(2) for r in range(QWEN3_30B_A3B.hidden_size)]
    import dataclasses
    for fewer in (128, 100):                       # fewer queues: one or two tiles of 8 rows per committing instruction, never more
        spans = [i.tile_N_end_idx - i.tile_N_start_idx for q in dataclasses.replace(mi355x_scheduler(QWEN3_30B_A3B), sm_count=fewer).queues(1)
                 for i in q if i.opcode() == 13]
        assert sum(spans) == QWEN3_30B_A3B.hidden_size // 8 and set(spans) <= {1, 2}
    # split-KV slices per KV head of that shape: 2, 4 for a request whose cache holds more than 256 tokens
    assert [mi355x_scheduler(QWEN3_30B_A3B, kv_capacity=c).num_partials for c in (None, 64, 256, 257, 528)] == [2, 2, 2, 4, 4]
    assert mi355x_scheduler(FULL, kv_capacity=1040).num_partials == 8
    holders = [ql for ql in tagged_stream if any(i.opcode() == 9 for i in ql)]
    assert len(holders) == 1
    ops = [(i.opcode(), i.padded()[1]) for i in holders[0]]
    at = ops.index((9, 0))                         # layer 0's report: behind layer 1's QKV rows, ahead of its O-projection rows
    assert ops[at - 1] == (1, 1) and ops[at + 1] == (4, 1) and ops[-1] == (9, 1)
    key = lambda ins: tuple(ins.padded())
    assert Counter(key(i) for q in queues for i in q) == Counter(key(i) for i in sched.instruction_list())
    phase = {1: 0, 2: 1, 3: 2, 4: 3, 8: 4, 9: 5, 10: 6, 12: 7, 11: 8, 13: 9, 14: 10, 7: 11}
    for q in queues:
        order = [(10 ** 6 if i.opcode() == 7 else i.padded()[1], phase[i.opcode()]) for i in q]
        assert order == sorted(order)
    layer0 = [[i for i in q if i.opcode() != 7 and i.padded()[1] == 0] for q in queues]
    side = [q for q in layer0 if any(i.opcode() in (8, 9) for i in q)]
    assert len(side) == 9 and not any(i.opcode() in (4, 10) for q in side for i in q)
    tiles = [sum(i.padded()[4] - i.padded()[3] for i in q if i.opcode() in (10, 12)) for q in layer0]
    assert max(tiles) == 3 and sum(tiles) == 2 * 352
    # weight rows of H per queue between the attention and the down projections (an up/gate output streams two): the routed
    # tiles fill the queues up to one level, 96 rows, as far as tiles of 16 outputs can (the queues of the router and the
    # top-k, which start last, get what the least loaded of the others gets)
    rows = [sum((i.padded()[4] - i.padded()[3]) * (16 if i.opcode() == 4 else 32) for i in q if i.opcode() in (4, 10, 12)) for q in layer0]
    main = [r for r, q in zip(rows, layer0) if not any(i.opcode() in (8, 9) for i in q)]
    assert sum(rows) == 256 * 96 and set(main) == {80, 96, 112} and Counter(main)[96] >= 119
    assert all(sum((i.padded()[4] - i.padded()[3]) for i in q if i.opcode() == 12) == 2 for q in side)


def _crafted(weights, layer=0):
    """Layer 0 of a request whose MoE block has a known answer: router rows that pick experts 5 and 2
    with prescribed logits, all experts equal to expert 0, and a shared gate of zero weights."""
    w = {k: v.clone() for k, v in weights.items()}
    w["expert_gate_up_proj_weights"][layer] = w["expert_gate_up_proj_weights"][layer, 0]
    w["expert_down_proj_weights"][layer] = w["expert_down_proj_weights"][layer, 0]
    w["shared_expert_gate_weights"][layer].zero_()
    g = _request(w)
    g.position_id = 17
    g.hidden_states.copy_(g.embed_tokens[3])
    return w, g


@pytest.mark.parametrize("route", ["fused", "vm"])
def test_moe_block_closed_form(weights, route):
    """With identical experts the routed sum is (sum of the top-k weights) x one expert's output; with
    a zero shared gate the shared output enters with sigmoid(0) = 1/2; the top-k weights are the
    softmax of the prescribed logits, not renormalised."""
    from fused_oracle import rms_norm

    w, g = _crafted(weights)
    s = SMALL
    oracle = FusedMoeOracle(s)
    oracle.qkv_rope(g, 0); oracle.attention(g, 0); oracle.oproj_residual(g, 0)
    normed = rms_norm(g.hidden_states, g.mlp_norm_weights[0], s.rms_norm_eps)
    # router rows along the normalised vector: logit_e = c_e * |normed|^2 / |normed|^2 = c_e
    unit = normed.float() / normed.float().pow(2).sum()
    want_logits = torch.tensor([0.0, -1.0, 2.0, -2.0, 0.5, 3.0, -0.5, 1.0])
    g.router_weights[0].copy_((want_logits[:, None] * unit[None, :]).to(torch.bfloat16))
    before = g.hidden_states.clone()
    if route == "fused":
        oracle.moe_block(g, 0)
    else:
        g.barriers[0, 3, 0] = s.num_hidden_blocks
        sched = S.reference_scheduler(s)
        MoeInstructionVM(s).run(g, sched.router_gemv(0) + sched.router_softmax_topk(0) + sched.shared_upgate(0) + sched.shared_downproj(0)
                                + sched.routed_upgate(0) + sched.routed_downproj(0) + sched.combine_commit(0))
    assert g.expert_indices.tolist() == [5, 2]
    probs = torch.softmax((g.router_weights[0].float() * normed.float()).sum(-1), dim=-1)
    assert torch.allclose(g.expert_weights, probs[[5, 2]], rtol=1e-5)
    assert abs(float(probs[5]) - float(torch.softmax(want_logits, 0)[5])) < 2e-2      # bf16 router rows
    # one expert and the shared expert, computed directly in fp32 from the same normalised row
    mid = s.moe_intermediate_size
    gu = w["expert_gate_up_proj_weights"][0, 0].float() @ normed.float()
    one = w["expert_down_proj_weights"][0, 0].float() @ (torch.nn.functional.silu(gu[:mid]) * gu[mid:])
    sh = torch.nn.functional.silu(w["shared_expert_gate_proj_weights"][0].float() @ normed.float()) * (w["shared_expert_up_proj_weights"][0].float() @ normed.float())
    shared = w["shared_expert_down_proj_weights"][0].float() @ sh
    want = before.float() + float(probs[5] + probs[2]) * one + 0.5 * shared
    got = g.hidden_states.float()
    assert float((got - want).abs().max()) <= 3e-2 * float(want.abs().max())
    # and the terms matter: dropping the gate or one expert is far outside that tolerance
    assert float((before.float() + float(probs[5]) * one + 0.5 * shared - got).abs().max()) > 3e-2 * float(want.abs().max())
    assert float((before.float() + float(probs[5] + probs[2]) * one + shared - got).abs().max()) > 3e-2 * float(want.abs().max())


def test_mk_of_the_moe_route_checks_its_arguments(weights):
    with pytest.raises(ImportError, match="missing prebuilt kernel"):
        mk_kernel.get_mk(ROOT / "tests")
    mk = mk_kernel.get_mk()
    g = _request(weights)
    g.instructions = torch.zeros(4, 1, 32, dtype=torch.int32)
    with pytest.raises(ValueError, match="must live on the GPU"):
        mk_kernel.call_mk(g, mk)
    with pytest.raises(TypeError, match="positional arguments"):
        mk(g.instructions, g.hidden_states)
