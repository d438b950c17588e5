"""Pin the CPU oracle against what the mathematics fixes.

Every check is chosen so that a plausible mistake in the oracle (a dropped
rounding, a swapped sign or index, the wrong pairing in RoPE, a transposed
weight) fails it.  bf16 rounding is re-implemented here on bit patterns, and all
reference values are fp64 brute force — nothing below calls the function it pins.
"""
import dataclasses
import math

import numpy as np
import pytest
import torch

from fused_oracle import FusedOracle, gemv, rms_norm, rotate_pairs
from pyvm_oracle import Counts, InstructionVM
from qimeng_megakernel_amd import synthetic
from qimeng_megakernel_amd.decode_schedule.instructions import instruction_defs as D
from qimeng_megakernel_amd.decode_schedule.instructions import scheduler as S
from qimeng_megakernel_amd.decode_schedule.model_config import LLAMA_3_2_1B, LlamaConfig


def bf16_round(x: np.ndarray) -> np.ndarray:
    """fp32/fp64 -> nearest-even bf16, returned as fp64 (independent of torch)."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) >> 16 << 16
    return u.astype(np.uint32).view(np.float32).astype(np.float64)


def f64(t: torch.Tensor) -> np.ndarray:
    return t.double().numpy()


def ulp_bf16(x):
    return 2.0 ** (np.floor(np.log2(np.maximum(np.abs(x), 1e-30))) - 7)


def test_bf16_round_helper_matches_torch():
    x = torch.randn(10000) * 3
    assert np.array_equal(bf16_round(x.numpy()), f64(x.bfloat16()))


def test_rms_norm_two_roundings():
    torch.manual_seed(0)
    x = (torch.randn(2048) * 1.7).bfloat16()
    w = (1 + 0.1 * torch.randn(2048)).bfloat16()
    got = f64(rms_norm(x, w, 1e-5))
    xs = f64(x)
    rstd = 1.0 / math.sqrt(float((xs ** 2).mean()) + 1e-5)
    n = bf16_round(xs * np.float32(rstd))
    want = bf16_round(f64(w) * n)
    # the fp32 reduction may differ from fp64 in the last bit of rstd: allow 1 bf16 ulp on a few elements
    diff = np.abs(got - want)
    assert (diff <= ulp_bf16(want)).all() and (diff > 0).mean() < 0.02
    # with unit weights the second rounding is the identity
    assert torch.equal(rms_norm(x, torch.ones(2048, dtype=torch.bfloat16), 1e-5),
                       (x.float() * torch.rsqrt(x.float().pow(2).mean() + 1e-5)).bfloat16())
    # a single-rounding implementation would differ somewhere
    single = bf16_round(f64(w) * xs * rstd)
    assert (single != want).any()


def test_rotate_pairs_sign_and_order():
    x = torch.arange(8.0)
    assert rotate_pairs(x).tolist() == [-1, 0, -3, 2, -5, 4, -7, 6]


def test_rope_tables_closed_form_and_hf_equivalence():
    shape = LLAMA_3_2_1B
    cos, sin = synthetic.rope_tables(shape, 64)
    d = shape.head_dim
    assert torch.equal(cos[0], torch.ones(d)) and torch.equal(sin[0], torch.zeros(d))
    for pos in (1, 17, 63):
        for i in (0, 5, 31):
            ang = np.float32(pos) * np.float32(1.0 / (np.float32(shape.rope_theta) ** np.float32(2 * i / d)))
            assert abs(float(cos[pos, 2 * i]) - math.cos(ang)) < 1e-6 and cos[pos, 2 * i] == cos[pos, 2 * i + 1]
            assert abs(float(sin[pos, 2 * i]) - math.sin(ang)) < 1e-6 and sin[pos, 2 * i] == sin[pos, 2 * i + 1]
    # interleaved rotation of interleaved vectors == HF rotate-half on the original order (textbook RoPE)
    torch.manual_seed(1)
    q, k = torch.randn(d, dtype=torch.float64), torch.randn(d, dtype=torch.float64)
    idx = synthetic.interleave_indices(d)
    pos_q, pos_k = 9, 4
    def hf(x, pos):
        inv = 1.0 / (shape.rope_theta ** (torch.arange(0, d, 2).double() / d))
        f = torch.cat((pos * inv, pos * inv))
        rot = torch.cat((-x[d // 2:], x[: d // 2]))
        return x * f.cos() + rot * f.sin()
    def ours(x, pos):
        xi = x[idx]
        return xi * cos[pos].double() + rotate_pairs(xi) * sin[pos].double()
    assert torch.allclose(ours(q, pos_q), hf(q, pos_q)[idx], atol=1e-6)
    assert abs(float(ours(q, pos_q) @ ours(k, pos_k)) - float(hf(q, pos_q) @ hf(k, pos_k))) < 1e-5
    # rotation preserves every pair's norm
    r = ours(q, pos_q)
    assert torch.allclose(r[0::2] ** 2 + r[1::2] ** 2, q[idx][0::2] ** 2 + q[idx][1::2] ** 2, atol=1e-6)


@pytest.fixture(scope="module")
def one_layer():
    shape = dataclasses.replace(LLAMA_3_2_1B, num_hidden_layers=1, vocab_size=512)
    w = synthetic.random_weights(shape, seed=3, max_positions=48)
    # non-trivial norm weights so that their use is observable
    gen = torch.Generator().manual_seed(5)
    for name in ("attn_norm_weights", "mlp_norm_weights", "lm_head_norm_weights"):
        w[name] = (1 + 0.2 * torch.randn(w[name].shape, generator=gen)).bfloat16()
    return shape, w


def _fresh(shape, w, pos=0, hidden_seed=0):
    g = synthetic.build_globals(w, shape, 48, "cpu")
    gen = torch.Generator().manual_seed(hidden_seed)
    g.hidden_states.copy_((torch.randn(shape.hidden_size, generator=gen) * 0.5).bfloat16())
    g.position_id = pos
    return g


def _near_bf16(got: np.ndarray, want_f64: np.ndarray, frac_off=0.01):
    """bf16 results of an fp32-accumulated dot product: equal to the bf16 rounding of the exact
    value except where the exact value sits next to a rounding boundary (then 1 ulp)."""
    want = bf16_round(want_f64)
    diff = np.abs(got - want)
    assert (diff <= ulp_bf16(want) * 1.001).all(), float(diff.max())
    assert (diff > 0).mean() <= frac_off


def test_qkv_rope_against_fp64(one_layer):
    shape, w = one_layer
    pos = 13
    g = _fresh(shape, w, pos)
    # make the KV row non-zero beforehand to see it overwritten
    g.k_cache.fill_(1.0); g.v_cache.fill_(1.0)
    FusedOracle(shape).qkv_rope(g, 0)
    y = f64(rms_norm(g.hidden_states, w["attn_norm_weights"][0], shape.rms_norm_eps))
    qkv = bf16_round(f64(w["qkv_weights"][0]) @ y)          # rounded BEFORE the rotation
    cos, sin = f64(w["rope_cos"][pos]), f64(w["rope_sin"][pos])
    def rope(v):
        v = v.reshape(-1, shape.head_dim)
        rot = np.stack((-v[:, 1::2], v[:, 0::2]), axis=-1).reshape(v.shape)
        return (v * cos + rot * sin).reshape(-1)
    nq, nkv, d = shape.num_attention_heads, shape.num_key_value_heads, shape.head_dim
    _near_bf16(f64(g.q_post_rope), rope(qkv[: nq * d]), 0.02)
    _near_bf16(f64(g.k_cache[0, 0, pos]).reshape(-1), rope(qkv[nq * d:(nq + nkv) * d]), 0.02)
    _near_bf16(f64(g.v_cache[0, 0, pos]).reshape(-1), qkv[(nq + nkv) * d:], 0.02)
    assert (g.k_cache[0, 0, pos + 1] == 1).all() and (g.k_cache[0, 0, pos - 1] == 1).all()
    # position 0 is the identity rotation: q equals the rounded projection
    g0 = _fresh(shape, w, 0)
    FusedOracle(shape).qkv_rope(g0, 0)
    _near_bf16(f64(g0.q_post_rope), qkv[: nq * d], 0.01)


def _brute_attention(q, K, V, ratio):
    """fp64 softmax attention, GQA: q [Hq, d], K/V [n, Hkv, d]."""
    out = np.zeros_like(q)
    for h in range(q.shape[0]):
        s = K[:, h // ratio] @ q[h] / math.sqrt(q.shape[1])
        p = np.exp(s - s.max()); p /= p.sum()
        out[h] = p @ V[:, h // ratio]
    return out


def test_attention_against_brute_force_and_invariants(one_layer):
    shape, w = one_layer
    nq, nkv, d = shape.num_attention_heads, shape.num_key_value_heads, shape.head_dim
    g = _fresh(shape, w, pos=36)
    gen = torch.Generator().manual_seed(2)
    g.q_post_rope.copy_(torch.randn(nq * d, generator=gen).bfloat16())
    g.k_cache[0, 0].copy_(torch.randn(48, nkv, d, generator=gen).bfloat16())
    g.v_cache[0, 0].copy_(torch.randn(48, nkv, d, generator=gen).bfloat16())
    o = FusedOracle(shape)
    o.attention(g, 0)
    want = _brute_attention(f64(g.q_post_rope).reshape(nq, d), f64(g.k_cache[0, 0, :37]), f64(g.v_cache[0, 0, :37]), nq // nkv)
    _near_bf16(f64(g.attn_out), want.reshape(-1), 0.01)      # tokens beyond pos are ignored
    # one token: output is V[0] of the KV head the query head maps to
    g.position_id = 0
    o.attention(g, 0)
    assert torch.equal(g.attn_out.view(nq, d), g.v_cache[0, 0, 0].repeat_interleave(nq // nkv, dim=0))
    # all V rows equal: output equals that row whatever the scores
    g.position_id = 20
    g.v_cache[0, 0, :21] = g.v_cache[0, 0, 5].clone()
    o.attention(g, 0)
    assert (g.attn_out.view(nq, d).float() - g.v_cache[0, 0, 5].repeat_interleave(nq // nkv, dim=0).float()).abs().max() <= 2 ** -7


def test_residual_gemvs_against_fp64(one_layer):
    shape, w = one_layer
    o = FusedOracle(shape)
    g = _fresh(shape, w)
    gen = torch.Generator().manual_seed(4)
    g.attn_out.copy_(torch.randn(shape.hidden_size, generator=gen).bfloat16())
    h0 = f64(g.hidden_states)
    o.oproj_residual(g, 0)
    delta = bf16_round(f64(w["o_proj_weights"][0]) @ f64(g.attn_out))   # first rounding
    _near_bf16(f64(g.hidden_states), h0 + delta, 0.02)                 # second rounding
    # MLP
    h1 = f64(g.hidden_states)
    o.mlp_upgate(g, 0)
    y = f64(rms_norm(g.hidden_states, w["mlp_norm_weights"][0], shape.rms_norm_eps))
    up = bf16_round(f64(w["up_proj_weights"][0]) @ y)
    gate = bf16_round(f64(w["gate_proj_weights"][0]) @ y)
    act = bf16_round(gate / (1 + np.exp(-gate)))
    _near_bf16(f64(g.silu_out), act * up, 0.03)
    # up and gate must not be swapped: silu(up) * gate differs
    swapped = bf16_round(bf16_round(up / (1 + np.exp(-up))) * gate)
    assert (np.abs(f64(g.silu_out) - swapped) > 2 * ulp_bf16(swapped)).mean() > 0.5
    o.mlp_down_residual(g, 0)
    delta = bf16_round(f64(w["down_proj_weights"][0]) @ f64(g.silu_out))
    _near_bf16(f64(g.hidden_states), h1 + delta, 0.02)
    # LM head
    o.lm_head(g)
    y = f64(rms_norm(g.hidden_states, w["lm_head_norm_weights"], shape.rms_norm_eps))
    _near_bf16(f64(g.logits), f64(w["lm_head_weights"]) @ y, 0.01)


def test_gemv_orientation():
    W = torch.arange(6.0).view(3, 2)
    assert gemv(W, torch.tensor([[1.0, 10.0]])).tolist() == [[10.0, 32.0, 54.0]]


def test_greedy_positions_and_first_index_ties(one_layer):
    shape, w = one_layer
    o = FusedOracle(shape)
    g = synthetic.build_globals(w, shape, 48, "cpu")
    prompt = synthetic.random_prompt(shape, 3, 4)
    toks = o.greedy(g, prompt, 5)
    assert len(toks) == 5 and g.position_id == 4 + 3        # the last embedded token sits at prompt_len + 3
    # replay by hand: token i of the continuation is embedded at position prompt_len + i
    h = synthetic.build_globals(w, shape, 48, "cpu")
    seq = prompt.tolist()
    for pos in range(4 + 4):
        o.embed(h, seq[pos]); h.position_id = pos; o.decode_step(h)
        if pos >= 3:
            seq.append(int(h.logits.argmax()))
    assert seq[4:] == toks
    assert int(torch.argmax(torch.tensor([1.0, 3.0, 3.0, 2.0]).bfloat16())) == 1


# ----------------------------------------------------- split-KV / LSE merge ----
@pytest.mark.parametrize("seq_len,P", [(1, 1), (1, 5), (16, 3), (17, 2), (37, 4), (37, 13), (40, 25), (33, 7)])
def test_split_merge_equals_unsplit(one_layer, seq_len, P):
    shape, w = one_layer
    nq, nkv, d = shape.num_attention_heads, shape.num_key_value_heads, shape.head_dim
    g = _fresh(shape, w, pos=seq_len - 1)
    gen = torch.Generator().manual_seed(seq_len * 31 + P)
    g.q_post_rope.copy_(torch.randn(nq * d, generator=gen).bfloat16())
    g.k_cache[0, 0].copy_(torch.randn(48, nkv, d, generator=gen).bfloat16())
    g.v_cache[0, 0].copy_(torch.randn(48, nkv, d, generator=gen).bfloat16())
    g.barriers[0, 0, :] = 4
    g.attn_lse_intermediates.fill_(123.0); g.attn_out_intermediates.fill_(-7.0)   # stale garbage must not leak
    vm = InstructionVM(shape, Counts())
    sched = S.DecodeScheduler(shape, D.REFERENCE_GEOMETRY, 108, P)
    ins = sched.attention_split_kv(0) + sched.attention_reduction(0)
    # any execution order of the partials, and any order of the merge list, gives the same answer
    rng = np.random.default_rng(P)
    split = ins[: nkv * P]; rng.shuffle(split)
    red = ins[nkv * P:]
    for r in red:
        perm = list(r.reduction_list); rng.shuffle(perm); r.reduction_list = perm
    vm.run(g, list(split) + red)
    want = _brute_attention(f64(g.q_post_rope).reshape(nq, d), f64(g.k_cache[0, 0, :seq_len]), f64(g.v_cache[0, 0, :seq_len]), nq // nkv)
    _near_bf16(f64(g.attn_out), want.reshape(-1), 0.02)
    total_blocks = math.ceil(seq_len / 16); per = math.ceil(total_blocks / P)
    for p in range(P):
        empty = p * per >= total_blocks
        assert bool(torch.isinf(g.attn_lse_intermediates[:, p]).all()) == empty
        if empty:
            assert (g.attn_out_intermediates[:, p] == 0).all()
    assert (g.barriers[0, 1, :nq] == P).all() and int(g.barriers[0, 2, 0]) == nq
    # partial LSEs are in the log2 domain: 2^lse sums to the full partition function
    s = (f64(g.k_cache[0, 0, :seq_len, 0]) @ f64(g.q_post_rope).reshape(nq, d)[0]) / 8.0
    z = sum(2.0 ** float(g.attn_lse_intermediates[0, p]) for p in range(P))
    assert abs(z / np.exp(s).sum() - 1) < 1e-4


def test_pyvm_matches_fused_and_counts(small_model):
    shape, w, prompt = small_model
    LlamaConfig.set_shape(shape)
    # (scheduler, hidden tolerance, logit tolerance): the K-sliced down projection of the reference
    # geometry adds four bf16-rounded partials per row, a few ulps away from the single fused add.
    for sched, tol_h, tol_l in ((S.mi355x_scheduler(shape, num_partials=3), 0.016, 0.04),
                                (S.reference_scheduler(shape), 0.07, 0.15)):
        a = synthetic.build_globals(w, shape, 96, "cpu")
        b = synthetic.build_globals(w, shape, 96, "cpu")
        fo, vm = FusedOracle(shape), InstructionVM(shape, Counts(*sched.expected_counts()))
        il = sched.instruction_list()
        for pos, tok in enumerate(prompt.tolist()[:3]):
            for g in (a, b):
                fo.embed(g, tok); g.position_id = pos
            fo.decode_step(a)
            b.barriers.zero_(); vm.run(b, il)
            # identical up to where a tile GEMV rounds differently from the full GEMV (and, for the
            # reference geometry, the four bf16-rounded K slices of the down projection)
            assert (a.hidden_states.float() - b.hidden_states.float()).abs().max() <= tol_h
            assert (a.logits.float() - b.logits.float()).abs().max() <= tol_l
        bph, opb, ubk, dwn = sched.expected_counts()
        assert int(b.barriers[1, 5, 0]) == dwn and int(b.barriers[0, 3, 0]) == opb
        assert (b.barriers[:, 0, : shape.num_heads] == bph).all()
        assert (b.barriers[:, 4, : sched.geometry.num_split_k(shape)] == ubk).all()
