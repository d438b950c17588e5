"""Full-size Llama-3.2-1B-shaped decode on the GPU against the golden fixtures.

The fixtures (tests/golden/llama1b_seed0.*) were written once from the imported reference
(fused route, `…/decode_schedule/fused/layer_scheduler.py:45-56`) on this repository's seeded
weights: 8-token prompt, 1024 forced-greedy tokens, per-step top-8 logits and margins, sampled
hidden states.  The reference's own bf16 logits tie exactly (margin 0) on ~5% of the steps and sit
within 2 bf16 ulps on ~18%, so a free-running trajectory is decided by accumulation-order noise at
those steps; the comparison is therefore teacher-forced, and strict wherever the margin is clear.
"""
import json

import numpy as np
import pytest
import torch

from conftest import GOLDEN
from gpu_helpers import rel_close, tensor_rel_close
from qimeng_megakernel_amd import decode, synthetic
from qimeng_megakernel_amd.decode_schedule import mk_kernel
from qimeng_megakernel_amd.decode_schedule.instructions import scheduler as S
from qimeng_megakernel_amd.decode_schedule.model_config import LLAMA_3_2_1B, LlamaConfig

pytestmark = pytest.mark.gpu

LOGIT_ULPS = 6.0   # see test_teacher_forced_1024_steps, point 1


def _bf16(bits: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(bits.astype(np.int32)).to(torch.int16).view(torch.bfloat16).float()


@pytest.fixture(scope="module")
def golden():
    meta = json.loads((GOLDEN / "llama1b_seed0.json").read_text())
    arrays = np.load(GOLDEN / "llama1b_seed0.npz")
    assert meta["complete"] and meta["new_tokens"] == 1024
    return meta, arrays


@pytest.fixture(scope="module")
def model(golden):
    meta, _ = golden
    shape = LLAMA_3_2_1B
    LlamaConfig.set_shape(shape)
    kv = meta["prompt_len"] + meta["new_tokens"]
    weights = synthetic.random_weights(shape, meta["seed"], max_positions=kv)
    prompt = synthetic.random_prompt(shape, meta["seed"], meta["prompt_len"])
    assert prompt.tolist() == meta["prompt"]
    return shape, synthetic.build_globals(weights, shape, kv, "cuda:0"), prompt


def test_teacher_forced_1024_steps(golden, model):
    meta, arrays = golden
    shape, g, prompt = model
    LlamaConfig.set_shape(shape)
    mk = mk_kernel.get_mk()
    S.build(g)
    tokens = meta["tokens"]                      # tokens[i] = i-th generated token (the first comes from prefill)
    seq = prompt.tolist() + tokens
    n_prompt, n_new = len(prompt), len(tokens)
    topk_ids = torch.from_numpy(arrays["topk_ids"].astype(np.int64)).cuda()
    got_argmax = torch.zeros(n_new, dtype=torch.long, device="cuda")
    got_topk = torch.zeros(n_new, 8, dtype=torch.float32, device="cuda")
    record = {0: "step0", 1: "step1", 127: "step127", 511: "step511"}
    hidden_at, logits_at = {}, {}
    ids = torch.tensor(seq, device="cuda")
    for pos in range(n_prompt + n_new - 1):
        g.hidden_states.copy_(g.embed_tokens[ids[pos]])
        g.position_id = pos
        mk_kernel.call_mk(g, mk)
        i = pos - (n_prompt - 1)                 # index of the token this step predicts
        if i >= 0:
            got_argmax[i] = g.logits.argmax()
            got_topk[i] = g.logits[topk_ids[i]].float()
            step = i - 1                         # fixture naming: decode step k predicts token k+1
            if step in record:
                hidden_at[record[step]] = g.hidden_states.clone()
                logits_at[record[step]] = g.logits[::501].clone()
    mk.check()

    got = got_argmax.cpu().tolist()
    want_topk = _bf16(arrays["topk_bits"])
    ulp = torch.exp2(torch.floor(torch.log2(want_topk[:, 0].abs())) - 7)
    margin_ulps = torch.tensor(meta["margins"]) / ulp
    mismatches = [i for i in range(n_new) if got[i] != tokens[i]]
    err_ulps = ((got_topk.cpu() - want_topk).abs() / ulp[:, None])
    print(f"mismatch margins (ulps): {sorted(float(margin_ulps[i]) for i in mismatches)}")
    print(f"top-8 logit error in ulps of the top logit: max {float(err_ulps.max()):.2f}, "
          f"99.9% {float(err_ulps.flatten().quantile(0.999)):.2f}, mean {float(err_ulps.mean()):.3f}")
    # 1. logits at the reference's top-8 ids: within LOGIT_ULPS bf16 ulps of the top logit.  Exact sums rounded
    #    where the reference rounds sit up to 5 ulps from the fixture and up to 6 from the kernel, 0.78 on average
    #    from either (test_kernel_against_exact_sums_beside_the_reference); the kernel sits up to 5 from the fixture.
    assert float(err_ulps.max()) <= LOGIT_ULPS
    # 2. top-1 identical wherever the reference's own margin exceeds that noise
    clear = [i for i in mismatches if margin_ulps[i] > LOGIT_ULPS]
    assert not clear, f"top-1 differs at clear margins: {[(i, float(margin_ulps[i])) for i in clear[:5]]}"
    # 3. a different pick is one of the reference's top-8 and its reference logit is within the noise of the top
    for i in mismatches:
        ids_i = arrays["topk_ids"][i].tolist()
        assert got[i] in ids_i, f"step {i}: kernel picked {got[i]}, not among the reference top-8"
        assert (want_topk[i, 0] - want_topk[i, ids_i.index(got[i])]) / ulp[i] <= LOGIT_ULPS
    agreement = 1 - len(mismatches) / n_new
    near = margin_ulps <= 2.0
    beyond = [i for i in mismatches if not near[i]]
    print(f"teacher-forced top-1 agreement {agreement:.4f} ({len(mismatches)} of {n_new} differ; "
          f"{int(near.sum())} steps have a reference margin <= 2 ulps, {int((margin_ulps == 0).sum())} exact ties; "
          f"{len(beyond)} mismatches at margins > 2 ulps)")
    for t in (0.0, 0.5, 1.0, 1.5, 2.0, 3.0):
        sel = margin_ulps > t
        bad = sum(1 for i in mismatches if sel[i])
        print(f"  steps with a reference margin > {t} ulps: {int(sel.sum())}, agreement {1 - bad / int(sel.sum()):.4f}")
    # 4. random-init logits are nearly flat: 50 steps are exact ties in the reference's own bf16 logits and 210 sit
    #    within 2 ulps.  The reference's own picks agree with exact sums on 0.930 of the steps (the kernel's on
    #    0.940), so no evaluation can be held to 0.95 over all 1024; it holds where the reference's top two logits
    #    are not tied, and tightens with the margin.
    assert agreement >= 0.93
    for floor_ulps, want_agreement in ((0.0, 0.95), (1.0, 0.975), (2.0, 0.99)):
        sel = margin_ulps > floor_ulps
        bad = sum(1 for i in mismatches if sel[i])
        assert 1 - bad / int(sel.sum()) >= want_agreement, (floor_ulps, bad, int(sel.sum()))
    # 4. residual stream after the last layer and sampled logits at the recorded steps
    for name in record.values():
        # 16 layers deep a second CPU evaluation of the reference (tests/golden/noise_floor_*.json,
        # final_hidden_max_diff_over_max_ref) sits at 2.0e-2 (step 0) .. 2.6e-2 (step 127) of the largest
        # element, and exact sums at 2.0e-2 .. 2.5e-2 from the fixture.  An elementwise ratio means nothing this
        # deep: where |exact| > 0.05 the reference's own elements are off by up to 3.5x their value.
        e = tensor_rel_close(hidden_at[name], _bf16(arrays[f"final_hidden_{name}"]), rel=3e-2, name=f"final hidden {name}")
        want_l = _bf16(arrays[f"logit_samples_{name}"])
        l_err = float((logits_at[name].float().cpu() - want_l).abs().max())
        print(f"{name}: final hidden max|diff|/max|ref| {e:.4f}; 256 sampled logits off by <= {l_err:.4f}")
        assert l_err <= LOGIT_ULPS * 2.0 ** -6      # LOGIT_ULPS ulps of a top logit in [2, 4)


class ExactEvaluator:
    """The decode step with exact sums: every dot product, norm and softmax in fp64 on the GPU, rounded to bf16 at
    exactly the points where the reference's fused route rounds (`…/single_batch/decode_schedule/fused/operations.py:
    126-321`: the normalised row, its product with the norm weight, every GEMV output, the rotated q/k, the attention
    output, each residual add, silu(gate) and its product with up, the logits).  Neither the reference's CPU
    accumulation order nor the kernel's enters: what is left is the arithmetic both approximate.  (fp64 -> bf16 goes
    through fp32; the double rounding can only matter within 2^-29 of a bf16 midpoint.)"""

    def __init__(self, g, shape):
        self.s = shape
        f64 = lambda t: t.to(torch.float64)
        self.w = {n: f64(getattr(g, n)) for n in ("attn_norm_weights", "qkv_weights", "o_proj_weights", "mlp_norm_weights", "up_proj_weights",
                                                   "gate_proj_weights", "down_proj_weights", "lm_head_norm_weights", "lm_head_weights")}
        self.embed, self.cos, self.sin = g.embed_tokens, f64(g.rope_cos), f64(g.rope_sin)
        L, S = shape.num_hidden_layers, g.k_cache.shape[2]
        self.k = torch.zeros(L, S, shape.num_key_value_heads, shape.head_dim, dtype=torch.float64, device=g.k_cache.device)
        self.v = torch.zeros_like(self.k)

    @staticmethod
    def r(x):   # one bf16 rounding, value kept in fp64
        return x.to(torch.float32).to(torch.bfloat16).to(torch.float64)

    def norm(self, x, w):
        return self.r(w * self.r(x * torch.rsqrt(x.pow(2).mean() + self.s.rms_norm_eps)))

    def rope(self, x, pos):   # pairs are neighbours: (x0, x1) -> (x0 c0 - x1 s0, x1 c1 + x0 s1)
        rot = torch.stack((-x[..., 1::2], x[..., 0::2]), dim=-1).reshape(x.shape)
        return self.r(x * self.cos[pos] + rot * self.sin[pos])

    def step(self, token: int, pos: int):
        s, w, r = self.s, self.w, self.r
        nq, nkv, d = s.num_attention_heads, s.num_key_value_heads, s.head_dim
        h = self.embed[token].to(torch.float64)
        for l in range(s.num_hidden_layers):
            qkv = r(w["qkv_weights"][l] @ self.norm(h, w["attn_norm_weights"][l]))
            q = self.rope(qkv[: nq * d].view(nq, d), pos)
            self.k[l, pos] = self.rope(qkv[nq * d : (nq + nkv) * d].view(nkv, d), pos)
            self.v[l, pos] = qkv[(nq + nkv) * d :].view(nkv, d)
            k = self.k[l, : pos + 1].repeat_interleave(nq // nkv, dim=1)             # [n, nq, d]
            v = self.v[l, : pos + 1].repeat_interleave(nq // nkv, dim=1)
            p = torch.softmax(torch.einsum("hi,shi->hs", q, k) / d ** 0.5, dim=-1)
            attn = r(torch.einsum("hs,sho->ho", p, v)).reshape(-1)
            h = r(h + r(w["o_proj_weights"][l] @ attn))
            y = self.norm(h, w["mlp_norm_weights"][l])
            gate, up = r(w["gate_proj_weights"][l] @ y), r(w["up_proj_weights"][l] @ y)
            act = r(r(gate * torch.sigmoid(gate)) * up)
            h = r(h + r(w["down_proj_weights"][l] @ act))
        return h, r(w["lm_head_weights"] @ self.norm(h, w["lm_head_norm_weights"]))


def test_kernel_against_exact_sums_beside_the_reference(golden, model):
    """Teacher-forced on the golden tokens, three evaluations of every step: the reference's (the fixture's top-8
    logits, CPU bf16 GEMVs), the kernel's, and exact sums rounded where the reference rounds.  The kernel must sit
    no farther from the exact evaluation than the reference itself does — in bf16 ulps of the step's top logit,
    maximum and mean over all 1024 steps x 8 logits — and so must the final residual stream at the recorded steps."""
    meta, arrays = golden
    shape, g, prompt = model
    LlamaConfig.set_shape(shape)
    mk = mk_kernel.get_mk()
    S.build(g)
    tokens = meta["tokens"]
    seq = prompt.tolist() + tokens
    n_prompt, n_new = len(prompt), len(tokens)
    exact = ExactEvaluator(g, shape)
    topk_ids = torch.from_numpy(arrays["topk_ids"].astype(np.int64)).cuda()
    kernel_topk = torch.zeros(n_new, 8, dtype=torch.float64, device="cuda")
    exact_topk = torch.zeros_like(kernel_topk)
    picks = torch.zeros(2, n_new, dtype=torch.long, device="cuda")          # kernel's, exact evaluation's
    record = {0: "step0", 1: "step1", 127: "step127", 511: "step511"}
    hidden = {}
    ids = torch.tensor(seq, device="cuda")
    with torch.no_grad():
        for pos in range(n_prompt + n_new - 1):
            g.hidden_states.copy_(g.embed_tokens[ids[pos]])
            g.position_id = pos
            mk_kernel.call_mk(g, mk)
            h, logits = exact.step(seq[pos], pos)
            i = pos - (n_prompt - 1)
            if i >= 0:
                kernel_topk[i] = g.logits[topk_ids[i]].double()
                exact_topk[i] = logits[topk_ids[i]]
                picks[0, i], picks[1, i] = g.logits.argmax(), logits.argmax()
                if i - 1 in record:
                    hidden[record[i - 1]] = (g.hidden_states.double().clone(), h.clone())
    mk.check()
    ref_topk = _bf16(arrays["topk_bits"]).double()
    ulp = torch.exp2(torch.floor(torch.log2(ref_topk[:, :1].abs())) - 7)
    err_kernel = ((kernel_topk.cpu() - exact_topk.cpu()).abs() / ulp)
    err_ref = ((ref_topk - exact_topk.cpu()).abs() / ulp)
    err_kr = ((kernel_topk.cpu() - ref_topk).abs() / ulp)
    q = lambda e: f"max {float(e.max()):.2f}, 99.9 % {float(e.flatten().quantile(0.999)):.2f}, mean {float(e.mean()):.3f}"
    print(f"top-8 logits in ulps of the step's top logit: kernel vs exact sums {q(err_kernel)}; reference vs exact sums {q(err_ref)}; "
          f"kernel vs reference {q(err_kr)}")
    want = torch.tensor(tokens)
    kernel_pick, exact_pick = picks[0].cpu(), picks[1].cpu()
    agree = lambda a, b: float((a == b).float().mean())
    print(f"top-1 agreement over {n_new} steps: kernel/exact {agree(kernel_pick, exact_pick):.4f}, reference/exact {agree(want, exact_pick):.4f}, "
          f"kernel/reference {agree(kernel_pick, want):.4f}")
    rel = {}
    for name, (got, exact_h) in hidden.items():
        ref_h = _bf16(arrays[f"final_hidden_{name}"]).double().cuda()
        big = exact_h.abs() > 0.05
        rms = lambda t: float(t.pow(2).mean().sqrt())
        rel[name] = (float(((got - exact_h).abs() / exact_h.abs())[big].max()), float(((ref_h - exact_h).abs() / exact_h.abs())[big].max()),
                     float((got - exact_h).abs().max() / exact_h.abs().max()), float((ref_h - exact_h).abs().max() / exact_h.abs().max()),
                     rms(got - exact_h) / rms(exact_h), rms(ref_h - exact_h) / rms(exact_h))
        print(f"{name}: final hidden vs exact sums, elementwise rel err where |exact| > 0.05: kernel {rel[name][0]:.4f}, reference {rel[name][1]:.4f}; "
              f"max|diff| / max|exact|: kernel {rel[name][2]:.4f}, reference {rel[name][3]:.4f}; rms(diff) / rms(exact): kernel {rel[name][4]:.5f}, "
              f"reference {rel[name][5]:.5f}")
    # The mean is a statistic of 8192 logits; the maximum and the 99.9 % point are single elements on a grid of half ulps.
    assert float(err_kernel.mean()) <= 1.02 * float(err_ref.mean())
    assert float(err_kernel.flatten().quantile(0.999)) <= float(err_ref.flatten().quantile(0.999)) + 0.5
    assert float(err_kernel.max()) <= float(err_ref.max()) + 1.0
    assert agree(kernel_pick, exact_pick) >= agree(want, exact_pick) - 0.01
    for name, (k_rel, r_rel, k_max, r_max, k_rms, r_rms) in rel.items():
        assert k_rms <= 1.25 * r_rms, name
        assert k_max <= 1.5 * r_max, name      # one element of 2048
    assert sum(v[4] for v in rel.values()) <= 1.05 * sum(v[5] for v in rel.values())


def test_per_layer_hidden_first_decode_step(golden, model):
    """Residual stream after every layer at decode step 0 (position 8) vs the reference's samples."""
    meta, arrays = golden
    shape, g, prompt = model
    LlamaConfig.set_shape(shape)
    mk = mk_kernel.get_mk()
    out = decode.decode(g, prompt, 2, mk=mk, decode_time=False)     # fills the KV cache for positions 0..8
    assert int(out["new_tokens"][0, 0]) == meta["tokens"][0]
    sched = S.scheduler_for(g)
    pos = len(prompt)
    start = g.embed_tokens[meta["tokens"][0]].clone()
    want = _bf16(arrays["hidden_samples_step0"])                    # [16 layers, 64 samples]
    for nl in range(1, shape.num_hidden_layers + 1):
        g.hidden_states.copy_(start)
        g.position_id = pos
        g.barriers.zero_()
        mk_kernel.run_instructions(g, sched.instruction_list(nl), mk=mk)
        # 2e-2 of the largest element while the stream is shallow; deeper in, the gate of the final
        # residual stream (1.5x the distance of a second CPU evaluation of the reference) applies
        e = tensor_rel_close(g.hidden_states[:: meta["sample_stride"]], want[nl - 1], rel=1e-2 if nl <= 4 else 2.5e-2,
                             name=f"hidden after layer {nl - 1}")
        print(f"layer {nl - 1}: max|diff| / max|ref| over the samples {e:.4f}")
        assert int(g.hidden_states.view(torch.int16).to(torch.int64).bitwise_and(0xFFFF).sum()) > 0
    g.barriers.zero_()
    g.instructions = None
    mk.check()


def test_free_running_divergence_only_at_near_ties(golden, model):
    meta, arrays = golden
    shape, g, prompt = model
    LlamaConfig.set_shape(shape)
    out = decode.decode(g, prompt, 256, decode_time=False)
    got = out["new_tokens"][0].tolist()
    want = meta["tokens"][:256]
    first = next((i for i in range(256) if got[i] != want[i]), 256)
    print(f"free-running greedy: identical prefix {first} of 256 tokens")
    want_topk = _bf16(arrays["topk_bits"])
    ulp = torch.exp2(torch.floor(torch.log2(want_topk[:256, 0].abs())) - 7)
    margin_ulps = torch.tensor(meta["margins"][:256]) / ulp
    if first < 256:
        # Free-running trajectories of two evaluations can only be compared up to the first step the reference itself
        # decides by less than its arithmetic noise: they must part at such a step (here: within 2 ulps of a tie;
        # teacher-forced, the kernel differs at larger margins on 5 of 1024 steps), never at a clear one.
        assert float(margin_ulps[first]) <= 2.0, f"the trajectories part at step {first}, margin {float(margin_ulps[first])} ulps"
    first_near_tie = next(i for i in range(256) if float(margin_ulps[i]) <= 2.0)
    assert first >= first_near_tie
