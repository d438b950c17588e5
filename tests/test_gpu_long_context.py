"""Split-KV attention stress (BASELINE config 3): one decode step over a KV cache of 4096 / 16384 / 32768
tokens, GQA 32:8, head_dim 64, K/V ~ N(0,1) in bf16.  Validates the split + log-sum-exp merge against
brute-force softmax attention and reports the attention-phase HBM rate."""
import dataclasses
import math

import pytest
import torch

from gpu_helpers import bf16_close
from qimeng_megakernel_amd import synthetic
from qimeng_megakernel_amd.decode_schedule import mk_kernel
from qimeng_megakernel_amd.decode_schedule.instructions import scheduler as S
from qimeng_megakernel_amd.decode_schedule.model_config import LLAMA_3_2_1B, LlamaConfig

pytestmark = pytest.mark.gpu


def _reference_attention(q, k, v, n_kv):
    """fp32 softmax attention on the GPU with the library routines (not the kernel under test)."""
    nq, d = q.shape
    ratio = nq // n_kv
    k = k.float().repeat_interleave(ratio, dim=1)            # [n, nq, d]
    v = v.float().repeat_interleave(ratio, dim=1)
    s = torch.einsum("hd,nhd->hn", q.float(), k) / math.sqrt(d)
    p = torch.softmax(s.double(), dim=-1)
    return torch.einsum("hn,nhd->hd", p, v.double()).float()


@pytest.mark.parametrize("context", [4096, 16384, 32768])
@pytest.mark.parametrize("merge", ["last", "separate"])
def test_long_context_attention(context, merge):
    shape = dataclasses.replace(LLAMA_3_2_1B, num_hidden_layers=1, vocab_size=256)
    LlamaConfig.set_shape(shape)
    w = synthetic.random_weights(shape, seed=5, max_positions=context)
    g = synthetic.build_globals(w, shape, context, "cuda:0", max_partials=32)
    gen = torch.Generator(device="cuda").manual_seed(context)
    g.k_cache.copy_(torch.randn(g.k_cache.shape, generator=gen, device="cuda").bfloat16())
    g.v_cache.copy_(torch.randn(g.v_cache.shape, generator=gen, device="cuda").bfloat16())
    g.q_post_rope.copy_((torch.randn(shape.hidden_size, generator=gen, device="cuda") * 0.4).bfloat16())
    g.position_id = context - 1
    sched = S.mi355x_scheduler(shape, kv_capacity=context, attention_merge=merge)
    assert sched.num_partials == min(25, -(-context // S.KV_TOKENS_PER_PASS))
    g.barriers[0, 0, :] = sched.expected_counts()[0]
    ins = sched.attention_split_kv(0) + sched.attention_reduction(0)
    mk = mk_kernel.get_mk(reset_barriers=False)
    mk_kernel.run_instructions(g, ins, mk=mk)                 # warm-up and correctness run
    mk.check()
    want = _reference_attention(g.q_post_rope.view(32, 64), g.k_cache[0, 0], g.v_cache[0, 0], 8)
    # attn_out = bf16 of an fp32 online-softmax sum over up to 32768 terms: 1 ulp of the rounding plus accumulation noise
    bf16_close(g.attn_out, want.bfloat16().reshape(-1), ulps=1.0, frac=0.05, name="attn_out")
    assert (g.attn_out.float() - want.reshape(-1)).abs().max() <= 2 ** -8 * max(1.0, float(want.abs().max()))
    # partial LSEs recombine to the full log-partition function (log2 domain); a partial is empty
    # (-inf, ignored by the merge) exactly when its first 16-token block lies beyond the context
    lse = g.attn_lse_intermediates[:, : sched.num_partials]
    blocks = -(-context // 16)
    per = -(-blocks // sched.num_partials)
    nonempty = torch.tensor([p * per < blocks for p in range(sched.num_partials)], device="cuda")
    assert torch.equal(torch.isfinite(lse), nonempty.expand_as(lse))
    k = g.k_cache[0, 0].float().repeat_interleave(4, dim=1)
    full = torch.logsumexp((torch.einsum("hd,nhd->hn", g.q_post_rope.view(32, 64).float(), k) / 8.0).double(), dim=-1) / math.log(2)
    merged = torch.log2(torch.exp2(lse.double() - lse.double().max(dim=1, keepdim=True).values).sum(dim=1)) + lse.double().max(dim=1).values
    assert (merged - full).abs().max() < 1e-3
    assert int(g.barriers[0, 2, 0]) == 32 and (g.barriers[0, 1, :32] == sched.num_partials).all()

    # attention-phase rate: K and V rows of the whole context, once
    reps = 20
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    total = 0.0
    for _ in range(reps):
        g.barriers.zero_(); g.barriers[0, 0, :] = sched.expected_counts()[0]
        start.record(); mk_kernel.call_mk(g, mk); stop.record()
        torch.cuda.synchronize()
        total += start.elapsed_time(stop)
    mk.check()
    nbytes = context * 8 * 64 * 2 * 2
    print(f"\ncontext {context} merge={merge}: {total / reps * 1e3:.1f} us per attention phase, "
          f"{nbytes / (total / reps * 1e-3) / 1e9:.0f} GB/s of K/V")


@pytest.mark.parametrize("context", [4096, 16384, 32768])
def test_long_context_default_path_through_the_oproj(context):
    """The path a request takes by default (and `bench.py --attention-stress` times): the fan-out
    ``scheduler_for`` picks for this cache, no merging instruction, every O-proj workgroup merging
    the partials of all heads itself.  Checked where that path ends — the residual stream after the
    O-proj — against fp64 attention -> bf16 -> fp64 O-proj GEMV -> bf16 -> residual add, and on the
    ``attn_out`` copy that the first O-proj workgroup leaves in memory."""
    shape = dataclasses.replace(LLAMA_3_2_1B, num_hidden_layers=1, vocab_size=256)
    LlamaConfig.set_shape(shape)
    w = synthetic.random_weights(shape, seed=6, max_positions=context)
    g = synthetic.build_globals(w, shape, context, "cuda:0", max_partials=32)
    gen = torch.Generator(device="cuda").manual_seed(context + 1)
    g.k_cache.copy_(torch.randn(g.k_cache.shape, generator=gen, device="cuda").bfloat16())
    g.v_cache.copy_(torch.randn(g.v_cache.shape, generator=gen, device="cuda").bfloat16())
    g.q_post_rope.copy_((torch.randn(shape.hidden_size, generator=gen, device="cuda") * 0.4).bfloat16())
    hidden0 = (torch.randn(shape.hidden_size, generator=gen, device="cuda") * 0.7).bfloat16()
    g.hidden_states.copy_(hidden0)
    g.position_id = context - 1
    sched = S.scheduler_for(g)
    assert sched.attention_merge == "oproj" and sched.oproj_spares_attention
    assert sched.num_partials == min(32, -(-context // S.KV_TOKENS_PER_PASS))      # 13, 32, 32
    g.barriers[0, 0, :] = sched.expected_counts()[0]
    ins = sched.attention_split_kv(0) + sched.attention_reduction(0) + sched.oproj(0, (8 * sched.num_partials) % sched.sm_count)
    assert not sched.attention_reduction(0)
    for xcd in (False, True):   # the reference's counter rows, then the per-XCD sub-counters of the default launch
        g.hidden_states.copy_(hidden0); g.attn_out.zero_(); g.barriers.zero_(); g.barriers[0, 0, :] = sched.expected_counts()[0]
        mk = mk_kernel.get_mk(geometry=sched.geometry, reset_barriers=False, xcd_counters=xcd)
        mk_kernel.run_instructions(g, ins, mk=mk, sm_count=sched.sm_count)
        mk.check()
        attn = _reference_attention(g.q_post_rope.view(32, 64), g.k_cache[0, 0], g.v_cache[0, 0], 8)
        bf16_close(g.attn_out, attn.bfloat16().reshape(-1), ulps=1.0, frac=0.05, name="attn_out")
        proj = (g.o_proj_weights[0].double() @ attn.bfloat16().reshape(-1).double()).float().bfloat16()
        want = (hidden0.float() + proj.float()).bfloat16()
        # a differently rounded attn_out element moves a 2048-term dot product by far less than an ulp of the sum
        bf16_close(g.hidden_states, want, ulps=1.0, frac=0.03, floor=1.0, name="hidden_states")
        assert (g.hidden_states.float() - want.float()).abs().max() <= 2.0 ** -7 * max(1.0, float(want.float().abs().max()))
