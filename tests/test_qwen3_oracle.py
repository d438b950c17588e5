"""The Qwen3 op set on the CPU: per-head QK RMSNorm, raw-QKV instruction split, schedule, fixture.

Reference: qimeng_megakernel/models/LLM/qwen/qwen3__0_6b/A100/single_batch/decode_schedule/
(fused/operations.py:52-215, instructions/python_vm.py:110-320).  The golden fixture was written by
tests/golden/make_fixtures_qwen3.py from the imported reference after a bit-for-bit lock-step with
this repository's oracle.
"""
import dataclasses
import json
from pathlib import Path

import pytest
import torch

from fused_oracle import FusedOracle, per_head_rms_norm, rotate_pairs
from pyvm_oracle import Counts, InstructionVM
from qimeng_megakernel_amd import synthetic
from qimeng_megakernel_amd.decode_schedule import mk_kernel
from qimeng_megakernel_amd.decode_schedule.instructions import scheduler as S
from qimeng_megakernel_amd.decode_schedule.model_config import LLAMA_3_2_1B, QWEN3_1_7B, LlamaConfig

GOLDEN = Path(__file__).parent / "golden" / "qwen3_reduced_seed0.json"


@pytest.fixture(autouse=True)
def _restore_shape():
    yield
    LlamaConfig.set_shape(LLAMA_3_2_1B)


def test_per_head_rms_norm_is_fp32_with_one_rounding():
    gen = torch.Generator().manual_seed(4)
    x = (torch.randn(24, 128, generator=gen) * 3).bfloat16()
    w = (1 + 0.1 * torch.randn(128, generator=gen)).bfloat16()
    got = per_head_rms_norm(x, w, 1e-6)
    xd, wd = x.double(), w.double()
    exact = wd * xd / torch.sqrt(xd.pow(2).mean(-1, keepdim=True) + 1e-6)
    # one bf16 rounding of the exact value: at most half an ulp away, up to fp32 noise at rounding boundaries
    ulp = torch.exp2(torch.floor(torch.log2(exact.abs().clamp_min(1e-30))) - 7)
    assert ((got.double() - exact).abs() <= 0.5 * ulp * (1 + 1e-4)).all()
    # the two-rounding form (round, then multiply by the weight) differs on a visible share of the elements
    two = (w * (x.float() * torch.rsqrt(x.float().pow(2).mean(-1, keepdim=True) + 1e-6)).bfloat16())
    assert (two != got).float().mean() > 0.02
    # scale invariance up to eps and exactness for a constant vector
    assert torch.equal(per_head_rms_norm(torch.full((1, 128), 2.0).bfloat16(), torch.ones(128).bfloat16(), 0.0), torch.ones(1, 128).bfloat16())


def test_interleaved_norm_and_rope_equal_the_checkpoint_order():
    """q_norm + rotate-half RoPE on the checkpoint's column order == the same on pair-interleaved columns,
    when weights, norm weights and tables are permuted alike (llama/preprocess.py:21-83 applied to Qwen3)."""
    d = 128
    shape = dataclasses.replace(QWEN3_1_7B, num_hidden_layers=1)
    cos_i, sin_i = synthetic.rope_tables(shape, 8)
    idx = synthetic.interleave_indices(d)
    gen = torch.Generator().manual_seed(9)
    q = torch.randn(16, d, generator=gen).bfloat16()
    w = (1 + 0.1 * torch.randn(d, generator=gen)).bfloat16()
    pos = 5
    inv = 1.0 / (shape.rope_theta ** (torch.arange(0, d, 2).float() / d))
    ang = torch.cat((pos * inv, pos * inv))
    qn = per_head_rms_norm(q, w, 1e-6)
    rot_half = torch.cat((-qn[:, d // 2:], qn[:, : d // 2]), dim=-1)
    want = (qn * ang.cos() + rot_half * ang.sin()).bfloat16()
    qi = per_head_rms_norm(q[:, idx], w[idx], 1e-6)
    got = (qi * cos_i[pos] + rotate_pairs(qi) * sin_i[pos]).bfloat16()
    assert torch.equal(got, want[:, idx])


def _reduced(layers=2, vocab=2048):
    shape = dataclasses.replace(QWEN3_1_7B, num_hidden_layers=layers, vocab_size=vocab)
    LlamaConfig.set_shape(shape)
    return shape


def test_schedule_for_the_qwen3_shape():
    shape = _reduced()
    sched = S.mi355x_scheduler(shape, num_partials=3)
    assert sched.geometry.upgate_tile_n == 8 and sched.geometry.split_k == 6144
    assert sched.expected_counts() == (32, 256, 768, 256)
    per_queue = [sum(len(i.tile_N_block_idxs) for i in q if i.opcode() == 5 and i.layer_idx == 0) for q in sched.queues()]
    assert set(per_queue) == {3}                       # 768 up/gate blocks: three for every workgroup
    qkv = [i for i in sched.qkvproj(0)]
    assert len(qkv) == 256 and all(i.tile_N_end_idx - i.tile_N_start_idx == 4 for i in qkv)
    assert mk_kernel._model_id(shape) == mk_kernel.QMK_MODEL_QWEN3_1_7B
    assert mk_kernel._model_id(LLAMA_3_2_1B) == mk_kernel.QMK_MODEL_LLAMA_3_2_1B
    with pytest.raises(ValueError, match="no kernel was compiled"):
        mk_kernel._model_id(dataclasses.replace(shape, head_dim=96))
    tied = synthetic.build_globals(synthetic.random_weights(shape, 1, 8), shape, 8, "cpu")
    assert tied.lm_head_weights is tied.embed_tokens and tied.qkv_raw.shape == (4096,)


def test_instruction_vm_agrees_with_the_fused_route():
    shape = _reduced()
    w = synthetic.random_weights(shape, 3, 16)
    a, b = (synthetic.build_globals(w, shape, 16, "cpu", max_partials=4) for _ in range(2))
    sched = S.mi355x_scheduler(shape, num_partials=4, attention_merge="separate")
    oracle, vm = FusedOracle(shape), InstructionVM(shape, Counts(*sched.expected_counts()))
    tok = 5
    for pos in range(3):
        for g in (a, b):
            oracle.embed(g, tok); g.position_id = pos
        oracle.decode_step(a)
        b.barriers.zero_()
        vm.run(b, sched.instruction_list())
        assert torch.equal(a.qkv_raw, b.qkv_raw) and torch.equal(a.q_post_rope, b.q_post_rope)
        assert torch.equal(a.k_cache, b.k_cache) and torch.equal(a.v_cache, b.v_cache)
        # four partials in both, but scored head by head there and per GQA group here: fp32 noise only
        diff = (a.attn_out.float() - b.attn_out.float()).abs()
        assert float(diff.max()) <= 2.0 ** -7 * float(a.attn_out.float().abs().max()) and float((diff > 0).float().mean()) < 0.02
        assert float((a.logits.float() - b.logits.float()).abs().max()) <= 2e-2 * float(a.logits.float().abs().max())
        tok = int(a.logits.argmax())


def test_oracle_reproduces_the_reference_trajectory():
    fix = json.loads(GOLDEN.read_text())
    shape = dataclasses.replace(QWEN3_1_7B, **{k: v for k, v in fix["shape"].items()})
    LlamaConfig.set_shape(shape)
    steps = fix["steps"]
    w = synthetic.random_weights(shape, fix["seed"], steps + 1)
    g = synthetic.build_globals(w, shape, steps + 1, "cpu", max_partials=fix["max_partials"])
    oracle = FusedOracle(shape)
    tok = fix["first_token"]
    for pos in range(steps):
        oracle.embed(g, tok); g.position_id = pos
        oracle.decode_step(g)
        ids = torch.tensor(fix["top4_ids"][pos])
        assert g.logits[ids].view(torch.int16).tolist() == fix["top4_bf16_bits"][pos], pos
        tok = int(g.logits.argmax())
        assert tok == fix["tokens"][pos], pos
    assert g.hidden_states.view(torch.int16)[::16].tolist() == fix["final_hidden_bf16_bits"]
