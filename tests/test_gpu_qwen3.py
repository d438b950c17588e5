"""The Qwen3 op set on the GPU (Qwen3-1.7B layer geometry, reduced depth and vocabulary).

Reference: qimeng_megakernel/models/LLM/qwen/qwen3__0_6b/A100/single_batch/ — opcode 1 leaves the raw
QKV vector (decode_kernel/rms_qkvproj_gemv.cu; python_vm.py:110-141), the split-KV attention
instruction applies the per-head RMSNorm of q and k and RoPE and writes the cache row
(python_vm.py:214-320).  Same gates as for the Llama shape (tests/test_gpu_decode.py).
"""
import dataclasses
import json
from pathlib import Path

import pytest
import torch

from fused_oracle import FusedOracle
from gpu_helpers import bf16_close, rel_close, run_both, sync_state, tensor_rel_close
from qimeng_megakernel_amd import decode, synthetic
from qimeng_megakernel_amd.decode_schedule import mk_kernel
from qimeng_megakernel_amd.decode_schedule.instructions import scheduler as S
from qimeng_megakernel_amd.decode_schedule.model_config import LLAMA_3_2_1B, QWEN3_1_7B, LlamaConfig

pytestmark = pytest.mark.gpu
GOLDEN = Path(__file__).parent / "golden" / "qwen3_reduced_seed0.json"
TRAJECTORY_REL = 4e-2


@pytest.fixture(autouse=True)
def _restore_shape():
    yield
    LlamaConfig.set_shape(LLAMA_3_2_1B)


@pytest.fixture(scope="module")
def qwen():
    shape = dataclasses.replace(QWEN3_1_7B, num_hidden_layers=2, vocab_size=2048)
    return shape, synthetic.random_weights(shape, 3, 96)


def _margin_ulps(logits):
    top = torch.topk(logits.float().cpu(), 2).values
    return float((top[0] - top[1]) / 2.0 ** (torch.floor(torch.log2(top[0].abs())) - 7))


def test_ops_raw_qkv_then_attention_prologue(qwen):
    """Opcode 1 and the split-KV instructions against the sequential VM, counters word for word."""
    shape, w = qwen
    LlamaConfig.set_shape(shape)
    cpu = synthetic.build_globals(w, shape, 96, "cpu")
    gpu = synthetic.build_globals(w, shape, 96, "cuda:0")
    gen = torch.Generator().manual_seed(2)
    cpu.hidden_states.copy_((torch.randn(shape.hidden_size, generator=gen) * 0.7).bfloat16())
    cpu.k_cache.copy_(torch.randn(cpu.k_cache.shape, generator=gen).bfloat16())
    cpu.v_cache.copy_(torch.randn(cpu.v_cache.shape, generator=gen).bfloat16())
    for pos, P in ((0, 1), (41, 3), (80, 13)):
        sched = S.mi355x_scheduler(shape, num_partials=P, attention_merge="separate")
        cpu.position_id = pos
        cpu.barriers.zero_()
        sync_state(cpu, gpu)
        run_both(cpu, gpu, sched, sched.qkvproj(0) + sched.attention_split_kv(0) + sched.attention_reduction(0))
        bf16_close(gpu.qkv_raw, cpu.qkv_raw, name="qkv_raw")
        # norm and RoPE amplify a 1-ulp difference of the raw vector to at most one more ulp
        bf16_close(gpu.q_post_rope, cpu.q_post_rope, ulps=2.0, frac=0.03, name="q_post_rope")
        bf16_close(gpu.k_cache[0, 0, pos], cpu.k_cache[0, 0, pos], ulps=2.0, frac=0.03, name="k row")
        bf16_close(gpu.v_cache[0, 0, pos], cpu.v_cache[0, 0, pos], name="v row")
        assert torch.equal(gpu.k_cache[0, 0, :pos].cpu(), cpu.k_cache[0, 0, :pos])
        assert torch.equal(gpu.k_cache[0, 0, pos + 1:].cpu(), cpu.k_cache[0, 0, pos + 1:])
        rel_close(gpu.attn_out, cpu.attn_out, rel=2e-2, name="attn_out")
        assert torch.equal(gpu.barriers.cpu(), cpu.barriers)


def test_teacher_forced_decode_matches_the_oracle(qwen):
    shape, w = qwen
    LlamaConfig.set_shape(shape)
    cpu = synthetic.build_globals(w, shape, 96, "cpu", max_partials=4)
    gpu = synthetic.build_globals(w, shape, 96, "cuda:0", max_partials=4)
    oracle, mk = FusedOracle(shape), mk_kernel.get_mk()
    tok, agree, steps = 5, 0, 50
    for pos in range(steps):
        for g in (cpu, gpu):
            g.hidden_states.copy_(g.embed_tokens[tok]); g.position_id = pos
        oracle.decode_step(cpu)
        mk_kernel.call_mk(gpu, mk)
        want, got = int(cpu.logits.argmax()), int(gpu.logits.argmax())
        if got == want:
            agree += 1
        else:
            assert _margin_ulps(cpu.logits) <= 2.0, f"step {pos}: kernel {got} vs oracle {want} at a clear margin"
        rel_close(gpu.logits, cpu.logits, rel=TRAJECTORY_REL, name=f"logits@{pos}")
        tok = want
    mk.check()
    assert mk._tagged and agree >= 0.85 * steps
    rel_close(gpu.hidden_states, cpu.hidden_states, rel=TRAJECTORY_REL, name="hidden")
    rel_close(gpu.k_cache[:, 0, :steps], cpu.k_cache[:, 0, :steps], rel=TRAJECTORY_REL, name="k_cache")
    rel_close(gpu.q_post_rope, cpu.q_post_rope, rel=TRAJECTORY_REL, name="q_post_rope")
    assert int(gpu.barriers.abs().sum()) == 0


def test_reference_trajectory_teacher_forced():
    """The fixture written from the imported reference: at every step the kernel's top-1 is the
    reference's wherever the reference's own margin exceeds the accumulation-order noise, and the
    reference's top-4 logits are reproduced within 8 bf16 ulps."""
    fix = json.loads(GOLDEN.read_text())
    shape = dataclasses.replace(QWEN3_1_7B, **fix["shape"])
    LlamaConfig.set_shape(shape)
    steps = fix["steps"]
    w = synthetic.random_weights(shape, fix["seed"], steps + 1)
    g = synthetic.build_globals(w, shape, steps + 1, "cuda:0")
    mk = mk_kernel.get_mk()
    tok, agree = fix["first_token"], 0
    for pos in range(steps):
        g.hidden_states.copy_(g.embed_tokens[tok]); g.position_id = pos
        mk_kernel.call_mk(g, mk)
        ids = torch.tensor(fix["top4_ids"][pos], device="cuda:0")
        ref = torch.tensor(fix["top4_bf16_bits"][pos], dtype=torch.int16).view(torch.bfloat16).float()
        got = g.logits[ids].float().cpu()
        ulp = 2.0 ** (torch.floor(torch.log2(ref.abs().clamp_min(2.0 ** -6))) - 7)
        assert float(((got - ref).abs() / ulp).max()) <= 8.0, pos
        mine = int(g.logits.argmax())
        if mine == fix["tokens"][pos]:
            agree += 1
        else:
            assert float((ref[0] - ref[1]) / ulp[0]) <= 8.0, f"step {pos}: different pick at a clear margin"
        tok = fix["tokens"][pos]
    mk.check()
    assert agree >= 0.9 * steps


def test_tagged_and_counter_modes_agree_bit_for_bit(qwen):
    shape, w = qwen
    LlamaConfig.set_shape(shape)
    out = []
    for tagged in (False, True):
        g = synthetic.build_globals(w, shape, 64, "cuda:0")
        mk = mk_kernel.get_mk(tagged=tagged)
        tok = 7
        for pos in range(20):
            g.hidden_states.copy_(g.embed_tokens[tok]); g.position_id = pos
            mk_kernel.call_mk(g, mk)
            tok = int(g.logits.argmax())
        mk.check()
        out.append(g)
    for name in ("hidden_states", "qkv_raw", "q_post_rope", "attn_out", "silu_out", "logits", "k_cache", "v_cache"):
        assert torch.equal(getattr(out[0], name), getattr(out[1], name)), name


def test_device_sampling_with_the_tied_head(qwen):
    shape, w = qwen
    LlamaConfig.set_shape(shape)
    prompt = torch.tensor([3, 99, 1024, 7])
    runs = []
    for kw in ({}, {"device_sampling": True}):
        g = synthetic.build_globals(w, shape, 64, "cuda:0")
        assert g.lm_head_weights.data_ptr() == g.embed_tokens.data_ptr()
        runs.append(decode.decode(g, prompt, 24, **kw)["new_tokens"].clone())
    assert torch.equal(runs[0], runs[1])


@pytest.mark.slow
def test_full_size_model_layer_by_layer():
    """BASELINE config 4's model as it is benchmarked — 28 layers, FFN 6144, the tied 151 936-row head — layer
    by layer from the oracle's residual stream (one layer's rounding differences are not amplified by the
    next): hidden states within the bf16 gate (max rel err 2e-2) after every layer, the appended K/V rows,
    logits within the gate after the LM head, and the oracle's greedy pick wherever it has a clear winner."""
    shape = QWEN3_1_7B
    LlamaConfig.set_shape(shape)
    capacity, pos = 96, 70
    w = synthetic.random_weights(shape, 4, capacity)
    cpu = synthetic.build_globals(w, shape, capacity, "cpu")
    gpu = synthetic.build_globals(w, shape, capacity, "cuda:0")
    assert gpu.lm_head_weights.data_ptr() == gpu.embed_tokens.data_ptr() and gpu.logits.numel() == 151936
    gen = torch.Generator().manual_seed(8)
    cpu.k_cache[:, :, :pos].copy_(torch.randn(cpu.k_cache[:, :, :pos].shape, generator=gen).bfloat16())
    cpu.v_cache[:, :, :pos].copy_(torch.randn(cpu.v_cache[:, :, :pos].shape, generator=gen).bfloat16())
    cpu.hidden_states.copy_(cpu.embed_tokens[4242])
    cpu.position_id = pos
    sync_state(cpu, gpu)
    oracle = FusedOracle(shape)
    sched = S.scheduler_for(gpu)
    assert sched.sm_count == 256
    mk = mk_kernel.get_mk(geometry=sched.geometry, reset_barriers=False, xcd_counters=False)
    done = sched.expected_counts()[3]
    for layer in range(shape.num_hidden_layers):
        gpu.hidden_states.copy_(cpu.hidden_states)
        oracle.decode_layer(cpu, layer)
        gpu.barriers.zero_()
        if layer:
            gpu.barriers[layer - 1, 5, 0] = done
        mk_kernel.run_instructions(gpu, sched.layer(layer), mk=mk, sm_count=sched.sm_count)
        mk.check()
        rel_close(gpu.hidden_states, cpu.hidden_states, name=f"hidden_states after layer {layer}")
        rel_close(gpu.k_cache[layer, 0, pos], cpu.k_cache[layer, 0, pos], name=f"k row of layer {layer}")
        bf16_close(gpu.v_cache[layer, 0, pos], cpu.v_cache[layer, 0, pos], frac=0.05, name=f"v row of layer {layer}")
    gpu.hidden_states.copy_(cpu.hidden_states)
    oracle.lm_head(cpu)
    gpu.barriers.zero_()
    gpu.barriers[shape.num_hidden_layers - 1, 5, 0] = done
    mk_kernel.run_instructions(gpu, sched.lmhead(), mk=mk, sm_count=sched.sm_count)
    mk.check()
    rel_close(gpu.logits, cpu.logits, name="logits")
    if _margin_ulps(cpu.logits) > 2.0:
        assert int(gpu.logits.argmax()) == int(cpu.logits.argmax())
    # the same step free-running through call_mk (tagged units, self-clearing counters): 28 layers deep
    cpu2 = synthetic.build_globals(w, shape, capacity, "cpu")
    cpu2.k_cache.copy_(cpu.k_cache); cpu2.v_cache.copy_(cpu.v_cache)
    cpu2.hidden_states.copy_(cpu2.embed_tokens[4242]); cpu2.position_id = pos
    sync_state(cpu2, gpu)
    gpu.barriers.zero_()
    gpu.instructions = None
    oracle.decode_step(cpu2)
    free = mk_kernel.get_mk()
    mk_kernel.call_mk(gpu, free)
    free.check()
    assert free._tagged
    # 28 layers of rounding differences deep, so the gate is on the tensor's scale (as for the Llama shape)
    err = tensor_rel_close(gpu.logits, cpu2.logits, rel=5e-2, name="free-running logits")
    print(f"free-running step: logits {err:.4f} of the tensor maximum")


def test_later_positions_of_a_request_run_a_wider_fan_out(qwen):
    """Heads of 128: `build` leaves streams with 8 and 12 split-KV slices per KV head beside the request's first one, and
    `call_mk` takes them from positions 480 and 800 on.  One free-running step at a position of each stream against
    the fused oracle from the same state: logits within the trajectory gate, the same pick at a clear margin."""
    shape, _ = qwen
    LlamaConfig.set_shape(shape)
    capacity = 1040
    w = synthetic.random_weights(shape, 5, capacity)
    gpu = synthetic.build_globals(w, shape, capacity, "cuda:0")
    S.build(gpu)
    base, later = gpu.instruction_plan
    assert base is gpu.instructions and [first for first, _ in later] == [480, 800]
    widths = [int((t[:, :, 0] == 2).sum()) // shape.num_hidden_layers // shape.num_key_value_heads for t in (base, later[0][1], later[1][1])]
    assert widths == [4, 8, 12]
    oracle = FusedOracle(shape)
    mk = mk_kernel.get_mk()
    gen = torch.Generator().manual_seed(11)
    cpu = synthetic.build_globals(w, shape, capacity, "cpu")
    cpu.k_cache.copy_(torch.randn(cpu.k_cache.shape, generator=gen).bfloat16())
    cpu.v_cache.copy_(torch.randn(cpu.v_cache.shape, generator=gen).bfloat16())
    for pos in (100, 479, 480, 700, 1000):
        cpu.hidden_states.copy_(cpu.embed_tokens[17 + pos]); cpu.position_id = pos
        sync_state(cpu, gpu)
        gpu.barriers.zero_()
        oracle.decode_step(cpu)
        mk_kernel.call_mk(gpu, mk)
        mk.check()
        tensor_rel_close(gpu.logits, cpu.logits, rel=TRAJECTORY_REL, name=f"logits at position {pos}")
        if _margin_ulps(cpu.logits) > 2.0:
            assert int(gpu.logits.argmax()) == int(cpu.logits.argmax())
        bf16_close(gpu.k_cache[0, 0, pos], cpu.k_cache[0, 0, pos], ulps=2.0, frac=0.03, name=f"k row at {pos}")
