"""MoE decode route on the GPU: the kernel behind ``qmk_decode_step_moe`` against the CPU oracles.

Mirrors the reference's verifier stages for this route
(`qimeng_megakernel/verifier/LLM/qwen/qwen1_5_moe_a2_7b/A100/single_batch/{pyvm_to_megakernel,e2e_generate}`):
the same instruction list runs on the sequential VM and through the C ABI; outputs agree within bf16
rounding, routing decisions and counters exactly; a whole request reproduces the tokens and the routing
recorded from the reference.
"""
import copy
import dataclasses
import hashlib
import json

import numpy as np
import pytest
import torch

from conftest import GOLDEN
from gpu_helpers import bf16_close, rel_close, tensor_rel_close
from pyvm_moe_oracle import MoeInstructionVM
from qimeng_megakernel_amd import synthetic
from qimeng_megakernel_amd.decode_schedule_moe import mk_kernel
from qimeng_megakernel_amd.decode_schedule_moe.instructions import scheduler as S
from qimeng_megakernel_amd.decode_schedule_moe.model_config import QWEN1_5_MOE_A2_7B, QwenMoeConfig, num_partials_for

pytestmark = pytest.mark.gpu

FIX = json.loads((GOLDEN / "moe_reduced_seed0.json").read_text())
SMALL = dataclasses.replace(QWEN1_5_MOE_A2_7B, **FIX["shape"])
MUTABLE = ("hidden_states", "q_post_rope", "attn_out", "logits", "k_cache", "v_cache", "attn_out_intermediates", "attn_lse_intermediates",
           "barriers", "router_logits_buf", "normed_hidden_states", "shared_expert_silu_out", "shared_out", "routed_silu_buffer",
           "routed_out_f32", "silu_out", "expert_indices", "expert_weights")


@pytest.fixture(autouse=True)
def _shape():
    QwenMoeConfig.set_shape(SMALL)
    with torch.no_grad():
        yield
    QwenMoeConfig.set_shape(QWEN1_5_MOE_A2_7B)


@pytest.fixture(scope="module")
def weights():
    return synthetic.random_moe_weights(SMALL, FIX["seed"], FIX["kv_capacity"])


def sync_state(src, dst):
    for name in MUTABLE:
        getattr(dst, name).copy_(getattr(src, name))
    dst.position_id = src.position_id


def make_pair(weights, shape=SMALL, position=41, token=99, capacity=None):
    capacity = capacity or FIX["kv_capacity"]
    cpu = synthetic.build_moe_globals(weights, shape, capacity, "cpu")
    gpu = synthetic.build_moe_globals(weights, shape, capacity, "cuda:0")
    gen = torch.Generator().manual_seed(5)
    cpu.k_cache.copy_(torch.randn(cpu.k_cache.shape, generator=gen).bfloat16())
    cpu.v_cache.copy_(torch.randn(cpu.v_cache.shape, generator=gen).bfloat16())
    cpu.hidden_states.copy_(cpu.embed_tokens[token])
    cpu.position_id = position
    sync_state(cpu, gpu)
    return cpu, gpu


def run_kernel(gpu, instructions, queues=256):
    mk = mk_kernel.get_mk(reset_barriers=False, spin_limit=1 << 18)
    mk_kernel.run_instructions(gpu, copy.deepcopy(instructions), mk=mk, queues=queues)
    mk.check()
    return mk


STAGES = ["qkvproj", "attention_split_kv", "attention_reduction", "oproj", "router_gemv", "router_softmax_topk", "shared_upgate",
          "shared_downproj", "routed_upgate", "routed_downproj", "combine_commit"]
BF16_OUT = {"qkvproj": ("q_post_rope", "k_cache", "v_cache"), "attention_reduction": ("attn_out",), "oproj": ("hidden_states",),
            "router_gemv": ("normed_hidden_states",), "shared_upgate": ("shared_expert_silu_out",),
            "routed_upgate": ("routed_silu_buffer", "silu_out"), "combine_commit": ("hidden_states", "shared_out")}


@pytest.mark.parametrize("stage", range(len(STAGES)), ids=STAGES)
@pytest.mark.parametrize("position", [41, 0, 95])
def test_one_op_against_the_vm(weights, stage, position):
    """Everything before the op runs on the VM; the op itself on both, from identical state."""
    cpu, gpu = make_pair(weights, position=position)
    sched = dataclasses.replace(mk_kernel.mi355x_scheduler(SMALL), merge_in_last=False, merge_in_oproj=False)     # the reference's protocol, op by op
    vm = MoeInstructionVM(SMALL)
    name = STAGES[stage]
    # the combine step uses what the router (the gate) and the two down projections (their terms) left in the launcher's
    # workspace: the whole MoE block runs on both sides then
    first = STAGES.index("router_gemv") if name == "combine_commit" else stage
    for earlier in STAGES[:first]:
        vm.run(cpu, getattr(sched, earlier)(0))
    sync_state(cpu, gpu)
    mine = [ins for part in STAGES[first : stage + 1] for ins in getattr(sched, part)(0)]
    vm.run(cpu, copy.deepcopy(mine))
    mk = run_kernel(gpu, mine)
    assert torch.equal(gpu.barriers.cpu(), cpu.barriers), "counters differ from the VM's"
    for out in BF16_OUT.get(name, ()):
        loose = out in ("q_post_rope", "k_cache", "shared_expert_silu_out", "routed_silu_buffer", "silu_out")
        floor = 2.0 ** -1 if out == "hidden_states" else 2.0 ** -6
        bf16_close(getattr(gpu, out), getattr(cpu, out), ulps=2.0 if loose else 1.0, floor=floor, name=out)
    H = SMALL.hidden_size
    if name == "attention_split_kv":
        g, w = gpu.attn_lse_intermediates.cpu(), cpu.attn_lse_intermediates
        assert torch.equal(torch.isinf(g), torch.isinf(w))
        assert float((g[~torch.isinf(w)] - w[~torch.isinf(w)]).abs().max()) <= 2e-3
        assert float((gpu.attn_out_intermediates.cpu() - cpu.attn_out_intermediates).abs().max()) <= 2e-3 * float(cpu.attn_out_intermediates.abs().max())
    if name == "router_gemv":
        assert torch.allclose(gpu.router_logits_buf.cpu(), cpu.router_logits_buf, rtol=1e-4, atol=1e-5)
    if name == "router_softmax_topk":
        assert gpu.expert_indices.tolist() == cpu.expert_indices.tolist()
        assert torch.allclose(gpu.expert_weights.cpu(), cpu.expert_weights, rtol=1e-5)
    if name == "shared_downproj":      # the K-slice terms wait in the workspace: added in slice order they are the VM's shared_out
        parts = mk._workspace[: SMALL.num_downproj_split_k_shared * H * 2].view(torch.bfloat16).view(-1, H).cpu()
        total = torch.zeros(H, dtype=torch.bfloat16)
        for k in range(parts.shape[0]):
            total = (total.float() + parts[k].float()).to(torch.bfloat16)
        bf16_close(total, cpu.shared_out, ulps=2.0, name="shared_out from the K-slice terms")
    if name == "routed_downproj":
        off = ((SMALL.num_downproj_split_k_shared * H * 2 + 127) // 128) * 128
        parts = mk._workspace[off : off + SMALL.num_experts_per_tok * H * 4].view(torch.float32).view(-1, H).cpu()
        total = torch.zeros(H)
        for j in range(parts.shape[0]):
            total += parts[j]
        assert float((total - cpu.routed_out_f32).abs().max()) <= 2.0 ** -8 * float(cpu.routed_out_f32.abs().max())
    if name == "combine_commit":
        assert float(gpu.routed_out_f32.abs().max()) == 0.0 == float(cpu.routed_out_f32.abs().max())


@pytest.mark.parametrize("position", [41, 0, 95])
def test_split_kv_whose_last_arrival_merges(weights, position):
    """A stream without reduction instructions: the last split-KV arrival of a KV head merges."""
    cpu, gpu = make_pair(weights, position=position)
    sched = dataclasses.replace(mk_kernel.mi355x_scheduler(SMALL), merge_in_last=True, merge_in_oproj=False, num_partials=16)
    assert not sched.attention_reduction(0)
    vm = MoeInstructionVM(SMALL)
    vm.run(cpu, sched.qkvproj(0))
    sync_state(cpu, gpu)
    mine = sched.attention_split_kv(0)
    assert all(i.padded()[5] == 1 for i in mine)
    vm.run(cpu, copy.deepcopy(mine))
    run_kernel(gpu, mine)
    assert torch.equal(gpu.barriers.cpu(), cpu.barriers) and int(cpu.barriers[0, 2, 0]) == SMALL.num_attention_heads
    bf16_close(gpu.attn_out, cpu.attn_out, name="attn_out")


@pytest.mark.parametrize("position,partials", [(41, 3), (0, 2), (95, 6)])
def test_oproj_that_merges_the_partials(weights, position, partials):
    """The other stream without reduction instructions: split-KV instructions that only count their arrival,
    O-projection instructions that merge the partials of all heads themselves."""
    cpu, gpu = make_pair(weights, position=position)
    sched = dataclasses.replace(mk_kernel.mi355x_scheduler(SMALL), num_partials=partials)
    assert sched.merge_in_oproj and not sched.merge_in_last
    assert not sched.attention_reduction(0)
    vm = MoeInstructionVM(SMALL)
    vm.run(cpu, sched.qkvproj(0))
    sync_state(cpu, gpu)
    mine = sched.attention_split_kv(0) + sched.oproj(0)
    assert all(i.padded()[5] == 2 for i in mine if i.opcode() == 2) and all(i.padded()[5] == partials for i in mine if i.opcode() == 4)
    vm.run(cpu, copy.deepcopy(mine))
    run_kernel(gpu, mine)
    assert torch.equal(gpu.barriers.cpu(), cpu.barriers)
    assert int(cpu.barriers[0, 2, 0]) == SMALL.num_key_value_heads * partials and int(cpu.barriers[0, 3, 0]) == SMALL.num_hidden_blocks
    bf16_close(gpu.attn_out, cpu.attn_out, name="attn_out")
    # each side multiplies its own merged attn_out (1 ulp apart at most) into the residual stream
    bf16_close(gpu.hidden_states, cpu.hidden_states, ulps=2.0, frac=0.05, floor=2.0 ** -1, name="hidden_states")


def test_lm_head_against_the_vm(weights):
    cpu, gpu = make_pair(weights)
    sched = mk_kernel.mi355x_scheduler(SMALL)
    cpu.barriers[SMALL.num_hidden_layers - 1, 13, 0] = SMALL.num_hidden_blocks
    sync_state(cpu, gpu)
    MoeInstructionVM(SMALL).run(cpu, sched.lmhead())
    run_kernel(gpu, sched.lmhead())
    bf16_close(gpu.logits, cpu.logits, name="logits")


@pytest.mark.parametrize("queues", [256, 108])
def test_whole_step(weights, queues):
    """One step of both layers and the LM head: the reference's stream on 108 queues unchanged (its QKV tiles of 16 rows:
    the launch takes the tile from the scheduler's shape), and the same order of instructions on 256 with this build's tiles."""
    cpu, gpu = make_pair(weights)
    sched = S.reference_scheduler(SMALL) if queues == 108 else S.MoeScheduler(SMALL, queues, num_partials_for(queues, SMALL))
    assert (sched.sm_count, sched.shape.qkv_tile) == ((108, 16) if queues == 108 else (256, SMALL.qkv_tile))
    QwenMoeConfig.set_shape(sched.shape)
    mine = sched.instruction_list()
    if queues == 108:     # word for word the list whose digest was recorded from the reference's scheduler
        assert hashlib.sha256(np.asarray([i.padded() for i in mine], dtype=np.int32).tobytes()).hexdigest() == FIX["instruction_list_sha256"]
    MoeInstructionVM(SMALL).run(cpu, copy.deepcopy(mine))
    run_kernel(gpu, mine, queues=queues)
    assert torch.equal(gpu.barriers.cpu(), cpu.barriers)
    assert gpu.expert_indices.tolist() == cpu.expert_indices.tolist()
    tensor_rel_close(gpu.hidden_states, cpu.hidden_states, name="hidden_states")
    rel_close(gpu.logits, cpu.logits, rel=4e-2, name="logits")
    assert int(gpu.logits.float().argmax()) == int(cpu.logits.float().argmax())


def test_request_of_the_reference_fixture(weights):
    """Six greedy steps through call_mk with one instruction tensor and self-clearing counters: the tokens,
    the last layer's routing and the top-4 logits recorded from the reference's VM."""
    g = synthetic.build_moe_globals(weights, SMALL, FIX["kv_capacity"], "cuda:0")
    gen = torch.Generator().manual_seed(FIX["seed"] + 1)
    g.k_cache.copy_(torch.randn(g.k_cache.shape, generator=gen).bfloat16())
    g.v_cache.copy_(torch.randn(g.v_cache.shape, generator=gen).bfloat16())
    mk = mk_kernel.get_mk(spin_limit=1 << 18)
    token = FIX["start_token"]
    for step, want in enumerate(FIX["steps"]):
        g.position_id = want["position"]
        g.hidden_states.copy_(g.embed_tokens[token])
        mk_kernel.call_mk(g, mk)
        mk.check()
        assert int(g.barriers.abs().sum()) == 0, "the last workgroup clears the counters"
        rec = want["my_vm"]
        if g.expert_indices.tolist() != rec["last_layer_experts"]["indices"]:
            # A routing decision may flip where two experts are next to tied (the normalised row differs from the
            # VM's in bf16 roundings): the disputed experts must then be that close, and the trajectories part here.
            probs = torch.softmax(g.router_logits_buf.cpu(), dim=-1)
            disputed = sorted(set(g.expert_indices.tolist()) ^ set(rec["last_layer_experts"]["indices"]))
            assert len(disputed) == 2 and abs(float(probs[disputed[0]] - probs[disputed[1]])) <= 0.03 * float(probs[disputed].max()), (step, disputed, probs.tolist())
            assert step >= 2, "the first steps of this request have clear routing margins"
            break
        assert torch.allclose(g.expert_weights.cpu(), torch.tensor(rec["last_layer_experts"]["weights"]), rtol=2e-2)
        got = g.logits[torch.tensor(rec["top_ids"], device=g.logits.device)].view(torch.int16).to(torch.int32).cpu()
        ref = torch.tensor(rec["top_bits"], dtype=torch.int32)
        ref = torch.where(ref >= 32768, ref - 65536, ref)
        assert int((got - ref).abs().max()) <= 8, (step, got.tolist(), ref.tolist())
        token = int(g.logits.float().argmax())
        assert token == rec["token"], step


def _request_both_ways(weights, shape, capacity, steps):
    """The same greedy request on two sets of buffers: through counters only, then with tagged hand-over."""
    from qimeng_megakernel_amd import decode_moe

    gen = torch.Generator().manual_seed(23)
    prompt = torch.randint(0, shape.vocab_size, (4,), generator=gen)
    out = []
    for tagged in (False, True):
        g = synthetic.build_moe_globals(weights, shape, capacity, "cuda:0")
        mk = mk_kernel.get_mk(tagged=tagged, spin_limit=1 << 18)
        toks = decode_moe.decode(g, prompt, steps, mk=mk, decode_time=False)["new_tokens"].clone()
        assert mk._tagged == tagged
        out.append((g, toks))
    return out


def test_tagged_and_counter_modes_agree_bit_for_bit(weights):
    """Tagged hand-over changes how values travel, not the values: every buffer of the request is identical."""
    (plain, toks_p), (tagged, toks_t) = _request_both_ways(weights, SMALL, FIX["kv_capacity"], 24)
    assert torch.equal(toks_p, toks_t)
    for name in MUTABLE:
        assert torch.equal(getattr(plain, name), getattr(tagged, name)), name
    assert int(tagged.barriers.abs().sum()) == 0


def test_tagged_and_counter_modes_agree_full_geometry():
    shape = dataclasses.replace(QWEN1_5_MOE_A2_7B, num_hidden_layers=3, vocab_size=4096)
    QwenMoeConfig.set_shape(shape)
    w = synthetic.random_moe_weights(shape, 4, 40)
    (plain, toks_p), (tagged, toks_t) = _request_both_ways(w, shape, 40, 10)
    assert torch.equal(toks_p, toks_t)
    for name in MUTABLE:
        assert torch.equal(getattr(plain, name), getattr(tagged, name)), name


def test_decode_loop_as_one_graph_moe(weights):
    """The request's loop (embedding row, kernel, argmax per step) as one HIP graph: the tokens of the loop run
    launch by launch, on three replays with eager work between them."""
    from qimeng_megakernel_amd import decode_moe

    g = synthetic.build_moe_globals(weights, SMALL, FIX["kv_capacity"], "cuda:0")
    gen = torch.Generator().manual_seed(17)
    prompt = torch.randint(0, SMALL.vocab_size, (5,), generator=gen)
    mk = mk_kernel.get_mk(spin_limit=1 << 18)
    want = decode_moe.decode(g, prompt, 12, mk=mk)["new_tokens"].clone()
    out = decode_moe.decode(g, prompt, 12, mk=mk, use_graph=True)
    assert torch.equal(out["new_tokens"], want)
    for _ in range(2):
        g.logits.zero_()
        g.hidden_states.zero_()
        torch.cuda.synchronize()
        again = out["replay"]()
        torch.cuda.synchronize()
        mk.check()
        assert torch.equal(again, want)


def test_full_geometry_layers_against_the_vm():
    """Qwen1.5-MoE-A2.7B layer geometry (60 experts of 1408, top-4, shared 5632), two layers, small vocabulary:
    layer by layer from the VM's residual stream, then the LM head."""
    shape = dataclasses.replace(QWEN1_5_MOE_A2_7B, num_hidden_layers=2, vocab_size=2048)
    QwenMoeConfig.set_shape(shape)
    w = synthetic.random_moe_weights(shape, 4, 160)
    cpu, gpu = make_pair(w, shape=shape, position=133, token=77, capacity=160)
    sched = mk_kernel.mi355x_scheduler(shape)
    vm = MoeInstructionVM(shape)
    for layer in range(2):
        gpu.hidden_states.copy_(cpu.hidden_states)
        vm.run(cpu, sched.layer(layer))
        gpu.barriers.zero_()
        if layer:
            gpu.barriers[layer - 1, 13, 0] = shape.num_hidden_blocks
        run_kernel(gpu, sched.layer(layer))
        assert gpu.expert_indices.tolist() == cpu.expert_indices.tolist(), layer
        assert torch.allclose(gpu.expert_weights.cpu(), cpu.expert_weights, rtol=2e-2)   # the router reads a bf16 row that differs in roundings
        rel_close(gpu.hidden_states, cpu.hidden_states, name=f"hidden_states after layer {layer}")
        assert torch.equal(gpu.barriers[layer].cpu(), cpu.barriers[layer])
    gpu.hidden_states.copy_(cpu.hidden_states)
    vm.run(cpu, sched.lmhead())
    gpu.barriers.zero_()
    gpu.barriers[1, 13, 0] = shape.num_hidden_blocks
    run_kernel(gpu, sched.lmhead())
    rel_close(gpu.logits, cpu.logits, name="logits")
    assert int(gpu.logits.float().argmax()) == int(cpu.logits.float().argmax())


# ---- error paths: forced from the host, every kernel still exits normally -----------------------------------------

def _launch(gpu, instructions, **opts):
    mk = mk_kernel.get_mk(reset_barriers=False, **opts)
    mk_kernel.run_instructions(gpu, copy.deepcopy(instructions), mk=mk, queues=8)
    return mk


def test_wait_timeout_drains_the_grid_moe(weights):
    """Routed up/gate instructions wait for a top-k that nobody runs: they run out of polls, say so and retire;
    the next well-formed launch works (the reference hangs: decode_kernel/mk.cu has no bounded wait)."""
    cpu, gpu = make_pair(weights)
    sched = mk_kernel.mi355x_scheduler(SMALL)
    mk = _launch(gpu, sched.routed_upgate(0)[:8], spin_limit=50)
    with pytest.raises(RuntimeError, match="counter wait ran out of polls") as err:
        mk.check()
    assert "opcode=12" in str(err.value)
    gpu.barriers.zero_()
    vm = MoeInstructionVM(SMALL)
    for stage in STAGES[: STAGES.index("oproj") + 1]:
        vm.run(cpu, getattr(sched, stage)(0))
    sync_state(cpu, gpu)
    vm.run(cpu, sched.router_gemv(0))
    run_kernel(gpu, sched.router_gemv(0))
    assert torch.equal(gpu.barriers.cpu(), cpu.barriers)


@pytest.mark.parametrize("bad, operand", [
    (S.Router_GEMV(9, 0, 1, 0), 1),                                        # layer out of range
    (S.Router_GEMV(0, 3, 2, 0), 2),                                        # experts end before they start
    (S.Router_SoftmaxTopK(9), 1),
    (S.SharedExpert_UpGate_SiLU(0, 0, 0, 4096, 0), 4),                     # rows beyond the shared expert's width
    (S.SharedExpert_DownProj(0, 0, 0, 4096, 0), 4),                        # rows beyond the hidden size
    (S.SharedExpert_DownProj(0, 0, 0, 1, 99), 5),                          # K slice beyond the launch's slices
    (S.RoutedExpert_UpGate_SiLU(0, 8, 0, 1), 2),                           # expert slot beyond top-k
    (S.RoutedExpert_UpGate_SiLU(0, 0, 0, 4096), 4),
    (S.RoutedExpert_DownProj(0, 8, 0, 0, 1), 2),
    (S.RoutedExpert_DownProj(0, 0, 0, 0, 4096), 5),
    (S.MoE_Combine_Commit(0, 0, 4096), 3),
])
def test_bad_operands_are_rejected_on_the_device_moe(weights, bad, operand):
    _, gpu = make_pair(weights)
    before = {n: getattr(gpu, n).clone() for n in MUTABLE if n != "barriers"}
    mk = _launch(gpu, [bad])
    with pytest.raises(RuntimeError, match="operand out of bounds") as err:
        mk.check()
    assert f"opcode={bad.opcode()}" in str(err.value) and f"operand={operand}" in str(err.value)
    for n, t in before.items():
        assert torch.equal(getattr(gpu, n), t), n                           # nothing was written
    assert int(gpu.barriers.abs().sum()) == 0


def test_expert_index_outside_the_layer_is_rejected(weights):
    """The routed ops take the physical expert from ``expert_indices`` at run time: a value no expert has
    (a buffer the caller overwrote) is refused before any weight row is addressed."""
    cpu, gpu = make_pair(weights)
    gpu.expert_indices.fill_(SMALL.num_experts + 3)
    gpu.barriers[0, 8, 0] = 1                                               # the top-k counts as done
    gpu.barriers[0, 3, 0] = SMALL.num_hidden_blocks
    before = gpu.routed_silu_buffer.clone()
    mk = _launch(gpu, [S.RoutedExpert_UpGate_SiLU(0, 0, 0, 1)])
    with pytest.raises(RuntimeError, match="operand out of bounds"):
        mk.check()
    assert torch.equal(gpu.routed_silu_buffer, before)


def test_host_side_checks_moe(weights):
    _, gpu = make_pair(weights)
    mk = mk_kernel.get_mk()
    mk_kernel.build(gpu)
    gpu.position_id = FIX["kv_capacity"]
    with pytest.raises(RuntimeError, match="pos_id outside"):
        mk_kernel.call_mk(gpu, mk)
    gpu.position_id = 3
    keep = gpu.instructions
    gpu.instructions = torch.zeros(4096, 1, 32, dtype=torch.int32, device="cuda:0")
    with pytest.raises(RuntimeError, match="co-resident"):
        mk_kernel.call_mk(gpu, mk)
    gpu.instructions = keep
    keep, gpu.barriers = gpu.barriers, gpu.barriers[:, :10].contiguous()    # the dense route's ten counter rows
    with pytest.raises(ValueError, match="barriers must be"):
        mk_kernel.call_mk(gpu, mk)
    gpu.barriers = keep
    mk_kernel.call_mk(gpu, mk)
    mk.check()
