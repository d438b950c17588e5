"""Batch route on the Qwen3-1.7B layer geometry on the GPU: ``qmk_decode_step_batch`` with QMK_MODEL_QWEN3_1_7B
against the CPU oracles (the Qwen3 op set per row: opcode 2 leaves raw QKV rows, opcode 3 applies the per-head
RMSNorm and RoPE and appends the cache rows; 16 query / 8 KV heads of 128, FFN 6144, tied 151 936-row head).

Same ladder as the Llama geometry's tests: single ops against the instruction VM from identical state (counters
word for word), whole steps against VM and fused oracle, the request recorded from the imported reference, the
full-size model layer by layer at batch 8 and free-running.
"""
import copy
import dataclasses
import json

import pytest
import torch

from conftest import GOLDEN
from fused_mb_oracle import FusedBatchOracle
from gpu_helpers import bf16_close, rel_close, tensor_rel_close
from pyvm_mb_oracle import BatchInstructionVM
from qimeng_megakernel_amd import synthetic
from qimeng_megakernel_amd.decode_schedule.model_config import QWEN3_1_7B, LlamaConfig
from qimeng_megakernel_amd.decode_schedule_mb import mk_kernel
from qimeng_megakernel_amd.decode_schedule_mb.instructions import scheduler as S
from qimeng_megakernel_amd.decode_schedule_mb.row_state import RowState

pytestmark = pytest.mark.gpu

FIX = json.loads((GOLDEN / "qwen3_mb_reduced_seed0.json").read_text())
FULL = QWEN3_1_7B
SMALL = dataclasses.replace(FULL, num_hidden_layers=FIX["layers"], vocab_size=FIX["vocab"])

MUTABLE = ("hidden_states", "qkv_raw", "q_post_rope", "attn_out", "silu_out", "logits", "k_cache", "v_cache", "attn_out_intermediates",
           "attn_lse_intermediates", "barriers", "attn_partial_valid", "attn_rms_out", "mlp_rms_out", "lm_head_rms_out",
           "position_ids", "active_mask")


def sync_state(src, dst):
    for name in MUTABLE:
        getattr(dst, name).copy_(getattr(src, name))


@pytest.fixture(autouse=True)
def _shape():
    LlamaConfig.set_shape(SMALL)
    with torch.no_grad():
        yield


@pytest.fixture(scope="module")
def weights():
    return synthetic.random_weights(SMALL, FIX["seed"], max_positions=FIX["kv_capacity"])


def make_pair(weights, rows, positions, *, inactive=(), capacity=None, shape=SMALL, seed=5, max_partials=27):
    capacity = capacity or FIX["kv_capacity"]
    cpu = synthetic.build_batch_globals(weights, shape, capacity, rows, "cpu", max_partials=max_partials)
    gpu = synthetic.build_batch_globals(weights, shape, capacity, rows, "cuda:0", max_partials=max_partials)
    gen = torch.Generator().manual_seed(seed)
    cpu.hidden_states.copy_((torch.randn(cpu.hidden_states.shape, generator=gen) * 0.7).bfloat16())
    cpu.k_cache.copy_(torch.randn(cpu.k_cache.shape, generator=gen).bfloat16())
    cpu.v_cache.copy_(torch.randn(cpu.v_cache.shape, generator=gen).bfloat16())
    cpu.position_ids.copy_(torch.tensor(positions, dtype=torch.int32))
    for r in inactive:
        cpu.active_mask[r] = False
    RowState.of(cpu)
    sync_state(cpu, gpu)
    return cpu, gpu


def vm_for(sched):
    return BatchInstructionVM(sched.shape, sched.oproj_tile, sched.down_tile)


def run_kernel(gpu, instructions, workers=256):
    mk = mk_kernel.get_mk(reset_barriers=False, spin_limit=1 << 18)
    mk_kernel.run_instructions(gpu, copy.deepcopy(instructions), mk=mk, workers=workers)
    mk.check()


def close_f32(got, want, name):
    g, w = got.cpu(), want
    assert torch.equal(torch.isinf(g), torch.isinf(w)), name
    finite = ~torch.isinf(w)
    assert float((g[finite] - w[finite]).abs().max()) <= 2e-3 * max(1.0, float(w[finite].abs().max())), name


# The ops of one layer in dependency order: (name, what it writes).
STAGES = [
    ("attn_rms", ("attn_rms_out",)),
    ("qkvproj", ("qkv_raw",)),
    ("attention_split_kv", ("q_post_rope", "k_cache", "v_cache", "attn_out_intermediates", "attn_lse_intermediates", "attn_partial_valid")),
    ("attention_reduction", ("attn_out",)),
    ("oproj", ("hidden_states",)),
    ("mlp_rms", ("mlp_rms_out",)),
    ("upgate", ("silu_out",)),
    ("downproj", ("hidden_states",)),
]
CASES = {"ragged3": (3, (70, 3, 130), ()), "inactive_row": (4, (9, 64, 0, 127), (2,)), "batch16": (16, tuple(range(5, 150, 9))[:16], (7,))}


def stage_instructions(sched, globs, name, layer=0):
    p = sched.partials_for_request(globs)
    if name == "attention_split_kv":
        return sched.attention_split_kv(layer, p, globs)
    if name == "attention_reduction":
        return sched.attention_reduction(layer, p, globs)
    return getattr(sched, name)(layer)


@pytest.mark.parametrize("stage", range(len(STAGES)), ids=[s[0] for s in STAGES])
@pytest.mark.parametrize("case", list(CASES))
def test_one_op_against_the_vm(weights, stage, case):
    """Everything before the op runs on the VM; the op itself on both, from identical state."""
    rows, positions, inactive = CASES[case]
    cpu, gpu = make_pair(weights, rows, positions, inactive=inactive)
    sched = S.mi355x_scheduler(rows, SMALL, merge_in_last=False)
    vm = vm_for(sched)
    for name, _ in STAGES[:stage]:
        vm.run(cpu, stage_instructions(sched, cpu, name))
    sync_state(cpu, gpu)
    gpu.residual_tiles = (sched.oproj_tile, sched.down_tile)
    mine = stage_instructions(sched, cpu, STAGES[stage][0])
    vm.run(cpu, copy.deepcopy(mine))
    run_kernel(gpu, mine)
    floor = 2.0 ** -1 if STAGES[stage][0] in ("oproj", "downproj") else 2.0 ** -6
    for name in MUTABLE:
        got, want = getattr(gpu, name), getattr(cpu, name)
        if name not in STAGES[stage][1]:
            assert torch.equal(got.cpu(), want), f"{name} moved"
        elif want.dtype == torch.bfloat16:
            # silu_out is a product of two rounded factors; q and k are rotations of normalised, rounded values
            loose = name in ("silu_out", "q_post_rope", "k_cache")
            bf16_close(got, want, floor=floor, ulps=2.0 if loose else 1.0, name=name)
        elif want.dtype == torch.float32:
            close_f32(got, want, name)
        else:
            assert torch.equal(got.cpu(), want), name
    assert torch.equal(gpu.barriers.cpu(), cpu.barriers), "counters differ from the VM's"


@pytest.mark.parametrize("case", list(CASES))
@pytest.mark.parametrize("template", [False, True], ids=["static", "runtime"])
def test_split_kv_whose_last_arrival_merges(weights, case, template):
    """The MI355X stream: no reduction instructions; the slice that holds a row's position appends the cache rows."""
    rows, positions, inactive = CASES[case]
    cpu, gpu = make_pair(weights, rows, positions, inactive=inactive)
    sched = S.mi355x_scheduler(rows, SMALL)
    vm = vm_for(sched)
    vm.run(cpu, sched.attn_rms(0) + sched.qkvproj(0))
    sync_state(cpu, gpu)
    p = sched.partials_for_capacity(FIX["kv_capacity"]) if template else sched.partials_for_request(cpu)
    mine = sched.attention_split_kv(0, p, None if template else cpu)
    assert not sched.attention_reduction(0, p)
    vm.run(cpu, copy.deepcopy(mine))
    run_kernel(gpu, mine)
    bf16_close(gpu.attn_out, cpu.attn_out, name="attn_out")
    for name in ("q_post_rope", "k_cache"):
        bf16_close(getattr(gpu, name), getattr(cpu, name), ulps=2.0, name=name)
    assert torch.equal(gpu.v_cache.cpu(), cpu.v_cache)
    assert torch.equal(gpu.attn_partial_valid.cpu(), cpu.attn_partial_valid)
    assert torch.equal(gpu.barriers.cpu(), cpu.barriers)
    assert int(cpu.barriers[0, 3, 0]) == SMALL.num_attention_heads


def test_lm_head_ops_against_the_vm(weights):
    cpu, gpu = make_pair(weights, 3, (70, 3, 130), inactive=(1,))
    sched = S.mi355x_scheduler(3, SMALL)
    last = SMALL.num_hidden_layers - 1
    cpu.barriers[last, 7, 0] = SMALL.hidden_size // sched.down_tile     # the last down projection is complete
    sync_state(cpu, gpu)
    gpu.residual_tiles = (sched.oproj_tile, sched.down_tile)
    mine = sched.lmhead_rms() + sched.lmhead()
    vm_for(sched).run(cpu, copy.deepcopy(mine))
    run_kernel(gpu, mine)
    bf16_close(gpu.lm_head_rms_out, cpu.lm_head_rms_out, name="lm_head_rms_out")
    bf16_close(gpu.logits, cpu.logits, name="logits")
    assert torch.equal(gpu.barriers.cpu(), cpu.barriers)
    assert bool((gpu.logits[1].float() == torch.tensor(-1e9).bfloat16().float()).all())


@pytest.mark.parametrize("make,workers", [(S.mi355x_scheduler, 256), (S.reference_scheduler, 216)])
def test_whole_step_static_list(weights, make, workers):
    cpu, gpu = make_pair(weights, 3, (70, 3, 130))
    sched = make(3, SMALL)
    mine = sched.instruction_list(cpu)
    vm_for(sched).run(cpu, copy.deepcopy(mine))
    run_kernel(gpu, mine, workers=workers)
    assert torch.equal(gpu.barriers.cpu(), cpu.barriers)
    tensor_rel_close(gpu.hidden_states, cpu.hidden_states, name="hidden_states")
    rel_close(gpu.logits, cpu.logits, rel=4e-2, name="logits")
    assert gpu.logits.float().argmax(-1).tolist() == cpu.logits.float().argmax(-1).tolist()
    assert torch.equal(gpu.attn_partial_valid.cpu(), cpu.attn_partial_valid)


def test_request_of_the_reference_fixture(weights):
    """Six steps of the recorded request through call_mk with one instruction tensor for the whole request and
    self-clearing counters: tokens, row state and the recorded top-4 logits of the fused route."""
    g = synthetic.build_batch_globals(weights, SMALL, FIX["kv_capacity"], FIX["rows"], "cuda:0")
    gen = torch.Generator().manual_seed(FIX["seed"] + 1)
    g.k_cache.copy_(torch.randn(g.k_cache.shape, generator=gen).bfloat16())
    g.v_cache.copy_(torch.randn(g.v_cache.shape, generator=gen).bfloat16())
    g.position_ids.copy_(torch.tensor(FIX["start_positions"], dtype=torch.int32))
    state = RowState.of(g)
    mk = mk_kernel.get_mk(spin_limit=1 << 18)
    tokens = list(FIX["start_tokens"])
    for step, want in enumerate(FIX["steps"]):
        assert g.position_ids.tolist() == want["positions"] and g.active_mask.tolist() == want["active"]
        g.hidden_states.copy_(g.embed_tokens[torch.tensor(tokens, device=g.embed_tokens.device)])
        mk_kernel.call_mk(g, mk)
        mk.check()
        assert int(g.barriers.abs().sum()) == 0, "the last workgroup clears the counters"
        ids = torch.tensor(want["fused"]["top_ids"], device=g.logits.device)
        got = g.logits.gather(1, ids).view(torch.int16).to(torch.int32).cpu()
        ref = torch.tensor(want["fused"]["top_bits"], dtype=torch.int32)
        ref = torch.where(ref >= 32768, ref - 65536, ref)
        assert int((got - ref).abs().max()) <= 8, (step, got.tolist(), ref.tolist())
        nxt = g.logits.float().argmax(dim=-1)
        assert nxt.tolist() == want["fused"]["tokens"], step
        state.advance(nxt, [FIX["eos_token"]] if step >= 1 else [])
        tokens = nxt.tolist()
    assert g.active_mask.tolist() == [True, False, True]


@pytest.fixture(scope="module")
def full_weights():
    return synthetic.random_weights(FULL, 3, max_positions=320)


@pytest.mark.parametrize("rows", [2, 8])
def test_full_size_layers_against_the_fused_oracle(full_weights, rows):
    """Qwen3-1.7B shape, ragged contexts.  Layer by layer from the oracle's residual stream (so that one layer's
    rounding differences are not amplified by the next): hidden states within the bf16 gate (max rel err 2e-2)
    after every layer, logits within it after the tied 151 936-row head, greedy picks identical wherever the
    oracle has a clear winner."""
    LlamaConfig.set_shape(FULL)
    capacity = 320
    positions = [(37 * r + 11) % 300 for r in range(rows)]
    cpu, gpu = make_pair(full_weights, rows, positions, inactive=(rows - 1,) if rows >= 8 else (), capacity=capacity, shape=FULL, seed=9,
                         max_partials=8)
    toks = torch.tensor([(977 * r + 13) % FULL.vocab_size for r in range(rows)])
    cpu.hidden_states.copy_(cpu.embed_tokens[toks])
    fused, sched = FusedBatchOracle(FULL), S.mi355x_scheduler(rows, FULL)
    live = [r for r in range(rows) if bool(cpu.active_mask[r])]
    done = FULL.hidden_size // sched.down_tile
    p = min(8, sched.partials_for_request(cpu))
    gpu.residual_tiles = (sched.oproj_tile, sched.down_tile)
    for layer in range(FULL.num_hidden_layers):
        gpu.hidden_states.copy_(cpu.hidden_states)
        before = cpu.hidden_states.clone()
        fused.decode_layer(cpu, layer)
        gpu.barriers.zero_()
        if layer:
            gpu.barriers[layer - 1, 7, 0] = done
        run_kernel(gpu, sched.attn_rms(layer) + sched.qkvproj(layer) + sched.attention_split_kv(layer, p, cpu)
                   + sched.attention_reduction(layer, p, cpu) + sched.oproj(layer) + sched.mlp_rms(layer)
                   + sched.upgate(layer) + sched.downproj(layer))
        rel_close(gpu.hidden_states[live], cpu.hidden_states[live], name=f"hidden_states after layer {layer}")
        for r in range(rows):
            if r in live:
                rel_close(gpu.k_cache[layer, r, positions[r]], cpu.k_cache[layer, r, positions[r]], name="k row")
                # the oracle's one-row bf16 GEMV on the host is itself a few ulps of the row's scale from the exact dot products
                rel_close(gpu.v_cache[layer, r, positions[r]], cpu.v_cache[layer, r, positions[r]], name="v row")
            else:
                assert torch.equal(gpu.hidden_states[r].cpu(), before[r])
    gpu.hidden_states.copy_(cpu.hidden_states)
    fused.lm_head(cpu)
    gpu.barriers.zero_()
    gpu.barriers[FULL.num_hidden_layers - 1, 7, 0] = done
    run_kernel(gpu, sched.lmhead_rms() + sched.lmhead())
    rel_close(gpu.logits[live], cpu.logits[live], name="logits")
    top2 = cpu.logits.float().topk(2, dim=-1).values
    for r in range(rows):
        if r not in live:
            assert bool((gpu.logits[r].float() == torch.tensor(-1e9).bfloat16().float()).all())
        elif float(top2[r, 0] - top2[r, 1]) > 2.0 ** -6 * float(top2[r, 0].abs()):   # a clear winner
            assert int(gpu.logits[r].float().argmax()) == int(cpu.logits[r].float().argmax()), r


def test_full_size_step_free_running(full_weights):
    """One whole step at batch 8 through call_mk (run-time template, self-clearing counters) against the fused
    oracle: 28 layers of rounding differences deep, so the gate is on the tensor's scale."""
    LlamaConfig.set_shape(FULL)
    rows, capacity = 8, 320
    positions = [(37 * r + 11) % 300 for r in range(rows)]
    cpu, gpu = make_pair(full_weights, rows, positions, inactive=(5,), capacity=capacity, shape=FULL, seed=9)
    toks = torch.tensor([(977 * r + 13) % FULL.vocab_size for r in range(rows)])
    cpu.hidden_states.copy_(cpu.embed_tokens[toks])
    sync_state(cpu, gpu)
    FusedBatchOracle(FULL).decode_step(cpu)
    mk = mk_kernel.get_mk(spin_limit=1 << 20)
    mk_kernel.call_mk(gpu, mk)
    mk.check()
    live = [r for r in range(rows) if r != 5]
    err_h = tensor_rel_close(gpu.hidden_states[live], cpu.hidden_states[live], rel=5e-2, name="hidden_states")
    err_l = tensor_rel_close(gpu.logits[live], cpu.logits[live], rel=5e-2, name="logits")
    print(f"free-running step: hidden {err_h:.4f}, logits {err_l:.4f} of the tensor maximum")
    assert torch.equal(gpu.hidden_states[5].cpu(), cpu.hidden_states[5])
    assert int(gpu.barriers.abs().sum()) == 0


def test_host_side_checks(weights):
    """The three tensors of the Qwen3 op set are part of the call; a Llama-shaped call with them is refused."""
    _, gpu = make_pair(weights, 3, (70, 3, 130))
    mk = mk_kernel.get_mk()
    keep, gpu.qkv_raw = gpu.qkv_raw, gpu.qkv_raw[:, :128].contiguous()
    with pytest.raises(ValueError, match="qkv_raw"):
        mk_kernel.call_mk(gpu, mk)
    gpu.qkv_raw = keep
    mk_kernel.call_mk(gpu, mk)
    mk.check()
