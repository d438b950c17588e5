"""Batch decode route on the GPU: the kernel behind ``qmk_decode_step_batch`` against the CPU oracles.

Mirrors the reference's verifier stages for this route
(`qimeng_megakernel/verifier/LLM/llama/llama3_2__1b/A100/multi_batch/{pyvm_to_megakernel,e2e_generate}`):
the same instruction list runs on the sequential VM and through the C ABI; outputs agree within bf16
rounding, the counters word for word; whole requests reproduce the tokens recorded from the reference.
"""
import copy
import ctypes
import dataclasses
import json

import pytest
import torch

from conftest import GOLDEN
from fused_mb_oracle import FusedBatchOracle
from gpu_helpers import bf16_close, rel_close, tensor_rel_close
from pyvm_mb_oracle import BatchInstructionVM
from qimeng_megakernel_amd import synthetic
from qimeng_megakernel_amd.decode_schedule.model_config import LLAMA_3_2_1B, LlamaConfig
from qimeng_megakernel_amd.decode_schedule_mb import mk_kernel
from qimeng_megakernel_amd.decode_schedule_mb.row_state import RowState
from qimeng_megakernel_amd.decode_schedule_mb.instructions import scheduler as S

pytestmark = pytest.mark.gpu

FIX = json.loads((GOLDEN / "mb_reduced_seed0.json").read_text())
MB_FULL = dataclasses.replace(LLAMA_3_2_1B, attn_kv_block_size=FIX["kv_block"])
MB_SMALL = dataclasses.replace(MB_FULL, num_hidden_layers=FIX["layers"], vocab_size=FIX["vocab"])

MUTABLE = ("hidden_states", "q_post_rope", "attn_out", "silu_out", "logits", "k_cache", "v_cache", "attn_out_intermediates",
           "attn_lse_intermediates", "barriers", "attn_partial_valid", "attn_rms_out", "mlp_rms_out", "lm_head_rms_out",
           "position_ids", "active_mask")


def sync_state(src, dst):
    for name in MUTABLE:
        getattr(dst, name).copy_(getattr(src, name))


@pytest.fixture(autouse=True)
def _shape():
    LlamaConfig.set_shape(MB_SMALL)
    with torch.no_grad():
        yield


@pytest.fixture(scope="module")
def weights():
    return synthetic.random_weights(MB_SMALL, FIX["seed"], max_positions=FIX["kv_capacity"])


@pytest.fixture(scope="module")
def full_weights():
    return synthetic.random_weights(MB_FULL, 3, max_positions=320)


def make_pair(weights, rows, positions, *, inactive=(), capacity=None, shape=MB_SMALL, seed=5, max_partials=27):
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


def compare(cpu, gpu, names, *, ulps=1.0, frac=0.02):
    for name in names:
        got, want = getattr(gpu, name), getattr(cpu, name)
        if want.dtype == torch.bfloat16:
            bf16_close(got, want, ulps=ulps, frac=frac, name=name)
        elif want.dtype == torch.float32:
            g, w = got.cpu(), want
            assert torch.equal(torch.isinf(g), torch.isinf(w)), name
            finite = ~torch.isinf(w)
            assert float((g[finite] - w[finite]).abs().max()) <= 2e-3 * max(1.0, float(w[finite].abs().max())), name
        else:
            assert torch.equal(got.cpu(), want), name
    assert torch.equal(gpu.barriers.cpu(), cpu.barriers), "counters differ from the VM's"


# The ops of one layer in dependency order, then the LM head: (name, what it writes).
STAGES = [
    ("attn_rms", ("attn_rms_out",)),
    ("qkvproj", ("q_post_rope", "k_cache", "v_cache")),
    ("attention_split_kv", ("attn_out_intermediates", "attn_lse_intermediates", "attn_partial_valid")),
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
@pytest.mark.parametrize("case", ["ragged3", "inactive_row", "batch16"])
@pytest.mark.parametrize("tile", [16, 8], ids=["blocks16", "residual_blocks8"])
def test_one_op_against_the_vm(weights, stage, case, tile):
    """Everything before the op runs on the VM; the op itself on both, from identical state."""
    rows, positions, inactive = CASES[case]
    if tile == 8 and STAGES[stage][0] not in ("oproj", "mlp_rms", "downproj"):
        pytest.skip("only the residual projections and what waits for them see the block size")
    cpu, gpu = make_pair(weights, rows, positions, inactive=inactive)
    sched = S.mi355x_scheduler(rows, MB_SMALL, merge_in_last=False, residual_tile=tile)
    vm = vm_for(sched)
    for name, _ in STAGES[:stage]:
        vm.run(cpu, stage_instructions(sched, cpu, name))
    sync_state(cpu, gpu)
    gpu.residual_tiles = (sched.oproj_tile, sched.down_tile)
    mine = stage_instructions(sched, cpu, STAGES[stage][0])
    vm.run(cpu, copy.deepcopy(mine))
    run_kernel(gpu, mine)
    floor = 2.0 ** -1 if STAGES[stage][0] in ("oproj", "downproj") else 2.0 ** -6
    for name in STAGES[stage][1]:
        if getattr(cpu, name).dtype == torch.bfloat16:
            # silu_out is a product of two rounded factors, each of which may sit one ulp apart; q and k are
            # rotations of two rounded GEMM outputs
            loose = name in ("silu_out", "q_post_rope", "k_cache")
            bf16_close(getattr(gpu, name), getattr(cpu, name), floor=floor, ulps=2.0 if loose else 1.0, name=name)
    compare(cpu, gpu, [n for n in MUTABLE if getattr(cpu, n).dtype != torch.bfloat16])
    # nothing else moved
    for name in MUTABLE:
        if name not in STAGES[stage][1] and getattr(cpu, name).dtype == torch.bfloat16:
            assert torch.equal(getattr(gpu, name).cpu(), getattr(cpu, name)), name


@pytest.mark.parametrize("case", list(CASES))
@pytest.mark.parametrize("template", [False, True], ids=["static", "runtime"])
def test_split_kv_whose_last_arrival_merges(weights, case, template):
    """The MI355X stream: no reduction instructions; lengths and activity in the words or left to the launch."""
    rows, positions, inactive = CASES[case]
    cpu, gpu = make_pair(weights, rows, positions, inactive=inactive)
    sched = S.mi355x_scheduler(rows, MB_SMALL)
    vm = vm_for(sched)
    vm.run(cpu, sched.attn_rms(0) + sched.qkvproj(0))
    sync_state(cpu, gpu)
    p = sched.partials_for_capacity(FIX["kv_capacity"]) if template else sched.partials_for_request(cpu)
    mine = sched.attention_split_kv(0, p, None if template else cpu)
    assert not sched.attention_reduction(0, p) and all(i.padded()[8] == 1 for i in mine)
    vm.run(cpu, copy.deepcopy(mine))
    run_kernel(gpu, mine)
    bf16_close(gpu.attn_out, cpu.attn_out, name="attn_out")
    compare(cpu, gpu, ("attn_out_intermediates", "attn_lse_intermediates", "attn_partial_valid"))
    assert int(cpu.barriers[0, 3, 0]) == MB_SMALL.num_attention_heads


def test_lm_head_ops_against_the_vm(weights):
    cpu, gpu = make_pair(weights, 3, (70, 3, 130), inactive=(1,))
    sched = S.mi355x_scheduler(3, MB_SMALL)
    last = MB_SMALL.num_hidden_layers - 1
    cpu.barriers[last, 7, 0] = MB_SMALL.hidden_size // sched.down_tile     # the last down projection is complete
    sync_state(cpu, gpu)
    gpu.residual_tiles = (sched.oproj_tile, sched.down_tile)
    mine = sched.lmhead_rms() + sched.lmhead()
    vm_for(sched).run(cpu, copy.deepcopy(mine))
    run_kernel(gpu, mine)
    compare(cpu, gpu, ("lm_head_rms_out", "logits"))
    assert bool((gpu.logits[1].float() == torch.tensor(-1e9).bfloat16().float()).all())


@pytest.mark.parametrize("make,workers", [(S.mi355x_scheduler, 256), (S.reference_scheduler, 216)])
def test_whole_step_static_list(weights, make, workers):
    """The step's instruction list as the reference builds it per step (lengths and activity fixed in the words)."""
    cpu, gpu = make_pair(weights, 3, (70, 3, 130))
    sched = make(3, MB_SMALL)
    mine = sched.instruction_list(cpu)
    vm_for(sched).run(cpu, copy.deepcopy(mine))
    run_kernel(gpu, mine, workers=workers)
    assert torch.equal(gpu.barriers.cpu(), cpu.barriers)
    tensor_rel_close(gpu.hidden_states, cpu.hidden_states, name="hidden_states")
    rel_close(gpu.logits, cpu.logits, rel=4e-2, name="logits")
    assert gpu.logits.float().argmax(-1).tolist() == cpu.logits.float().argmax(-1).tolist()
    assert torch.equal(gpu.attn_partial_valid.cpu(), cpu.attn_partial_valid)


def test_step_run_column_by_column_equals_the_step_run_whole(weights):
    """`mk_step` / `mk_step_loop` (…/multi_batch/decode_kernel/mk.h:44-115): the step's instruction tensor one column per
    launch, the counters carrying the step from launch to launch, against the same tensor in one launch: every buffer and
    every counter bit for bit; a window without lasting counters and a column outside the tensor are refused."""
    sched = S.mi355x_scheduler(3, MB_SMALL)
    results = []
    for by_column in (False, True):
        cpu, gpu = make_pair(weights, 3, (70, 3, 130), inactive=(1,))
        mk = mk_kernel.get_mk(reset_barriers=False, spin_limit=1 << 18)
        mk_kernel.tensorize_instructions(gpu, S.deal(sched.instruction_list(cpu), 64))   # 64 queues: a couple of dozen columns
        gpu.residual_tiles = (sched.oproj_tile, sched.down_tile)
        gpu.barriers.zero_()
        mk_kernel.call_mk(gpu, mk, column_by_column=by_column)
        mk.check()
        results.append(gpu)
    whole, cols = results
    assert int(whole.instructions.shape[1]) > 10
    for f in dataclasses.fields(whole):
        a, b = getattr(whole, f.name), getattr(cols, f.name)
        if isinstance(a, torch.Tensor):
            assert torch.equal(a, b), f.name
    assert int(whole.barriers.abs().sum()) > 0
    clearing = mk_kernel.get_mk(spin_limit=1 << 18)
    with pytest.raises(ValueError):
        mk_kernel.call_mk(cols, clearing, column_by_column=True)
    args = mk_kernel.QmkBatchArgs()
    ctypes.memmove(ctypes.byref(args), ctypes.byref(mk._args), ctypes.sizeof(args))
    args.first_inst, args.inst_count = int(whole.instructions.shape[1]) - 1, 2      # past the last column
    assert mk._lib.qmk_decode_step_batch(ctypes.byref(args)) != 0
    args.first_inst, args.inst_count, args.flags = 1, 1, 0                           # a window, but counters that are cleared
    assert mk._lib.qmk_decode_step_batch(ctypes.byref(args)) != 0


def test_arrivals_counted_per_xcd_change_no_result(weights):
    """The blocks of the O-projection, the up/gate and the down projection counted on eight sub-counters of their rows
    (QMK_FLAG_XCD_COUNTERS; taken by default when the kernel clears the counters and a row has 256 words) against the
    same step counted on word 0: every buffer bit for bit, the counters cleared; a launch that keeps the counters
    stays with the reference's words, and rows too short for the sub-counters are refused."""
    rows = 8
    sched = S.mi355x_scheduler(rows, MB_SMALL)
    results = []
    for per_xcd in (False, True):
        cpu, gpu = make_pair(weights, rows, (70, 3, 130, 64, 0, 17, 150, 99), inactive=(2,))
        mk = mk_kernel.get_mk(spin_limit=1 << 18, xcd_counters=per_xcd)
        mk_kernel.tensorize_instructions(gpu, sched.runtime_queues(int(gpu.k_cache.shape[2])))
        gpu.residual_tiles = (sched.oproj_tile, sched.down_tile)
        mk_kernel.call_mk(gpu, mk)
        mk.check()
        assert bool(mk._args.flags & 2) == per_xcd
        assert int(gpu.barriers.abs().sum()) == 0
        results.append((gpu, mk))
    (plain, _), (spread, mk) = results
    for f in dataclasses.fields(plain):
        a, b = getattr(plain, f.name), getattr(spread, f.name)
        if isinstance(a, torch.Tensor):
            assert torch.equal(a, b), f.name
    keeping = mk_kernel.get_mk(reset_barriers=False, spin_limit=1 << 18)
    spread.barriers.zero_()
    mk_kernel.call_mk(spread, keeping)
    keeping.check()
    assert keeping._args.flags == 1
    blocks = MB_SMALL.intermediate_size // 16
    assert spread.barriers[:, 6, 0].tolist() == [blocks] * MB_SMALL.num_hidden_layers and int(spread.barriers[:, 6, 1:].abs().sum()) == 0
    args = mk_kernel.QmkBatchArgs()
    ctypes.memmove(ctypes.byref(args), ctypes.byref(mk._args), ctypes.sizeof(args))
    assert args.flags & 2 and args.barrier_slots >= 256
    args.barrier_slots = 255
    assert mk._lib.qmk_decode_step_batch(ctypes.byref(args)) != 0


def test_request_of_the_reference_fixture(weights):
    """Six steps of the recorded request through call_mk with one instruction tensor for the whole request
    and self-clearing counters: tokens, row state and the recorded top-4 logits."""
    g = synthetic.build_batch_globals(weights, MB_SMALL, FIX["kv_capacity"], FIX["rows"], "cuda:0")
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
        ids = torch.tensor(want["my_vm"]["top_ids"], device=g.logits.device)
        got = g.logits.gather(1, ids).view(torch.int16).to(torch.int32).cpu()
        ref = torch.tensor(want["my_vm"]["top_bits"], dtype=torch.int32)
        ref = torch.where(ref >= 32768, ref - 65536, ref)
        assert int((got - ref).abs().max()) <= 8, (step, got.tolist(), ref.tolist())
        nxt = g.logits.float().argmax(dim=-1)
        assert nxt.tolist() == want["my_vm"]["tokens"], step
        state.advance(nxt, [FIX["eos_token"]] if step >= 1 else [])
        tokens = nxt.tolist()
    assert g.active_mask.tolist() == [True, False, True]


@pytest.mark.parametrize("rows", [1, 2, 8, 16])
def test_full_size_layers_against_the_fused_oracle(full_weights, rows):
    """Llama-3.2-1B shape, every batch size class, ragged contexts.  Layer by layer from the oracle's
    residual stream (so that one layer's rounding differences are not amplified by the next):
    hidden states within the bf16 gate (max rel err 2e-2) after every layer, logits within it after the
    LM head, greedy picks identical wherever the oracle has a clear winner."""
    LlamaConfig.set_shape(MB_FULL)
    capacity, w = 320, full_weights
    positions = [(37 * r + 11) % 300 for r in range(rows)]
    cpu, gpu = make_pair(w, rows, positions, inactive=(rows - 1,) if rows >= 8 else (), capacity=capacity, shape=MB_FULL, seed=9)
    toks = torch.tensor([(977 * r + 13) % MB_FULL.vocab_size for r in range(rows)])
    cpu.hidden_states.copy_(cpu.embed_tokens[toks])
    fused, sched = FusedBatchOracle(MB_FULL), S.mi355x_scheduler(rows, MB_FULL)
    live = [r for r in range(rows) if bool(cpu.active_mask[r])]
    done = MB_FULL.hidden_size // sched.down_tile
    p = sched.partials_for_request(cpu)
    gpu.residual_tiles = (sched.oproj_tile, sched.down_tile)
    for layer in range(MB_FULL.num_hidden_layers):
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
                rel_close(gpu.k_cache[layer, r, positions[r]], cpu.k_cache[layer, r, positions[r]], name="k row")   # a rotation: small outputs of larger inputs
                bf16_close(gpu.v_cache[layer, r, positions[r]], cpu.v_cache[layer, r, positions[r]], frac=0.05, name="v row")
            else:
                assert torch.equal(gpu.hidden_states[r].cpu(), before[r])
    gpu.hidden_states.copy_(cpu.hidden_states)
    fused.lm_head(cpu)
    gpu.barriers.zero_()
    gpu.barriers[MB_FULL.num_hidden_layers - 1, 7, 0] = done
    run_kernel(gpu, sched.lmhead_rms() + sched.lmhead())
    rel_close(gpu.logits[live], cpu.logits[live], name="logits")
    top2 = cpu.logits.float().topk(2, dim=-1).values
    for r in range(rows):
        if r not in live:
            assert bool((gpu.logits[r].float() == torch.tensor(-1e9).bfloat16().float()).all())
        elif float(top2[r, 0] - top2[r, 1]) > 2.0 ** -6 * float(top2[r, 0].abs()):   # a clear winner
            assert int(gpu.logits[r].float().argmax()) == int(cpu.logits[r].float().argmax()), r


def test_full_size_step_free_running(full_weights):
    """One whole step at batch 8 through call_mk (run-time template, self-clearing counters) against the
    fused oracle: sixteen layers of rounding differences deep, so the gate is on the tensor's scale."""
    LlamaConfig.set_shape(MB_FULL)
    rows, capacity = 8, 320
    positions = [(37 * r + 11) % 300 for r in range(rows)]
    cpu, gpu = make_pair(full_weights, rows, positions, inactive=(5,), capacity=capacity, shape=MB_FULL, seed=9)
    toks = torch.tensor([(977 * r + 13) % MB_FULL.vocab_size for r in range(rows)])
    cpu.hidden_states.copy_(cpu.embed_tokens[toks])
    sync_state(cpu, gpu)
    FusedBatchOracle(MB_FULL).decode_step(cpu)
    mk = mk_kernel.get_mk(spin_limit=1 << 20)
    mk_kernel.call_mk(gpu, mk)
    mk.check()
    live = [r for r in range(rows) if r != 5]
    err_h = tensor_rel_close(gpu.hidden_states[live], cpu.hidden_states[live], rel=5e-2, name="hidden_states")
    err_l = tensor_rel_close(gpu.logits[live], cpu.logits[live], rel=5e-2, name="logits")
    print(f"free-running step: hidden {err_h:.4f}, logits {err_l:.4f} of the tensor maximum")
    assert torch.equal(gpu.hidden_states[5].cpu(), cpu.hidden_states[5])
    assert int(gpu.barriers.abs().sum()) == 0


def test_decode_loop_as_one_graph(weights):
    """The whole loop of a request — embedding rows, kernel, argmax, row state with one row retiring on an EOS
    token — captured into one HIP graph: the same tokens and row state as launch by launch, on three replays
    with eager work between them."""
    from qimeng_megakernel_amd import decode_batch

    rows, new_tokens = 4, 12
    g = synthetic.build_batch_globals(weights, MB_SMALL, FIX["kv_capacity"], rows, "cuda:0")
    prompts = torch.stack([synthetic.random_prompt(MB_SMALL, 3 + r, 5) for r in range(rows)])
    mk = mk_kernel.get_mk(spin_limit=1 << 18)
    free = decode_batch.decode(g, prompts, new_tokens, mk=mk)["new_tokens"].clone()
    eos = [int(free[2, 4])]                                  # row 2 retires after its fifth new token
    eager = decode_batch.decode(g, prompts, new_tokens, mk=mk, eos_token_ids=eos)
    want, want_active = eager["new_tokens"].clone(), g.active_mask.clone()
    assert not bool(want_active[2]) and bool(want_active[0])
    out = decode_batch.decode(g, prompts, new_tokens, mk=mk, eos_token_ids=eos, use_graph=True)
    assert torch.equal(out["new_tokens"], want) and torch.equal(g.active_mask, want_active)
    for _ in range(2):
        g.logits.zero_()                                     # eager work between replays
        torch.cuda.synchronize()
        again = out["replay"]()
        torch.cuda.synchronize()
        mk.check()
        assert torch.equal(again, want) and torch.equal(g.active_mask, want_active)


def test_position_outside_the_cache_is_reported_not_executed(weights):
    cpu, gpu = make_pair(weights, 3, (70, 3, 130))
    gpu.position_ids[1] = FIX["kv_capacity"]          # one past the last cache row
    before = gpu.hidden_states.clone()
    mk = mk_kernel.get_mk(spin_limit=1 << 12)
    mk_kernel.call_mk(gpu, mk)
    with pytest.raises(RuntimeError, match="operand"):
        mk.check()
    assert torch.equal(gpu.hidden_states, before)
    gpu.barriers.zero_()


# ---- more error paths: forced from the host, every kernel still exits normally -------------------------------------

def _launch(gpu, instructions, **opts):
    mk = mk_kernel.get_mk(reset_barriers=False, **opts)
    mk_kernel.run_instructions(gpu, copy.deepcopy(instructions), mk=mk, workers=8)
    return mk


def test_wait_timeout_drains_the_grid_batch(weights):
    """O-projection tiles wait for attention heads that nobody merges: they run out of polls, say so and retire;
    a well-formed launch afterwards works (the reference's kernel has no bounded wait)."""
    cpu, gpu = make_pair(weights, 3, (70, 3, 130))
    sched = S.mi355x_scheduler(3, MB_SMALL)
    mk = _launch(gpu, sched.oproj(0)[:8], spin_limit=50)
    with pytest.raises(RuntimeError, match="counter wait ran out of polls") as err:
        mk.check()
    assert "opcode=5" in str(err.value)
    gpu.barriers.zero_()
    first = sched.attn_rms(0)
    vm_for(sched).run(cpu, copy.deepcopy(first))
    run_kernel(gpu, first)
    compare(cpu, gpu, ("attn_rms_out",))


def _bad_batch_instructions():
    from qimeng_megakernel_amd.decode_schedule_mb.instructions import instruction_defs as D

    return [
        (D.QKVProj_GEMM_RoPE(9, 3, 0, 0, 1), 1),                                   # layer out of range
        (D.QKVProj_GEMM_RoPE(0, 5, 0, 0, 1), 2),                                   # not the launch's batch size
        (D.QKVProj_GEMM_RoPE(0, 3, 0, 0, 4096), 4),                                # tiles beyond the QKV matrix
        (D.QKVProj_GEMM_RoPE(0, 3, 0, 0, 1, tile_N_granularity=4), 7),             # a tile the kernel is not built for
        (D.DecodeAttentionSplitKV(0, 7, 0, 1, 0), 2),                              # row beyond the batch
        (D.DecodeAttentionSplitKV(0, 0, 99, 1, 0), 3),                             # kv head out of range
        (D.DecodeAttentionSplitKV(0, 0, 0, 999, 0), 4),                            # more partials than the workspace holds
        (D.DecodeAttentionReduction(0, 0, 999, 1, [0]), 3),                        # head group beyond the last head
        (D.DecodeAttentionReduction(0, 0, 0, 1, [999]), 6),                        # partial index beyond the workspace
        (D.OProj_GEMM_Residual(0, 3, 0, 0, 4096, 0), 4),
        (D.UpGateProj_GEMM_SiLU(0, 3, 0, [1 << 20]), 5),                           # block beyond the intermediate size
        (D.DownProj_GEMM_Residual(0, 3, 0, 0, 4096), 4),
        (D.LMHeadProj_GEMM(3, 0, 1 << 20), 3),                                     # rows beyond the vocabulary
    ]


@pytest.mark.parametrize("case", range(13))
def test_bad_operands_are_rejected_on_the_device_batch(weights, case):
    bad, operand = _bad_batch_instructions()[case]
    _, gpu = make_pair(weights, 3, (70, 3, 130))
    names = ("hidden_states", "logits", "q_post_rope", "silu_out", "attn_out", "k_cache", "v_cache")
    before = {n: getattr(gpu, n).clone() for n in names}
    mk = _launch(gpu, [bad])
    with pytest.raises(RuntimeError, match="operand out of bounds") as err:
        mk.check()
    assert f"opcode={bad.opcode()}" in str(err.value) and f"operand={operand}" in str(err.value)
    for n, t in before.items():
        assert torch.equal(getattr(gpu, n), t), n                                   # nothing was written
    assert int(gpu.barriers.abs().sum()) == 0


def test_host_side_checks_batch(weights):
    _, gpu = make_pair(weights, 3, (70, 3, 130))
    mk = mk_kernel.get_mk()
    mk_kernel.build(gpu)
    keep = gpu.instructions
    gpu.instructions = torch.zeros(4096, 1, 32, dtype=torch.int32, device="cuda:0")
    with pytest.raises(RuntimeError, match="co-resident"):
        mk_kernel.call_mk(gpu, mk)
    gpu.instructions = torch.zeros(4, 0, 32, dtype=torch.int32, device="cuda:0")
    mk_kernel.call_mk(gpu, mk)                                                      # empty queues: nothing to launch
    gpu.instructions = keep
    keep, gpu.barriers = gpu.barriers, gpu.barriers[:, :7].contiguous()             # the batch-1 route's counter rows
    with pytest.raises((RuntimeError, ValueError), match="barriers|dimension out of range"):
        mk_kernel.call_mk(gpu, mk)
    gpu.barriers = keep
    mk_kernel.call_mk(gpu, mk)
    mk.check()
