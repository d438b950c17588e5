"""Kernel vs sequential VM, one op at a time, with the counters pre-filled.

Mirrors the reference's pyvm_to_megakernel stage
(`qimeng_megakernel/verifier/LLM/llama/llama3_2__1b/A100/single_batch/pyvm_to_megakernel/`,
barrier fills per `verifier/common/barrier_fill.py:67-119`): the same instruction
list runs on the CPU VM and through the C ABI on the GPU; outputs must agree
within bf16 rounding and the counters must be identical.
"""
import dataclasses

import pytest
import torch

from gpu_helpers import bf16_close, pair, rel_close, run_both, sync_state
from qimeng_megakernel_amd import synthetic
from qimeng_megakernel_amd.decode_schedule.instructions import instruction_defs as D
from qimeng_megakernel_amd.decode_schedule.instructions import scheduler as S
from qimeng_megakernel_amd.decode_schedule.model_config import LlamaConfig

pytestmark = pytest.mark.gpu


def _sched(shape, which, P=3):
    if which == "mi355x":            # the O-proj workgroups merge the split-KV partials themselves
        return S.mi355x_scheduler(shape, sm_count=256, num_partials=P)
    if which == "mi355x_last":       # the last split-KV arrival of a head group merges
        return S.mi355x_scheduler(shape, sm_count=256, num_partials=P, attention_merge="last")
    if which == "mi355x_unfused":    # MI355X tiles, separate reduction instructions
        return S.mi355x_scheduler(shape, sm_count=256, num_partials=P, attention_merge="separate")
    return S.DecodeScheduler(shape, D.REFERENCE_GEOMETRY, 108, P)


@pytest.fixture()
def state(small_model):
    shape, w, _ = small_model
    LlamaConfig.set_shape(shape)
    cpu, gpu = pair(w, shape)
    gen = torch.Generator().manual_seed(21)
    cpu.hidden_states.copy_((torch.randn(shape.hidden_size, generator=gen) * 0.7).bfloat16())
    cpu.attn_out.copy_(torch.randn(shape.hidden_size, generator=gen).bfloat16())
    cpu.silu_out.copy_((torch.randn(shape.intermediate_size, generator=gen) * 0.3).bfloat16())
    cpu.q_post_rope.copy_(torch.randn(shape.hidden_size, generator=gen).bfloat16())
    cpu.k_cache.copy_(torch.randn(cpu.k_cache.shape, generator=gen).bfloat16())
    cpu.v_cache.copy_(torch.randn(cpu.v_cache.shape, generator=gen).bfloat16())
    cpu.position_id = 41
    return shape, cpu, gpu


@pytest.mark.parametrize("which", ["mi355x", "reference"])
def test_op_qkv_rope(state, which):
    shape, cpu, gpu = state
    sched = _sched(shape, which)
    sync_state(cpu, gpu)
    run_both(cpu, gpu, sched, sched.qkvproj(0))
    bf16_close(gpu.q_post_rope, cpu.q_post_rope, name="q_post_rope")
    bf16_close(gpu.k_cache[0, 0, 41], cpu.k_cache[0, 0, 41], name="k row")
    bf16_close(gpu.v_cache[0, 0, 41], cpu.v_cache[0, 0, 41], name="v row")
    # only the row of this position was touched
    assert torch.equal(gpu.k_cache[0, 0, :41].cpu(), cpu.k_cache[0, 0, :41])
    assert torch.equal(gpu.k_cache[0, 0, 42:].cpu(), cpu.k_cache[0, 0, 42:])
    assert torch.equal(gpu.barriers.cpu(), cpu.barriers)


@pytest.mark.parametrize("which", ["mi355x", "mi355x_last", "mi355x_unfused", "reference"])
@pytest.mark.parametrize("pos,P", [(0, 1), (0, 4), (15, 2), (16, 3), (41, 3), (80, 13), (95, 25)])
def test_op_attention_split_and_reduce(state, which, pos, P):
    shape, cpu, gpu = state
    sched = _sched(shape, which, P)
    cpu.position_id = pos
    cpu.barriers[0, 0, :] = sched.expected_counts()[0]
    cpu.attn_lse_intermediates.fill_(55.0)
    cpu.attn_out_intermediates.fill_(-3.0)
    sync_state(cpu, gpu)
    ins = sched.attention_split_kv(0) + sched.attention_reduction(0)
    if sched.attention_merge == "oproj":
        ins = ins + sched.oproj(0)           # the merge happens in the O-proj prologue
    run_both(cpu, gpu, sched, ins)
    lse_c, lse_g = cpu.attn_lse_intermediates[:, :P], gpu.attn_lse_intermediates[:, :P].cpu()
    assert torch.equal(torch.isinf(lse_c), torch.isinf(lse_g))
    fin = torch.isfinite(lse_c)
    assert (lse_c[fin] - lse_g[fin]).abs().max() < 2e-4
    assert (cpu.attn_out_intermediates[:, :P] - gpu.attn_out_intermediates[:, :P].cpu()).abs().max() < 2e-4
    bf16_close(gpu.attn_out, cpu.attn_out, name="attn_out", frac=0.03)
    assert torch.equal(gpu.barriers.cpu(), cpu.barriers)


@pytest.mark.parametrize("pos,P", [(95, 32), (33, 32), (7, 32), (64, 40)])
def test_op_attention_fan_out_beyond_the_reduction_list(state, pos, P):
    """With the O-proj workgroups merging the partials themselves no instruction lists them, so the
    fan-out may exceed the 25 entries a reduction instruction holds (up to one workgroup per CU and
    KV head); most slices are then shorter than one 16-token tile, many are empty."""
    shape, cpu, gpu = state
    cpu2, gpu2 = pair(synthetic.random_weights(shape, 0, 96), shape, max_partials=P)
    for name in ("hidden_states", "q_post_rope", "k_cache", "v_cache"):
        getattr(cpu2, name).copy_(getattr(cpu, name))
    sched = _sched(shape, "mi355x", P)
    cpu2.position_id = pos
    cpu2.barriers[0, 0, :] = sched.expected_counts()[0]
    sync_state(cpu2, gpu2)
    run_both(cpu2, gpu2, sched, sched.attention_split_kv(0) + sched.oproj(0))
    lse_c, lse_g = cpu2.attn_lse_intermediates[:, :P], gpu2.attn_lse_intermediates[:, :P].cpu()
    assert torch.equal(torch.isinf(lse_c), torch.isinf(lse_g))
    fin = torch.isfinite(lse_c)
    assert (lse_c[fin] - lse_g[fin]).abs().max() < 2e-4
    assert (cpu2.attn_out_intermediates[:, :P] - gpu2.attn_out_intermediates[:, :P].cpu()).abs().max() < 2e-4
    bf16_close(gpu2.attn_out, cpu2.attn_out, name="attn_out", frac=0.03)
    assert torch.equal(gpu2.barriers.cpu(), cpu2.barriers)


@pytest.mark.parametrize("which", ["mi355x", "reference"])
def test_op_oproj(state, which):
    shape, cpu, gpu = state
    sched = _sched(shape, which)
    sched = dataclasses.replace(sched, attention_merge="separate")   # the plain GEMV; the merging form is covered above
    cpu.barriers[0, 2, 0] = shape.num_attention_heads
    sync_state(cpu, gpu)
    run_both(cpu, gpu, sched, sched.oproj(0))
    # addends (hidden ~0.7, projection ~0.9) are O(1): 1 ulp at magnitude 1, wherever the sum lands
    bf16_close(gpu.hidden_states, cpu.hidden_states, floor=1.0, name="hidden")
    assert torch.equal(gpu.barriers.cpu(), cpu.barriers)
    # from a zero residual the result is the rounded projection itself: 1 ulp at its own magnitude
    cpu.hidden_states.zero_(); cpu.barriers.zero_(); cpu.barriers[0, 2, 0] = shape.num_attention_heads
    sync_state(cpu, gpu)
    run_both(cpu, gpu, sched, sched.oproj(0))
    bf16_close(gpu.hidden_states, cpu.hidden_states, name="projection")


@pytest.mark.parametrize("which", ["mi355x", "reference"])
def test_op_upgate(state, which):
    shape, cpu, gpu = state
    sched = _sched(shape, which)
    cpu.barriers[0, 3, 0] = sched.expected_counts()[1]
    sync_state(cpu, gpu)
    run_both(cpu, gpu, sched, sched.upgate(0))
    # silu_out = bf16(bf16(silu(gate)) * up): a 1-ulp difference in up or gate moves the product by up to 2 ulps
    bf16_close(gpu.silu_out, cpu.silu_out, ulps=2.0, frac=0.03, name="silu_out")
    assert torch.equal(gpu.barriers.cpu(), cpu.barriers)


@pytest.mark.parametrize("which", ["mi355x", "reference"])
def test_op_down(state, which):
    shape, cpu, gpu = state
    sched = _sched(shape, which)
    cpu.barriers[0, 4, : sched.geometry.num_split_k(shape)] = sched.expected_counts()[2]
    sync_state(cpu, gpu)
    run_both(cpu, gpu, sched, sched.downproj(0))
    if which == "mi355x":
        bf16_close(gpu.hidden_states, cpu.hidden_states, floor=1.0, name="hidden")
    else:
        # four K slices arrive in any order and every add rounds to bf16: the legal results span a
        # few ulps of the addends' magnitude (the reference gates this with an arrival-order
        # envelope, verifier/common/reduction_order.py:161-243)
        bf16_close(gpu.hidden_states, cpu.hidden_states, ulps=3.0, frac=0.6, floor=1.0, name="hidden")
    assert torch.equal(gpu.barriers.cpu(), cpu.barriers)
    if which == "mi355x":
        cpu.hidden_states.zero_(); cpu.barriers.zero_()
        cpu.barriers[0, 4, : sched.geometry.num_split_k(shape)] = sched.expected_counts()[2]
        sync_state(cpu, gpu)
        run_both(cpu, gpu, sched, sched.downproj(0))
        bf16_close(gpu.hidden_states, cpu.hidden_states, name="projection")


@pytest.mark.parametrize("which", ["mi355x", "reference"])
def test_op_lm_head(state, which):
    shape, cpu, gpu = state
    sched = _sched(shape, which)
    cpu.barriers[shape.num_hidden_layers - 1, 5, 0] = sched.expected_counts()[3]
    sync_state(cpu, gpu)
    run_both(cpu, gpu, sched, sched.lmhead())
    bf16_close(gpu.logits, cpu.logits, name="logits")
    assert torch.equal(gpu.barriers.cpu(), cpu.barriers)


@pytest.mark.parametrize("which", ["mi355x", "reference"])
def test_whole_layer_and_counters(state, which):
    shape, cpu, gpu = state
    sched = _sched(shape, which, P=5)
    sync_state(cpu, gpu)
    run_both(cpu, gpu, sched, sched.instruction_list())
    # one layer from identical state; the reference geometry's four rounded K slices widen the band
    rel = 2e-2 if which == "mi355x" else 4e-2
    rel_close(gpu.hidden_states, cpu.hidden_states, rel=rel, name="hidden")
    rel_close(gpu.logits, cpu.logits, rel=rel, name="logits")
    assert torch.equal(gpu.barriers.cpu(), cpu.barriers)


def test_xcd_sub_counters(state):
    """With room in `barriers`, the all-to-all edges count on eight per-XCD lines: same results,
    rows 3..5 of the protocol untouched, the sub-counters of a GEMV edge summing to its final count, each of the
    attention edge's holding all of it."""
    shape, cpu, gpu = state
    sched = _sched(shape, "mi355x", P=4)
    sync_state(cpu, gpu)
    run_both(cpu, gpu, sched, sched.instruction_list(), xcd_counters=True)
    rel_close(gpu.hidden_states, cpu.hidden_states, rel=2e-2, name="hidden")
    rel_close(gpu.logits, cpu.logits, rel=2e-2, name="logits")
    b = gpu.barriers.cpu()
    assert torch.equal(b[:, :2], cpu.barriers[:, :2])          # per-head rows are the plain protocol
    assert int(b[:, 2:6].abs().sum()) == 0
    bph, opb, ubk, dwn = sched.expected_counts()
    for layer in range(shape.num_hidden_layers):
        flat = b[layer, 10:54].reshape(-1)
        region, flags = flat[: 4 * 8 * 32].reshape(4, 8, 32), flat[4 * 8 * 32 : 8 * 8 * 32].reshape(4, 8, 32)
        # the GEMV edges: an arrival on the sender's XCD's line; the attention edge: every arrival on all eight lines
        assert region[1:, :, 0].sum(dim=1).tolist() == [opb, ubk, dwn]
        assert region[0, :, 0].tolist() == [shape.num_key_value_heads * sched.num_partials] * 8
        assert (region[1:, :, 0] > 0).all()                     # every XCD took part in the GEMV edges
        assert int(region[:, :, 1:].abs().sum()) == 0
        assert set(flags[:, :, 0].reshape(-1).tolist()) <= {0, 1}   # the XCD's ready flag, on a line of its own
        assert int(flags[:, :, 1:].abs().sum()) == 0


def test_single_queue_and_odd_queue_counts(state):
    """The same stream dealt onto 1, 7 and 256 queues gives the same result (in-order queues, no deadlock)."""
    shape, cpu, gpu = state
    sched = S.mi355x_scheduler(shape, num_partials=2)
    results = []
    for sm in (1, 7, 256):
        sync_state(cpu, gpu)
        from qimeng_megakernel_amd.decode_schedule import mk_kernel
        mk = mk_kernel.get_mk(geometry=sched.geometry, reset_barriers=False)
        mk_kernel.run_instructions(gpu, sched.instruction_list(), mk=mk, sm_count=sm)
        mk.check()
        results.append((gpu.hidden_states.clone(), gpu.logits.clone()))
    for h, l in results[1:]:
        assert torch.equal(h, results[0][0]) and torch.equal(l, results[0][1])


def test_parked_upgate_rows_with_ragged_instructions(state):
    """An O-proj that has a wait ahead leaves rows of the up/gate instruction behind it in LDS.  Up/gate instructions
    whose rows are not whole rounds of the eight waves (blocks of 2 outputs dealt for 100 queues: 104, 60 and 56 rows
    per instruction, so the parked rows and the ring's refills exist for some waves only), on few queues so that every
    queue has O-proj instructions in front of its up/gate instructions: the silu vector equals the VM's, and 7 and 13
    queues give bit for bit what 256 give."""
    shape, cpu, gpu = state
    start_hidden, start_silu = cpu.hidden_states.clone(), cpu.silu_out.clone()
    base = S.mi355x_scheduler(shape, sm_count=100, num_partials=2)
    sched = dataclasses.replace(base, geometry=dataclasses.replace(base.geometry, upgate_tile_n=2),
                                attention_merge="separate")   # the plain O-proj GEMV: attn_out is given
    rows = sorted({4 * len(i.tile_N_block_idxs) for i in sched.upgate(0)})
    assert any(r % 8 for r in rows) and max(rows) > 8 * 6      # ragged, and longer than ring + parked rows
    from qimeng_megakernel_amd.decode_schedule import mk_kernel
    first = None
    for sm in (7, 13, 256):
        cpu.barriers.zero_(); cpu.barriers[0, 2, 0] = shape.num_attention_heads
        sync_state(cpu, gpu)
        if first is None:
            run_both(cpu, gpu, sched, [*sched.oproj(0), *sched.upgate(0)], sm_count=sm)
            bf16_close(gpu.silu_out, cpu.silu_out, ulps=2.0, frac=0.03, name="silu_out")
            bf16_close(gpu.hidden_states, cpu.hidden_states, floor=1.0, name="hidden after the O-proj")
            first = (gpu.silu_out.clone(), gpu.hidden_states.clone())
            # the VM has advanced the CPU state: put back what the runs start from
            cpu.hidden_states.copy_(start_hidden); cpu.silu_out.copy_(start_silu)
        else:
            mk = mk_kernel.get_mk(geometry=sched.geometry, reset_barriers=False)
            mk_kernel.run_instructions(gpu, [*sched.oproj(0), *sched.upgate(0)], mk=mk, sm_count=sm)
            mk.check()
            assert torch.equal(gpu.silu_out, first[0]) and torch.equal(gpu.hidden_states, first[1])
