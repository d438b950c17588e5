"""Error paths: every failure is forced from the host and every kernel still exits normally.

A consumer whose counter can never fill (nothing produces it) runs out of its poll budget, records
QMK_DEV_WAIT_TIMEOUT and retires its workgroup; malformed instructions are rejected operand by
operand before any memory is touched.  The reference traps or hangs in these cases
(decode_kernel/mk.cu:82-90; debug/barrier_watchdog.cuh:12-47).
"""
import pytest
import torch

from gpu_helpers import pair
from qimeng_megakernel_amd import synthetic
from qimeng_megakernel_amd.decode_schedule import mk_kernel
from qimeng_megakernel_amd.decode_schedule.instructions import instruction_defs as D
from qimeng_megakernel_amd.decode_schedule.instructions import scheduler as S
from qimeng_megakernel_amd.decode_schedule.model_config import LlamaConfig

pytestmark = pytest.mark.gpu


@pytest.fixture()
def gpu(small_model):
    shape, w, _ = small_model
    LlamaConfig.set_shape(shape)
    g = synthetic.build_globals(w, shape, 32, "cuda:0")
    g.position_id = 3
    return shape, g


def _run(g, instructions, sm_count=4, **opts):
    mk = mk_kernel.get_mk(reset_barriers=False, **opts)
    mk_kernel.run_instructions(g, instructions, mk=mk, sm_count=sm_count)
    return mk


def test_wait_timeout_drains_the_grid(gpu):
    shape, g = gpu
    sched = S.mi355x_scheduler(shape, num_partials=1)
    # O-proj instructions wait for 32 attention heads that nobody will ever publish.
    mk = _run(g, sched.oproj(0)[:8], spin_limit=50)
    with pytest.raises(RuntimeError, match="counter wait ran out of polls") as err:
        mk.check()
    assert "opcode=4" in str(err.value)
    # the status word was cleared by the fetch; a well-formed launch afterwards works
    g.barriers.zero_()
    g.barriers[0, 2, 0] = shape.num_attention_heads
    mk = _run(g, sched.oproj(0), sm_count=64, xcd_counters=False)
    mk.check()
    assert int(g.barriers[0, 3, 0]) == sched.expected_counts()[1]


def test_a_failed_step_leaves_nothing_behind_for_the_next_one(small_model):
    """A whole step that aborts half way (its wait budget is too small for the real waits) leaves counters, an
    arrival word and tagged units of a step that never finished; check() clears them, so the same request
    simply carries on and ends where an undisturbed one ends."""
    shape, w, _ = small_model
    LlamaConfig.set_shape(shape)

    def request(fail_at):
        g = synthetic.build_globals(w, shape, 32, "cuda:0")
        S.build(g)
        mk, tok = mk_kernel.get_mk(), 7
        for pos in range(6):
            g.hidden_states.copy_(g.embed_tokens[tok]); g.position_id = pos
            if pos == fail_at:
                keep = (g.hidden_states.clone(), g.k_cache.clone(), g.v_cache.clone())
                broken = mk.with_options(spin_limit=1)
                mk_kernel.call_mk(g, broken)
                with pytest.raises(RuntimeError, match="ran out of polls|cleared"):
                    broken.check()
                assert int(g.barriers.abs().sum()) == 0
                g.hidden_states.copy_(keep[0]); g.k_cache.copy_(keep[1]); g.v_cache.copy_(keep[2])
            mk_kernel.call_mk(g, mk)
            tok = int(g.logits.argmax())
        mk.check()
        return g, tok

    (plain, tok_plain), (hurt, tok_hurt) = request(None), request(3)
    assert tok_plain == tok_hurt
    for name in ("hidden_states", "logits", "k_cache", "v_cache", "attn_out", "silu_out"):
        assert torch.equal(getattr(plain, name), getattr(hurt, name)), name


def test_xcd_edge_wait_timeout(gpu):
    shape, g = gpu
    sched = S.mi355x_scheduler(shape, num_partials=1)
    mk = mk_kernel.get_mk(reset_barriers=False, spin_limit=20, xcd_counters=True)
    mk_kernel.run_instructions(g, sched.upgate(0)[:32], mk=mk, sm_count=32)   # leaders and followers, nothing arrives
    with pytest.raises(RuntimeError, match="counter wait ran out of polls"):
        mk.check()
    g.barriers.zero_()


@pytest.mark.parametrize("bad, operand", [
    (D.RMS_QKVProj_GEMV_RoPE(7, 0, 0, 4, tile_N_granularity=4), 1),              # layer out of range
    (D.RMS_QKVProj_GEMV_RoPE(0, 0, 700, 800, tile_N_granularity=4), 4),          # rows beyond the QKV matrix
    (D.RMS_QKVProj_GEMV_RoPE(0, 0, 0, 4, tile_N_granularity=6), 6),              # tile does not divide a head
    (D.OProj_GEMV_Residual(0, 0, 0, 300, 0, tile_N_granularity=8), 4),
    (D.DecodeAttentionSplitKV(0, 9, 1, 0), 2),                                   # kv head out of range
    (D.DecodeAttentionSplitKV(0, 0, 64, 0), 3),                                  # more partials than the workspace holds
    (D.DecodeAttentionReduction(0, 30, 1, [0]), 2),                              # head group beyond the last head
    (D.DecodeAttentionReduction(0, 0, 1, [99]), 5),                              # partial index beyond the workspace
    (D.RMS_UpGateProj_GEMV_SiLU(0, 0, [4096], tile_N_granularity=16), 4),        # block beyond the intermediate size
    (D.DownProj_GEMV_Residual(0, 0, 0, 8, 1, tile_N_granularity=8, split_K_granularity=8192), 5),
    (D.DownProj_GEMV_Residual(0, 0, 0, 8, 0, tile_N_granularity=8, split_K_granularity=1000), 8),
    (D.RMS_LMHead_GEMV(0, 5000, tile_N_granularity=16), 2),                      # rows beyond the vocabulary
])
def test_bad_operands_are_rejected_on_the_device(gpu, bad, operand):
    shape, g = gpu
    before = {n: getattr(g, n).clone() for n in ("hidden_states", "logits", "q_post_rope", "silu_out", "attn_out")}
    mk = _run(g, [bad], sm_count=1, xcd_counters=False)
    with pytest.raises(RuntimeError, match="operand out of bounds") as err:
        mk.check()
    assert f"opcode={bad.opcode()}" in str(err.value) and f"operand={operand}" in str(err.value)
    for n, t in before.items():
        assert torch.equal(getattr(g, n), t), n                                   # nothing was written
    g.barriers.zero_()


def test_bad_opcode(gpu):
    shape, g = gpu
    S.tensorize_instructions(g, [[D.NoOp()]])
    g.instructions[0, 0, 0] = 9
    mk = mk_kernel.get_mk()
    mk_kernel.call_mk(g, mk)
    with pytest.raises(RuntimeError, match="unknown opcode"):
        mk.check()


def test_host_side_checks(gpu):
    shape, g = gpu
    mk = mk_kernel.get_mk()
    S.build(g)
    g.position_id = 32                                        # == KV capacity
    with pytest.raises(RuntimeError, match="pos_id outside"):
        mk_kernel.call_mk(g, mk)
    g.position_id = 3
    g.instructions = torch.zeros(4096, 1, 32, dtype=torch.int32, device="cuda:0")
    with pytest.raises(RuntimeError, match="co-resident"):
        mk_kernel.call_mk(g, mk)
    g.instructions = torch.zeros(4, 0, 32, dtype=torch.int32, device="cuda:0")
    mk_kernel.call_mk(g, mk)                                  # empty queues: nothing to launch
    g.instructions = None
    assert mk.query(mk_kernel.QMK_QUERY_CU_COUNT) == 256
    assert mk.query(mk_kernel.QMK_QUERY_MAX_QUEUES) >= 256
    mk.check()
