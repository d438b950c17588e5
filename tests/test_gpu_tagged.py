"""Tagged activation hand-over (QMK_FLAG_TAGGED) against the counter protocol.

Both modes execute the same arithmetic in the same order, so whole decode requests must agree
bit for bit in every buffer the caller owns; what differs is only how a workgroup learns that
another one's output has landed.  The reference has one mode (counters,
decode_kernel/*.cu `wait_barrier`/`signal_barrier` sites); the tagged mode has no counterpart there.
"""
import ctypes

import pytest
import torch

from qimeng_megakernel_amd import synthetic
from qimeng_megakernel_amd.decode_schedule import mk_kernel
from qimeng_megakernel_amd.decode_schedule.instructions import scheduler as S
from qimeng_megakernel_amd.decode_schedule.model_config import LLAMA_3_2_1B, LlamaConfig

pytestmark = pytest.mark.gpu

CALLER_BUFFERS = ("hidden_states", "q_post_rope", "attn_out", "silu_out", "logits", "k_cache", "v_cache",
                  "attn_out_intermediates", "attn_lse_intermediates")


def _two_requests(shape, w, steps, kv_capacity=64):
    """The same greedy request on two sets of buffers: counters only, then tagged."""
    LlamaConfig.set_shape(shape)
    out = []
    for tagged in (False, True):
        g = synthetic.build_globals(w, shape, kv_capacity, "cuda:0")
        mk = mk_kernel.get_mk(tagged=tagged)
        tok, toks = 7, []
        for pos in range(steps):
            g.hidden_states.copy_(g.embed_tokens[tok]); g.position_id = pos
            mk_kernel.call_mk(g, mk)
            tok = int(g.logits.argmax()); toks.append(tok)
        mk.check()
        assert mk._tagged == tagged
        out.append((g, toks))
    return out


def test_tagged_and_counter_modes_agree_bit_for_bit(small_model):
    shape, w, _ = small_model
    (plain, toks_p), (tagged, toks_t) = _two_requests(shape, w, steps=24)
    assert toks_p == toks_t
    for name in CALLER_BUFFERS:
        assert torch.equal(getattr(plain, name), getattr(tagged, name)), name
    assert int(tagged.barriers.abs().sum()) == 0 and int(plain.barriers.abs().sum()) == 0


@pytest.mark.slow
def test_tagged_and_counter_modes_agree_full_model():
    shape = LLAMA_3_2_1B
    w = synthetic.random_weights(shape, 0, 40)
    (plain, toks_p), (tagged, toks_t) = _two_requests(shape, w, steps=12, kv_capacity=40)
    assert toks_p == toks_t
    for name in CALLER_BUFFERS:
        assert torch.equal(getattr(plain, name), getattr(tagged, name)), name


def test_tag_that_never_arrives_times_out_and_the_workspace_is_cleared(small_model):
    """Up/gate instructions alone: nobody announces the residual stream they poll for."""
    shape, w, _ = small_model
    LlamaConfig.set_shape(shape)
    g = synthetic.build_globals(w, shape, 32, "cuda:0")
    g.position_id = 3
    sched = S.mi355x_scheduler(shape, num_partials=1)
    mk = mk_kernel.get_mk(spin_limit=40)
    S.tensorize_instructions(g, [[ins] for ins in sched.upgate(0)[:16]])
    mk_kernel.call_mk(g, mk)
    assert mk._tagged
    with pytest.raises(RuntimeError, match="counter wait ran out of polls") as err:
        mk.check()
    assert "opcode=5" in str(err.value)
    assert int(mk._workspace.view(torch.int32).abs().sum()) == 0
    # a whole step afterwards runs and matches the counter protocol
    g.barriers.zero_()
    g.instructions = None
    ref = synthetic.build_globals(w, shape, 32, "cuda:0")
    for gg, m in ((g, mk_kernel.get_mk()), (ref, mk_kernel.get_mk(tagged=False))):
        gg.hidden_states.copy_(gg.embed_tokens[11]); gg.position_id = 0
        mk_kernel.call_mk(gg, m)
        m.check()
    assert torch.equal(g.logits, ref.logits)


def test_tagged_mode_host_side_checks(small_model):
    shape, w, _ = small_model
    LlamaConfig.set_shape(shape)
    g = synthetic.build_globals(w, shape, 32, "cuda:0")
    g.hidden_states.copy_(g.embed_tokens[3]); g.position_id = 0
    mk = mk_kernel.get_mk()
    mk_kernel.call_mk(g, mk)
    mk.check()
    a = mk._args
    assert a.flags & mk_kernel.QMK_FLAG_TAGGED and a.workspace_bytes == mk._lib.qmk_workspace_bytes(0)
    lib, saved = mk._lib, (a.flags, a.workspace, a.workspace_bytes)
    a.flags |= mk_kernel.QMK_FLAG_KEEP_BARRIERS
    assert lib.qmk_decode_step(ctypes.byref(a)) == 3          # QMK_ERR_SHAPE: needs self-clearing counters
    a.flags = saved[0]
    a.workspace_bytes = saved[2] - 8
    assert lib.qmk_decode_step(ctypes.byref(a)) == 3          # workspace too small
    a.workspace_bytes = saved[2]
    a.workspace = saved[1] + 8
    assert lib.qmk_decode_step(ctypes.byref(a)) == 3          # not 128-byte aligned
    a.workspace = None
    assert lib.qmk_decode_step(ctypes.byref(a)) == 1          # QMK_ERR_NULL_ARG
    a.workspace = saved[1]
    torch.cuda.synchronize()
