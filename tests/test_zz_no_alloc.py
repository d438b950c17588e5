"""qmk_decode_step_static: the decode step with the library's own static workspace, against qmk_decode_step.

The static entry point has no counterpart in the reference; it exists for callers that cannot allocate
device memory.  Both entry points run the same kernels on the same arguments, so every buffer the caller
owns must come out bit for bit the same — in the tagged mode, whose units live in the workspace, and
with device-side sampling, whose candidates do.  Two requests in a row go through the static array, the
second one smaller (fewer layers, a smaller vocabulary, fewer queues), so that it runs on what the first
one left behind: units with old tags, candidates of queues that no longer exist.
"""
import ctypes

import pytest
import torch

from qimeng_megakernel_amd import synthetic
from qimeng_megakernel_amd.decode_schedule import mk_kernel
from qimeng_megakernel_amd.decode_schedule.instructions import scheduler as S
from qimeng_megakernel_amd.decode_schedule.model_config import LlamaConfig

pytestmark = pytest.mark.gpu

CALLER_BUFFERS = ("hidden_states", "q_post_rope", "attn_out", "silu_out", "logits", "k_cache", "v_cache",
                  "attn_out_intermediates", "attn_lse_intermediates", "barriers")


def _request(shape, weights, *, static, steps, queues, kv_capacity=48):
    """Greedy steps with the token picked on the device; returns the buffers and the tokens."""
    LlamaConfig.set_shape(shape)
    g = synthetic.build_globals(weights, shape, kv_capacity, "cuda:0")
    sched = S.mi355x_scheduler(shape, sm_count=queues, kv_capacity=kv_capacity)
    S.tensorize_instructions(g, sched.queues())
    mk = mk_kernel.get_mk(geometry=sched.geometry, static_scratch=static)
    tokens = torch.zeros(steps + 1, dtype=torch.long, device="cuda:0")
    tokens[0] = 7
    g.hidden_states.copy_(g.embed_tokens[7])
    for pos in range(steps):
        g.position_id = pos
        mk.greedy_into(g.embed_tokens, tokens, pos + 1)
        mk_kernel.call_mk(g, mk)
    mk.check()
    assert mk._tagged
    assert (mk._workspace is None) == static
    return g, tokens.tolist()


def _same(a, b):
    for name in CALLER_BUFFERS:
        assert torch.equal(getattr(a, name), getattr(b, name)), name


def test_static_scratch_entry_point_matches_the_allocating_one_twice():
    big = synthetic.reduced_shape(num_layers=3, vocab_size=4096)
    small = synthetic.reduced_shape(num_layers=2, vocab_size=2048)
    w_big = synthetic.random_weights(big, seed=21, max_positions=48)
    w_small = synthetic.random_weights(small, seed=22, max_positions=48)

    want_big, toks_big = _request(big, w_big, static=False, steps=10, queues=256)
    got_big, toks_big_static = _request(big, w_big, static=True, steps=10, queues=256)
    assert toks_big_static == toks_big
    _same(got_big, want_big)

    # the second call: smaller model, half the queues, on the array the first request left behind
    want_small, toks_small = _request(small, w_small, static=False, steps=6, queues=128)
    got_small, toks_small_static = _request(small, w_small, static=True, steps=6, queues=128)
    assert toks_small_static == toks_small
    _same(got_small, want_small)
    assert len(set(toks_small)) > 1 and len(set(toks_big)) > 1


def test_static_scratch_rejects_what_the_array_cannot_hold(small_model):
    shape, w, _ = small_model
    LlamaConfig.set_shape(shape)
    g = synthetic.build_globals(w, shape, 32, "cuda:0")
    S.build(g)
    mk = mk_kernel.get_mk(static_scratch=True)
    g.hidden_states.copy_(g.embed_tokens[3]); g.position_id = 0
    mk_kernel.call_mk(g, mk)           # binds the argument block
    mk.check()
    a = mk._args
    a.flags = mk_kernel.QMK_FLAG_TAGGED
    a.num_layers = 64                  # a tag keeps six bits for the layer
    assert mk._lib.qmk_decode_step_static(ctypes.byref(a)) == 9     # QMK_ERR_SCRATCH
    assert b"static scratch" in mk._lib.qmk_error_string(9)
    a.num_layers = 2
    assert mk._lib.qmk_decode_step_static(ctypes.byref(a)) == 0
    mk.check()


def _chained_request(shape, weights, *, static, steps, tagged=True, capture=False, replays=1, kv_capacity=48):
    """``steps`` chained greedy launches (the kernel writes each token and the next embedding row itself), eager or
    captured into one HIP graph that is replayed ``replays`` times with eager work in between."""
    LlamaConfig.set_shape(shape)
    g = synthetic.build_globals(weights, shape, kv_capacity, "cuda:0")
    sched = S.mi355x_scheduler(shape, sm_count=256, kv_capacity=kv_capacity)
    S.tensorize_instructions(g, sched.queues())
    mk = mk_kernel.get_mk(geometry=sched.geometry, static_scratch=static, tagged=tagged)
    assert mk.query(4) > 0        # QMK_QUERY_MAX_QUEUES: the device is looked up here, outside any capture
    tokens = torch.zeros(steps + 1, dtype=torch.long, device="cuda:0")
    first = g.embed_tokens[7].clone()

    def launches():
        for pos in range(steps):
            g.position_id = pos
            mk.greedy_into(g.embed_tokens, tokens, pos + 1)
            mk_kernel.call_mk(g, mk)

    g.hidden_states.copy_(first)
    if not capture:
        launches()
        mk.check()
        return g, [tokens.tolist()]
    launches()                    # binds the argument block before the capture
    mk.check()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        launches()
    seen = []
    for _ in range(replays):
        g.hidden_states.copy_(first)
        tokens.zero_()
        graph.replay()
        torch.cuda.synchronize()
        mk.check()
        seen.append(tokens.tolist())
        torch.randn(1024, device="cuda:0").sum().item()   # eager work and a synchronisation between replays
    return g, seen


def test_static_entry_point_under_graph_capture_replays_like_the_eager_loop(small_model):
    shape, w, _ = small_model
    want, (toks,) = _chained_request(shape, w, static=False, steps=8)
    got, seen = _chained_request(shape, w, static=True, steps=8, capture=True, replays=3)
    assert all(t == toks for t in seen), (toks, seen)
    _same(got, want)
    assert len(set(toks[1:])) > 1


def test_static_entry_point_sampling_only_without_tagged_units(small_model):
    """Counters carry the hand-overs; only the greedy candidates live in the library's array."""
    shape, w, _ = small_model
    want, (toks,) = _chained_request(shape, w, static=False, steps=6, tagged=False)
    got, (toks_static,) = _chained_request(shape, w, static=True, steps=6, tagged=False)
    assert toks_static == toks
    _same(got, want)
    again, (toks_tagged,) = _chained_request(shape, w, static=True, steps=6, tagged=True)
    assert toks_tagged == toks     # tagged and counter launches agree bit for bit, also through the array
    _same(again, want)
