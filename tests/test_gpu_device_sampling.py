"""Greedy step chaining on the device: argmax + embedding lookup folded into the kernel's retirement.

The reference does both on the host between launches (`models/LLM/decode.py:1386-1397`:
``logits.argmax()`` written into the token buffer, then the embedding row copied into
``hidden_states``); the checks below hold the device path to exactly that: the first index of the
largest bf16 logit, and that token's embedding row, bit for bit.
"""
import ctypes

import pytest
import torch

from qimeng_megakernel_amd import decode, synthetic
from qimeng_megakernel_amd.decode_schedule import mk_kernel
from qimeng_megakernel_amd.decode_schedule.model_config import LlamaConfig

pytestmark = pytest.mark.gpu


def _globals(shape, w, kv=64):
    LlamaConfig.set_shape(shape)
    return synthetic.build_globals(w, shape, kv, "cuda:0")


def test_device_token_is_torch_argmax_and_hidden_is_its_embedding(small_model):
    shape, w, _ = small_model
    g = _globals(shape, w)
    mk = mk_kernel.get_mk()
    tokens = torch.full((1, 40), -1, dtype=torch.long, device="cuda:0")
    tok = 5
    for pos in range(30):
        g.hidden_states.copy_(g.embed_tokens[tok]); g.position_id = pos
        mk.greedy_into(g.embed_tokens, tokens, pos + 1)
        mk_kernel.call_mk(g, mk)
        want = int(g.logits.argmax())
        assert int(tokens[0, pos + 1]) == want, pos
        assert torch.equal(g.hidden_states, g.embed_tokens[want]), pos
        tok = want
    mk.check()
    assert int(tokens[0, 0]) == -1 and (tokens[0, 31:] == -1).all()      # nothing else was written
    # a step without greedy_into leaves tokens and hidden_states to the host, as before
    g.hidden_states.copy_(g.embed_tokens[tok]); g.position_id = 30
    mk_kernel.call_mk(g, mk)
    mk.check()
    assert int(tokens[0, 31]) == -1
    assert not torch.equal(g.hidden_states, g.embed_tokens[int(g.logits.argmax())])


def test_ties_go_to_the_first_row_across_workgroups(small_model):
    """Identical LM-head rows give identical logits in every workgroup: the answer must be row 0;
    with row 0 made smaller, the first of the remaining equals."""
    shape, w, _ = small_model
    g = _globals(shape, w)                      # device copies: the fixture's weights stay as they are
    row = g.lm_head_weights[7].clone()
    g.lm_head_weights.copy_(row.expand_as(g.lm_head_weights))
    mk = mk_kernel.get_mk()
    tokens = torch.zeros(1, 4, dtype=torch.long, device="cuda:0")
    g.hidden_states.copy_(g.embed_tokens[3]); g.position_id = 0
    mk.greedy_into(g.embed_tokens, tokens, 1)
    mk_kernel.call_mk(g, mk)
    mk.check()
    assert float(g.logits.float().max()) == float(g.logits.float().min())
    assert int(tokens[0, 1]) == 0 == int(g.logits.argmax())
    # now rows 0..36 lose: flip their sign (or zero them if the common logit is negative/zero)
    common = float(g.logits[0])
    g.lm_head_weights[:37] = -row if common > 0 else torch.zeros_like(row)
    if common <= 0:
        pytest.skip("common logit not positive for this seed; the first case already covered ties")
    g.hidden_states.copy_(g.embed_tokens[3]); g.position_id = 1
    mk.greedy_into(g.embed_tokens, tokens, 2)
    mk_kernel.call_mk(g, mk)
    mk.check()
    assert int(tokens[0, 2]) == 37 == int(g.logits.argmax())


def test_device_sampled_request_equals_host_sampled_request(small_model):
    shape, w, prompt = small_model
    runs = []
    for kw in ({}, {"device_sampling": True}, {"use_graph": True}):
        g = _globals(shape, w, kv=96)
        out = decode.decode(g, prompt, 48, **kw)
        runs.append((out["new_tokens"].clone(), g.k_cache.clone(), g.logits.clone(), out["timing"]))
    for tokens, k_cache, logits, _ in runs[1:]:
        assert torch.equal(tokens, runs[0][0])
        assert torch.equal(k_cache, runs[0][1]) and torch.equal(logits, runs[0][2])
    assert runs[1][3]["kernel_tok_s"] > 0 and runs[2][3]["kernel_tok_s"] == 0 and runs[2][3]["effective_tok_s_gpu"] > 0


def test_graph_of_steps_replays_identically(small_model):
    """One captured graph of 12 chained steps, replayed three times with eager work and
    synchronisation in between; every replay must reproduce the eager request."""
    shape, w, prompt = small_model
    g = _globals(shape, w, kv=64)
    mk = mk_kernel.get_mk()
    n, plen = 12, int(prompt.numel())
    eager = torch.zeros(1, plen + n + 1, dtype=torch.long, device="cuda:0")
    eager[0, :plen] = prompt.to("cuda:0")
    decode.prefill_by_decode(g, mk, prompt, sample_into=(eager, plen))
    start_hidden = g.hidden_states.clone()
    decode.generate_greedy_on_device(g, eager, plen, n, mk=mk)
    mk.check()
    want_tokens, want_logits, want_k = eager.clone(), g.logits.clone(), g.k_cache.clone()

    replayed = torch.zeros_like(eager)
    replayed[0, : plen + 1] = eager[0, : plen + 1]
    g.hidden_states.copy_(start_hidden)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        decode.generate_greedy_on_device(g, replayed, plen, n, mk=mk)
    for _ in range(3):
        replayed[0, plen + 1:] = 0
        g.k_cache[:, :, plen:] = 0
        g.hidden_states.copy_(start_hidden)               # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        mk.check()
        assert torch.equal(replayed, want_tokens)
        assert torch.equal(g.logits, want_logits) and torch.equal(g.k_cache, want_k)


def test_sampling_argument_checks(small_model):
    shape, w, _ = small_model
    g = _globals(shape, w)
    tokens = torch.zeros(4, dtype=torch.long, device="cuda:0")
    with pytest.raises(ValueError, match="self-clearing"):
        mk_kernel.get_mk(reset_barriers=False).greedy_into(g.embed_tokens, tokens, 0)
    mk = mk_kernel.get_mk()
    with pytest.raises(TypeError):
        mk.greedy_into(g.embed_tokens.float(), tokens, 0)
    with pytest.raises(TypeError):
        mk.greedy_into(g.embed_tokens, tokens.int(), 0)
    with pytest.raises(IndexError):
        mk.greedy_into(g.embed_tokens, tokens, 4)
    g.hidden_states.copy_(g.embed_tokens[3]); g.position_id = 0
    mk_kernel.call_mk(g, mk)
    mk.check()
    a = mk._args
    a.token_out = tokens.data_ptr()                              # without the embedding table
    assert mk._lib.qmk_decode_step(ctypes.byref(a)) == 1         # QMK_ERR_NULL_ARG
    a.token_out = None
    torch.cuda.synchronize()
