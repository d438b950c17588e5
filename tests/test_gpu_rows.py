"""The batch route at 1..4 rows on the row-streaming engine (qmk_decode_step_rows) on the GPU.

The reference's batch route (…/llama3_2__1b/A100/multi_batch/) defines a step of B rows as its batch-1 arithmetic per row
(fused/__init__.py runs the single-batch fused operations on [B, H] activations), so the oracle of a row is the batch-1
route on that row.  Every buffer of every active row must equal — bit for bit — what the batch-1 kernel (pinned against the
fused oracle, the VM and the reference's fixture in tests/test_gpu_ops.py, test_gpu_decode.py, test_gpu_golden.py,
test_gpu_qwen3.py) leaves when it decodes the row alone; the logits are also held against the fused batch oracle directly.
"""
import dataclasses

import pytest
import torch

from fused_mb_oracle import FusedBatchOracle
from gpu_helpers import rel_close
from qimeng_megakernel_amd import decode, decode_batch, synthetic
from qimeng_megakernel_amd.decode_schedule import mk_kernel as mk1
from qimeng_megakernel_amd.decode_schedule.instructions import scheduler as S1
from qimeng_megakernel_amd.decode_schedule.instructions.scheduler import tensorize_instructions
from qimeng_megakernel_amd.decode_schedule.model_config import LLAMA_3_2_1B, QWEN3_1_7B, LlamaConfig
from qimeng_megakernel_amd.decode_schedule_mb import rows_kernel

pytestmark = pytest.mark.gpu

SHAPES = {"llama": dataclasses.replace(LLAMA_3_2_1B, num_hidden_layers=2, vocab_size=2048),
          "qwen3": dataclasses.replace(QWEN3_1_7B, num_hidden_layers=2, vocab_size=2048)}
ROW_STATE = ("hidden_states", "q_post_rope", "attn_out", "silu_out", "logits", "attn_out_intermediates", "attn_lse_intermediates")


def _past(g, rows, seed):
    gen = torch.Generator().manual_seed(seed)
    g.k_cache.copy_(torch.randn(g.k_cache.shape, generator=gen).bfloat16())
    g.v_cache.copy_(torch.randn(g.v_cache.shape, generator=gen).bfloat16())
    tokens = torch.randint(0, g.embed_tokens.shape[0], (rows,), generator=gen)
    g.hidden_states.copy_(g.embed_tokens[tokens.to(g.embed_tokens.device)])


def _row_alone(g, weights, shape, row, pos, partials, merge_in_oproj, capacity):
    """Row ``row`` of the batch buffers ``g`` stepped once by the batch-1 kernel on its own copy of the row's state."""
    one = synthetic.build_globals(weights, shape, capacity, "cuda:0", max_partials=int(g.attn_lse_intermediates.shape[-1]))
    one.hidden_states.copy_(g.hidden_states[row])
    one.k_cache.copy_(g.k_cache[:, row : row + 1])
    one.v_cache.copy_(g.v_cache[:, row : row + 1])
    one.position_id = pos
    sched = S1.mi355x_scheduler(shape, num_partials=partials, attention_merge="oproj" if merge_in_oproj else "last", oproj_spares_attention=False)
    tensorize_instructions(one, sched.queues())
    mk = mk1.get_mk(geometry=sched.geometry, spin_limit=1 << 20)
    mk1.call_mk(one, mk)
    mk.check()
    assert mk._tagged
    return one


def _same_row(g, row, one, shape):
    for name in ROW_STATE + (("qkv_raw",) if shape.qk_norm else ()):
        assert torch.equal(getattr(g, name)[row], getattr(one, name)), (row, name)
    assert torch.equal(g.k_cache[:, row], one.k_cache[:, 0]) and torch.equal(g.v_cache[:, row], one.v_cache[:, 0]), row


@pytest.mark.parametrize("merge_in_oproj", [False, True])
@pytest.mark.parametrize("model, positions", [("llama", (41, 41, 41, 41)), ("llama", (70, 3, 41)), ("llama", (0, 95)), ("qwen3", (17, 64, 5, 33)),
                                              ("qwen3", (9,))])
def test_one_step_of_ragged_rows_equals_each_row_alone(model, positions, merge_in_oproj):
    shape = SHAPES[model]
    LlamaConfig.set_shape(shape)
    rows, capacity = len(positions), 96
    w = synthetic.random_weights(shape, 4, capacity)
    g = synthetic.build_batch_globals(w, shape, capacity, rows, "cuda:0")
    _past(g, rows, seed=rows)
    g.position_ids.copy_(torch.tensor(positions, dtype=torch.int32))
    alone = [_row_alone(g, w, shape, r, pos, 2, merge_in_oproj, capacity) for r, pos in enumerate(positions)]
    rows_kernel.build(g, num_partials=2, merge_in_oproj=merge_in_oproj)
    mk = rows_kernel.get_mk(spin_limit=1 << 20)
    rows_kernel.call_mk(g, mk)
    mk.check()
    for r in range(rows):
        _same_row(g, r, alone[r], shape)
    assert int(g.barriers.abs().sum()) == 0


def test_an_inactive_row_is_left_alone():
    shape = SHAPES["llama"]
    LlamaConfig.set_shape(shape)
    w = synthetic.random_weights(shape, 4, 96)
    g = synthetic.build_batch_globals(w, shape, 96, 3, "cuda:0")
    _past(g, 3, seed=9)
    positions = (30, 50, 12)
    g.position_ids.copy_(torch.tensor(positions, dtype=torch.int32))
    g.active_mask.copy_(torch.tensor([True, False, True]))
    before = {n: getattr(g, n)[1].clone() for n in ("hidden_states", "q_post_rope", "attn_out")}
    k_before = g.k_cache[:, 1].clone()
    alone = [_row_alone(g, w, shape, r, positions[r], 2, False, 96) for r in (0, 2)]
    rows_kernel.build(g, num_partials=2)
    mk = rows_kernel.get_mk(spin_limit=1 << 20)
    rows_kernel.call_mk(g, mk)
    mk.check()
    _same_row(g, 0, alone[0], shape)
    _same_row(g, 2, alone[1], shape)
    for n, t in before.items():
        assert torch.equal(getattr(g, n)[1], t), n
    assert torch.equal(g.k_cache[:, 1], k_before)
    assert float(g.logits[1].float().max()) < -9e8 and int(g.silu_out[1].float().abs().sum()) == 0


@pytest.mark.parametrize("model", ["llama", "qwen3"])
def test_requests_decoded_together_equal_the_requests_alone(model):
    """Through the decode loop: every row's tokens, logits and cache rows equal the request decoded alone by the batch-1
    kernel (the stream with the same merge of the split-KV partials); the loop as one HIP graph gives the same tokens."""
    shape = SHAPES[model]
    LlamaConfig.set_shape(shape)
    capacity, new = 64, 12
    w = synthetic.random_weights(shape, 6, capacity)
    prompts = torch.tensor([[3, 99, 1024, 7], [5, 5, 5, 5], [2047, 0, 1, 2], [77, 1500, 300, 9]])
    g = synthetic.build_batch_globals(w, shape, capacity, 4, "cuda:0")
    mk = rows_kernel.get_mk(spin_limit=1 << 20)
    together = decode_batch.decode(g, prompts, new, mk=mk, timed_steps=4)
    assert together["timing"]["engine"] == "rows" and together["timing"]["kernel_steps"] == 4
    tokens = together["new_tokens"].clone()
    logits, cache = g.logits.clone(), g.k_cache.clone()
    for r in range(4):
        one = synthetic.build_globals(w, shape, capacity, "cuda:0")
        S1.build(one)
        sched = dataclasses.replace(S1.scheduler_for(one), attention_merge="last", oproj_spares_attention=False,
                                    num_partials=rows_kernel.mi355x_scheduler(4, shape, kv_capacity=capacity).num_partials)
        mk_one = mk1.get_mk(geometry=sched.geometry, spin_limit=1 << 20)
        toks, tok = [], None
        for pos in range(4 + new - 1):
            tok = int(prompts[r, pos]) if pos < 4 else toks[-1]
            one.hidden_states.copy_(one.embed_tokens[tok]); one.position_id = pos
            tensorize_instructions(one, sched.queues()) if pos == 0 else None
            mk1.call_mk(one, mk_one)
            if pos >= 3:
                toks.append(int(one.logits.argmax()))
        mk_one.check()
        assert tokens[r].tolist() == toks, r
        assert torch.equal(logits[r], one.logits) and torch.equal(cache[:, r], one.k_cache[:, 0]), r
    graphed = decode_batch.decode(g, prompts, new, mk=mk, use_graph=True)
    assert torch.equal(graphed["new_tokens"], tokens)
    for _ in range(2):
        torch.cuda.synchronize()
        assert torch.equal(graphed["replay"](), tokens)
    mk.check()


def test_a_row_that_retires_stops_and_the_others_go_on():
    """An end-of-sequence token retires its row (the row state clears its active flag on the device): from then on the row
    is a hole — position frozen, logits -1e9, so token 0 — and the other rows' tokens are those of the run without it."""
    shape = SHAPES["llama"]
    LlamaConfig.set_shape(shape)
    w = synthetic.random_weights(shape, 6, 64)
    prompts = torch.tensor([[3, 99, 1024, 7], [5, 5, 5, 5], [2047, 0, 1, 2]])
    g = synthetic.build_batch_globals(w, shape, 64, 3, "cuda:0")
    mk = rows_kernel.get_mk(spin_limit=1 << 20)
    free = decode_batch.decode(g, prompts, 14, mk=mk, decode_time=False)["new_tokens"].clone()
    eos = int(free[1, 5])                       # the token row 1 produces at step 5 retires it there
    first = next(i for i in range(14) if int(free[1, i]) == eos)
    out = decode_batch.decode(g, prompts, 14, mk=mk, eos_token_ids=[eos], decode_time=False)["new_tokens"]
    others = [r for r in (0, 2) if eos not in free[r].tolist()]
    assert others, "the chosen token retires every row: pick another seed"
    for r in others:
        assert torch.equal(out[r], free[r]), r
    assert out[1, : first + 1].tolist() == free[1, : first + 1].tolist() and out[1, first + 1 :].abs().sum() == 0
    assert int(g.position_ids[1]) == 4 + first - 1 and not bool(g.active_mask[1])     # frozen where it produced the token


def test_rows_against_the_fused_batch_oracle():
    """Independently of the batch-1 kernel: three ragged rows stepped six times against the fused batch oracle
    (oracle/fused_mb_oracle.py, pinned against the imported reference): logits within the bf16 gate, picks at clear margins."""
    shape = SHAPES["llama"]
    LlamaConfig.set_shape(shape)
    w = synthetic.random_weights(shape, 8, 64)
    cpu = synthetic.build_batch_globals(w, shape, 64, 3, "cpu")
    gpu = synthetic.build_batch_globals(w, shape, 64, 3, "cuda:0")
    _past(cpu, 3, seed=2)
    gpu.k_cache.copy_(cpu.k_cache); gpu.v_cache.copy_(cpu.v_cache)
    oracle = FusedBatchOracle(shape)
    mk = rows_kernel.get_mk(spin_limit=1 << 20)
    start = torch.tensor([40, 3, 21], dtype=torch.int32)
    tokens = torch.tensor([17, 900, 5])
    with torch.no_grad():
        for step in range(6):
            for g in (cpu, gpu):
                g.hidden_states.copy_(g.embed_tokens[tokens.to(g.embed_tokens.device)])
                g.position_ids.copy_(start + step)
            oracle.decode_step(cpu)
            rows_kernel.call_mk(gpu, mk)
            for r in range(3):
                rel_close(gpu.logits[r], cpu.logits[r], rel=4e-2, name=f"logits of row {r} at step {step}")
                top2 = cpu.logits[r].float().topk(2).values
                if float(top2[0] - top2[1]) > 2.0 ** -5:
                    assert int(gpu.logits[r].argmax()) == int(cpu.logits[r].argmax()), (r, step)
            tokens = cpu.logits.argmax(dim=-1)
    mk.check()


def test_error_paths():
    """A row the launch does not have is refused on the device before anything is written; five rows on the host."""
    shape = SHAPES["llama"]
    LlamaConfig.set_shape(shape)
    w = synthetic.random_weights(shape, 4, 32)
    g = synthetic.build_batch_globals(w, shape, 32, 2, "cuda:0")
    _past(g, 2, seed=1)
    before = g.hidden_states.clone()
    bad = rows_kernel.DecodeAttentionSplitKVRow(0, 0, 2, 0, 1, batch_row=2)
    tensorize_instructions(g, S1._round_robin_assign_to_sms([bad], 8))
    mk = rows_kernel.get_mk(spin_limit=1 << 10)
    rows_kernel.call_mk(g, mk)
    with pytest.raises(RuntimeError, match="operand out of bounds") as err:
        mk.check()
    assert "opcode=2" in str(err.value) and "operand=6" in str(err.value) and torch.equal(g.hidden_states, before)
    g.instructions = None
    g.position_ids.copy_(torch.tensor([3, 32], dtype=torch.int32))           # outside the cache
    rows_kernel.call_mk(g, mk)
    with pytest.raises(RuntimeError, match="operand out of bounds") as err:
        mk.check()
    assert "instruction=-1" in str(err.value) and "operand=1" in str(err.value)
    g.position_ids.fill_(3)
    rows_kernel.call_mk(g, rows_kernel.get_mk(spin_limit=1 << 20))            # and a whole step on the same buffers works
    torch.cuda.synchronize()
    assert torch.isfinite(g.logits.float()).all()
    with pytest.raises(ValueError, match="rows"):
        rows_kernel.mi355x_scheduler(5)
    g5 = synthetic.build_batch_globals(w, shape, 32, 5, "cuda:0")
    with pytest.raises(ValueError, match="rows"):
        rows_kernel.call_mk(g5, rows_kernel.get_mk())


@pytest.mark.slow
def test_full_size_llama_four_rows_equal_the_rows_alone():
    """The whole Llama-3.2-1B shape (16 layers, vocabulary 128 256), four rows at contexts up to 1000 over random pasts:
    one launch against one batch-1 launch per row, every buffer of every row bit for bit."""
    shape = LLAMA_3_2_1B
    LlamaConfig.set_shape(shape)
    capacity, positions = 1032, (1000, 17, 480, 256)
    w = synthetic.random_weights(shape, 0, capacity)
    g = synthetic.build_batch_globals(w, shape, capacity, 4, "cuda:0")
    _past(g, 4, seed=13)
    g.position_ids.copy_(torch.tensor(positions, dtype=torch.int32))
    rows_kernel.build(g)
    p = int((g.instructions[..., 0] == 2).sum()) // (16 * 4 * 8)
    alone = [_row_alone(g, w, shape, r, pos, p, False, capacity) for r, pos in enumerate(positions)]
    mk = rows_kernel.get_mk(spin_limit=1 << 20)
    rows_kernel.call_mk(g, mk)
    mk.check()
    for r in range(4):
        _same_row(g, r, alone[r], shape)
