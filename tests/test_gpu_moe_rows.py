"""Several MoE requests in ONE launch per step (qmk_decode_step_moe_rows) on the GPU: BASELINE config 5 at batch 4.

The reference has no MoE route for batch sizes above one.  A step of B rows is defined as its batch-1 route
(…/qwen/qwen1_5_moe_a2_7b/A100/single_batch/decode_schedule/instructions/python_vm.py:331-530 behind the Qwen3 op
set's attention, …/qwen/qwen3__0_6b/A100/single_batch/decode_schedule/fused/operations.py:52-215) run for every row
on that row's own buffers, so the oracle of a row is the batch-1 oracle on that row: every buffer of every row must
equal — bit for bit — what the batch-1 kernel (itself pinned against the fused oracle and the VM in
tests/test_gpu_qwen3_moe.py) leaves when it decodes the row alone, and the logits are held against the fused oracle
directly as well.
"""
import dataclasses

import pytest
import torch

from fused_moe_oracle import FusedMoeOracle
from gpu_helpers import rel_close
from qimeng_megakernel_amd import decode_moe, synthetic
from qimeng_megakernel_amd.decode_schedule.instructions.scheduler import tensorize_instructions
from qimeng_megakernel_amd.decode_schedule_moe import mk_kernel, rows_kernel
from qimeng_megakernel_amd.decode_schedule_moe.instructions import instruction_defs as D
from qimeng_megakernel_amd.decode_schedule_moe.instructions import scheduler as S
from qimeng_megakernel_amd.decode_schedule_moe.model_config import QWEN1_5_MOE_A2_7B, QWEN3_30B_A3B, QwenMoeConfig

pytestmark = pytest.mark.gpu

SMALL = dataclasses.replace(QWEN3_30B_A3B, num_hidden_layers=2, vocab_size=2048, num_experts=16, num_experts_per_tok=4,
                            moe_intermediate_size=256)
# every buffer a step leaves behind for its request (the split-KV workspaces included: same fan-out on both sides)
ROW_STATE = ("hidden_states", "qkv_raw", "q_post_rope", "attn_out", "logits", "k_cache", "v_cache", "attn_out_intermediates",
             "attn_lse_intermediates", "router_logits_buf", "normed_hidden_states", "routed_silu_buffer", "routed_out_f32", "silu_out",
             "expert_indices", "expert_weights")


@pytest.fixture(autouse=True)
def _shape():
    QwenMoeConfig.set_shape(SMALL)
    with torch.no_grad():
        yield
    QwenMoeConfig.set_shape(QWEN1_5_MOE_A2_7B)


@pytest.fixture(scope="module")
def weights():
    return synthetic.random_moe_weights(SMALL, 0, 96)


def _fill_state(g, rows, seed):
    """A random past for every row: KV caches ~N(0,1), residual streams from embedding rows."""
    gen = torch.Generator().manual_seed(seed)
    g.k_cache.copy_(torch.randn(g.k_cache.shape, generator=gen).bfloat16())
    g.v_cache.copy_(torch.randn(g.v_cache.shape, generator=gen).bfloat16())
    tokens = torch.randint(0, g.embed_tokens.shape[0], (rows,), generator=gen)
    g.hidden_states.copy_(g.embed_tokens[tokens.to(g.embed_tokens.device)])


def _rows_alone(g, shape, positions, partials, merge_in_oproj):
    """Every row of ``g`` stepped once by the batch-1 kernel on a copy of the row's buffers; the copies.  The batch-1
    stream merges the split-KV partials where the rows stream does (in the O-projection workgroups, or by the last arrival
    of a KV head: ``num * (1 / den)`` there, ``num / den`` here)."""
    out = []
    for r, pos in enumerate(positions):
        view = rows_kernel.row_view(g, r)
        alone = dataclasses.replace(view)
        for name in ROW_STATE:
            setattr(alone, name, getattr(view, name).clone())
        alone.position_id = pos
        sched = dataclasses.replace(mk_kernel.mi355x_scheduler(shape, kv_capacity=int(g.k_cache.shape[3])), num_partials=partials,
                                    merge_in_oproj=merge_in_oproj, merge_in_last=not merge_in_oproj)
        tensorize_instructions(alone, sched.queues())
        mk = mk_kernel.get_mk(spin_limit=1 << 20)
        mk_kernel.call_mk(alone, mk)
        mk.check()
        assert mk._tagged
        out.append(alone)
    return out


@pytest.mark.parametrize("merge_in_oproj", [False, True])
@pytest.mark.parametrize("positions", [(41, 41, 41, 41), (70, 3, 41), (0, 95), (17,)])
def test_one_step_of_ragged_rows_equals_each_row_alone(weights, positions, merge_in_oproj):
    """Rows at different positions over random pasts: one launch for all of them against one batch-1 launch per row."""
    rows = len(positions)
    g = rows_kernel.build_rows_globals(weights, SMALL, 96, rows, "cuda:0", max_partials=8)
    _fill_state(g, rows, seed=3 + rows)
    g.position_ids.copy_(torch.tensor(positions, dtype=torch.int32))
    alone = _rows_alone(g, SMALL, positions, partials=2, merge_in_oproj=merge_in_oproj)
    rows_kernel.build(g, num_partials=2, merge_in_oproj=merge_in_oproj)
    mk = rows_kernel.get_mk(spin_limit=1 << 20)
    mk(g)
    mk.check()
    for r in range(rows):
        for name in ROW_STATE:
            assert torch.equal(getattr(g, name)[r], getattr(alone[r], name)), (r, name)
    assert int(g.barriers.abs().sum()) == 0                                  # the last workgroup cleared the counters
    picks = {int(e) for e in g.expert_indices.flatten().tolist()}            # the last layer's picks of all rows
    assert int(g.distinct_experts[SMALL.num_hidden_layers - 1]) == len(picks)
    assert all(1 <= int(n) <= rows * SMALL.num_experts_per_tok for n in g.distinct_experts.tolist())
    for r in range(rows):
        assert abs(float(g.expert_weights[r].sum()) - 1.0) < 1e-6            # renormalised


def test_requests_decoded_together_equal_the_requests_alone(weights):
    """Four requests through the decode loop, one launch per step: every row's tokens, logits and caches equal the
    request decoded alone on the batch-1 kernel; rows that pick the same expert share its rows."""
    new = 10
    prompts = torch.tensor([[3, 99, 1024, 7], [5, 5, 5, 5], [2047, 0, 1, 2], [77, 1500, 300, 9]])
    g = rows_kernel.build_rows_globals(weights, SMALL, 64, 4, "cuda:0", max_partials=8)
    together = decode_moe.decode_batch(g, prompts, new, timed_steps=4, merge_in_oproj=True)   # the default batch-1 request's bits
    t = together["timing"]
    assert t["kernel_steps"] == 4 and t["kernel_launches"] == 4 and t["first_timed_context"] == 4 + (new - 1 - 4) + 1
    assert 1.0 <= t["distinct_experts_per_layer"] <= 16.0
    assert t["algorithmic_bytes"] < t["moved_if_rows_alone"]
    for r in range(4):
        alone = synthetic.build_moe_globals(weights, SMALL, 64, "cuda:0", max_partials=8)
        want = decode_moe.decode(alone, prompts[r], new, decode_time=False)["new_tokens"]
        assert torch.equal(together["new_tokens"][r], want), r
        assert torch.equal(g.logits[r], alone.logits) and torch.equal(g.k_cache[r], alone.k_cache) and torch.equal(g.v_cache[r], alone.v_cache), r
    assert len({tuple(x) for x in together["new_tokens"].tolist()}) == 4
    # identical requests pick identical experts: the list of distinct experts is as long as one row's picks
    same = torch.tensor([[3, 99, 1024, 7]] * 3)
    g3 = rows_kernel.build_rows_globals(weights, SMALL, 64, 3, "cuda:0", max_partials=8)
    out = decode_moe.decode_batch(g3, same, 6, timed_steps=2, merge_in_oproj=True)
    assert out["timing"]["distinct_experts_per_layer"] == SMALL.num_experts_per_tok
    assert torch.equal(out["new_tokens"][0], out["new_tokens"][1]) and torch.equal(out["new_tokens"][0], out["new_tokens"][2])
    assert torch.equal(out["new_tokens"][0], together["new_tokens"][0][:6])


class _RecordingOracle(FusedMoeOracle):
    """The fused oracle, noting per step how clearly it routed: the smallest relative gap, over the layers, between the
    last expert it picked and the first one it did not."""

    def router(self, g, layer, normed):
        super().router(g, layer, normed)
        logits = torch.nn.functional.linear(normed.float().unsqueeze(0), g.router_weights[layer].float()).squeeze(0)
        p = torch.softmax(logits, dim=-1).sort(descending=True).values
        k = self.shape.num_experts_per_tok
        self.gap = min(getattr(self, "gap", 1.0), float((p[k - 1] - p[k]) / p[k - 1]))


def test_teacher_forced_rows_follow_the_fused_oracle(weights):
    """Independently of the batch-1 kernel: three rows teacher-forced with the oracle's tokens, every row's logits
    within the bf16 gate of the fused oracle run on that row alone and the same pick at clear margins — on every step
    the oracle itself routes clearly (its k-th and (k+1)-th expert more than 3 % apart in every layer: each side routes
    on its own bf16 residual stream, and two experts that close may change places, which changes the step's output)."""
    rows, steps = 3, 10
    prompts = [[3, 99], [5, 1500], [2047, 0]]
    g = rows_kernel.build_rows_globals(weights, SMALL, 32, rows, "cuda:0", max_partials=8)
    rows_kernel.build(g)
    mk = rows_kernel.get_mk(spin_limit=1 << 20)
    oracle = _RecordingOracle(SMALL)
    cpus = [synthetic.build_moe_globals(weights, SMALL, 32, "cpu", max_partials=8) for _ in range(rows)]
    tokens = [list(p) for p in prompts]
    clear = total = 0
    for pos in range(len(prompts[0]) + steps):
        feed = torch.tensor([tokens[r][pos] for r in range(rows)])
        g.hidden_states.copy_(g.embed_tokens[feed.to("cuda:0")])
        g.position_ids.fill_(pos)
        mk(g)
        for r in range(rows):
            cpus[r].hidden_states.copy_(cpus[r].embed_tokens[feed[r]])
            cpus[r].position_id = pos
            oracle.gap = 1.0
            oracle.decode_step(cpus[r])
            total += 1
            if oracle.gap > 0.03:
                clear += 1
                rel_close(g.logits[r], cpus[r].logits, rel=4e-2, name=f"logits of row {r} at position {pos}")
                top2 = cpus[r].logits.float().topk(2).values
                if float(top2[0] - top2[1]) > 2.0 ** -5:
                    assert int(g.logits[r].argmax()) == int(cpus[r].logits.argmax()), (r, pos)
            if pos + 1 >= len(prompts[r]):
                tokens[r].append(int(cpus[r].logits.argmax()))
    mk.check()
    assert clear >= 0.6 * total, (clear, total)
    # the caches hold what every step appended, whatever the routing did afterwards in its layer... of layer 0 exactly so
    for r in range(rows):
        rel_close(g.k_cache[r, 0, 0, : len(prompts[0]) + steps], cpus[r].k_cache[0, 0, : len(prompts[0]) + steps], rel=4e-2, name=f"k rows of row {r}")


@pytest.mark.parametrize("bad, opcode, operand", [
    (D.DecodeAttentionSplitKVRow(0, 0, 2, 0, merge_in_last=2, batch_row=2), 2, 6),   # a row the launch does not have
    (D.Router_SoftmaxTopKRow(0, batch_row=-1), 9, 2),
    (D.RoutedExperts_UpGate_Rows(0, 8, 8), 15, 2),                                   # part 8 of 8
    (D.RoutedExperts_DownCommit_Rows(0, 0, 3, 8), 16, 3),                            # more than 16 rows
    (D.RoutedExperts_DownCommit_Rows(0, 0, 1, 4), 16, 3),                            # tiles of 8 or 16 rows only
    (D.OProj_GEMV_Residual(0, 0, 0, 1, 65, tile_N_granularity=8), 4, 5),             # a fan-out beyond what a workgroup merges
])
def test_bad_instructions_are_rejected_on_the_device(weights, bad, opcode, operand):
    """Error paths forced from the host: the kernel refuses the instruction before it writes anything and exits normally."""
    g = rows_kernel.build_rows_globals(weights, SMALL, 32, 2, "cuda:0", max_partials=8)
    _fill_state(g, 2, seed=1)
    before = {n: getattr(g, n).clone() for n in ("hidden_states", "k_cache", "routed_silu_buffer", "logits")}
    tensorize_instructions(g, S.deal([bad], 8))
    mk = rows_kernel.get_mk(spin_limit=1 << 10)
    mk(g)
    with pytest.raises(RuntimeError, match="operand out of bounds") as err:
        mk.check()
    assert f"opcode={opcode}" in str(err.value) and f"operand={operand}" in str(err.value)
    for n, t in before.items():
        assert torch.equal(getattr(g, n), t), n


def test_a_wait_that_cannot_complete_runs_out_of_polls_and_the_next_step_works(weights):
    """Nobody runs the router: the gate/up instruction's looks run out of polls, it says so and the grid drains; the
    launcher clears counters and workspace, and a whole step on the same buffers then works.  A position outside the
    cache is refused before anything runs."""
    g = rows_kernel.build_rows_globals(weights, SMALL, 32, 2, "cuda:0", max_partials=8)
    _fill_state(g, 2, seed=2)
    before = g.hidden_states.clone()
    tensorize_instructions(g, S.deal([D.RoutedExperts_UpGate_Rows(0, q, 8) for q in range(8)], 8))
    mk = rows_kernel.get_mk(spin_limit=64)
    mk(g)
    with pytest.raises(RuntimeError, match="ran out of polls") as err:
        mk.check()
    assert "opcode=15" in str(err.value) and torch.equal(g.hidden_states, before)
    assert int(mk._workspace.view(torch.int32).abs().sum()) == 0 and int(g.barriers.abs().sum()) == 0
    g.instructions = None
    mk = rows_kernel.get_mk(spin_limit=1 << 20)
    g.position_ids.copy_(torch.tensor([5, 9], dtype=torch.int32))
    mk(g)
    mk.check()
    assert torch.isfinite(g.logits.float()).all()
    g.position_ids.copy_(torch.tensor([5, 32], dtype=torch.int32))
    mk(g)
    with pytest.raises(RuntimeError, match="operand out of bounds") as err:
        mk.check()
    assert "instruction=-1" in str(err.value) and "operand=1" in str(err.value)


def test_host_side_checks(weights):
    g = rows_kernel.build_rows_globals(weights, SMALL, 32, 2, "cuda:0", max_partials=8)
    rows_kernel.build(g)
    mk = rows_kernel.get_mk()
    g.position_ids = g.position_ids.long()
    with pytest.raises(ValueError, match="position_ids"):
        mk(g)
    g.position_ids = torch.zeros(2, dtype=torch.int32, device="cuda:0")
    g.logits = g.logits[:1].contiguous()
    with pytest.raises(ValueError, match="logits has"):
        mk(g)
    with pytest.raises(ValueError, match="rows"):
        rows_kernel.build_rows_globals(weights, SMALL, 32, 5, "cuda:0")
    QwenMoeConfig.set_shape(QWEN1_5_MOE_A2_7B)
    with pytest.raises(ValueError, match="shared expert"):
        rows_kernel.mi355x_scheduler(2)


@pytest.mark.slow
def test_full_layer_geometry_four_rows_equal_the_rows_alone():
    """128 experts of 768, renormalised top-8, 32/4 heads of 128 — the benchmarked layer, three of them and a reduced
    vocabulary: four rows at different positions in one launch against the batch-1 kernel row by row, every buffer bit
    for bit; the four rows' 32 picks per layer land on fewer distinct experts than that only by coincidence, never more."""
    shape = dataclasses.replace(QWEN3_30B_A3B, num_hidden_layers=3, vocab_size=4096)
    QwenMoeConfig.set_shape(shape)
    w = synthetic.random_moe_weights(shape, 2, 300)
    positions = (290, 12, 131, 64)
    g = rows_kernel.build_rows_globals(w, shape, 300, 4, "cuda:0", max_partials=8)
    _fill_state(g, 4, seed=11)
    g.position_ids.copy_(torch.tensor(positions, dtype=torch.int32))
    alone = _rows_alone(g, shape, positions, partials=4, merge_in_oproj=False)
    rows_kernel.build(g)
    assert int((g.instructions[..., 0] == 2).sum()) == 3 * 4 * 4 * 4        # layers x rows x KV heads x slices
    mk = rows_kernel.get_mk(spin_limit=1 << 20)
    mk(g)
    mk.check()
    for r in range(4):
        for name in ROW_STATE:
            assert torch.equal(getattr(g, name)[r], getattr(alone[r], name)), (r, name)
    assert all(8 <= int(n) <= 32 for n in g.distinct_experts.tolist())
