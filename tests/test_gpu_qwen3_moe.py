"""The Qwen3-30B-A3B geometry of the MoE route on the GPU (BASELINE config 5): 32 query heads over 4 KV heads of
128 with the Qwen3 op set's attention, 128 experts of 768 with renormalised top-8 routing, no shared expert.

The reference has no route for this shape; it is its Qwen3 route (attention half:
…/qwen/qwen3__0_6b/A100/single_batch/decode_schedule/{fused/operations.py:52-215, instructions/python_vm.py:110-320})
in front of its MoE route (MoE half: …/qwen/qwen1_5_moe_a2_7b/A100/single_batch/decode_schedule/instructions/
python_vm.py:331-530) with ``norm_topk_prob`` (…/fused/operations.py:405) and without the shared expert's
instructions.  Same checks as for the reference's own MoE shape (tests/test_gpu_moe.py): every op alone against the
sequential VM with counters word for word, whole steps, a request against the fused oracle, the full layer geometry.
"""
import copy
import dataclasses
import json

import pytest
import torch

from conftest import GOLDEN
from fused_moe_oracle import FusedMoeOracle
from gpu_helpers import bf16_close, rel_close, tensor_rel_close
from pyvm_moe_oracle import MoeInstructionVM
from qimeng_megakernel_amd import decode_moe, synthetic
from qimeng_megakernel_amd.decode_schedule_moe import mk_kernel
from qimeng_megakernel_amd.decode_schedule_moe.instructions import scheduler as S
from qimeng_megakernel_amd.decode_schedule_moe.model_config import QWEN1_5_MOE_A2_7B, QWEN3_30B_A3B, QwenMoeConfig, num_partials_for

pytestmark = pytest.mark.gpu

SMALL = dataclasses.replace(QWEN3_30B_A3B, num_hidden_layers=2, vocab_size=2048, num_experts=16, num_experts_per_tok=4,
                            moe_intermediate_size=256)
CAPACITY = 96
MUTABLE = ("hidden_states", "qkv_raw", "q_post_rope", "attn_out", "logits", "k_cache", "v_cache", "attn_out_intermediates",
           "attn_lse_intermediates", "barriers", "router_logits_buf", "normed_hidden_states", "routed_silu_buffer", "routed_out_f32",
           "silu_out", "expert_indices", "expert_weights")


@pytest.fixture(autouse=True)
def _shape():
    QwenMoeConfig.set_shape(SMALL)
    with torch.no_grad():
        yield
    QwenMoeConfig.set_shape(QWEN1_5_MOE_A2_7B)


@pytest.fixture(scope="module")
def weights():
    return synthetic.random_moe_weights(SMALL, 0, CAPACITY)


def sync_state(src, dst):
    for name in MUTABLE:
        getattr(dst, name).copy_(getattr(src, name))
    dst.position_id = src.position_id


def make_pair(weights, shape=SMALL, position=41, token=99, capacity=CAPACITY, max_partials=27):
    cpu = synthetic.build_moe_globals(weights, shape, capacity, "cpu", max_partials=max_partials)
    gpu = synthetic.build_moe_globals(weights, shape, capacity, "cuda:0", max_partials=max_partials)
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


STAGES = ["qkvproj", "attention_split_kv", "attention_reduction", "oproj", "router_gemv", "router_softmax_topk", "routed_upgate",
          "routed_downproj", "combine_commit"]
BF16_OUT = {"qkvproj": ("qkv_raw",), "attention_split_kv": ("q_post_rope", "k_cache", "v_cache"), "attention_reduction": ("attn_out",),
            "oproj": ("hidden_states",), "router_gemv": ("normed_hidden_states",), "routed_upgate": ("routed_silu_buffer", "silu_out"),
            "combine_commit": ("hidden_states",)}


def test_the_stream_has_no_shared_expert_instructions():
    for sched in (S.reference_scheduler(SMALL), mk_kernel.mi355x_scheduler(SMALL), mk_kernel.mi355x_scheduler(QWEN3_30B_A3B)):
        opcodes = {ins.opcode() for ins in sched.instruction_list(1)}
        # (a stream for tagged launches commits in its routed down projections: no opcode 14)
        assert opcodes == {1, 2, 4, 8, 9, 12, 13} | (set() if sched.commit_in_down else {14}) | ({3} if not (sched.merge_in_last or sched.merge_in_oproj) else set())
    full = mk_kernel.mi355x_scheduler(QWEN3_30B_A3B)
    tiles = [ins.tile_N_end_idx - ins.tile_N_start_idx for ins in full.routed_upgate(0)]
    per_queue = [sum(i.tile_N_end_idx - i.tile_N_start_idx for i in q if i.opcode() == 12) for q in full.queues(1)]
    assert sum(tiles) == 8 * 96 and set(per_queue) == {3}          # 768 tiles of 8 outputs: three per queue


@pytest.mark.parametrize("stage", range(len(STAGES)), ids=STAGES)
@pytest.mark.parametrize("position", [41, 0, 95])
def test_one_op_against_the_vm(weights, stage, position):
    """Everything before the op runs on the VM; the op itself on both, from identical state."""
    cpu, gpu = make_pair(weights, position=position)
    sched = dataclasses.replace(mk_kernel.mi355x_scheduler(SMALL, tagged=False), merge_in_last=False, merge_in_oproj=False)
    vm = MoeInstructionVM(SMALL)
    name = STAGES[stage]
    # the combine step adds what the routed down projections left in the launcher's workspace: both run on both sides then
    first = STAGES.index("routed_downproj") if name == "combine_commit" else stage
    for earlier in STAGES[:first]:
        vm.run(cpu, getattr(sched, earlier)(0))
    sync_state(cpu, gpu)
    mine = [ins for part in STAGES[first : stage + 1] for ins in getattr(sched, part)(0)]
    vm.run(cpu, copy.deepcopy(mine))
    mk = run_kernel(gpu, mine)
    assert torch.equal(gpu.barriers.cpu(), cpu.barriers), "counters differ from the VM's"
    for out in BF16_OUT.get(name, ()):
        loose = out in ("q_post_rope", "k_cache", "routed_silu_buffer", "silu_out")
        floor = 2.0 ** -1 if out == "hidden_states" else 2.0 ** -6
        bf16_close(getattr(gpu, out), getattr(cpu, out), ulps=2.0 if loose else 1.0, floor=floor, name=out)
    H = SMALL.hidden_size
    if name == "attention_split_kv":
        g, w = gpu.attn_lse_intermediates.cpu(), cpu.attn_lse_intermediates
        assert torch.equal(torch.isinf(g), torch.isinf(w))
        assert float((g[~torch.isinf(w)] - w[~torch.isinf(w)]).abs().max()) <= 2e-3
        assert float((gpu.attn_out_intermediates.cpu() - cpu.attn_out_intermediates).abs().max()) <= 2e-3 * float(cpu.attn_out_intermediates.abs().max())
        # only the row of this position was written
        assert torch.equal(gpu.k_cache[:, :, :position].cpu(), cpu.k_cache[:, :, :position])
        assert torch.equal(gpu.k_cache[:, :, position + 1:].cpu(), cpu.k_cache[:, :, position + 1:])
    if name == "router_gemv":
        assert torch.allclose(gpu.router_logits_buf.cpu(), cpu.router_logits_buf, rtol=1e-4, atol=1e-5)
    if name == "router_softmax_topk":
        assert gpu.expert_indices.tolist() == cpu.expert_indices.tolist()
        assert torch.allclose(gpu.expert_weights.cpu(), cpu.expert_weights, rtol=1e-5)
        # renormalised: the weights are the picks' softmax probabilities over their own sum
        probs = torch.softmax(gpu.router_logits_buf.cpu().double(), dim=-1)[gpu.expert_indices.cpu()]
        assert torch.allclose(gpu.expert_weights.cpu().double(), probs / probs.sum(), rtol=1e-5)
        assert abs(float(gpu.expert_weights.sum()) - 1.0) < 1e-6
    if name == "routed_downproj":
        parts = mk._workspace[: SMALL.num_experts_per_tok * H * 4].view(torch.float32).view(-1, H).cpu()   # no shared terms in front
        total = torch.zeros(H)
        for j in range(parts.shape[0]):
            total += parts[j]
        assert float((total - cpu.routed_out_f32).abs().max()) <= 2.0 ** -8 * float(cpu.routed_out_f32.abs().max())
    if name == "combine_commit":
        assert float(gpu.routed_out_f32.abs().max()) == 0.0 == float(cpu.routed_out_f32.abs().max())


@pytest.mark.parametrize("tile", [16, 8, 4, 2])
def test_qkv_tiles_of_every_size_give_the_same_rows(weights, tile):
    """The rows per QKV tile are the stream's choice (``QmkMoeArgs.qkv_tile`` fixes what a head's counter ends at): the
    projection's output is the same bits whatever the tile, the counters are the VM's, and the attention that waits on
    them runs.  A stream whose tile is not the launch's is refused on the device; a tile the ABI does not list by the host."""
    shape = dataclasses.replace(SMALL, qkv_tile=tile)
    QwenMoeConfig.set_shape(shape)
    cpu, gpu = make_pair(weights, shape=shape)
    sched = mk_kernel.mi355x_scheduler(shape, tagged=False)
    stream = sched.qkvproj(0) + sched.attention_split_kv(0)
    assert all(i.tile_N_granularity == tile for i in sched.qkvproj(0))
    MoeInstructionVM(shape).run(cpu, copy.deepcopy(stream))
    run_kernel(gpu, stream)
    assert torch.equal(gpu.barriers.cpu(), cpu.barriers) and int(cpu.barriers[0, 0, 0]) == shape.head_dim // tile
    bf16_close(gpu.qkv_raw, cpu.qkv_raw, ulps=1.0, floor=2.0 ** -6, name="qkv_raw")
    if tile != 16:
        QwenMoeConfig.set_shape(SMALL if SMALL.qkv_tile != tile else dataclasses.replace(SMALL, qkv_tile=16))
        other = make_pair(weights)[1]
        QwenMoeConfig.set_shape(shape)
        run_kernel(other, stream)
        assert torch.equal(other.qkv_raw, gpu.qkv_raw)                      # the same rows from tiles of another size
    wrong = dataclasses.replace(shape, qkv_tile=16 if tile != 16 else 8)    # the launch says one tile, the stream another
    QwenMoeConfig.set_shape(wrong)
    mk = mk_kernel.get_mk(reset_barriers=False, spin_limit=1 << 18)
    gpu.barriers.zero_()
    mk_kernel.run_instructions(gpu, copy.deepcopy(sched.qkvproj(0)), mk=mk)
    with pytest.raises(RuntimeError, match="operand"):
        mk.check()
    QwenMoeConfig.set_shape(dataclasses.replace(shape, qkv_tile=6))
    with pytest.raises(RuntimeError, match="dimension out of range"):
        mk_kernel.run_instructions(gpu, copy.deepcopy(sched.qkvproj(0)), mk=mk_kernel.get_mk(reset_barriers=False))


@pytest.mark.parametrize("position,partials", [(41, 3), (0, 2), (95, 6), (95, 8)])
@pytest.mark.parametrize("mode", ["oproj", "last"])
def test_streams_without_reduction_instructions(weights, position, partials, mode):
    """The O-projection instructions merge the partials of all 32 heads themselves (two items per thread), or the
    last split-KV arrival of a KV head merges its eight heads."""
    cpu, gpu = make_pair(weights, position=position)
    sched = dataclasses.replace(mk_kernel.mi355x_scheduler(SMALL, tagged=False), num_partials=partials, merge_in_oproj=mode == "oproj",
                                merge_in_last=mode == "last")
    assert not sched.attention_reduction(0)
    vm = MoeInstructionVM(SMALL)
    vm.run(cpu, sched.qkvproj(0))
    sync_state(cpu, gpu)
    mine = sched.attention_split_kv(0) + sched.oproj(0)
    vm.run(cpu, copy.deepcopy(mine))
    run_kernel(gpu, mine)
    assert torch.equal(gpu.barriers.cpu(), cpu.barriers)
    assert int(cpu.barriers[0, 3, 0]) == SMALL.num_oproj_blocks == 256
    bf16_close(gpu.attn_out, cpu.attn_out, name="attn_out")
    bf16_close(gpu.q_post_rope, cpu.q_post_rope, ulps=2.0, frac=0.03, name="q_post_rope")
    bf16_close(gpu.hidden_states, cpu.hidden_states, ulps=2.0, frac=0.05, floor=2.0 ** -1, name="hidden_states")


def test_lm_head_against_the_vm(weights):
    cpu, gpu = make_pair(weights)
    sched = mk_kernel.mi355x_scheduler(SMALL, tagged=False)
    cpu.barriers[SMALL.num_hidden_layers - 1, 13, 0] = SMALL.num_hidden_blocks
    sync_state(cpu, gpu)
    MoeInstructionVM(SMALL).run(cpu, sched.lmhead())
    run_kernel(gpu, sched.lmhead())
    bf16_close(gpu.logits, cpu.logits, name="logits")


@pytest.mark.parametrize("which", ["dealt_256", "dealt_108", "placed"])
def test_whole_step(weights, which):
    """One step of both layers and the LM head: dealt round-robin on 256 and 108 queues (the reference's protocol with
    reduction instructions), and this build's placed stream."""
    cpu, gpu = make_pair(weights)
    if which == "placed":
        sched, queues = mk_kernel.mi355x_scheduler(SMALL, tagged=False), 256   # a launch on counters: top-k ahead of its consumers
        mine, per_queue = [i for q in sched.queues() for i in q], sched.queues()
    else:
        queues = int(which.split("_")[1])
        sched = S.MoeScheduler(SMALL, queues, min(25, num_partials_for(queues, SMALL)))   # 25: what a reduction instruction lists
        mine, per_queue = sched.instruction_list(), None
    MoeInstructionVM(SMALL).run(cpu, copy.deepcopy(sched.instruction_list()))
    if per_queue is None:
        run_kernel(gpu, mine, queues=queues)
    else:
        from qimeng_megakernel_amd.decode_schedule.instructions.scheduler import tensorize_instructions

        tensorize_instructions(gpu, copy.deepcopy(per_queue))
        mk = mk_kernel.get_mk(reset_barriers=False, spin_limit=1 << 18)
        mk_kernel.call_mk(gpu, mk)
        mk.check()
    assert torch.equal(gpu.barriers.cpu(), cpu.barriers)
    assert gpu.expert_indices.tolist() == cpu.expert_indices.tolist()
    tensor_rel_close(gpu.hidden_states, cpu.hidden_states, name="hidden_states")
    rel_close(gpu.logits, cpu.logits, rel=4e-2, name="logits")
    assert int(gpu.logits.float().argmax()) == int(cpu.logits.float().argmax())


def _margin_ulps(logits):
    top = torch.topk(logits.float().cpu(), 2).values
    return float((top[0] - top[1]) / 2.0 ** (torch.floor(torch.log2(top[0].abs())) - 7))


def test_teacher_forced_request_against_the_fused_oracle(weights):
    """Greedy steps through call_mk (placed stream, tagged units, self-clearing counters) against the fused oracle:
    same routing wherever the oracle's choice is clear, same pick wherever its margin is, logits within the bf16 gate."""
    cpu = synthetic.build_moe_globals(weights, SMALL, CAPACITY, "cpu", max_partials=8)
    gpu = synthetic.build_moe_globals(weights, SMALL, CAPACITY, "cuda:0", max_partials=8)
    oracle, mk = FusedMoeOracle(SMALL), mk_kernel.get_mk(spin_limit=1 << 18)
    tok, agree, steps = 5, 0, 40
    for pos in range(steps):
        for g in (cpu, gpu):
            g.hidden_states.copy_(g.embed_tokens[tok]); g.position_id = pos
        oracle.decode_step(cpu)
        mk_kernel.call_mk(gpu, mk)
        want, got = int(cpu.logits.argmax()), int(gpu.logits.argmax())
        if got == want:
            agree += 1
        else:
            assert _margin_ulps(cpu.logits) <= 2.0, f"step {pos}: kernel {got} vs oracle {want} at a clear margin"
        rel_close(gpu.logits, cpu.logits, rel=4e-2, name=f"logits@{pos}")
        tok = want
    mk.check()
    assert mk._tagged and agree >= 0.85 * steps
    assert int(gpu.barriers.abs().sum()) == 0
    rel_close(gpu.k_cache[:, 0, :steps], cpu.k_cache[:, 0, :steps], rel=4e-2, name="k_cache")


def test_request_of_the_reference_fixture():
    """The request recorded from the reference's own functions put together (tests/golden/make_fixtures_qwen3_moe.py),
    teacher-forced through call_mk: the last layer's routing, the top-4 logits within 8 bf16 ulps, the greedy token
    wherever the reference's margin is clear.  A routing decision may flip only where the reference has the two
    experts within 3 % of each other."""
    fix = json.loads((GOLDEN / "qwen3_moe_reduced_seed0.json").read_text())
    shape = dataclasses.replace(QWEN3_30B_A3B, **fix["shape"])
    QwenMoeConfig.set_shape(shape)
    w = synthetic.random_moe_weights(shape, fix["seed"], fix["kv_capacity"])
    g = synthetic.build_moe_globals(w, shape, fix["kv_capacity"], "cuda:0", max_partials=fix["max_partials"])
    gen = torch.Generator().manual_seed(fix["seed"] + 1)
    g.k_cache.copy_(torch.randn(g.k_cache.shape, generator=gen).bfloat16())
    g.v_cache.copy_(torch.randn(g.v_cache.shape, generator=gen).bfloat16())
    mk = mk_kernel.get_mk(spin_limit=1 << 18)
    token, agree = fix["start_token"], 0
    for step, want in enumerate(fix["steps"]):
        g.position_id = want["position"]
        g.hidden_states.copy_(g.embed_tokens[token])
        mk_kernel.call_mk(g, mk)
        mk.check()
        assert int(g.barriers.abs().sum()) == 0, "the last workgroup clears the counters"
        got_experts, ref_experts = g.expert_indices.tolist(), want["experts_per_layer"][-1]
        if sorted(got_experts) != sorted(ref_experts):
            probs = torch.softmax(g.router_logits_buf.cpu(), dim=-1)
            disputed = sorted(set(got_experts) ^ set(ref_experts))
            assert len(disputed) == 2 and abs(float(probs[disputed[0]] - probs[disputed[1]])) <= 0.03 * float(probs[disputed].max()), (step, disputed)
        else:
            ref_w = dict(zip(ref_experts, want["weights_per_layer"][-1]))
            assert torch.allclose(g.expert_weights.cpu(), torch.tensor([ref_w[e] for e in got_experts]), rtol=2e-2)
            assert abs(float(g.expert_weights.sum()) - 1.0) < 1e-6
        got = g.logits[torch.tensor(want["top_ids"], device=g.logits.device)].view(torch.int16).to(torch.int32).cpu()
        ref = torch.tensor(want["top_bits"], dtype=torch.int32)
        ref = torch.where(ref >= 32768, ref - 65536, ref)
        assert int((got - ref).abs().max()) <= 8, (step, got.tolist(), ref.tolist())
        mine = int(g.logits.float().argmax())
        if mine == want["token"]:
            agree += 1
        else:
            assert int(ref[0] - ref[1]) <= 8, f"step {step}: different pick at a clear margin"
        token = want["token"]
    assert mk._tagged and agree >= len(fix["steps"]) - 1


def test_tagged_and_counter_modes_agree_bit_for_bit(weights):
    out = []
    for tagged in (False, True):
        g = synthetic.build_moe_globals(weights, SMALL, 64, "cuda:0", max_partials=8)
        mk = mk_kernel.get_mk(tagged=tagged, spin_limit=1 << 18)
        tok, toks = 7, []
        for pos in range(16):
            g.hidden_states.copy_(g.embed_tokens[tok]); g.position_id = pos
            mk_kernel.call_mk(g, mk)
            tok = int(g.logits.argmax()); toks.append(tok)
        mk.check()
        assert mk._tagged == tagged
        out.append((g, toks))
    assert out[0][1] == out[1][1]
    for name in ("hidden_states", "qkv_raw", "q_post_rope", "attn_out", "logits", "k_cache", "v_cache", "expert_indices", "expert_weights"):
        assert torch.equal(getattr(out[0][0], name), getattr(out[1][0], name)), name


def test_committing_down_projection_of_sixteen_rows(weights):
    """The tagged stream on 128 queues: every committing down-projection instruction takes two tiles of 8 rows (the
    most the op accepts).  Same bits as the 256-queue stream, whose instructions take one."""
    from qimeng_megakernel_amd.decode_schedule.instructions.scheduler import tensorize_instructions

    out = []
    for queues in (256, 128):
        g = synthetic.build_moe_globals(weights, SMALL, 64, "cuda:0", max_partials=8)
        sched = dataclasses.replace(mk_kernel.mi355x_scheduler(SMALL), sm_count=queues)
        rows = {i.tile_N_granularity * (i.tile_N_end_idx - i.tile_N_start_idx) for q in sched.queues() for i in q if i.opcode() == 13}
        assert rows == ({8} if queues == 256 else {16})
        tensorize_instructions(g, sched.queues())
        mk = mk_kernel.get_mk(spin_limit=1 << 18)
        tok, toks = 7, []
        for pos in range(12):
            g.hidden_states.copy_(g.embed_tokens[tok]); g.position_id = pos
            mk_kernel.call_mk(g, mk)
            tok = int(g.logits.argmax()); toks.append(tok)
        mk.check()
        assert mk._tagged and int(g.instructions.shape[0]) == queues
        out.append((g, toks))
    assert out[0][1] == out[1][1]
    for name in ("hidden_states", "logits", "k_cache", "v_cache", "expert_indices", "expert_weights"):
        assert torch.equal(getattr(out[0][0], name), getattr(out[1][0], name)), name


@pytest.mark.parametrize("bad, operand, tagged", [
    (S.RoutedExpert_DownProj(0, 0, 2, 0, 1, tile_N_granularity=8), 3, False),     # the committing form in a launch on counters
    (S.RoutedExpert_DownProj(0, 1, 2, 0, 1, tile_N_granularity=8), 3, True),      # ... names a slot: it takes all of them
    (S.RoutedExpert_DownProj(0, 0, 2, 0, 3, tile_N_granularity=8), 5, True),      # more than 16 rows
    (S.RoutedExpert_DownProj(0, 0, 2, 0, 1, tile_N_granularity=4), 5, True),      # tiles of 8 or 16 rows only
    (S.RoutedExpert_DownProj(0, 0, 2, 256, 257, tile_N_granularity=8), 5, True),  # rows beyond the hidden size
    (S.RoutedExpert_DownProj(0, 0, 3, 0, 1), 3, True),                            # no such form
])
def test_bad_committing_instructions_are_rejected_on_the_device(weights, bad, operand, tagged):
    """Error paths forced from the host: the kernel refuses the instruction before it writes anything and exits normally."""
    _, gpu = make_pair(weights)
    names = ("hidden_states", "routed_out_f32", "routed_silu_buffer", "k_cache", "logits")
    before = {n: getattr(gpu, n).clone() for n in names}
    from qimeng_megakernel_amd.decode_schedule.instructions.scheduler import tensorize_instructions

    tensorize_instructions(gpu, S.deal([copy.deepcopy(bad)], 8))
    mk = mk_kernel.get_mk(spin_limit=1 << 10) if tagged else mk_kernel.get_mk(reset_barriers=False, spin_limit=1 << 10)
    mk_kernel.call_mk(gpu, mk)
    with pytest.raises(RuntimeError, match="operand out of bounds") as err:
        mk.check()
    assert mk._tagged == tagged and "opcode=13" in str(err.value) and f"operand={operand}" in str(err.value)
    for n, t in before.items():
        assert torch.equal(getattr(gpu, n), t), n


def test_committing_instruction_whose_inputs_never_arrive_runs_out_of_polls(weights):
    """Nobody runs the router: the committing instruction's looks at the logits run out of polls, it says so and the
    grid drains; the launcher clears the workspace, and the next well-formed step works."""
    from qimeng_megakernel_amd.decode_schedule.instructions.scheduler import tensorize_instructions

    _, gpu = make_pair(weights)
    before = gpu.hidden_states.clone()
    tensorize_instructions(gpu, S.deal([S.RoutedExpert_DownProj(0, 0, 2, 0, 1, tile_N_granularity=8)], 8))
    mk = mk_kernel.get_mk(spin_limit=64)
    mk_kernel.call_mk(gpu, mk)
    with pytest.raises(RuntimeError, match="ran out of polls") as err:
        mk.check()
    assert "opcode=13" in str(err.value) and torch.equal(gpu.hidden_states, before)
    assert int(mk._workspace.view(torch.int32).abs().sum()) == 0 and int(gpu.barriers.abs().sum()) == 0
    gpu.instructions = None
    mk = mk_kernel.get_mk(spin_limit=1 << 18)
    mk_kernel.call_mk(gpu, mk)                      # a whole step on the same buffers
    mk.check()
    assert torch.isfinite(gpu.logits.float()).all()


def test_decode_loop_and_graph(weights):
    g = synthetic.build_moe_globals(weights, SMALL, 64, "cuda:0", max_partials=8)
    prompt = torch.tensor([3, 99, 1024, 7])
    mk = mk_kernel.get_mk(spin_limit=1 << 18)
    eager = decode_moe.decode(g, prompt, 12, mk=mk)
    want = eager["new_tokens"].clone()
    assert eager["timing"]["kernel_steps"] == 11 and eager["timing"]["algorithmic_bytes"] > 0
    out = decode_moe.decode(g, prompt, 12, mk=mk, use_graph=True)
    assert torch.equal(out["new_tokens"], want)
    for _ in range(2):
        g.logits.zero_()
        torch.cuda.synchronize()
        assert torch.equal(out["replay"](), want)
    mk.check()


def test_rows_side_by_side_equal_the_rows_alone(weights):
    """Four requests side by side over one copy of the weights (BASELINE's batch 4 on this route: one launch per row and
    step): every row's tokens, logits and cache equal that request decoded alone, and the first row's step follows the
    fused oracle teacher-forced like the batch-1 request does."""
    rows_n, new = 4, 10
    first = synthetic.build_moe_globals(weights, SMALL, 64, "cuda:0", max_partials=8)
    rows = decode_moe.share_weights(first, SMALL, 64, rows_n, max_partials=8)
    assert all(g.qkv_weights.data_ptr() == first.qkv_weights.data_ptr() for g in rows)          # one copy of the weights
    assert len({g.k_cache.data_ptr() for g in rows}) == rows_n                                   # ... and a cache per row
    prompts = torch.tensor([[3, 99, 1024, 7], [5, 5, 5, 5], [2047, 0, 1, 2], [77, 1500, 300, 9]])
    together = decode_moe.decode_rows(rows, prompts, new, timed_steps=4)
    t = together["timing"]
    assert t["kernel_steps"] == 4 and t["kernel_launches"] == 4 * rows_n and t["first_timed_context"] == 4 + (new - 1 - 4) + 1
    assert t["algorithmic_bytes"] == rows_n * sum(SMALL.step_bytes(c) for c in range(t["first_timed_context"], t["last_timed_context"] + 1))
    for r in range(rows_n):
        alone = synthetic.build_moe_globals(weights, SMALL, 64, "cuda:0", max_partials=8)
        want = decode_moe.decode(alone, prompts[r], new, decode_time=False)["new_tokens"]
        assert torch.equal(together["new_tokens"][r], want), r
        assert torch.equal(rows[r].logits, alone.logits) and torch.equal(rows[r].k_cache, alone.k_cache), r
    assert len({tuple(x) for x in together["new_tokens"].tolist()}) == rows_n                    # four different requests


@pytest.mark.slow
def test_full_layer_geometry_layer_by_layer():
    """128 experts of 768, top-8 renormalised, 32/4 heads of 128 — the benchmarked layer, three of them and a reduced
    vocabulary — layer by layer from the VM's residual stream: hidden states within the bf16 gate, identical routing,
    weights that sum to one; then the LM head and the greedy pick at a clear margin."""
    shape = dataclasses.replace(QWEN3_30B_A3B, num_hidden_layers=3, vocab_size=4096)
    QwenMoeConfig.set_shape(shape)
    capacity, pos = 80, 70
    w = synthetic.random_moe_weights(shape, 2, capacity)
    cpu, gpu = make_pair(w, shape=shape, position=pos, token=1234, capacity=capacity, max_partials=8)
    sched, vm = mk_kernel.mi355x_scheduler(shape, tagged=False), MoeInstructionVM(shape)
    assert sched.merge_in_oproj
    from qimeng_megakernel_amd.decode_schedule.instructions.scheduler import tensorize_instructions

    mk = mk_kernel.get_mk(reset_barriers=False, spin_limit=1 << 20)
    for layer in range(shape.num_hidden_layers):
        gpu.hidden_states.copy_(cpu.hidden_states)
        vm.run(cpu, sched.layer(layer))
        gpu.barriers.zero_()
        if layer:
            gpu.barriers[layer - 1, 13, 0] = shape.num_hidden_blocks
        queues = [[] for _ in range(sched.sm_count)]
        sched._place_layer(queues, layer)
        tensorize_instructions(gpu, queues)
        mk_kernel.call_mk(gpu, mk)
        mk.check()
        assert abs(float(gpu.expert_weights.sum()) - 1) < 1e-6
        got, want = gpu.expert_indices.tolist(), cpu.expert_indices.tolist()
        if got != want:
            # each side routes on its own attention output (bf16 roundings apart): with 128 experts two of them can be
            # close enough to change places — only ever two whose probabilities the VM itself has within 3 %
            probs = torch.softmax(cpu.router_logits_buf.double(), dim=-1)
            for a, b in zip(got, want):
                assert a == b or abs(float(probs[a] - probs[b])) <= 0.03 * float(probs[b]), (layer, got, want)
        if sorted(got) != sorted(want):
            continue    # another expert took part: the layer's output is not comparable (the next layer starts from the VM's again)
        if got == want:
            assert torch.allclose(gpu.expert_weights.cpu(), cpu.expert_weights, rtol=5e-3)
        rel_close(gpu.hidden_states, cpu.hidden_states, name=f"hidden_states after layer {layer}")
        rel_close(gpu.k_cache[layer, 0, pos], cpu.k_cache[layer, 0, pos], name=f"k row of layer {layer}")
        bf16_close(gpu.v_cache[layer, 0, pos], cpu.v_cache[layer, 0, pos], frac=0.05, name=f"v row of layer {layer}")
    gpu.hidden_states.copy_(cpu.hidden_states)
    vm.run(cpu, sched.lmhead())
    gpu.barriers.zero_()
    gpu.barriers[shape.num_hidden_layers - 1, 13, 0] = shape.num_hidden_blocks
    run_kernel(gpu, sched.lmhead())
    rel_close(gpu.logits, cpu.logits, name="logits")
    if _margin_ulps(cpu.logits) > 2.0:
        assert int(gpu.logits.argmax()) == int(cpu.logits.argmax())
