"""Whole decode requests on the GPU vs the fused CPU oracle (reduced model: 2 layers, vocab 2048)."""
import pytest
import torch

from fused_oracle import FusedOracle
from gpu_helpers import bf16_close, pair
from qimeng_megakernel_amd import decode, synthetic
from qimeng_megakernel_amd.decode_schedule import mk_kernel
from qimeng_megakernel_amd.decode_schedule.model_config import LlamaConfig

pytestmark = pytest.mark.gpu


def test_greedy_matches_oracle_teacher_forced(small_model):
    shape, w, prompt = small_model
    LlamaConfig.set_shape(shape)
    cpu, gpu = pair(w, shape)
    oracle = FusedOracle(shape)
    steps = 40
    want = oracle.greedy(cpu, prompt, steps)
    out = decode.decode(gpu, prompt, steps, decode_time=True)
    got = out["new_tokens"][0].tolist()
    assert got == want, f"first difference at {next(i for i, (a, b) in enumerate(zip(got, want)) if a != b)}"
    # final state: residual stream and logits within bf16 rounding noise accumulated over 2 layers
    assert (gpu.hidden_states.float().cpu() - cpu.hidden_states.float()).abs().max() <= 0.04
    assert (gpu.logits.float().cpu() - cpu.logits.float()).abs().max() <= 0.06
    # KV cache rows written for every position, untouched beyond
    n = prompt.numel() + steps - 1
    assert (gpu.k_cache[:, 0, :n].float().cpu() - cpu.k_cache[:, 0, :n].float()).abs().max() <= 0.07
    assert (gpu.k_cache[:, 0, n:] == 0).all() and (gpu.v_cache[:, 0, n:] == 0).all()
    t = out["timing"]
    assert t["kernel_steps"] == steps - 1 and t["kernel_tok_s"] > 0 and t["decode_window_new_tokens"] == steps - 1
    # the kernel cleared its counters itself
    assert int(gpu.barriers.abs().sum()) == 0


def test_rel_err_per_layer_and_top1(small_model):
    """north-star gate: per-layer hidden max rel err <= 2e-2 (|ref| > 0.05), logit top-1 identical."""
    shape, w, prompt = small_model
    LlamaConfig.set_shape(shape)
    cpu, gpu = pair(w, shape)
    oracle = FusedOracle(shape)
    mk = mk_kernel.get_mk()
    from qimeng_megakernel_amd.decode_schedule.instructions import scheduler as S
    sched = S.scheduler_for(gpu)
    for pos, tok in enumerate(prompt.tolist()):
        for g in (cpu, gpu):
            g.hidden_states.copy_(g.embed_tokens[tok]); g.position_id = pos
        per_layer = []
        oracle.decode_layers(cpu, on_layer=lambda l, g: per_layer.append(g.hidden_states.clone()))
        oracle.lm_head(cpu)
        # the kernel, layer prefix by layer prefix, from the same starting state
        start = gpu.embed_tokens[tok].clone()
        kv = (gpu.k_cache.clone(), gpu.v_cache.clone())
        for nl in range(1, shape.num_hidden_layers + 1):
            gpu.hidden_states.copy_(start); gpu.k_cache.copy_(kv[0]); gpu.v_cache.copy_(kv[1])
            gpu.barriers.zero_()
            mk_kernel.run_instructions(gpu, sched.instruction_list(nl), mk=mk)
            ref = per_layer[nl - 1].float()
            got = gpu.hidden_states.float().cpu()
            big = ref.abs() > 0.05
            assert ((got - ref).abs()[big] / ref.abs()[big]).max() <= 2e-2
            assert (got - ref).abs()[~big].max() <= 2e-3
        gpu.barriers.zero_()
        assert int(gpu.logits.argmax()) == int(cpu.logits.argmax())
        gpu.instructions = None
    mk.check()


def test_reference_built_instruction_stream_runs_unchanged(small_model):
    """An instruction tensor from the A100 scheduler (108 queues, 16-row tiles, 4 K slices) is a valid input."""
    shape, w, prompt = small_model
    LlamaConfig.set_shape(shape)
    cpu, gpu = pair(w, shape)
    from qimeng_megakernel_amd.decode_schedule.instructions import instruction_defs as D
    from qimeng_megakernel_amd.decode_schedule.instructions import scheduler as S
    sched = S.reference_scheduler(shape)
    S.tensorize_instructions(gpu, sched.queues())
    assert tuple(gpu.instructions.shape[::2]) == (108, 32)
    mk = mk_kernel.get_mk(geometry=D.REFERENCE_GEOMETRY)
    oracle = FusedOracle(shape)
    for pos, tok in enumerate(prompt.tolist()):
        for g in (cpu, gpu):
            g.hidden_states.copy_(g.embed_tokens[tok]); g.position_id = pos
        oracle.decode_step(cpu)
        mk_kernel.call_mk(gpu, mk)
        assert int(gpu.logits.argmax()) == int(cpu.logits.argmax())
    mk.check()
    assert (gpu.hidden_states.float().cpu() - cpu.hidden_states.float()).abs().max() <= 0.1
