"""Helpers shared by the GPU parity tests (imported, not collected)."""
from __future__ import annotations

import copy

import torch

from pyvm_oracle import Counts, InstructionVM
from qimeng_megakernel_amd import synthetic
from qimeng_megakernel_amd.decode_schedule import mk_kernel
from qimeng_megakernel_amd.decode_schedule.instructions import scheduler as S

MUTABLE = ("hidden_states", "q_post_rope", "attn_out", "silu_out", "logits", "k_cache", "v_cache",
           "attn_out_intermediates", "attn_lse_intermediates", "barriers")


def sync_state(src, dst) -> None:
    """Copy every mutable buffer of ``src`` onto ``dst`` (across devices)."""
    for name in MUTABLE + ("qkv_raw",):
        if getattr(src, name, None) is not None:
            getattr(dst, name).copy_(getattr(src, name))
    dst.position_id = src.position_id


def pair(weights, shape, kv_capacity=96, max_partials=32):
    cpu = synthetic.build_globals(weights, shape, kv_capacity, "cpu", max_partials=max_partials)
    gpu = synthetic.build_globals(weights, shape, kv_capacity, "cuda:0", max_partials=max_partials)
    return cpu, gpu


def run_both(cpu, gpu, sched, instructions, *, sm_count=None, xcd_counters=False):
    """Execute the same instruction list on the CPU VM and on the kernel, counters kept.

    By default the kernel counts on the reference protocol's rows, so the counter end state can be
    compared word for word; ``xcd_counters=True`` exercises the per-XCD sub-counters instead."""
    vm = InstructionVM(sched.shape, Counts(*sched.expected_counts()))
    vm.run(cpu, copy.deepcopy(instructions))
    mk = mk_kernel.get_mk(geometry=sched.geometry, reset_barriers=False, xcd_counters=xcd_counters)
    mk_kernel.run_instructions(gpu, copy.deepcopy(instructions), mk=mk, sm_count=sm_count or sched.sm_count)
    mk.check()
    return mk


def bf16_close(got: torch.Tensor, want: torch.Tensor, *, ulps: float = 1.0, frac: float = 0.02,
               floor: float = 2.0 ** -6, name: str = "tensor"):
    """bf16 tensors that come from fp32-accumulated dot products of the same inputs: equal except
    where the exact value sits next to a rounding boundary; there, at most ``ulps`` bf16 ulps.
    Tolerance: |diff| <= ulps * ulp_bf16(max(|want|, floor)); at most ``frac`` of the elements differ.
    ``floor`` is the magnitude of the operands that were rounded on the way (for a residual add
    the addends, not the possibly cancelled sum)."""
    got, want = got.detach().float().cpu().reshape(-1), want.detach().float().cpu().reshape(-1)
    assert torch.isfinite(got).all(), f"{name}: non-finite values"
    scale = torch.maximum(want.abs(), torch.tensor(float(floor)))
    ulp = torch.exp2(torch.floor(torch.log2(scale)) - 7)
    diff = (got - want).abs()
    worst = float((diff / ulp).max())
    assert worst <= ulps * 1.001, f"{name}: {worst:.2f} ulps off (allowed {ulps})"
    off = float((diff > 0).float().mean())
    assert off <= frac, f"{name}: {off:.4f} of the elements differ (allowed {frac})"
    return worst, off


def rel_close(got: torch.Tensor, want: torch.Tensor, *, rel: float = 2e-2, name: str = "tensor"):
    """The bf16 gate of the decode path: elementwise |diff| <= rel * max(|want_i|, rms(want)).

    Relative error is taken against the element where it is large enough to carry a meaningful
    ratio and against the tensor's RMS otherwise: the residual stream adds O(1) terms whose own
    bf16 rounding (2^-8 relative) lands on elements that happen to cancel to nearly zero."""
    got, want = got.detach().float().cpu().reshape(-1), want.detach().float().cpu().reshape(-1)
    assert torch.isfinite(got).all(), f"{name}: non-finite values"
    rms = float(want.pow(2).mean().sqrt())
    bound = rel * torch.maximum(want.abs(), torch.tensor(rms))
    ratio = float(((got - want).abs() / bound).max()) * rel
    assert ratio <= rel, f"{name}: max rel err {ratio:.4g} > {rel} (rms {rms:.4g})"
    return ratio


def tensor_rel_close(got: torch.Tensor, want: torch.Tensor, *, rel: float = 2e-2, name: str = "tensor"):
    """max|diff| <= rel * max|want|: the gate for states that are many bf16-rounded residual adds deep
    (after 16 layers the residual stream has taken 32 roundings at magnitudes up to ~16; their
    accumulation-order differences random-walk to a few ulps of the largest elements)."""
    got, want = got.detach().float().cpu().reshape(-1), want.detach().float().cpu().reshape(-1)
    assert torch.isfinite(got).all(), f"{name}: non-finite values"
    err = float((got - want).abs().max()) / float(want.abs().max())
    assert err <= rel, f"{name}: max|diff|/max|ref| = {err:.4g} > {rel}"
    return err
