"""``Globals``: every tensor one decode step touches — the tensor ABI of the route.

Field names and meanings are the reference's
(`…/A100/single_batch/decode_schedule/globs.py:8-41`); shapes for the
Llama-3.2-1B shape are given per field.  Python owns all of it; the kernel
borrows raw device pointers for the duration of one launch.
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass
from typing import Iterator, Optional

import torch

Tensor = torch.Tensor

_WEIGHT_FIELDS = frozenset(
    {
        "attn_norm_weights", "qkv_weights", "rope_cos", "rope_sin", "o_proj_weights",
        "mlp_norm_weights", "up_proj_weights", "gate_proj_weights", "down_proj_weights",
        "lm_head_norm_weights", "lm_head_weights", "q_norm_weights", "k_norm_weights",
    }
)


@dataclass
class Globals:
    # --- instruction stream and inter-workgroup counters -------------------
    instructions: Optional[Tensor] = None            # int32 [queues, len, 32]
    barriers: Optional[Tensor] = None                # int32 [L, 10, 48]
    position_id: Optional[int] = None                # host int: index of the token being decoded

    # --- weights, in the order a layer consumes them ------------------------
    attn_norm_weights: Optional[Tensor] = None       # bf16 [L, H]
    qkv_weights: Optional[Tensor] = None             # bf16 [L, (Hq+2Hkv)*D, H], q/k rows pair-interleaved
    q_norm_weights: Optional[Tensor] = None          # bf16 [L, D]  per-head RMSNorm of q (Qwen3 op set), pair-interleaved
    k_norm_weights: Optional[Tensor] = None          # bf16 [L, D]  per-head RMSNorm of k
    rope_cos: Optional[Tensor] = None                # f32  [max_pos, D], pair-interleaved
    rope_sin: Optional[Tensor] = None                # f32  [max_pos, D]
    o_proj_weights: Optional[Tensor] = None          # bf16 [L, H, H]
    mlp_norm_weights: Optional[Tensor] = None        # bf16 [L, H]
    up_proj_weights: Optional[Tensor] = None         # bf16 [L, F, H]
    gate_proj_weights: Optional[Tensor] = None       # bf16 [L, F, H]
    down_proj_weights: Optional[Tensor] = None       # bf16 [L, H, F]
    lm_head_norm_weights: Optional[Tensor] = None    # bf16 [H]
    lm_head_weights: Optional[Tensor] = None         # bf16 [V, H]

    # --- state and scratch, in the order a layer touches them ---------------
    k_cache: Optional[Tensor] = None                 # bf16 [L, 1, S, Hkv, D]
    v_cache: Optional[Tensor] = None                 # bf16 [L, 1, S, Hkv, D]
    hidden_states: Optional[Tensor] = None           # bf16 [H]   residual stream, in/out
    qkv_raw: Optional[Tensor] = None                 # bf16 [(Hq+2Hkv)*D]  QKV before QK-norm and RoPE (Qwen3 op set)
    q_post_rope: Optional[Tensor] = None             # bf16 [Hq*D]
    attn_out: Optional[Tensor] = None                # bf16 [Hq*D]
    attn_out_intermediates: Optional[Tensor] = None  # f32  [Hq, max_partials, D]
    attn_lse_intermediates: Optional[Tensor] = None  # f32  [Hq, max_partials]   (log2 domain)
    silu_out: Optional[Tensor] = None                # bf16 [F]
    logits: Optional[Tensor] = None                  # bf16 [V]

    # --- prefill-only, sequence-sized (unused by the decode kernel) ---------
    hidden_states_seq: Optional[Tensor] = None
    prefill_q_seq: Optional[Tensor] = None
    attn_out_seq: Optional[Tensor] = None

    def tensor_fields(self) -> Iterator[tuple[str, Tensor]]:
        for f in dataclasses.fields(self):
            value = getattr(self, f.name)
            if isinstance(value, Tensor):
                yield f.name, value

    def diff(self, other: "Globals", skip_kv_cache: bool = False) -> dict[str, tuple[float, float]]:
        """Print and return (max abs diff, mean symmetric rel diff) of every mutable tensor."""
        report: dict[str, tuple[float, float]] = {}
        for name, mine in self.tensor_fields():
            if name in _WEIGHT_FIELDS or (skip_kv_cache and "cache" in name):
                continue
            theirs = getattr(other, name)
            if not isinstance(theirs, Tensor):
                continue
            _, adiff, rdiff = diff_tensors(mine, theirs, name)
            report[name] = (float(adiff.max()), float(rdiff.mean()))
        return report


def diff_tensors(a: Tensor, b: Tensor, name: str):
    a, b = a.float().cpu(), b.float().cpu()
    diff = a - b
    adiff = diff.abs()
    rdiff = 2 * adiff / (a.abs() + b.abs() + 1e-6)
    print(f"{name}: max adiff: {adiff.max()}, mean rdiff: {rdiff.mean()}")
    return diff, adiff, rdiff
