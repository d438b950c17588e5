"""Seeded random-init weights and ``Globals`` allocation for the decode route.

Stands in for the reference's checkpoint loader and buffer allocation when no
checkpoint is available:

* weight layout: per-layer matrices stacked ``[L, out, in]``, q/k rows of the
  QKV matrix pair-interleaved per head (`LLM/llama/preprocess.py:21-83`);
* RoPE tables: plain-theta ``cos/sin(pos * theta^(-2i/d))`` in fp32, columns
  pair-interleaved the same way (`LLM/llama/load_weights.py:37-74`);
* buffers: `…/A100/fused_prefill.py:38-160` (KV cache ``[L,1,S,Hkv,D]``, fp32
  split-KV workspaces, int32 counters ``[L,10,48]``).

Random weights are drawn on a CPU generator, so a seed names the same model on
every machine.  A random-init matrix is its own interleaved version in
distribution, so no row permutation is applied to it.
"""
from __future__ import annotations

import dataclasses
from typing import Any

import torch

from .decode_schedule.globs import Globals
from .decode_schedule.model_config import DecodeShape, LlamaConfig

BARRIER_ROWS = 10          # the reference's allocation
XCD_COUNTER_ROWS = 54      # rows 10..53 hold the per-XCD sub-counters of the all-to-all edges
WEIGHT_STD = 0.02


def interleave_indices(head_dim: int) -> torch.Tensor:
    """Column order [0, d/2, 1, d/2+1, ...]: rotate-half partners become neighbours."""
    half = head_dim // 2
    return torch.stack((torch.arange(half), torch.arange(half) + half), dim=1).reshape(-1)


def rope_tables(shape: DecodeShape, max_positions: int) -> tuple[torch.Tensor, torch.Tensor]:
    """fp32 ``[max_positions, head_dim]`` cos/sin in the pair-interleaved layout."""
    d = shape.head_dim
    inv_freq = 1.0 / (shape.rope_theta ** (torch.arange(0, d, 2, dtype=torch.int64).float() / d))
    freqs = torch.outer(torch.arange(max_positions, dtype=torch.float32), inv_freq)
    emb = torch.cat((freqs, freqs), dim=-1)
    idx = interleave_indices(d)
    return emb.cos()[:, idx].contiguous(), emb.sin()[:, idx].contiguous()


def _normal_bf16(gen: torch.Generator, *size: int) -> torch.Tensor:
    # Drawn layer by layer in fp32, stored as bf16: peak host memory stays at one matrix.
    return (torch.randn(*size, generator=gen, dtype=torch.float32) * WEIGHT_STD).to(torch.bfloat16)


def random_weights(shape: DecodeShape, seed: int, max_positions: int) -> dict[str, torch.Tensor]:
    """bf16 ~N(0, 0.02) projections and embeddings, unit norm weights, untied LM head (CPU tensors)."""
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed)
    L, H, F, V = shape.num_hidden_layers, shape.hidden_size, shape.intermediate_size, shape.vocab_size
    w: dict[str, torch.Tensor] = {}
    w["embed_tokens"] = _normal_bf16(gen, V, H)
    w["qkv_weights"] = torch.stack([_normal_bf16(gen, shape.qkv_out_dim, H) for _ in range(L)])
    w["o_proj_weights"] = torch.stack([_normal_bf16(gen, H, shape.num_attention_heads * shape.head_dim) for _ in range(L)])
    w["up_proj_weights"] = torch.stack([_normal_bf16(gen, F, H) for _ in range(L)])
    w["gate_proj_weights"] = torch.stack([_normal_bf16(gen, F, H) for _ in range(L)])
    w["down_proj_weights"] = torch.stack([_normal_bf16(gen, H, F) for _ in range(L)])
    w["lm_head_weights"] = w["embed_tokens"] if shape.tie_word_embeddings else _normal_bf16(gen, V, H)
    if shape.qk_norm:
        # Not all ones: a per-head norm whose weights do nothing would hide a wrong column order.
        for name in ("q_norm_weights", "k_norm_weights"):
            w[name] = (1.0 + 0.1 * torch.randn(L, shape.head_dim, generator=gen, dtype=torch.float32)).to(torch.bfloat16)
    w["attn_norm_weights"] = torch.ones(L, H, dtype=torch.bfloat16)
    w["mlp_norm_weights"] = torch.ones(L, H, dtype=torch.bfloat16)
    w["lm_head_norm_weights"] = torch.ones(H, dtype=torch.bfloat16)
    w["rope_cos"], w["rope_sin"] = rope_tables(shape, max_positions)
    return w


def random_prompt(shape: DecodeShape, seed: int, length: int) -> torch.Tensor:
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed + 1_000_003)
    return torch.randint(0, shape.vocab_size, (length,), generator=gen, dtype=torch.long)


def build_globals(
    weights: dict[str, torch.Tensor],
    shape: DecodeShape,
    kv_capacity: int,
    device: torch.device | str,
    *,
    max_partials: int = 32,
    globals_cls: Any = Globals,
    barrier_rows: int = XCD_COUNTER_ROWS,
) -> Any:
    """Allocate every decode buffer on ``device`` and attach the weights (moved there)."""
    device = torch.device(device)
    bf16 = torch.bfloat16
    L, H = shape.num_hidden_layers, shape.hidden_size
    nq, nkv, d = shape.num_attention_heads, shape.num_key_value_heads, shape.head_dim

    def zeros(*size: int, dtype: torch.dtype = bf16) -> torch.Tensor:
        return torch.zeros(*size, dtype=dtype, device=device)

    on_device = {k: v.to(device).contiguous() for k, v in weights.items()}
    g = globals_cls(
        position_id=0,
        barriers=zeros(L, barrier_rows, shape.num_heads, dtype=torch.int32),
        k_cache=zeros(L, 1, kv_capacity, nkv, d),
        v_cache=zeros(L, 1, kv_capacity, nkv, d),
        hidden_states=zeros(H),
        q_post_rope=zeros(nq * d),
        attn_out=zeros(nq * d),
        attn_out_intermediates=zeros(nq, max_partials, d, dtype=torch.float32),
        attn_lse_intermediates=zeros(nq, max_partials, dtype=torch.float32),
        silu_out=zeros(shape.intermediate_size),
        logits=zeros(shape.vocab_size),
        **{k: v for k, v in on_device.items() if k != "embed_tokens"},
    )
    g.embed_tokens = on_device["embed_tokens"]
    if shape.tie_word_embeddings:
        g.lm_head_weights = g.embed_tokens          # one matrix on the device, as in the tied checkpoint
    if shape.qk_norm:
        g.qkv_raw = zeros(shape.qkv_out_dim)
    return g


def build_batch_globals(
    weights: dict[str, torch.Tensor],
    shape: DecodeShape,
    kv_capacity: int,
    batch_size: int,
    device: torch.device | str,
    *,
    max_partials: int = 27,
    globals_cls: Any = None,
) -> Any:
    """Buffers of the batch route for ``batch_size`` rows (allocation as the reference's
    `…/A100/fused_prefill.py:93-160` for batch sizes above one); all rows active, positions 0."""
    if globals_cls is None:
        from .decode_schedule_mb.globs import Globals as globals_cls
    device = torch.device(device)
    bf16 = torch.bfloat16
    L, H, B = shape.num_hidden_layers, shape.hidden_size, batch_size
    nq, nkv, d = shape.num_attention_heads, shape.num_key_value_heads, shape.head_dim

    def zeros(*size: int, dtype: torch.dtype = bf16) -> torch.Tensor:
        return torch.zeros(*size, dtype=dtype, device=device)

    on_device = {k: v.to(device).contiguous() for k, v in weights.items()}
    g = globals_cls(
        position_id=0,
        barriers=zeros(L, 10, (nq + 2 * nkv) * B, dtype=torch.int32),
        k_cache=zeros(L, B, kv_capacity, nkv, d),
        v_cache=zeros(L, B, kv_capacity, nkv, d),
        hidden_states=zeros(B, H),
        q_post_rope=zeros(B, nq * d),
        attn_out=zeros(B, nq * d),
        attn_out_intermediates=zeros(B, nq, max_partials, d, dtype=torch.float32),
        attn_lse_intermediates=zeros(B, nq, max_partials, dtype=torch.float32),
        silu_out=zeros(B, shape.intermediate_size),
        logits=zeros(B, shape.vocab_size),
        position_ids=zeros(B, dtype=torch.int32),
        active_mask=torch.ones(B, dtype=torch.bool, device=device),
        attn_partial_valid=zeros(B, nq, max_partials, dtype=torch.bool),
        attn_rms_out=zeros(B, H),
        mlp_rms_out=zeros(B, H),
        lm_head_rms_out=zeros(B, H),
        **{k: v for k, v in on_device.items() if k != "embed_tokens"},
    )
    g.embed_tokens = on_device["embed_tokens"]
    if shape.qk_norm:
        g.qkv_raw = zeros(B, shape.qkv_out_dim)
    return g


def build_synthetic_globals(
    shape: DecodeShape | None = None,
    *,
    seed: int = 0,
    kv_capacity: int = 136,
    device: torch.device | str = "cuda",
    max_partials: int = 32,
) -> Any:
    """Convenience: weights of ``seed`` + buffers; also points ``LlamaConfig`` at ``shape``."""
    shape = shape or LlamaConfig.shape()
    LlamaConfig.set_shape(shape)
    weights = random_weights(shape, seed, max_positions=kv_capacity)
    return build_globals(weights, shape, kv_capacity, device, max_partials=max_partials)


def reduced_shape(num_layers: int = 2, vocab_size: int = 2048, **overrides: Any) -> DecodeShape:
    """Llama-3.2-1B layer geometry with fewer layers and a small vocabulary (fast CPU checks)."""
    return dataclasses.replace(LlamaConfig.shape().__class__(), num_hidden_layers=num_layers, vocab_size=vocab_size, **overrides)


#: what ``random_moe_weights`` may return beside ``embed_tokens`` (the read-only tensors of the MoE route's ``Globals``)
MOE_WEIGHT_NAMES = ("qkv_weights", "qkv_bias", "o_proj_weights", "router_weights", "shared_expert_gate_proj_weights",
                    "shared_expert_up_proj_weights", "shared_expert_down_proj_weights", "shared_expert_gate_weights",
                    "expert_gate_up_proj_weights", "expert_down_proj_weights", "lm_head_weights", "attn_norm_weights",
                    "mlp_norm_weights", "lm_head_norm_weights", "q_norm_weights", "k_norm_weights", "rope_cos", "rope_sin")


def random_moe_weights(shape: Any, seed: int, max_positions: int, device: torch.device | str = "cpu") -> dict[str, torch.Tensor]:
    """Seeded random-init weights of the MoE route (``decode_schedule_moe.MoeShape``): bf16 ~N(0, 0.02)
    projections, router and experts (gate rows first in ``expert_gate_up_proj_weights``), QKV bias
    ~N(0, 0.02) where the shape has one, norm weights near one (not all ones: the router and the shared
    gate read the normalised row directly), untied LM head; the tensors of a shared expert and of the
    per-head QK norm only for shapes that have them.

    ``device`` "cpu" (default): drawn on a CPU generator, so a seed names the same model on every machine.
    On a GPU the draws come from that device's generator, one layer of experts at a time — for models
    whose weights (61 GB for the Qwen3-30B-A3B shape) should not pass through host memory."""
    device = torch.device(device)
    gen = torch.Generator(device=device)
    gen.manual_seed(seed)

    def normal(*size: int) -> torch.Tensor:
        return (torch.randn(*size, generator=gen, dtype=torch.float32, device=device) * WEIGHT_STD).to(torch.bfloat16)

    def stacked(count: int, *size: int) -> torch.Tensor:
        out = torch.empty(count, *size, dtype=torch.bfloat16, device=device)
        for i in range(count):
            out[i] = normal(*size)
        return out

    L, H, V = shape.num_hidden_layers, shape.hidden_size, shape.vocab_size
    F, Fm, E = shape.intermediate_size, shape.moe_intermediate_size, shape.num_experts
    w: dict[str, torch.Tensor] = {}
    w["embed_tokens"] = normal(V, H)
    w["qkv_weights"] = stacked(L, shape.qkv_out_dim, H)
    if shape.qkv_bias:
        w["qkv_bias"] = stacked(L, shape.qkv_out_dim)
    w["o_proj_weights"] = stacked(L, H, shape.num_attention_heads * shape.head_dim)
    w["router_weights"] = stacked(L, E, H)
    if shape.has_shared_expert:
        w["shared_expert_gate_proj_weights"] = stacked(L, F, H)
        w["shared_expert_up_proj_weights"] = stacked(L, F, H)
        w["shared_expert_down_proj_weights"] = stacked(L, H, F)
        w["shared_expert_gate_weights"] = stacked(L, 1, H)
    w["expert_gate_up_proj_weights"] = torch.empty(L, E, 2 * Fm, H, dtype=torch.bfloat16, device=device)
    for layer in range(L):
        for e in range(E):
            w["expert_gate_up_proj_weights"][layer, e] = normal(2 * Fm, H)
    w["expert_down_proj_weights"] = torch.empty(L, E, H, Fm, dtype=torch.bfloat16, device=device)
    for layer in range(L):
        for e in range(E):
            w["expert_down_proj_weights"][layer, e] = normal(H, Fm)
    w["lm_head_weights"] = normal(V, H)
    norms = [("attn_norm_weights", (L, H)), ("mlp_norm_weights", (L, H)), ("lm_head_norm_weights", (H,))]
    if shape.qk_norm:
        norms += [("q_norm_weights", (L, shape.head_dim)), ("k_norm_weights", (L, shape.head_dim))]
    for name, size in norms:
        w[name] = (1.0 + 0.1 * torch.randn(*size, generator=gen, dtype=torch.float32, device=device)).to(torch.bfloat16)
    rope_shape = DecodeShape(head_dim=shape.head_dim, rope_theta=shape.rope_theta)
    cos, sin = rope_tables(rope_shape, max_positions)
    w["rope_cos"], w["rope_sin"] = cos.to(device), sin.to(device)
    return w


def build_moe_globals(weights: dict[str, torch.Tensor], shape: Any, kv_capacity: int, device: torch.device | str, *,
                      max_partials: int = 27, globals_cls: Any = None) -> Any:
    """Buffers of the MoE route (`…/qwen1_5_moe_a2_7b/A100/single_batch/decode_schedule/globs.py:79-120`)."""
    if globals_cls is None:
        from .decode_schedule_moe.globs import Globals as globals_cls
    from .decode_schedule_moe.model_config import NUM_OPCODE_ROWS

    device = torch.device(device)
    bf16 = torch.bfloat16
    L, H = shape.num_hidden_layers, shape.hidden_size
    nq, nkv, d, k = shape.num_attention_heads, shape.num_key_value_heads, shape.head_dim, shape.num_experts_per_tok

    def zeros(*size: int, dtype: torch.dtype = bf16) -> torch.Tensor:
        return torch.zeros(*size, dtype=dtype, device=device)

    on_device = {name: t.to(device).contiguous() for name, t in weights.items()}
    g = globals_cls(
        position_id=0,
        barriers=zeros(L, NUM_OPCODE_ROWS, max(shape.barrier_slots, shape.num_heads), dtype=torch.int32),
        k_cache=zeros(L, 1, kv_capacity, nkv, d),
        v_cache=zeros(L, 1, kv_capacity, nkv, d),
        hidden_states=zeros(H),
        q_post_rope=zeros(nq * d),
        attn_out=zeros(nq * d),
        attn_out_intermediates=zeros(nq, max_partials, d, dtype=torch.float32),
        attn_lse_intermediates=zeros(nq, max_partials, dtype=torch.float32),
        router_logits_buf=zeros(shape.num_experts, dtype=torch.float32),
        normed_hidden_states=zeros(H),
        **(dict(shared_expert_silu_out=zeros(shape.intermediate_size), shared_out=zeros(H)) if shape.has_shared_expert else {}),
        **(dict(qkv_raw=zeros(shape.qkv_out_dim)) if shape.qk_norm else {}),
        routed_out=zeros(H),
        routed_out_f32=zeros(H, dtype=torch.float32),
        routed_silu_buffer=zeros(k, shape.moe_intermediate_size),
        expert_indices=zeros(k, dtype=torch.int64),
        expert_weights=zeros(k, dtype=torch.float32),
        silu_out=zeros(shape.moe_intermediate_size),
        logits=zeros(shape.vocab_size),
        **{name: t for name, t in on_device.items() if name != "embed_tokens"},
    )
    g.embed_tokens = on_device["embed_tokens"]
    return g
