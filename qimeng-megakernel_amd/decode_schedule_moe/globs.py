"""``Globals`` of the MoE decode route: the tensor ABI
(`…/qwen1_5_moe_a2_7b/A100/single_batch/decode_schedule/globs.py:9-77`).

Shapes (Qwen1.5-MoE-A2.7B): ``qkv_weights [L, 6144, 2048]`` + ``qkv_bias [L, 6144]``,
``router_weights [L, E, H]``, ``expert_gate_up_proj_weights [L, E, 2*1408, H]`` (gate rows first),
``expert_down_proj_weights [L, E, H, 1408]``, shared expert ``[L, 5632, H]`` x2 and ``[L, H, 5632]``,
``shared_expert_gate_weights [L, 1, H]``; buffers ``router_logits_buf [E]`` f32,
``expert_indices [k]`` int64, ``expert_weights [k]`` f32, ``normed_hidden_states [H]``,
``shared_expert_silu_out [5632]``, ``shared_out [H]``, ``routed_silu_buffer [k, 1408]``,
``routed_out_f32 [H]`` f32, ``barriers [L, 15, 128]``.  A shape without a shared expert (Qwen3-30B-A3B) leaves the
six shared-expert fields ``None``; a shape with the Qwen3 op set's attention adds ``qkv_raw`` and the two per-head
norm weights, as the dense Qwen3 route does (`…/qwen/qwen3__0_6b/A100/single_batch/decode_schedule/globs.py`).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

import torch

Tensor = torch.Tensor


@dataclass
class Globals:
    instructions: Optional[Tensor] = None
    barriers: Optional[Tensor] = None
    position_id: Optional[int] = None
    attn_norm_weights: Optional[Tensor] = None
    qkv_weights: Optional[Tensor] = None
    qkv_bias: Optional[Tensor] = None
    qkv_raw: Optional[Tensor] = None                 # Qwen3 op set: bf16 [(Hq+2Hkv)*D], QKV before norm and RoPE
    q_norm_weights: Optional[Tensor] = None          # Qwen3 op set: bf16 [L, D]
    k_norm_weights: Optional[Tensor] = None
    rope_cos: Optional[Tensor] = None
    rope_sin: Optional[Tensor] = None
    o_proj_weights: Optional[Tensor] = None
    mlp_norm_weights: Optional[Tensor] = None
    shared_expert_gate_proj_weights: Optional[Tensor] = None
    shared_expert_up_proj_weights: Optional[Tensor] = None
    shared_expert_down_proj_weights: Optional[Tensor] = None
    shared_expert_gate_weights: Optional[Tensor] = None
    router_weights: Optional[Tensor] = None
    router_logits_buf: Optional[Tensor] = None
    expert_gate_up_proj_weights: Optional[Tensor] = None
    expert_down_proj_weights: Optional[Tensor] = None
    lm_head_norm_weights: Optional[Tensor] = None
    lm_head_weights: Optional[Tensor] = None
    k_cache: Optional[Tensor] = None
    v_cache: Optional[Tensor] = None
    hidden_states: Optional[Tensor] = None
    q_post_rope: Optional[Tensor] = None
    attn_out: Optional[Tensor] = None
    attn_out_intermediates: Optional[Tensor] = None
    attn_lse_intermediates: Optional[Tensor] = None
    normed_hidden_states: Optional[Tensor] = None
    shared_expert_silu_out: Optional[Tensor] = None
    shared_out: Optional[Tensor] = None
    routed_out: Optional[Tensor] = None
    routed_out_f32: Optional[Tensor] = None
    routed_silu_buffer: Optional[Tensor] = None
    expert_indices: Optional[Tensor] = None
    expert_weights: Optional[Tensor] = None
    silu_out: Optional[Tensor] = None
    logits: Optional[Tensor] = None
    embed_tokens: Optional[Tensor] = None
    # several requests in one launch (rows_kernel.py): every per-request buffer above then has a leading row dimension
    position_ids: Optional[Tensor] = None            # int32 [rows]
    distinct_experts: Optional[Tensor] = None        # int32 [L]: distinct experts each layer streamed in the last launch
