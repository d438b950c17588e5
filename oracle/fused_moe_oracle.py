"""CPU oracle of the MoE decode route (fused form) — TEST INFRASTRUCTURE, not product code.

Only ``tests/`` and the ``cpu_baseline`` leg of ``bench.py`` may import this module: as the checker and as
the timed CPU baseline, never as part of the product path.

Restates the reference's fused PyTorch operations
(``…/qwen/qwen1_5_moe_a2_7b/A100/single_batch/decode_schedule/fused/operations.py``):

===========================  ================================================================
``qkv_rope``                 :40-87   RMSNorm, one linear with bias (one rounding), RoPE, KV append
``attention``                :90-131  softmax attention over the cache rows [0, pos]
``oproj_residual``           :134-138
``shared_mlp``               :155-178 silu(gate) * up in fp32, one rounding, down projection
``router``                   :181-202 fp32 logits, softmax, top-k (weights not renormalised)
``routed_expert``            :205-252 per selected expert: fused gate|up rows, fp32 weighted sum
``moe_block``                :255-290 routed sum rounded to bf16, shared output scaled by a bf16 sigmoid gate
``lm_head``                  :141-152
===========================  ================================================================

A shape with ``qk_norm`` (Qwen3-30B-A3B) has no route in the reference; its step is the reference's two routes
put together: the attention half is the Qwen3 route's (``FusedOracle.qkv_rope`` / ``attention_split_merge`` /
``oproj_residual`` of oracle/fused_oracle.py, restating …/qwen/qwen3__0_6b/A100/single_batch/decode_schedule/
fused/operations.py:52-215), the MoE half is the block above with the two switches that shape sets:
``norm_topk_prob`` — the top-k probabilities divided by their sum in fp32, the one line the reference has for it
(…/qwen1_5_moe_a2_7b/…/fused/operations.py:405, in its prefill block) — and no shared expert (the block's shared
terms dropped; with all-zero shared weights the reference's block computes the same bits).

Pinning: tests/test_moe_oracle.py — closed forms (a router whose logits are given, experts that
are multiples of each other), the instruction VM of oracle/pyvm_moe_oracle.py on the same inputs,
and the fixture written by tests/golden/make_fixtures_moe.py from the imported reference while
this oracle ran in lock-step with it.
"""
from __future__ import annotations

import math
from typing import Any

import torch
import torch.nn.functional as F

from fused_oracle import FusedOracle, rms_norm, rotate_pairs

Tensor = torch.Tensor


class FusedMoeOracle:
    def __init__(self, shape: Any):
        self.shape = shape
        self._qwen3 = FusedOracle(shape) if getattr(shape, "qk_norm", False) else None   # the Qwen3 route's attention half

    def qkv_rope(self, g: Any, layer: int) -> None:
        s = self.shape
        if self._qwen3 is not None:
            return self._qwen3.qkv_rope(g, layer)
        nq, nkv, d, pos = s.num_attention_heads, s.num_key_value_heads, s.head_dim, int(g.position_id or 0)
        y = rms_norm(g.hidden_states, g.attn_norm_weights[layer], s.rms_norm_eps)
        bias = None if g.qkv_bias is None else g.qkv_bias[layer]
        qkv = F.linear(y.view(1, -1), g.qkv_weights[layer], bias).reshape(-1)      # the bias belongs to the projection: one rounding
        q = qkv[: nq * d].view(nq, d)
        k = qkv[nq * d : (nq + nkv) * d].view(nkv, d)
        v = qkv[(nq + nkv) * d :].view(nkv, d)
        cos, sin = g.rope_cos[pos].view(1, -1), g.rope_sin[pos].view(1, -1)
        g.q_post_rope.copy_((q * cos + rotate_pairs(q) * sin).reshape(-1).to(g.q_post_rope.dtype))
        g.k_cache[layer, 0, pos].copy_((k * cos + rotate_pairs(k) * sin).to(g.k_cache.dtype))
        g.v_cache[layer, 0, pos].copy_(v.to(g.v_cache.dtype))

    def attention(self, g: Any, layer: int) -> None:
        """torch's scaled-dot-product attention on fp32 copies, grouped heads, no mask (`:90-131`)."""
        s = self.shape
        if self._qwen3 is not None:
            return self._qwen3.attention_split_merge(g, layer)
        nq, d, n = s.num_attention_heads, s.head_dim, int(g.position_id or 0) + 1
        q = g.q_post_rope.view(1, nq, 1, d).float()
        k = g.k_cache[layer, 0, :n].permute(1, 0, 2).unsqueeze(0).float()
        v = g.v_cache[layer, 0, :n].permute(1, 0, 2).unsqueeze(0).float()
        out = F.scaled_dot_product_attention(q, k, v, is_causal=False, enable_gqa=True)
        g.attn_out.copy_(out.squeeze(0).squeeze(1).reshape(-1).to(g.attn_out.dtype))

    def oproj_residual(self, g: Any, layer: int) -> None:
        if self._qwen3 is not None:
            return self._qwen3.oproj_residual(g, layer)
        g.hidden_states += F.linear(g.attn_out.unsqueeze(0), g.o_proj_weights[layer]).squeeze(0).to(g.hidden_states.dtype)

    def shared_mlp(self, g: Any, layer: int, normed: Tensor) -> None:
        gate = F.linear(normed.unsqueeze(0), g.shared_expert_gate_proj_weights[layer]).squeeze(0)
        up = F.linear(normed.unsqueeze(0), g.shared_expert_up_proj_weights[layer]).squeeze(0)
        x = (F.silu(gate.float()) * up.float()).to(g.shared_out.dtype)
        g.shared_out.copy_(F.linear(x.unsqueeze(0), g.shared_expert_down_proj_weights[layer]).squeeze(0).to(g.shared_out.dtype))

    def router(self, g: Any, layer: int, normed: Tensor) -> None:
        logits = F.linear(normed.float().unsqueeze(0), g.router_weights[layer].float()).squeeze(0)
        top_p, top_i = torch.topk(F.softmax(logits, dim=-1), self.shape.num_experts_per_tok, dim=-1)
        if getattr(self.shape, "norm_topk_prob", False):
            top_p = top_p / top_p.sum(dim=-1, keepdim=True)
        g.expert_indices.copy_(top_i.to(g.expert_indices.dtype))
        g.expert_weights.copy_(top_p.to(g.expert_weights.dtype))

    def routed_expert(self, g: Any, layer: int, slot: int, normed: Tensor, accum: Tensor) -> None:
        mid = self.shape.moe_intermediate_size
        eid = int(g.expert_indices[slot])
        gate_up = F.linear(normed.unsqueeze(0), g.expert_gate_up_proj_weights[layer, eid]).squeeze(0)
        g.silu_out.copy_((F.silu(gate_up[:mid].float()) * gate_up[mid:].float()).to(g.silu_out.dtype))
        out = F.linear(g.silu_out.unsqueeze(0), g.expert_down_proj_weights[layer, eid]).squeeze(0)
        accum.add_(out.float() * g.expert_weights[slot])

    def moe_block(self, g: Any, layer: int) -> None:
        s = self.shape
        normed = rms_norm(g.hidden_states, g.mlp_norm_weights[layer], s.rms_norm_eps)
        shared = getattr(s, "has_shared_expert", True)
        if shared:
            self.shared_mlp(g, layer, normed)
        self.router(g, layer, normed)
        accum = torch.zeros(g.routed_out.shape, dtype=torch.float32)
        for slot in range(s.num_experts_per_tok):
            self.routed_expert(g, layer, slot, normed, accum)
        g.routed_out.copy_(accum.to(g.routed_out.dtype))
        if not shared:
            g.hidden_states.add_(g.routed_out)
            return
        gate_logit = (g.shared_expert_gate_weights[layer].squeeze(0).float() * normed.float()).sum()
        gate_scale = torch.sigmoid(gate_logit).to(g.hidden_states.dtype)
        g.hidden_states.add_(g.routed_out)
        g.hidden_states.add_(g.shared_out * gate_scale)

    def lm_head(self, g: Any) -> None:
        y = rms_norm(g.hidden_states, g.lm_head_norm_weights, self.shape.rms_norm_eps)
        g.logits.copy_(F.linear(y.unsqueeze(0), g.lm_head_weights).squeeze(0).to(g.logits.dtype))

    def decode_layer(self, g: Any, layer: int) -> None:
        self.qkv_rope(g, layer)
        self.attention(g, layer)
        self.oproj_residual(g, layer)
        self.moe_block(g, layer)

    def decode_step(self, g: Any, num_layers: int | None = None) -> None:
        layers = self.shape.num_hidden_layers if num_layers is None else num_layers
        for layer in range(layers):
            self.decode_layer(g, layer)
        if layers == self.shape.num_hidden_layers:
            self.lm_head(g)
