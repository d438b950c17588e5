"""CPU oracle of the decode path — TEST INFRASTRUCTURE, not product code.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module, and only as the checker.  Nothing the
library ships routes through it.

It restates, in plain PyTorch on whatever device the tensors live on (CPU in
every test), the reference's fused full-layer decode route with its exact bf16
rounding points.  Citations are into
``qimeng_megakernel/models/LLM/llama/llama3_2__1b/A100/single_batch/decode_schedule/``:

=========================  =====================================================
``rms_norm``               fused/operations.py:126-131
``rotate_pairs``           fused/operations.py:134-139
``qkv_rope``               fused/operations.py:151-215  (batch-1, all rows active)
``attention``              fused/operations.py:218-248
``oproj_residual``         fused/operations.py:251-262, 63-68
``mlp_upgate``             fused/operations.py:265-282
``mlp_down_residual``      fused/operations.py:285-295
``lm_head``                fused/operations.py:303-321
``decode_layers/step``     fused/layer_scheduler.py:32-56
``greedy``                 qimeng_megakernel/models/LLM/decode.py:1340-1400
=========================  =====================================================

Pinning (see tests/test_oracle_*.py): every function is checked against
closed forms / fp64 brute force with explicit bf16 rounding; the full greedy
trajectory is additionally pinned by fixtures written once from the imported
reference (tests/golden/).  GEMV accumulation order is whatever the executing
torch build does for a bf16 ``einsum`` — the reference leaves it unspecified.
"""
from __future__ import annotations

import math
from typing import Any

import torch
import torch.nn.functional as F

Tensor = torch.Tensor


def gemv(weight: Tensor, x_bh: Tensor) -> Tensor:
    """``[O, I] x [B, I] -> [B, O]`` in the operands' dtype (the reference's einsum 'o i, b i -> b o')."""
    return torch.einsum("oi,bi->bo", weight, x_bh)


def rms_norm(x: Tensor, weight: Tensor, eps: float) -> Tensor:
    dtype = x.dtype
    xf = x.to(torch.float32)
    var = xf.pow(2).mean(-1, keepdim=True)
    xf = xf * torch.rsqrt(var + eps)
    return weight * xf.to(dtype)


def per_head_rms_norm(x: Tensor, weight: Tensor, eps: float) -> Tensor:
    """RMSNorm over the last dim with one shared weight vector, all in fp32, ONE rounding at the end
    (qwen3__0_6b/…/fused/operations.py:52-63 — unlike ``rms_norm``, which rounds before the weight)."""
    xf = x.to(torch.float32)
    xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
    return (weight.to(torch.float32) * xf).to(x.dtype)


def rotate_pairs(x: Tensor) -> Tensor:
    """(x0, x1, x2, x3, ...) -> (-x1, x0, -x3, x2, ...)."""
    even, odd = x[..., 0::2], x[..., 1::2]
    return torch.stack((-odd, even), dim=-1).reshape(x.shape)


class FusedOracle:
    """One decode step on a ``Globals``-shaped object ``g`` (attribute access only)."""

    def __init__(self, shape: Any):
        self.shape = shape

    # ---- single ops ---------------------------------------------------------
    def qkv_rope(self, g: Any, layer: int) -> None:
        s = self.shape
        nq, nkv, d = s.num_attention_heads, s.num_key_value_heads, s.head_dim
        y = rms_norm(g.hidden_states, g.attn_norm_weights[layer], s.rms_norm_eps).unsqueeze(0)
        qkv = gemv(g.qkv_weights[layer], y)  # bf16 before RoPE
        q = qkv[:, : nq * d].view(1, nq, d)
        k = qkv[:, nq * d : (nq + nkv) * d].view(1, nkv, d)
        v = qkv[:, (nq + nkv) * d :].view(1, nkv, d)
        if getattr(s, "qk_norm", False):
            # Qwen3 op set: the raw vector is kept, q and k get a per-head RMSNorm before RoPE
            # (qwen3__0_6b/…/fused/operations.py:65-120).
            g.qkv_raw.copy_(qkv.reshape(-1).to(g.qkv_raw.dtype))
            q = per_head_rms_norm(q, g.q_norm_weights[layer], s.rms_norm_eps)
            k = per_head_rms_norm(k, g.k_norm_weights[layer], s.rms_norm_eps)
        pos = int(g.position_id or 0)
        cos = g.rope_cos[pos].view(1, 1, -1)  # fp32: the products below are fp32
        sin = g.rope_sin[pos].view(1, 1, -1)
        q_rot = (q * cos) + (rotate_pairs(q) * sin)
        k_rot = (k * cos) + (rotate_pairs(k) * sin)
        g.q_post_rope.copy_(q_rot.reshape(-1).to(g.q_post_rope.dtype))
        g.k_cache[layer, 0, pos].copy_(k_rot[0].to(g.k_cache.dtype))
        g.v_cache[layer, 0, pos].copy_(v[0].to(g.v_cache.dtype))

    def attention_split_merge(self, g: Any, layer: int) -> None:
        """The Qwen3 route's fused attention: always split into as many partials as the workspace
        has columns and merged in the log2 domain (qwen3__0_6b/…/fused/operations.py:123-215)."""
        s = self.shape
        nq, nkv, d = s.num_attention_heads, s.num_key_value_heads, s.head_dim
        ratio, block = nq // nkv, s.attn_kv_block_size
        n = int(g.position_id or 0) + 1
        parts = int(g.attn_lse_intermediates.shape[1])
        total_blocks = math.ceil(n / block)
        per_part = math.ceil(total_blocks / parts)
        q = g.q_post_rope.view(nq, d).float()
        k_full, v_full = g.k_cache[layer, 0, :n].float(), g.v_cache[layer, 0, :n].float()
        scale = 1.0 / math.sqrt(d)
        for h in range(nq):
            k, v = k_full[:, h // ratio], v_full[:, h // ratio]
            for p in range(parts):
                t0 = p * per_part * block
                t1 = min(min((p + 1) * per_part, total_blocks) * block, n)
                if t0 >= t1:
                    g.attn_lse_intermediates[h, p] = -float("inf")
                    g.attn_out_intermediates[h, p] = 0.0
                    continue
                sc = torch.einsum("hi,ki->hk", q[h : h + 1], k[t0:t1]) * scale
                g.attn_lse_intermediates[h, p] = torch.log2(torch.sum(torch.exp(sc), dim=-1) + 1e-12).squeeze(0)
                g.attn_out_intermediates[h, p] = torch.einsum("hk,ko->ho", torch.softmax(sc, dim=-1), v[t0:t1]).squeeze(0)
        step = s.attn_reduction_size  # the reference merges one reduction group of heads at a time
        for h0 in range(0, nq, step):
            lses, outs = g.attn_lse_intermediates[h0 : h0 + step], g.attn_out_intermediates[h0 : h0 + step]
            lses = torch.where(torch.isposinf(lses), torch.full_like(lses, 1e10), lses)
            top = torch.clamp(lses.max(dim=1, keepdim=True).values, min=-1e10)
            weights = (lses - top).exp2()
            denom = weights.sum(dim=1, keepdim=True).clamp(min=1e-12)
            merged = (outs * weights.unsqueeze(-1)).sum(dim=1) / denom
            g.attn_out.view(nq, d)[h0 : h0 + step] = merged.to(g.attn_out.dtype)

    def attention(self, g: Any, layer: int) -> None:
        s = self.shape
        if getattr(s, "qk_norm", False):
            return self.attention_split_merge(g, layer)
        nq, nkv, d = s.num_attention_heads, s.num_key_value_heads, s.head_dim
        ratio = nq // nkv
        n = int(g.position_id or 0) + 1
        q = g.q_post_rope.view(nq, d).float()
        k = g.k_cache[layer, 0, :n].float().unsqueeze(2).expand(-1, -1, ratio, -1).reshape(n, nq, d)
        v = g.v_cache[layer, 0, :n].float().unsqueeze(2).expand(-1, -1, ratio, -1).reshape(n, nq, d)
        scores = torch.einsum("hi,shi->hs", q, k) * (1 / math.sqrt(d))
        probs = torch.softmax(scores, dim=-1)
        out = torch.einsum("hs,sho->ho", probs, v)
        g.attn_out.copy_(out.reshape(-1).to(g.attn_out.dtype))

    def oproj_residual(self, g: Any, layer: int) -> None:
        delta = gemv(g.o_proj_weights[layer], g.attn_out.unsqueeze(0))
        g.hidden_states.add_(delta.squeeze(0).to(g.hidden_states.dtype))

    def mlp_upgate(self, g: Any, layer: int) -> None:
        y = rms_norm(g.hidden_states, g.mlp_norm_weights[layer], self.shape.rms_norm_eps).unsqueeze(0)
        up = gemv(g.up_proj_weights[layer], y)
        gate = gemv(g.gate_proj_weights[layer], y)
        act = F.silu(gate) * up
        g.silu_out.copy_(act.reshape(-1).to(g.silu_out.dtype))

    def mlp_down_residual(self, g: Any, layer: int) -> None:
        delta = gemv(g.down_proj_weights[layer], g.silu_out.unsqueeze(0))
        g.hidden_states.add_(delta.squeeze(0).to(g.hidden_states.dtype))

    def lm_head(self, g: Any) -> None:
        y = rms_norm(g.hidden_states, g.lm_head_norm_weights, self.shape.rms_norm_eps).unsqueeze(0)
        g.logits.copy_(gemv(g.lm_head_weights, y).to(g.logits.dtype).squeeze(0))

    # ---- step ---------------------------------------------------------------
    def decode_layer(self, g: Any, layer: int) -> None:
        self.qkv_rope(g, layer)
        self.attention(g, layer)
        self.oproj_residual(g, layer)
        self.mlp_upgate(g, layer)
        self.mlp_down_residual(g, layer)

    def decode_layers(self, g: Any, num_layers: int | None = None, on_layer=None) -> None:
        layers = self.shape.num_hidden_layers if num_layers is None else num_layers
        for layer in range(layers):
            self.decode_layer(g, layer)
            if on_layer is not None:
                on_layer(layer, g)

    def decode_step(self, g: Any, on_layer=None) -> None:
        self.decode_layers(g, on_layer=on_layer)
        self.lm_head(g)

    # ---- request ------------------------------------------------------------
    @staticmethod
    def embed(g: Any, token: int | Tensor) -> None:
        row = g.embed_tokens[int(token)]
        g.hidden_states.copy_(row.to(g.hidden_states.dtype))

    def prefill_by_decode(self, g: Any, prompt_ids: Tensor) -> int:
        """KV cache for the prompt via the single-token path; returns the first generated token."""
        for pos, tok in enumerate(prompt_ids.tolist()):
            self.embed(g, tok)
            g.position_id = pos
            self.decode_step(g)
        return int(torch.argmax(g.logits))

    def greedy(self, g: Any, prompt_ids: Tensor, max_new_tokens: int, on_step=None) -> list[int]:
        """Forced greedy continuation (no EOS stop); token ``prompt_len+i`` is embedded at that position."""
        prompt_len = int(prompt_ids.numel())
        tokens = [self.prefill_by_decode(g, prompt_ids)]
        if on_step is not None:
            on_step(-1, g)
        for i in range(max_new_tokens - 1):
            self.embed(g, tokens[-1])
            g.position_id = prompt_len + i
            self.decode_step(g)
            tokens.append(int(torch.argmax(g.logits)))  # first index on ties
            if on_step is not None:
                on_step(i, g)
        return tokens
