"""CPU oracle of the batch decode route (B rows) — TEST INFRASTRUCTURE, not product code.

Only ``tests/`` and the ``cpu_baseline`` leg of ``bench.py`` may import this module: as the checker and as
the timed CPU baseline, never as part of the product path.

The reference has no separate fused route for batch sizes above one: its single-batch fused
operations work on ``[B, H]`` activations
(``…/A100/multi_batch/decode_schedule/fused/__init__.py:1-18`` re-exports
``…/A100/single_batch/decode_schedule/fused/operations.py``).  Restated here, per function:

=========================  =====================================================
``qkv_rope``               fused/operations.py:151-215  (per-row position, inactive rows write nothing)
``attention``              fused/operations.py:218-248  (inactive rows: attn_out row zeroed)
``oproj_residual``         fused/operations.py:251-262  (inactive rows add zero)
``mlp_upgate``             fused/operations.py:265-282  (inactive rows: silu_out row zeroed)
``mlp_down_residual``      fused/operations.py:285-295
``lm_head``                fused/operations.py:303-321  (inactive rows: logits -1e9)
=========================  =====================================================

A shape with the Qwen3 op set (``qk_norm``: Qwen3-1.7B) has no batch route in the reference, and the Qwen3
route's fused operations take one row (…/qwen/qwen3__0_6b/A100/single_batch/decode_schedule/fused/operations.py:
``"o i, i -> o"`` throughout).  Its batch step is therefore that route run row by row: every live row goes through
``fused_oracle.FusedOracle`` (restating operations.py:52-250 of that route, pinned by its own fixture) on a
batch-1 view of the row's buffers, at the row's position.  Inactive rows as in the batch route above: nothing
written but a zeroed ``attn_out`` and ``silu_out`` row and logits of -1e9.  Pinned by the fixture of
tests/golden/make_fixtures_qwen3_mb.py: the imported functions of the Qwen3 route on the same row views, in
lock-step, bit for bit.

Pinning: tests/test_mb_oracle.py checks every row of a batch against the batch-1 oracle
(``fused_oracle.FusedOracle``, itself pinned against closed forms and the imported reference) on
the same weights — bit for bit where the reference's arithmetic is row-wise, which is everywhere
except the accumulation order inside a GEMM with B columns, left unspecified by the reference — and
against the fixture that tests/golden/make_fixtures_mb.py wrote from the imported reference while
stepping this oracle in lock-step with it.
"""
from __future__ import annotations

import math
from typing import Any

import torch
import torch.nn.functional as F

from fused_oracle import FusedOracle, gemv, rms_norm, rotate_pairs

Tensor = torch.Tensor


def _row_active(g: Any, b: int) -> bool:
    mask = getattr(g, "active_mask", None)
    return True if mask is None else bool(mask[b])


def _pos(g: Any, b: int) -> int:
    ids = getattr(g, "position_ids", None)
    return int(ids[b]) if ids is not None else int(g.position_id or 0)


_ROW_BUFFERS = ("hidden_states", "qkv_raw", "q_post_rope", "attn_out", "attn_lse_intermediates", "attn_out_intermediates",
                "silu_out", "logits")


class RowView:
    """Row ``b`` of the batch buffers as the batch-1 buffers of the Qwen3 route (views: writes land in the batch's)."""

    def __init__(self, g: Any, b: int):
        self.__dict__["_g"], self.__dict__["_b"] = g, b

    def __getattr__(self, name: str) -> Any:
        g, b = self._g, self._b
        if name in _ROW_BUFFERS:
            return getattr(g, name)[b]
        if name in ("k_cache", "v_cache"):
            return getattr(g, name)[:, b : b + 1]
        if name == "position_id":
            return _pos(g, b)
        return getattr(g, name)

    def __setattr__(self, name: str, value: Any) -> None:
        raise AttributeError("a row view is read-only: buffers are written in place")


class FusedBatchOracle:
    def __init__(self, shape: Any):
        self.shape = shape
        self._qwen3 = FusedOracle(shape) if getattr(shape, "qk_norm", False) else None   # the Qwen3 route's attention half, per row

    def _row_by_row(self, g: Any, op: str, *args: Any) -> None:
        for b in range(g.hidden_states.shape[0]):
            if _row_active(g, b):
                getattr(self._qwen3, op)(RowView(g, b), *args)

    def qkv_rope(self, g: Any, layer: int) -> None:
        s = self.shape
        if self._qwen3 is not None:
            return self._row_by_row(g, "qkv_rope", layer)
        nq, nkv, d = s.num_attention_heads, s.num_key_value_heads, s.head_dim
        y = rms_norm(g.hidden_states, g.attn_norm_weights[layer], s.rms_norm_eps)
        qkv = gemv(g.qkv_weights[layer], y)                       # bf16 [B, (nq + 2 nkv) d]: rounded before RoPE
        B = qkv.shape[0]
        q = qkv[:, : nq * d].view(B, nq, d)
        k = qkv[:, nq * d : (nq + nkv) * d].view(B, nkv, d)
        v = qkv[:, (nq + nkv) * d :].view(B, nkv, d)
        for b in range(B):
            if not _row_active(g, b):
                continue
            pos = _pos(g, b)
            cos, sin = g.rope_cos[pos].view(1, -1), g.rope_sin[pos].view(1, -1)   # fp32: the products are fp32
            qr = q[b] * cos + rotate_pairs(q[b]) * sin
            kr = k[b] * cos + rotate_pairs(k[b]) * sin
            g.q_post_rope[b].copy_(qr.reshape(-1).to(g.q_post_rope.dtype))
            g.k_cache[layer, b, pos].copy_(kr.to(g.k_cache.dtype))
            g.v_cache[layer, b, pos].copy_(v[b].to(g.v_cache.dtype))

    def attention(self, g: Any, layer: int) -> None:
        s = self.shape
        nq, d, ratio = s.num_attention_heads, s.head_dim, s.num_attention_heads // s.num_key_value_heads
        for b in range(g.hidden_states.shape[0]):
            if not _row_active(g, b):
                g.attn_out[b].zero_()
                continue
            if self._qwen3 is not None:
                self._qwen3.attention_split_merge(RowView(g, b), layer)
                continue
            n = _pos(g, b) + 1
            q = g.q_post_rope[b].view(nq, d).float()
            k = g.k_cache[layer, b, :n].float().repeat_interleave(ratio, dim=1)   # [n, nq, d]
            v = g.v_cache[layer, b, :n].float().repeat_interleave(ratio, dim=1)
            scores = torch.einsum("hi,shi->hs", q, k) * (1 / math.sqrt(d))
            out = torch.einsum("hs,sho->ho", torch.softmax(scores, dim=-1), v)
            g.attn_out[b].copy_(out.reshape(-1).to(g.attn_out.dtype))

    def _masked(self, g: Any, rows: Tensor, fill: float = 0.0) -> Tensor:
        for b in range(rows.shape[0]):
            if not _row_active(g, b):
                rows[b] = fill
        return rows

    def oproj_residual(self, g: Any, layer: int) -> None:
        if self._qwen3 is not None:
            return self._row_by_row(g, "oproj_residual", layer)
        g.hidden_states.add_(self._masked(g, gemv(g.o_proj_weights[layer], g.attn_out)).to(g.hidden_states.dtype))

    def mlp_upgate(self, g: Any, layer: int) -> None:
        if self._qwen3 is not None:
            g.silu_out.zero_()
            return self._row_by_row(g, "mlp_upgate", layer)
        y = rms_norm(g.hidden_states, g.mlp_norm_weights[layer], self.shape.rms_norm_eps)
        up, gate = gemv(g.up_proj_weights[layer], y), gemv(g.gate_proj_weights[layer], y)
        g.silu_out.copy_(self._masked(g, F.silu(gate) * up).to(g.silu_out.dtype))

    def mlp_down_residual(self, g: Any, layer: int) -> None:
        if self._qwen3 is not None:
            return self._row_by_row(g, "mlp_down_residual", layer)
        g.hidden_states.add_(self._masked(g, gemv(g.down_proj_weights[layer], g.silu_out)).to(g.hidden_states.dtype))

    def lm_head(self, g: Any) -> None:
        if self._qwen3 is not None:
            g.logits.fill_(-1e9)
            return self._row_by_row(g, "lm_head")
        y = rms_norm(g.hidden_states, g.lm_head_norm_weights, self.shape.rms_norm_eps)
        g.logits.copy_(self._masked(g, gemv(g.lm_head_weights, y).to(g.logits.dtype), -1e9))

    def decode_layer(self, g: Any, layer: int) -> None:
        self.qkv_rope(g, layer)
        self.attention(g, layer)
        self.oproj_residual(g, layer)
        self.mlp_upgate(g, layer)
        self.mlp_down_residual(g, layer)

    def decode_step(self, g: Any, num_layers: int | None = None) -> None:
        layers = self.shape.num_hidden_layers if num_layers is None else num_layers
        for layer in range(layers):
            self.decode_layer(g, layer)
        if layers == self.shape.num_hidden_layers:
            self.lm_head(g)
