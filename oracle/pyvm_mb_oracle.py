"""Sequential instruction VM of the batch decode route — TEST INFRASTRUCTURE, not product code.

Only ``tests/`` may import this module, and only as the checker.

Restates the reference's handlers
(``…/A100/multi_batch/decode_schedule/instructions/python_vm.py``): the same arithmetic as the
fused route, cut into the tiles the instructions name, plus the counter protocol — every handler
first checks that its producers' counters are complete and then adds to its own.

=============================  ==========================
``attn_rms / mlp_rms``         python_vm.py:139-160, 614-634
``lmhead_rms``                 python_vm.py:668-690
``qkvproj_gemm_rope``          python_vm.py:163-266   (Qwen3 op set: the raw rows only)
``decode_attention_split_kv``  python_vm.py:269-359   (Qwen3 op set: per-head norm, RoPE and cache rows first)
``decode_attention_reduction`` python_vm.py:442-551
``oproj / down``               python_vm.py:554-611
``upgate``                     python_vm.py:637-665
``lmhead_proj_gemm``           python_vm.py:693-715
=============================  ==========================

Pinning: tests/test_mb_oracle.py — against the fused batch oracle (same inputs, every
instruction stream of the scheduler), and against the fixture written from the imported
reference by tests/golden/make_fixtures_mb.py, which ran the reference's VM on the same
instruction list in lock-step with this one (bit-identical buffers and counters).
"""
from __future__ import annotations

import math
from typing import Any, Iterable

import torch
import torch.nn.functional as F

from fused_oracle import per_head_rms_norm, rms_norm, rotate_pairs

Tensor = torch.Tensor
TILE = 16                      # output rows per GEMM block
INACTIVE_LSE = float("-inf")   # what an empty or inactive partial leaves in the LSE workspace
NONCONTRIBUTING_LSE = -79.0    # without a validity buffer: partials at or below this do not count
MERGED_EMPTY_LSE = NONCONTRIBUTING_LSE - 1.0


def _gemm(mat: Tensor, rows_bk: Tensor, r0: int, r1: int) -> Tensor:
    return torch.einsum("oi,bi->bo", mat[r0:r1], rows_bk)


class _MergeAll:
    """What a reduction instruction over all partials of a head group would say."""

    def __init__(self, layer: int, b: int, h0: int, num_partials: int):
        self.layer_idx, self.batch_idx, self.head_start_idx, self.num_partials = layer, b, h0, num_partials
        self.reduction_list, self.is_terminal, self.output_partial_idx, self.is_active = list(range(num_partials)), True, 0, -1


class BatchInstructionVM:
    def __init__(self, shape: Any, oproj_tile: int = TILE, down_tile: int = TILE):
        """``oproj_tile`` / ``down_tile``: rows per block of the two residual projections in the stream
        (16 in the reference's; they fix the counter values the RMSNorm rows wait for)."""
        self.shape = shape
        self.oproj_blocks, self.down_blocks = shape.hidden_size // oproj_tile, shape.hidden_size // down_tile
        self.stride = shape.num_attention_heads + 2 * shape.num_key_value_heads   # counter slots per batch row

    # ---- state ---------------------------------------------------------------
    @staticmethod
    def _active(g: Any, b: int) -> bool:
        mask = getattr(g, "active_mask", None)
        return True if mask is None else bool(mask[b])

    @staticmethod
    def _pos(g: Any, b: int) -> int:
        ids = getattr(g, "position_ids", None)
        return int(ids[b]) if ids is not None else int(g.position_id or 0)

    def _instruction_active(self, flag: int, g: Any, b: int) -> bool:
        return False if flag == 0 else (True if flag == 1 else self._active(g, b))

    # ---- dispatcher ------------------------------------------------------------
    def run(self, g: Any, instructions: Iterable[Any]) -> None:
        table = {0: lambda g, i: None, 1: self.attn_rms, 2: self.qkvproj_gemm_rope, 3: self.decode_attention_split_kv,
                 4: self.decode_attention_reduction, 5: self.oproj_gemm_residual, 6: self.mlp_rms,
                 7: self.upgate_proj_gemm_silu, 8: self.down_proj_residual, 9: self.lmhead_rms, 10: self.lmhead_proj_gemm}
        for ins in instructions:
            table[ins.opcode()](g, ins)

    # ---- 1, 6, 9: RMSNorm rows ---------------------------------------------------
    def _rms_row(self, g: Any, dst: Tensor, row: int, weight: Tensor) -> None:
        if self._active(g, row):
            dst[row] = rms_norm(g.hidden_states[row], weight, self.shape.rms_norm_eps).to(dst.dtype)
        else:
            dst[row].zero_()

    def attn_rms(self, g: Any, ins: Any) -> None:
        if ins.layer_idx > 0:
            assert int(g.barriers[ins.layer_idx - 1, 7, 0]) == self.down_blocks
        self._rms_row(g, g.attn_rms_out, ins.batch_row, g.attn_norm_weights[ins.layer_idx])
        g.barriers[ins.layer_idx, 0, 0] += 1

    def mlp_rms(self, g: Any, ins: Any) -> None:
        assert int(g.barriers[ins.layer_idx, 4, 0]) == self.oproj_blocks
        self._rms_row(g, g.mlp_rms_out, ins.batch_row, g.mlp_norm_weights[ins.layer_idx])
        g.barriers[ins.layer_idx, 5, 0] += 1

    def lmhead_rms(self, g: Any, ins: Any) -> None:
        last = self.shape.num_hidden_layers - 1
        assert int(g.barriers[last, 7, 0]) == self.down_blocks
        self._rms_row(g, g.lm_head_rms_out, ins.batch_row, g.lm_head_norm_weights)
        g.barriers[last, 8, 0] += 1

    # ---- 2 -------------------------------------------------------------------------
    def qkvproj_gemm_rope(self, g: Any, ins: Any) -> None:
        s = self.shape
        layer, B, d, tile = ins.layer_idx, ins.batch_size, s.head_dim, ins.tile_N_granularity
        assert int(g.barriers[layer, 0, 0]) == B
        assert ins.tile_M_granularity == TILE, "one M tile covers the batch"
        k_start = s.num_attention_heads * d
        v_start = k_start + s.num_key_value_heads * d
        row, end = ins.tile_N_start_idx * tile, ins.tile_N_end_idx * tile
        while row < end:
            # one chunk never leaves its head, nor its q / k / v segment
            stop = min((row // d + 1) * d, end)
            seg = "q" if row < k_start else ("k" if row < v_start else "v")
            out = _gemm(g.qkv_weights[layer], g.attn_rms_out, row, stop)        # bf16 [B, chunk]
            for b in range(B):
                if not self._active(g, b):
                    continue
                pos, mine = self._pos(g, b), out[b]
                if getattr(s, "qk_norm", False):
                    # Qwen3 op set (qwen3__0_6b/…/instructions/python_vm.py:110-141, per row): the raw vector
                    # only; norm, RoPE and the cache rows belong to the attention instruction.
                    g.qkv_raw[b, row:stop] = mine.to(g.qkv_raw.dtype)
                    continue
                if seg != "v":
                    # RoPE pairs are neighbours, so a chunk that starts on an even column is closed under it
                    h0 = row % d
                    cos, sin = g.rope_cos[pos][h0 : h0 + stop - row], g.rope_sin[pos][h0 : h0 + stop - row]
                    mine = mine * cos + rotate_pairs(mine) * sin
                if seg == "q":
                    g.q_post_rope[b, row:stop] = mine.to(g.q_post_rope.dtype)
                elif seg == "k":
                    g.k_cache[layer, b, pos].view(-1)[row - k_start : stop - k_start] = mine.to(g.k_cache.dtype)
                else:
                    g.v_cache[layer, b, pos].view(-1)[row - v_start : stop - v_start] = mine.to(g.v_cache.dtype)
            for blk in range(row // tile, (stop + tile - 1) // tile):
                g.barriers[layer, 1, blk // (d // tile)] += 1
            row = stop

    # ---- 3 -------------------------------------------------------------------------
    def decode_attention_split_kv(self, g: Any, ins: Any) -> None:
        s = self.shape
        ratio, d = s.num_attention_heads // s.num_key_value_heads, s.head_dim
        layer, b, kvh, part = ins.layer_idx, ins.batch_idx, ins.kv_head_idx, ins.partial_idx
        per_head = d // TILE
        qkv_done = g.barriers[layer, 1]
        for i in range(ratio):
            assert int(qkv_done[kvh * ratio + i]) == per_head
        assert int(qkv_done[s.num_attention_heads + kvh]) == per_head
        assert int(qkv_done[s.num_attention_heads + s.num_key_value_heads + kvh]) == per_head
        h0, h1 = kvh * ratio, (kvh + 1) * ratio
        mine = g.barriers[layer, 2, b * self.stride : (b + 1) * self.stride]
        seq_len = ins.seq_len if ins.seq_len >= 0 else self._pos(g, b) + 1

        def arrive() -> None:
            mine[h0:h1] += 1
            # extension of this build: the arrival that completes the group merges it
            if getattr(ins, "merge_in_last", 0) and int(mine[h0]) == ins.num_partials:
                self.decode_attention_reduction(g, _MergeAll(layer, b, h0, ins.num_partials))   # the row's flag decides, not this slice's

        def leave_empty() -> None:
            g.attn_lse_intermediates[b, h0:h1, part] = INACTIVE_LSE
            g.attn_out_intermediates[b, h0:h1, part] = 0.0
            if g.attn_partial_valid is not None:
                g.attn_partial_valid[b, h0:h1, part] = False
            arrive()

        if not self._instruction_active(ins.is_active, g, b):
            return leave_empty()
        kvb = s.attn_kv_block_size
        total = max(1, math.ceil(seq_len / kvb))
        per = max(1, math.ceil(total / ins.num_partials))
        t0 = part * per * kvb
        t1 = min(min(part * per + per, total) * kvb, seq_len)
        if t0 >= t1:
            return leave_empty()
        if getattr(s, "qk_norm", False):
            # Qwen3 op set (qwen3__0_6b/…/instructions/python_vm.py:214-320, per row): q and k of this KV head get
            # their per-head RMSNorm and RoPE here and K/V of the row's position enter the cache.  Every slice
            # with work computes the same values, so the sequential VM simply writes them each time.
            nq, nkv, pos = s.num_attention_heads, s.num_key_value_heads, self._pos(g, b)
            raw = g.qkv_raw[b]
            k_off, v_off = (nq + kvh) * d, (nq + nkv + kvh) * d
            cos, sin = g.rope_cos[pos].unsqueeze(0), g.rope_sin[pos].unsqueeze(0)
            qn = per_head_rms_norm(raw[h0 * d : h1 * d].view(ratio, d), g.q_norm_weights[layer], s.rms_norm_eps)
            kn = per_head_rms_norm(raw[k_off : k_off + d].view(1, d), g.k_norm_weights[layer], s.rms_norm_eps)
            g.q_post_rope[b].view(nq, d)[h0:h1] = ((qn * cos) + (rotate_pairs(qn) * sin)).to(g.q_post_rope.dtype)
            g.k_cache[layer, b, pos, kvh] = ((kn * cos) + (rotate_pairs(kn) * sin)).view(-1).to(g.k_cache.dtype)
            g.v_cache[layer, b, pos, kvh] = raw[v_off : v_off + d].to(g.v_cache.dtype)
        k = g.k_cache[layer, b, t0:t1, kvh].float()
        v = g.v_cache[layer, b, t0:t1, kvh].float()
        q = g.q_post_rope[b].view(s.num_attention_heads, d)[h0:h1].float()
        scores = torch.einsum("hi,ki->hk", q, k) * (1 / math.sqrt(d))
        g.attn_lse_intermediates[b, h0:h1, part] = torch.log2(torch.exp(scores).sum(dim=-1))
        g.attn_out_intermediates[b, h0:h1, part] = torch.einsum("hk,ko->ho", torch.softmax(scores, dim=-1), v)
        if g.attn_partial_valid is not None:
            g.attn_partial_valid[b, h0:h1, part] = True
        arrive()

    # ---- 4 -------------------------------------------------------------------------
    def decode_attention_reduction(self, g: Any, ins: Any) -> None:
        s = self.shape
        layer, b, h0, R = ins.layer_idx, ins.batch_idx, ins.head_start_idx, s.attn_reduction_size
        if not self._instruction_active(ins.is_active, g, b):
            g.attn_out[b].view(s.num_attention_heads, -1)[h0 : h0 + R].zero_()
            g.barriers[layer, 3, b] += R
            return
        assert int(g.barriers[layer, 2, b * self.stride + h0]) == ins.num_partials
        idx = torch.as_tensor(ins.reduction_list, dtype=torch.long).reshape(-1)
        lses = g.attn_lse_intermediates[b, h0 : h0 + R][:, idx]
        outs = g.attn_out_intermediates[b, h0 : h0 + R][:, idx]
        if g.attn_partial_valid is not None:
            valid = g.attn_partial_valid[b, h0 : h0 + R][:, idx].to(torch.bool)
        else:
            valid = torch.isfinite(lses) & (lses > NONCONTRIBUTING_LSE)
        # log2-domain merge over the valid partials only
        mx = torch.where(valid, lses, torch.full_like(lses, -1e9)).max(dim=-1, keepdim=True).values
        any_valid = valid.any(dim=-1, keepdim=True)
        mx = torch.where(any_valid, mx, torch.full_like(mx, INACTIVE_LSE))
        wgt = torch.where(valid, (lses - mx).exp2(), torch.zeros_like(lses))
        den = wgt.sum(dim=-1, keepdim=True)
        merged = (outs * wgt.unsqueeze(-1)).sum(dim=-2) / den
        if ins.is_terminal:
            g.attn_out[b].view(s.num_attention_heads, -1)[h0 : h0 + R] = merged.to(g.attn_out.dtype)
        else:
            dead = 0.0 if g.attn_partial_valid is not None else MERGED_EMPTY_LSE
            new_lse = torch.where(any_valid.squeeze(-1), mx.squeeze(-1) + torch.log2(den.squeeze(-1)),
                                  torch.full_like(den.squeeze(-1), dead))
            slot = ins.output_partial_idx
            g.attn_lse_intermediates[b, h0 : h0 + R, slot] = new_lse
            g.attn_out_intermediates[b, h0 : h0 + R, slot] = merged
            if g.attn_partial_valid is not None:
                g.attn_partial_valid[b, h0 : h0 + R, slot] = any_valid.squeeze(-1)
        g.barriers[layer, 3, b] += R

    # ---- 5, 8: GEMM + residual -------------------------------------------------------
    def _gemm_residual(self, g: Any, ins: Any, mat: Tensor, act: Tensor, my_row: int) -> None:
        B, tile = ins.batch_size, ins.tile_N_granularity
        for blk in range(ins.tile_N_start_idx, ins.tile_N_end_idx):
            out = _gemm(mat, act[:B], blk * tile, (blk + 1) * tile).to(g.hidden_states.dtype)
            for b in range(B):
                if not self._active(g, b):
                    out[b].zero_()
            g.hidden_states[:B, blk * tile : (blk + 1) * tile] += out
            g.barriers[ins.layer_idx, my_row, 0] += 1

    def oproj_gemm_residual(self, g: Any, ins: Any) -> None:
        assert bool(torch.all(g.barriers[ins.layer_idx, 3, : ins.batch_size] == self.shape.num_attention_heads))
        assert ins.reduction_block_idx == 0
        self._gemm_residual(g, ins, g.o_proj_weights[ins.layer_idx], g.attn_out, 4)

    def down_proj_residual(self, g: Any, ins: Any) -> None:
        assert int(g.barriers[ins.layer_idx, 6, 0]) == self.shape.intermediate_size // TILE
        self._gemm_residual(g, ins, g.down_proj_weights[ins.layer_idx], g.silu_out, 7)

    # ---- 7 -------------------------------------------------------------------------
    def upgate_proj_gemm_silu(self, g: Any, ins: Any) -> None:
        B, tile, layer = ins.batch_size, ins.tile_N_granularity, ins.layer_idx
        assert int(g.barriers[layer, 5, 0]) == B
        y = g.mlp_rms_out[:B]
        for blk in ins.tile_N_block_idxs:
            r0, r1 = blk * tile, (blk + 1) * tile
            out = (F.silu(_gemm(g.gate_proj_weights[layer], y, r0, r1)) * _gemm(g.up_proj_weights[layer], y, r0, r1)).to(g.silu_out.dtype)
            for b in range(B):
                if not self._active(g, b):
                    out[b].zero_()
            g.silu_out[:B, r0:r1] = out
            g.barriers[layer, 6, 0] += 1

    # ---- 10 ------------------------------------------------------------------------
    def lmhead_proj_gemm(self, g: Any, ins: Any) -> None:
        last = self.shape.num_hidden_layers - 1
        assert int(g.barriers[last, 8, 0]) == ins.batch_size
        tile = ins.tile_N_granularity
        for blk in range(ins.start_output_block_idx, ins.end_output_block_idx):
            out = _gemm(g.lm_head_weights, g.lm_head_rms_out, blk * tile, (blk + 1) * tile).to(g.logits.dtype)
            if getattr(g, "active_mask", None) is not None:
                for b in range(out.shape[0]):
                    if not self._active(g, b):
                        out[b] = -1e9
            g.logits[:, blk * tile : (blk + 1) * tile] = out
