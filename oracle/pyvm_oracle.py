"""Sequential instruction VM — TEST INFRASTRUCTURE, not product code.

Only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline``
leg may import this module, and only as the checker.

Executes a decode instruction list one instruction at a time on a
``Globals``-shaped object, tile by tile, asserting every counter it consumes and
bumping every counter it produces: the specification of the device kernel at
instruction granularity.  Restates the reference's Python VM
(``qimeng_megakernel/models/LLM/llama/llama3_2__1b/A100/single_batch/decode_schedule/instructions/python_vm.py``):

================================  ========================
``oproj_gemv_residual``           python_vm.py:109-134
``down_proj_residual``            python_vm.py:137-171
``rms_upgate_proj_gemv_silu``     python_vm.py:174-214
``rms_qkvproj_gemv_rope``         python_vm.py:217-343
``rms_lmhead_gemv``               python_vm.py:346-370
``decode_attention_split_kv``     python_vm.py:373-436
``decode_attention_reduction``    python_vm.py:439-488
================================  ========================

Differences, all forced by running schedules other than the A100 one: the final
counter values a consumer asserts are computed from the producing instruction's
tile size (``counts``) instead of module constants, and instructions are
recognised by ``opcode()`` and attribute names, not by class identity.  A
non-terminal reduction (never scheduled) stores ``max + log2(denominator)`` so
that a later merge is consistent; the reference stores ``ln(denominator)``.

Pinning: the split-KV/merge algebra is checked against brute-force softmax
attention for every partition (tests/test_oracle_math.py); the GEMV tiles must
reproduce the fused oracle bit for bit when a schedule does not split K; the
counter end state is a pure-integer known answer.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Iterable

import torch
import torch.nn.functional as F

from fused_oracle import per_head_rms_norm, rms_norm, rotate_pairs

Tensor = torch.Tensor

ROW_QKV, ROW_SPLITKV, ROW_REDUCE, ROW_OPROJ, ROW_UPGATE, ROW_DOWN = range(6)


@dataclass(frozen=True)
class Counts:
    """Final counter values implied by the scheduler's tile geometry."""

    qkv_blocks_per_head: int = 4
    oproj_blocks: int = 128
    upgate_blocks_per_bucket: int = 128
    down_arrivals: int = 512


def _tile_gemv(mat: Tensor, vec: Tensor, r0: int, r1: int, k0: int | None = None, k1: int | None = None) -> Tensor:
    m = mat[r0:r1] if k0 is None else mat[r0:r1, k0:k1]
    v = vec if k0 is None else vec[k0:k1]
    return torch.einsum("oi,i->o", m, v)


class InstructionVM:
    def __init__(self, shape: Any, counts: Counts = Counts()):
        self.shape = shape
        self.counts = counts

    # ---- dispatcher -----------------------------------------------------------
    def run(self, g: Any, instructions: Iterable[Any]) -> None:
        table = {
            0: lambda g, i: None,
            1: self.rms_qkvproj_gemv_rope,
            2: self.decode_attention_split_kv,
            3: self.decode_attention_reduction,
            4: self.oproj_gemv_residual,
            5: self.rms_upgate_proj_gemv_silu,
            6: self.down_proj_residual,
            7: self.rms_lmhead_gemv,
        }
        for ins in instructions:
            table[ins.opcode()](g, ins)

    # ---- 4 --------------------------------------------------------------------
    def oproj_gemv_residual(self, g: Any, ins: Any) -> None:
        s = self.shape
        if ins.reduction_block_idx == 0:
            assert int(g.barriers[ins.layer_idx, ROW_REDUCE, 0]) == s.num_attention_heads
        else:
            # Extension: this instruction merges the split-KV partials itself (all heads); the
            # reduction row then counts one arrival per split-KV instruction.
            P = ins.reduction_block_idx
            assert int(g.barriers[ins.layer_idx, ROW_REDUCE, 0]) == s.num_key_value_heads * P
            for h0 in range(0, s.num_attention_heads, s.attn_reduction_size):
                self._merge(g, ins.layer_idx, h0, list(range(P)), True, 0, count=False)
        tile = ins.tile_N_granularity
        w = g.o_proj_weights[ins.layer_idx]
        for blk in range(ins.tile_N_start_idx, ins.tile_N_end_idx):
            r0, r1 = blk * tile, (blk + 1) * tile
            out = _tile_gemv(w, g.attn_out, r0, r1, 0, s.hidden_size)
            g.hidden_states[r0:r1] += out.to(g.hidden_states.dtype)
            g.barriers[ins.layer_idx, ROW_OPROJ, 0] += 1

    # ---- 6 --------------------------------------------------------------------
    def down_proj_residual(self, g: Any, ins: Any) -> None:
        s = self.shape
        assert int(g.barriers[ins.layer_idx, ROW_UPGATE, ins.split_K_idx]) == self.counts.upgate_blocks_per_bucket
        tile, kg = ins.tile_N_granularity, ins.split_K_granularity
        k0 = ins.split_K_idx * kg
        k1 = min(k0 + kg, s.intermediate_size)
        w = g.down_proj_weights[ins.layer_idx]
        for blk in range(ins.tile_N_start_idx, ins.tile_N_end_idx):
            r0, r1 = blk * tile, (blk + 1) * tile
            out = _tile_gemv(w, g.silu_out, r0, r1, k0, k1)
            g.hidden_states[r0:r1] += out.to(g.hidden_states.dtype)
            g.barriers[ins.layer_idx, ROW_DOWN, 0] += 1

    # ---- 5 --------------------------------------------------------------------
    def rms_upgate_proj_gemv_silu(self, g: Any, ins: Any) -> None:
        s = self.shape
        assert int(g.barriers[ins.layer_idx, ROW_OPROJ, 0]) == self.counts.oproj_blocks
        y = rms_norm(g.hidden_states, g.mlp_norm_weights[ins.layer_idx], s.rms_norm_eps)
        tile = ins.tile_N_granularity
        for blk in ins.tile_N_block_idxs:
            r0, r1 = blk * tile, (blk + 1) * tile
            up = _tile_gemv(g.up_proj_weights[ins.layer_idx], y, r0, r1)
            gate = _tile_gemv(g.gate_proj_weights[ins.layer_idx], y, r0, r1)
            g.silu_out[r0:r1] = F.silu(gate) * up
            g.barriers[ins.layer_idx, ROW_UPGATE, blk // self.counts.upgate_blocks_per_bucket] += 1

    # ---- 1 --------------------------------------------------------------------
    def rms_qkvproj_gemv_rope(self, g: Any, ins: Any) -> None:
        s = self.shape
        layer = ins.layer_idx
        if layer > 0:
            assert int(g.barriers[layer - 1, ROW_DOWN, 0]) == self.counts.down_arrivals
        assert ins.tile_M_granularity == 1
        y = rms_norm(g.hidden_states, g.attn_norm_weights[layer], s.rms_norm_eps)
        pos = int(g.position_id)
        d, tile = s.head_dim, ins.tile_N_granularity
        k_start = s.num_attention_heads * d
        v_start = k_start + s.num_key_value_heads * d
        blocks_per_head = d // tile
        cos, sin = g.rope_cos[pos], g.rope_sin[pos]
        row, end = ins.tile_N_start_idx * tile, ins.tile_N_end_idx * tile
        while row < end:
            # one chunk never leaves its head, nor its q / k / v segment
            stop = min((row // d + 1) * d, end)
            seg = "q" if row < k_start else ("k" if row < v_start else "v")
            out = _tile_gemv(g.qkv_weights[layer], y, row, stop, 0, s.hidden_size)
            if getattr(s, "qk_norm", False):
                # Qwen3 op set (qwen3__0_6b/…/instructions/python_vm.py:110-141): the raw vector only;
                # norm, RoPE and the cache write belong to the attention instruction.
                g.qkv_raw[row:stop] = out.to(g.qkv_raw.dtype)
                for blk in range(row // tile, (stop + tile - 1) // tile):
                    g.barriers[layer, ROW_QKV, blk // blocks_per_head] += 1
                row = stop
                continue
            if seg != "v":
                head = torch.zeros(1, d, dtype=out.dtype)
                a = row % d
                head[:, a : a + (stop - row)] = out.view(1, -1)
                rot = (head * cos.unsqueeze(0)) + (rotate_pairs(head) * sin.unsqueeze(0))
                out = rot[:, a : a + (stop - row)].reshape(-1)
            if seg == "q":
                g.q_post_rope[row:stop] = out.to(g.q_post_rope.dtype)
            elif seg == "k":
                g.k_cache[layer, :, pos].view(-1)[row - k_start : stop - k_start] = out.to(g.k_cache.dtype)
            else:
                g.v_cache[layer, :, pos].view(-1)[row - v_start : stop - v_start] = out.to(g.v_cache.dtype)
            for blk in range(row // tile, (stop + tile - 1) // tile):
                g.barriers[layer, ROW_QKV, blk // blocks_per_head] += 1
            row = stop

    # ---- 7 --------------------------------------------------------------------
    def rms_lmhead_gemv(self, g: Any, ins: Any) -> None:
        s = self.shape
        assert int(g.barriers[s.num_hidden_layers - 1, ROW_DOWN, 0]) == self.counts.down_arrivals
        y = rms_norm(g.hidden_states, g.lm_head_norm_weights, s.rms_norm_eps)
        tile = ins.tile_N_granularity
        for blk in range(ins.start_output_block_idx, ins.end_output_block_idx):
            r0, r1 = blk * tile, (blk + 1) * tile
            g.logits[r0:r1] = torch.einsum("oi,i->o", g.lm_head_weights[r0:r1], y)

    # ---- 2 --------------------------------------------------------------------
    def decode_attention_split_kv(self, g: Any, ins: Any) -> None:
        s = self.shape
        nq, nkv, d = s.num_attention_heads, s.num_key_value_heads, s.head_dim
        ratio = nq // nkv
        row0 = g.barriers[ins.layer_idx, ROW_QKV]
        bph = self.counts.qkv_blocks_per_head
        for i in range(ratio):
            assert int(row0[ins.kv_head_idx * ratio + i]) == bph
        assert int(row0[nq + ins.kv_head_idx]) == bph
        assert int(row0[nq + nkv + ins.kv_head_idx]) == bph

        seq_len = int(g.position_id or 0) + 1
        block = s.attn_kv_block_size
        total_blocks = math.ceil(seq_len / block)
        per_partial = math.ceil(total_blocks / ins.num_partials)
        b0 = ins.partial_idx * per_partial
        b1 = min(b0 + per_partial, total_blocks)
        t0, t1 = b0 * block, min(b1 * block, seq_len)

        h0, h1 = ins.kv_head_idx * ratio, (ins.kv_head_idx + 1) * ratio
        if getattr(s, "qk_norm", False):
            # Qwen3 op set (qwen3__0_6b/…/instructions/python_vm.py:214-320): q and k of this KV head
            # get their per-head RMSNorm and RoPE here; K/V of this position enter the cache.  Every
            # partial computes the same values, so the sequential VM simply writes them each time.
            pos = int(g.position_id or 0)
            raw = g.qkv_raw
            k_off, v_off = nq * d + ins.kv_head_idx * d, (nq + nkv) * d + ins.kv_head_idx * d
            cos, sin = g.rope_cos[pos].unsqueeze(0), g.rope_sin[pos].unsqueeze(0)
            qn = per_head_rms_norm(raw[h0 * d : h1 * d].view(ratio, d), g.q_norm_weights[ins.layer_idx], s.rms_norm_eps)
            kn = per_head_rms_norm(raw[k_off : k_off + d].view(1, d), g.k_norm_weights[ins.layer_idx], s.rms_norm_eps)
            g.q_post_rope.view(nq, d)[h0:h1] = ((qn * cos) + (rotate_pairs(qn) * sin)).to(g.q_post_rope.dtype)
            g.k_cache[ins.layer_idx, 0, pos, ins.kv_head_idx] = ((kn * cos) + (rotate_pairs(kn) * sin)).view(-1).to(g.k_cache.dtype)
            g.v_cache[ins.layer_idx, 0, pos, ins.kv_head_idx] = raw[v_off : v_off + d].to(g.v_cache.dtype)
        q = g.q_post_rope.view(nq, -1)[h0:h1].float()
        k = g.k_cache[ins.layer_idx, 0, t0:t1, ins.kv_head_idx].float()
        v = g.v_cache[ins.layer_idx, 0, t0:t1, ins.kv_head_idx].float()
        scores = torch.einsum("hi,ki->hk", q, k) * (1 / math.sqrt(d))
        probs = torch.softmax(scores, dim=-1)
        lse2 = torch.log2(torch.sum(torch.exp(scores), dim=-1))  # -inf for an empty slice
        out = torch.einsum("hk,ko->ho", probs, v)               # zeros for an empty slice
        g.attn_lse_intermediates[h0:h1, ins.partial_idx] = lse2
        g.attn_out_intermediates[h0:h1, ins.partial_idx] = out
        # Extension of this build's schedules (operand word 5, zero in the reference's streams):
        # 1 = the arrival that completes the head group merges all partials itself;
        # 2 = arrive on the reduction row only, the O-proj instructions merge.
        mode = getattr(ins, "merge_in_last", 0)
        if mode == 2:
            g.barriers[ins.layer_idx, ROW_REDUCE, 0] += 1
            return
        g.barriers[ins.layer_idx, ROW_SPLITKV, h0:h1] += 1
        if mode == 1 and int(g.barriers[ins.layer_idx, ROW_SPLITKV, h0]) == ins.num_partials:
            self._merge(g, ins.layer_idx, h0, list(range(ins.num_partials)), True, 0)

    # ---- 3 --------------------------------------------------------------------
    def decode_attention_reduction(self, g: Any, ins: Any) -> None:
        s = self.shape
        h0 = ins.head_start_idx
        assert int(g.barriers[ins.layer_idx, ROW_SPLITKV, h0]) == ins.num_partials
        self._merge(g, ins.layer_idx, h0, ins.reduction_list, ins.is_terminal, ins.output_partial_idx)

    def _merge(self, g: Any, layer: int, h0: int, reduction_list, is_terminal, output_partial_idx, count=True) -> None:
        s = self.shape
        h1 = h0 + s.attn_reduction_size
        idx = torch.tensor(list(reduction_list), dtype=torch.long)
        lses = g.attn_lse_intermediates[h0:h1][:, idx]
        outs = g.attn_out_intermediates[h0:h1][:, idx]
        top = lses.max(dim=-1, keepdim=True).values
        factors = (lses - top).exp2()
        denom = factors.sum(dim=-1, keepdim=True)
        merged = (outs * factors.unsqueeze(-1)).sum(dim=1) / denom
        if is_terminal:
            g.attn_out.view(s.num_attention_heads, -1)[h0:h1] = merged
        else:
            g.attn_lse_intermediates[h0:h1, output_partial_idx] = (top + denom.log2()).squeeze(-1)
            g.attn_out_intermediates[h0:h1, output_partial_idx] = merged
        if count:
            g.barriers[layer, ROW_REDUCE, 0] += s.attn_reduction_size
