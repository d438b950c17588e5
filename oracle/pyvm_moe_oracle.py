"""Sequential instruction VM of the MoE decode route — TEST INFRASTRUCTURE, not product code.

Only ``tests/`` may import this module, and only as the checker.

Restates the reference's handlers
(``…/qwen/qwen1_5_moe_a2_7b/A100/single_batch/decode_schedule/instructions/python_vm.py``): the fused
route's arithmetic cut into the tiles the instructions name, plus the counter protocol.  Where the VM
(and the reference's kernel) differs from the fused route, the VM is followed: the shared down
projection is split along K and accumulates bf16 partial sums, and the combine step adds
``hidden + routed_f32 + sigmoid(gate) * shared`` in fp32 with one rounding.

===============================  =====================
``rms_qkvproj_gemv_rope``        python_vm.py:109-207
``decode_attention_split_kv``    python_vm.py:210-267
``decode_attention_reduction``   python_vm.py:270-306
``oproj_gemv_residual``          python_vm.py:309-327
``router_gemv``                  python_vm.py:331-357
``router_softmax_topk``          python_vm.py:360-372
``shared_expert_upgate_silu``    python_vm.py:375-396
``shared_expert_downproj``       python_vm.py:399-418
``routed_expert_upgate_silu``    python_vm.py:421-464
``routed_expert_downproj``       python_vm.py:467-489
``moe_combine_commit``           python_vm.py:492-530
``rms_lmhead_gemv``              python_vm.py:533-546
===============================  =====================

A shape with ``qk_norm`` takes the Qwen3 route's protocol for opcodes 1 and 2 (…/qwen/qwen3__0_6b/A100/
single_batch/decode_schedule/instructions/python_vm.py:110-141, 214-320): opcode 1 leaves the raw QKV vector, every
split-KV instruction normalises and rotates the q heads and the K row of its KV head and writes the cache rows.
``norm_topk_prob`` divides the top-k probabilities by their sum (…/fused/operations.py:405); a shape without a
shared expert has no opcodes 10/11 and opcode 14 adds the routed experts only.

Pinning: tests/test_moe_oracle.py — against the fused MoE oracle within bf16 tolerance, final
counter values, and the fixture written by tests/golden/make_fixtures_moe.py from the imported
reference, which ran the reference's VM on the same instruction list in lock-step with this one.
"""
from __future__ import annotations

import math
from typing import Any, Iterable

import torch
import torch.nn.functional as F

from fused_oracle import per_head_rms_norm, rms_norm, rotate_pairs

Tensor = torch.Tensor
TILE = 16


def _rows(mat: Tensor, vec: Tensor, r0: int, r1: int, k0: int | None = None, k1: int | None = None) -> Tensor:
    vec = vec.reshape(-1).to(mat.dtype)
    if k0 is not None:
        return torch.matmul(mat[r0:r1, k0:k1], vec[k0:k1])
    return torch.matmul(mat[r0:r1], vec)


class MoeInstructionVM:
    def __init__(self, shape: Any):
        self.shape = shape

    def run(self, g: Any, instructions: Iterable[Any]) -> None:
        table = {0: lambda g, i: None, 1: self.rms_qkvproj_gemv_rope, 2: self.decode_attention_split_kv,
                 3: self.decode_attention_reduction, 4: self.oproj_gemv_residual, 7: self.rms_lmhead_gemv, 8: self.router_gemv,
                 9: self.router_softmax_topk, 10: self.shared_expert_upgate_silu, 11: self.shared_expert_downproj,
                 12: self.routed_expert_upgate_silu, 13: self.routed_expert_downproj, 14: self.moe_combine_commit}
        for ins in instructions:
            table[ins.opcode()](g, ins)

    # ---- 1 -----------------------------------------------------------------------
    def rms_qkvproj_gemv_rope(self, g: Any, ins: Any) -> None:
        s = self.shape
        layer, d, tile = ins.layer_idx, s.head_dim, ins.tile_N_granularity
        assert tile % 2 == 0 and d % tile == 0     # a tile holds whole RoPE pairs of one head
        self._qkv_tile = tile                      # a head's counter ends at d / (the stream's tile): 16 rows in the reference
        if layer > 0:
            assert self._layer_complete(g, layer - 1)
        y = rms_norm(g.hidden_states.reshape(-1), g.attn_norm_weights[layer], s.rms_norm_eps).reshape(-1)
        pos = int(g.position_id or 0)
        k_start = s.num_attention_heads * d
        v_start = k_start + s.num_key_value_heads * d
        row, end = ins.tile_N_start_idx * tile, ins.tile_N_end_idx * tile
        bar = g.barriers[layer, 0]
        while row < end:
            stop = min(row + tile, end)
            if row < v_start:   # a chunk never leaves its head, nor the q / k segment
                stop = min(stop, k_start if row < k_start else v_start, (row // d + 1) * d)
            seg = "q" if row < k_start else ("k" if row < v_start else "v")
            bias = None if g.qkv_bias is None else g.qkv_bias[layer, row:stop].to(g.qkv_weights.dtype)
            out = F.linear(y, g.qkv_weights[layer, row:stop], bias)
            if getattr(s, "qk_norm", False):   # the raw vector only; norm, RoPE and the cache write belong to opcode 2
                g.qkv_raw[row:stop] = out.to(g.qkv_raw.dtype)
                for blk in range(row // tile, (stop + tile - 1) // tile):
                    bar[blk // (d // tile)] += 1
                row = stop
                continue
            if seg != "v":
                # RoPE on a head-sized row that is zero outside the chunk: pairs are neighbours
                head = torch.zeros(1, d, dtype=out.dtype)
                h0 = row % d
                head[:, h0 : h0 + stop - row] = out.view(1, -1)
                cos, sin = g.rope_cos[pos].unsqueeze(0), g.rope_sin[pos].unsqueeze(0)
                out = (head * cos + rotate_pairs(head) * sin)[:, h0 : h0 + stop - row].view(-1)
            if seg == "q":
                g.q_post_rope.reshape(-1)[row:stop] = out.to(g.q_post_rope.dtype)
            else:
                at = row - (k_start if seg == "k" else v_start)
                cache = g.k_cache if seg == "k" else g.v_cache
                cache[layer, 0, pos, at // d, at % d : at % d + stop - row] = out.to(cache.dtype)
            for blk in range(row // tile, (stop + tile - 1) // tile):
                bar[blk // (d // tile)] += 1
            row = stop

    # ---- 2, 3 --------------------------------------------------------------------
    def decode_attention_split_kv(self, g: Any, ins: Any) -> None:
        s = self.shape
        ratio, d = s.num_attention_heads // s.num_key_value_heads, s.head_dim
        layer, kvh = ins.layer_idx, ins.kv_head_idx
        done = g.barriers[layer, 0]
        per_head = d // getattr(self, "_qkv_tile", TILE)
        for i in range(ratio):
            assert int(done[kvh * ratio + i]) == per_head
        assert int(done[s.num_attention_heads + kvh]) == per_head
        assert int(done[s.num_attention_heads + s.num_key_value_heads + kvh]) == per_head
        seq_len = int(g.position_id or 0) + 1
        total = math.ceil(seq_len / s.attn_kv_block_size)
        per = math.ceil(total / ins.num_partials)
        b0 = ins.partial_idx * per
        t0, t1 = b0 * s.attn_kv_block_size, min(min(b0 + per, total) * s.attn_kv_block_size, seq_len)
        h0, h1 = kvh * ratio, (kvh + 1) * ratio
        if getattr(s, "qk_norm", False):
            # every partial computes the same values, so the sequential VM simply writes them each time
            nq, nkv, pos, raw = s.num_attention_heads, s.num_key_value_heads, int(g.position_id or 0), g.qkv_raw
            k_off, v_off = nq * d + kvh * d, (nq + nkv) * d + kvh * d
            cos, sin = g.rope_cos[pos].unsqueeze(0), g.rope_sin[pos].unsqueeze(0)
            qn = per_head_rms_norm(raw[h0 * d : h1 * d].view(ratio, d), g.q_norm_weights[layer], s.rms_norm_eps)
            kn = per_head_rms_norm(raw[k_off : k_off + d].view(1, d), g.k_norm_weights[layer], s.rms_norm_eps)
            g.q_post_rope.view(nq, d)[h0:h1] = ((qn * cos) + (rotate_pairs(qn) * sin)).to(g.q_post_rope.dtype)
            g.k_cache[layer, 0, pos, kvh] = ((kn * cos) + (rotate_pairs(kn) * sin)).view(-1).to(g.k_cache.dtype)
            g.v_cache[layer, 0, pos, kvh] = raw[v_off : v_off + d].to(g.v_cache.dtype)
        if t1 <= t0:
            lse = torch.full((ratio,), float("-inf"), dtype=torch.float32)
            out = torch.zeros(ratio, d, dtype=g.attn_out_intermediates.dtype)
        else:
            q = g.q_post_rope.view(s.num_attention_heads, -1)[h0:h1].float()
            k = g.k_cache[layer, 0, t0:t1, kvh].float()
            v = g.v_cache[layer, 0, t0:t1, kvh].float()
            scores = torch.einsum("hi,ki->hk", q, k) * (1 / math.sqrt(d))
            lse = torch.logsumexp(scores, dim=-1) / math.log(2)
            out = torch.einsum("hk,ko->ho", torch.softmax(scores, dim=-1), v)
        g.attn_lse_intermediates[h0:h1, ins.partial_idx] = lse
        g.attn_out_intermediates[h0:h1, ins.partial_idx] = out
        # extensions of this build (word 5; 0 in the reference's streams) --
        mode = getattr(ins, "merge_in_last", 0)
        if mode == 2:      # one arrival on the reduction row; the O-projection instructions merge
            g.barriers[layer, 2, 0] += 1
            return
        g.barriers[layer, 1][h0:h1] += 1
        if mode == 1 and int(g.barriers[layer, 1, h0]) == ins.num_partials:   # the completing arrival merges its heads
            self._merge_all(g, layer, h0, h1, ins.num_partials)
            g.barriers[layer, 2, 0] += ratio

    def _merge_all(self, g: Any, layer: int, h0: int, h1: int, partials: int) -> None:
        s = self.shape
        idx = torch.arange(partials)
        lses, outs = g.attn_lse_intermediates[h0:h1][:, idx], g.attn_out_intermediates[h0:h1][:, idx]
        wgt = (lses - lses.max(dim=-1, keepdim=True).values).exp2()
        g.attn_out.view(s.num_attention_heads, -1)[h0:h1] = ((outs * wgt.unsqueeze(-1)).sum(dim=1) / wgt.sum(dim=-1, keepdim=True)).to(g.attn_out.dtype)

    def decode_attention_reduction(self, g: Any, ins: Any) -> None:
        s = self.shape
        layer, h0, R = ins.layer_idx, ins.head_start_idx, s.attn_reduction_size
        assert int(g.barriers[layer, 1, h0]) == ins.num_partials
        idx = torch.tensor(ins.reduction_list, dtype=torch.long)
        lses = g.attn_lse_intermediates[h0 : h0 + R][:, idx]
        outs = g.attn_out_intermediates[h0 : h0 + R][:, idx]
        wgt = (lses - lses.max(dim=-1, keepdim=True).values).exp2()
        den = wgt.sum(dim=-1, keepdim=True)
        merged = (outs * wgt.unsqueeze(-1)).sum(dim=1) / den
        if ins.is_terminal:
            g.attn_out.view(s.num_attention_heads, -1)[h0 : h0 + R] = merged.to(g.attn_out.dtype)
        else:
            g.attn_lse_intermediates[h0 : h0 + R, ins.output_partial_idx] = den.log().squeeze(-1)
            g.attn_out_intermediates[h0 : h0 + R, ins.output_partial_idx] = merged
        g.barriers[layer, 2, 0] += R

    # ---- 4 -----------------------------------------------------------------------
    def oproj_gemv_residual(self, g: Any, ins: Any) -> None:
        s = self.shape
        if ins.reduction_block_idx == 0:
            assert int(g.barriers[ins.layer_idx, 2, 0]) == s.num_attention_heads
        else:   # extension of this build: this instruction merges the split-KV partials of all heads itself
            assert int(g.barriers[ins.layer_idx, 2, 0]) == s.num_key_value_heads * ins.reduction_block_idx
            self._merge_all(g, ins.layer_idx, 0, s.num_attention_heads, ins.reduction_block_idx)
        hidden = g.hidden_states.reshape(-1)
        for blk in range(ins.tile_N_start_idx, ins.tile_N_end_idx):
            r0, r1 = blk * ins.tile_N_granularity, (blk + 1) * ins.tile_N_granularity
            delta = _rows(g.o_proj_weights[ins.layer_idx], g.attn_out, r0, r1, 0, s.num_attention_heads * s.head_dim)
            hidden[r0:r1] = (delta.float() + hidden[r0:r1].float()).to(hidden.dtype)
            g.barriers[ins.layer_idx, 3, 0] += 1

    # ---- 8, 9 --------------------------------------------------------------------
    def router_gemv(self, g: Any, ins: Any) -> None:
        s, layer = self.shape, ins.layer_idx
        assert int(g.barriers[layer, 3, 0]) == s.hidden_size // getattr(s, "oproj_tile", TILE)
        normed = rms_norm(g.hidden_states.reshape(-1), g.mlp_norm_weights[layer], s.rms_norm_eps)
        e0 = ins.tile_N_start_idx * ins.tile_N_granularity
        e1 = min(ins.tile_N_end_idx * ins.tile_N_granularity, s.num_experts)
        for e in range(e0, e1):
            g.router_logits_buf[e] = (g.router_weights[layer, e].float() * normed.float()).sum().item()
        g.barriers[layer, 7, 0] += e1 - e0
        if ins.write_normed_hidden:
            g.normed_hidden_states.copy_(normed.to(g.normed_hidden_states.dtype))
            g.barriers[layer, 7, 1] += 1

    def router_softmax_topk(self, g: Any, ins: Any) -> None:
        s, layer = self.shape, ins.layer_idx
        assert int(g.barriers[layer, 7, 0]) == s.num_experts
        top_p, top_i = torch.topk(F.softmax(g.router_logits_buf, dim=-1), s.num_experts_per_tok, dim=-1)
        if getattr(s, "norm_topk_prob", False):
            top_p = top_p / top_p.sum(dim=-1, keepdim=True)
        g.expert_indices.copy_(top_i.to(g.expert_indices.dtype))
        g.expert_weights.copy_(top_p.to(g.expert_weights.dtype))
        g.barriers[layer, 8, 0] = 1

    # ---- 10, 11 ------------------------------------------------------------------
    def shared_expert_upgate_silu(self, g: Any, ins: Any) -> None:
        layer = ins.layer_idx
        if ins.init_shared_out:
            g.shared_out.zero_()
        assert int(g.barriers[layer, 7, 1]) == 1
        normed = g.normed_hidden_states.reshape(-1)
        for blk in range(ins.tile_N_start_idx, ins.tile_N_end_idx):
            r0, r1 = blk * ins.tile_N_granularity, (blk + 1) * ins.tile_N_granularity
            gate = _rows(g.shared_expert_gate_proj_weights[layer], normed, r0, r1)
            up = _rows(g.shared_expert_up_proj_weights[layer], normed, r0, r1)
            g.shared_expert_silu_out.reshape(-1)[r0:r1] = (F.silu(gate.float()) * up.float()).to(g.shared_expert_silu_out.dtype)
            g.barriers[layer, 9, 0] += 1

    def shared_expert_downproj(self, g: Any, ins: Any) -> None:
        s, layer = self.shape, ins.layer_idx
        assert int(g.barriers[layer, 9, 0]) == s.intermediate_size // ins.tile_N_granularity
        k0 = ins.split_K_idx * ins.split_K_granularity
        k1 = min(k0 + ins.split_K_granularity, s.intermediate_size)
        shared = g.shared_out.reshape(-1)
        for blk in range(ins.tile_N_start_idx, ins.tile_N_end_idx):
            r0, r1 = blk * ins.tile_N_granularity, (blk + 1) * ins.tile_N_granularity
            part = _rows(g.shared_expert_down_proj_weights[layer], g.shared_expert_silu_out, r0, r1, k0, k1)
            shared[r0:r1] = (shared[r0:r1].float() + part.float()).to(shared.dtype)
            g.barriers[layer, 10, blk] += 1

    # ---- 12, 13 ------------------------------------------------------------------
    def routed_expert_upgate_silu(self, g: Any, ins: Any) -> None:
        s, layer = self.shape, ins.layer_idx
        assert int(g.barriers[layer, 8, 0]) == 1
        normed = g.normed_hidden_states.reshape(-1)
        eid, mid = int(g.expert_indices[ins.expert_idx]), s.moe_intermediate_size
        gate_up = g.expert_gate_up_proj_weights[layer, eid]
        for blk in range(ins.tile_N_start_idx, ins.tile_N_end_idx):
            r0, r1 = blk * ins.tile_N_granularity, (blk + 1) * ins.tile_N_granularity
            gate, up = _rows(gate_up[:mid], normed, r0, r1), _rows(gate_up[mid:], normed, r0, r1)
            piece = (F.silu(gate.float()) * up.float()).to(g.silu_out.dtype)
            g.silu_out.reshape(-1)[r0:r1] = piece            # the single buffer of the fused route is kept up to date too
            g.routed_silu_buffer[ins.expert_idx, r0:r1] = piece
        g.barriers[layer, 11, 0] += ins.tile_N_end_idx - ins.tile_N_start_idx
        g.barriers[layer, 14, ins.expert_idx] += ins.tile_N_end_idx - ins.tile_N_start_idx   # this build's per-slot count

    def routed_expert_downproj(self, g: Any, ins: Any) -> None:
        s, layer = self.shape, ins.layer_idx
        per_slot = s.moe_intermediate_size // getattr(s, "routed_upgate_tile", TILE)
        if ins.tile_M_idx == 2:
            # This build's streams for tagged launches without a shared expert: all expert slots of the instruction's
            # rows and the commit in one — the handler below for every slot in slot order, then opcode 14's arithmetic
            # on the same rows (`:467-530`).  Such a launch keeps no counters; here the rows committed are counted in
            # slot 1 of the combine row, in tiles of the instruction's granularity.
            assert not getattr(s, "has_shared_expert", True) and ins.expert_idx == 0
            assert int(g.barriers[layer, 11, 0]) == s.num_experts_per_tok * per_slot
            r0, r1 = ins.tile_N_start_idx * ins.tile_N_granularity, ins.tile_N_end_idx * ins.tile_N_granularity
            acc = torch.zeros(r1 - r0, dtype=torch.float32)
            for slot in range(s.num_experts_per_tok):
                mat = g.expert_down_proj_weights[layer, int(g.expert_indices[slot])].contiguous()
                vec = g.routed_silu_buffer[slot].reshape(-1).contiguous()
                acc += _rows(mat, vec, r0, r1).float() * g.expert_weights[slot].to(torch.float32)
            hidden = g.hidden_states.reshape(-1)
            hidden[r0:r1] = (hidden[r0:r1].float() + acc).to(hidden.dtype)
            g.routed_out_f32.reshape(-1)[r0:r1] = 0.0
            g.barriers[layer, 13, 1] += (r1 - r0) // ins.tile_N_granularity
            self._commit_tile = ins.tile_N_granularity
            return
        if ins.tile_M_idx == 1:     # this build's streams: the slot's own tiles are enough
            assert int(g.barriers[layer, 14, ins.expert_idx]) == per_slot
        else:
            assert int(g.barriers[layer, 11, 0]) == s.num_experts_per_tok * per_slot
        eid = int(g.expert_indices[ins.expert_idx])
        w = g.expert_weights[ins.expert_idx].to(torch.float32)
        mat = g.expert_down_proj_weights[layer, eid].contiguous()
        vec = g.routed_silu_buffer[ins.expert_idx].reshape(-1).contiguous()
        acc = g.routed_out_f32.reshape(-1)
        for blk in range(ins.tile_N_start_idx, ins.tile_N_end_idx):
            r0, r1 = blk * ins.tile_N_granularity, (blk + 1) * ins.tile_N_granularity
            acc[r0:r1] += _rows(mat, vec, r0, r1).float() * w
            g.barriers[layer, 12, blk] += 1

    def _layer_complete(self, g: Any, layer: int) -> bool:
        """Every row of the residual stream committed: by opcode 14 (16-row tiles, slot 0 of its counter row) or by
        opcode 13's committing form (tiles of its own granularity, slot 1)."""
        s = self.shape
        if int(g.barriers[layer, 13, 0]) == s.num_hidden_blocks:
            return True
        tile = getattr(self, "_commit_tile", TILE)
        return int(g.barriers[layer, 13, 1]) == s.hidden_size // tile

    # ---- 14 ----------------------------------------------------------------------
    def moe_combine_commit(self, g: Any, ins: Any) -> None:
        s, layer = self.shape, ins.layer_idx
        has_shared = getattr(s, "has_shared_expert", True)
        for blk in range(ins.tile_N_start_idx, ins.tile_N_end_idx):
            assert int(g.barriers[layer, 10, blk]) == (s.num_downproj_split_k_shared if has_shared else 0)
            assert int(g.barriers[layer, 12, blk]) == s.num_experts_per_tok
        r0, r1 = ins.tile_N_start_idx * ins.tile_N_granularity, ins.tile_N_end_idx * ins.tile_N_granularity
        hidden, routed = g.hidden_states.reshape(-1), g.routed_out_f32.reshape(-1)
        if has_shared:
            gate = torch.sigmoid((g.shared_expert_gate_weights[layer].reshape(-1).float() * g.normed_hidden_states.reshape(-1).float()).sum())
            hidden[r0:r1] = (hidden[r0:r1].float() + routed[r0:r1] + gate * g.shared_out.reshape(-1)[r0:r1].float()).to(hidden.dtype)
        else:
            hidden[r0:r1] = (hidden[r0:r1].float() + routed[r0:r1]).to(hidden.dtype)
        routed[r0:r1] = 0.0
        g.barriers[layer, 13, 0] += ins.tile_N_end_idx - ins.tile_N_start_idx

    # ---- 7 -----------------------------------------------------------------------
    def rms_lmhead_gemv(self, g: Any, ins: Any) -> None:
        s = self.shape
        assert self._layer_complete(g, s.num_hidden_layers - 1)
        y = rms_norm(g.hidden_states.reshape(-1), g.lm_head_norm_weights, s.rms_norm_eps)
        for blk in range(ins.start_output_block_idx, ins.end_output_block_idx):
            r0, r1 = blk * ins.tile_N_granularity, (blk + 1) * ins.tile_N_granularity
            g.logits.reshape(-1)[r0:r1] = _rows(g.lm_head_weights, y, r0, r1).to(g.logits.dtype)
