#!/usr/bin/env python3
"""Write tests/golden/qwen3_moe_reduced_seed0.json from the imported reference (Qwen3-30B-A3B geometry of the MoE route).

Runs ONLY in the build container, where the reference checkout is mounted at /root/reference; the fixture it
writes is plain JSON.  The reference has no route for this shape, so the step is put together from the functions
of its two routes, unchanged:

* attention half — the Qwen3 route's fused operations (…/qwen/qwen3__0_6b/A100/single_batch/decode_schedule/fused/
  operations.py: ``fused_rms_qkvproj_gemv``, ``fused_qknorm_rope_writecache``, ``fused_decode_attention``,
  ``fused_oproj_gemv_residual``) with its config pointed at 32 query / 4 KV heads of 128;
* MoE half — the MoE route's ``fused_moe_block`` (…/qwen/qwen1_5_moe_a2_7b/A100/single_batch/decode_schedule/fused/
  operations.py:255-290) with an all-zero shared expert, its ``fused_router`` followed by the renormalisation the
  reference applies under ``norm_topk_prob`` (``top_probs / top_probs.sum(dim=-1, keepdim=True)``, `:405`).  That line
  lives in the reference's prefill block, so the renormalised weights are also checked against what that block
  itself computes for a one-token sequence (it keeps them in bf16: compared after the same rounding);
* LM head — the MoE route's ``fused_rms_lmhead_gemv``.

This repository's fused MoE oracle runs the same request in lock-step on a shape without a shared expert; every
buffer must agree bit for bit after every layer, or nothing is written.  Reduced shape: 2 layers, vocabulary 2048,
16 experts of 256 with top-4 routing.

usage: python tests/golden/make_fixtures_qwen3_moe.py [--steps 8]
"""
from __future__ import annotations

import argparse
import dataclasses
import importlib
import json
import sys
from pathlib import Path

import torch

ROOT = Path(__file__).resolve().parents[2]
REFERENCE = Path("/root/reference")
OUT = Path(__file__).resolve().parent
Q3 = "qimeng_megakernel.models.LLM.qwen.qwen3__0_6b.A100.single_batch.decode_schedule"
MOE = "qimeng_megakernel.models.LLM.qwen.qwen1_5_moe_a2_7b.A100.single_batch.decode_schedule"
REDUCED = dict(num_hidden_layers=2, vocab_size=2048, num_experts=16, num_experts_per_tok=4, moe_intermediate_size=256)
SEED, CAPACITY, START_POS, START_TOK, PARTIALS, SHARED = 0, 96, 37, 5, 8, 512


def bits(t: torch.Tensor) -> list:
    return t.contiguous().view(torch.int16).to(torch.int32).bitwise_and(0xFFFF).tolist()


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--steps", type=int, default=8)
    args = ap.parse_args()
    sys.path.insert(0, str(ROOT))
    sys.path.insert(0, str(ROOT / "oracle"))
    sys.path.insert(0, str(REFERENCE))
    from __graft_entry__ import load_package

    load_package()
    from fused_moe_oracle import FusedMoeOracle
    from qimeng_megakernel_amd import synthetic
    from qimeng_megakernel_amd.decode_schedule_moe.model_config import QWEN3_30B_A3B, QwenMoeConfig

    torch.set_grad_enabled(False)
    shape = dataclasses.replace(QWEN3_30B_A3B, **REDUCED)
    QwenMoeConfig.set_shape(shape)

    q3_cfg = importlib.import_module(Q3 + ".model_config").Qwen3Config
    q3_cfg.update_from_dict(dict(num_hidden_layers=shape.num_hidden_layers, hidden_size=shape.hidden_size, intermediate_size=SHARED,
                                 head_dim=shape.head_dim, num_attention_heads=shape.num_attention_heads,
                                 num_key_value_heads=shape.num_key_value_heads, vocab_size=shape.vocab_size,
                                 rms_norm_eps=shape.rms_norm_eps, attn_reduction_size=shape.attn_reduction_size))
    q3_ops = importlib.import_module(Q3 + ".fused.operations")
    moe_cfg = importlib.import_module(MOE + ".model_config").QwenMoeConfig
    for name, value in dict(REDUCED, hidden_size=shape.hidden_size, head_dim=shape.head_dim, num_attention_heads=shape.num_attention_heads,
                            num_key_value_heads=shape.num_key_value_heads, intermediate_size=SHARED, rms_norm_eps=shape.rms_norm_eps,
                            norm_topk_prob=True).items():
        setattr(moe_cfg, name, value)
    moe_cfg.num_heads = shape.num_heads
    moe_cfg.qkv_out_dim = shape.qkv_out_dim
    moe_cfg._recompute_derived()
    moe_ops = importlib.import_module(MOE + ".fused.operations")

    # the reference's decode router, followed by the renormalisation of its line 405 (fused_moe_block calls it by name)
    plain_router = moe_ops.fused_router

    def router_renormalised(globs, layer_idx, normed=None):
        plain_router(globs, layer_idx, normed=normed)
        top_probs = globs.expert_weights
        globs.expert_weights.copy_(top_probs / top_probs.sum(dim=-1, keepdim=True))

    moe_ops.fused_router = router_renormalised

    weights = synthetic.random_moe_weights(shape, SEED, CAPACITY)
    L, H = shape.num_hidden_layers, shape.hidden_size
    zero_shared = dict(
        shared_expert_gate_proj_weights=torch.zeros(L, SHARED, H, dtype=torch.bfloat16),
        shared_expert_up_proj_weights=torch.zeros(L, SHARED, H, dtype=torch.bfloat16),
        shared_expert_down_proj_weights=torch.zeros(L, H, SHARED, dtype=torch.bfloat16),
        shared_expert_gate_weights=(torch.randn(L, 1, H, generator=torch.Generator().manual_seed(9)) * 0.02).bfloat16(),
    )
    with_shared = dataclasses.replace(shape, intermediate_size=SHARED, num_downproj_split_k_shared=4)

    def fresh(for_reference: bool):
        w = dict(weights, **zero_shared) if for_reference else weights
        g = synthetic.build_moe_globals(w, with_shared if for_reference else shape, CAPACITY, "cpu", max_partials=PARTIALS)
        if for_reference:
            g.qkv_raw = torch.zeros(shape.qkv_out_dim, dtype=torch.bfloat16)
            g.qkv_bias = None
        gen = torch.Generator().manual_seed(SEED + 1)
        g.k_cache.copy_(torch.randn(g.k_cache.shape, generator=gen).bfloat16())
        g.v_cache.copy_(torch.randn(g.v_cache.shape, generator=gen).bfloat16())
        return g

    ref, mine = fresh(True), fresh(False)
    oracle = FusedMoeOracle(shape)
    tok, steps = START_TOK, []
    for step in range(args.steps):
        pos = START_POS + step
        for g in (ref, mine):
            g.position_id = pos
            g.hidden_states.copy_(g.embed_tokens[tok])
        routing, weights_per_layer = [], []
        for layer in range(L):
            q3_ops.fused_rms_qkvproj_gemv(ref, layer)
            q3_ops.fused_qknorm_rope_writecache(ref, layer)
            q3_ops.fused_decode_attention(ref, layer)
            q3_ops.fused_oproj_gemv_residual(ref, layer)
            # the renormalisation as the reference's own prefill block computes it for this token (bf16 there)
            seq = type("Seq", (), {})()
            for name in ("mlp_norm_weights", "router_weights", "expert_gate_up_proj_weights", "expert_down_proj_weights",
                         "shared_expert_gate_proj_weights", "shared_expert_up_proj_weights", "shared_expert_down_proj_weights",
                         "shared_expert_gate_weights"):
                setattr(seq, name, getattr(ref, name))
            seq.hidden_states_seq = ref.hidden_states.clone().unsqueeze(0)
            seq.hidden_states, seq.routed_out, seq.shared_out = ref.hidden_states.clone(), ref.routed_out.clone(), ref.shared_out.clone()
            seq.expert_indices, seq.expert_weights = ref.expert_indices.clone(), torch.zeros_like(ref.expert_weights)
            moe_ops.fused_prefill_moe_block(seq, layer, 1)
            moe_ops.fused_moe_block(ref, layer)
            if ref.expert_indices.tolist() != seq.expert_indices.tolist():
                raise SystemExit(f"step {step} layer {layer}: decode and prefill blocks of the reference route differently")
            if not torch.equal(ref.expert_weights.to(torch.bfloat16).float(), seq.expert_weights.float()):
                raise SystemExit(f"step {step} layer {layer}: renormalised weights differ from the reference's prefill block")
            oracle.decode_layer(mine, layer)
            for name in ("qkv_raw", "q_post_rope", "attn_out", "hidden_states", "expert_indices", "expert_weights", "routed_out", "silu_out"):
                if not torch.equal(getattr(ref, name), getattr(mine, name)):
                    raise SystemExit(f"step {step} layer {layer}: {name} differs from the reference")
            if float(ref.shared_out.abs().max()) != 0.0:
                raise SystemExit("the all-zero shared expert produced something")
            routing.append(mine.expert_indices.tolist())
            weights_per_layer.append(mine.expert_weights.tolist())
        moe_ops.fused_rms_lmhead_gemv(ref)
        oracle.lm_head(mine)
        if not (torch.equal(ref.logits, mine.logits) and torch.equal(ref.k_cache, mine.k_cache) and torch.equal(ref.v_cache, mine.v_cache)):
            raise SystemExit(f"step {step}: logits or KV cache differ from the reference")
        top = mine.logits.float().topk(4)
        tok = int(mine.logits.float().argmax())
        steps.append({"position": pos, "token": tok, "top_ids": top.indices.tolist(), "top_bits": bits(mine.logits[top.indices]),
                      "experts_per_layer": routing, "weights_per_layer": weights_per_layer,
                      "hidden_bits_sampled": bits(mine.hidden_states[::128])})
    out = {"shape": REDUCED, "seed": SEED, "kv_capacity": CAPACITY, "start_position": START_POS, "start_token": START_TOK,
           "max_partials": PARTIALS, "steps": steps}
    path = OUT / "qwen3_moe_reduced_seed0.json"
    path.write_text(json.dumps(out, indent=1))
    print("lock-step identical for", len(steps), "steps; wrote", path, "tokens", [s["token"] for s in steps])


if __name__ == "__main__":
    main()
