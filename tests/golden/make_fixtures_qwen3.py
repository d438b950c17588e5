#!/usr/bin/env python3
"""Write tests/golden/qwen3_reduced_seed0.json from the imported reference (Qwen3 op set).

Runs ONLY in the build container, where the reference checkout is mounted at /root/reference; the
fixture it writes is plain JSON.  It pins what no closed form pins for the Qwen3 route: the greedy
token trajectory and the top-4 bf16 logits of the reference's fused decode step
(qwen3__0_6b/A100/single_batch/decode_schedule/fused/layer_scheduler.py:10-26) on this repository's
seeded synthetic weights, for the Qwen3-1.7B layer geometry (hidden 2048, 16 query / 8 KV heads of
128, FFN 6144, per-head QK RMSNorm, tied LM head) reduced to 3 layers and a 4096-token vocabulary so
that the fixture stays small.  While it runs, this repository's oracle is stepped in lock-step and
compared bit for bit (raw QKV, q after norm and RoPE, the KV rows, the hidden state after every
layer, the logits); any difference aborts before anything is written.

usage: python tests/golden/make_fixtures_qwen3.py [--steps 48]
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
LAYERS, VOCAB, SEED, PARTIALS = 3, 4096, 0, 8


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--steps", type=int, default=48)
    args = ap.parse_args()
    sys.path.insert(0, str(ROOT))
    sys.path.insert(0, str(ROOT / "oracle"))
    sys.path.insert(0, str(REFERENCE))
    from __graft_entry__ import load_package

    load_package()
    from fused_oracle import FusedOracle
    from qimeng_megakernel_amd import synthetic
    from qimeng_megakernel_amd.decode_schedule.model_config import QWEN3_1_7B

    ops = importlib.import_module(Q3 + ".fused.operations")
    cfg = importlib.import_module(Q3 + ".model_config").Qwen3Config
    globs_mod = importlib.import_module(Q3 + ".globs")
    torch.set_grad_enabled(False)

    shape = dataclasses.replace(QWEN3_1_7B, num_hidden_layers=LAYERS, vocab_size=VOCAB)
    cfg.update_from_dict(dict(num_hidden_layers=LAYERS, hidden_size=shape.hidden_size, intermediate_size=shape.intermediate_size,
                              head_dim=shape.head_dim, num_attention_heads=shape.num_attention_heads,
                              num_key_value_heads=shape.num_key_value_heads, vocab_size=VOCAB, rms_norm_eps=shape.rms_norm_eps,
                              attn_reduction_size=shape.attn_reduction_size))
    kv = args.steps + 1
    weights = synthetic.random_weights(shape, SEED, max_positions=kv)
    ref = synthetic.build_globals(weights, shape, kv, "cpu", globals_cls=globs_mod.Globals, max_partials=PARTIALS)
    mine = synthetic.build_globals(weights, shape, kv, "cpu", max_partials=PARTIALS)
    oracle = FusedOracle(shape)

    tokens, top_ids, top_bits = [], [], []
    tok = 7
    for pos in range(args.steps):
        for g in (ref, mine):
            g.hidden_states.copy_(g.embed_tokens[tok]); g.position_id = pos
        for layer in range(LAYERS):
            ops.fused_rms_qkvproj_gemv(ref, layer)
            ops.fused_qknorm_rope_writecache(ref, layer)
            ops.fused_decode_attention(ref, layer)
            ops.fused_oproj_gemv_residual(ref, layer)
            ops.fused_mlp(ref, layer)
            oracle.decode_layer(mine, layer)
            for name in ("qkv_raw", "q_post_rope", "attn_out", "silu_out", "hidden_states"):
                if not torch.equal(getattr(ref, name), getattr(mine, name)):
                    raise SystemExit(f"step {pos} layer {layer}: {name} differs from the reference")
        ops.fused_rms_lmhead_gemv(ref)
        oracle.lm_head(mine)
        if not (torch.equal(ref.logits, mine.logits) and torch.equal(ref.k_cache, mine.k_cache) and torch.equal(ref.v_cache, mine.v_cache)):
            raise SystemExit(f"step {pos}: logits or KV cache differ from the reference")
        top = torch.topk(ref.logits.float(), 4)
        tok = int(ref.logits.argmax())
        tokens.append(tok)
        top_ids.append(top.indices.tolist())
        top_bits.append(ref.logits[top.indices].view(torch.int16).tolist())
    out = {
        "shape": {k: v for k, v in dataclasses.asdict(shape).items()},
        "seed": SEED, "first_token": 7, "max_partials": PARTIALS, "steps": args.steps,
        "tokens": tokens, "top4_ids": top_ids, "top4_bf16_bits": top_bits,
        "final_hidden_bf16_bits": ref.hidden_states.view(torch.int16)[::16].tolist(),
    }
    (OUT / "qwen3_reduced_seed0.json").write_text(json.dumps(out))
    print(f"lock-step identical for {args.steps} steps; wrote qwen3_reduced_seed0.json; tokens[:8] = {tokens[:8]}")


if __name__ == "__main__":
    main()
