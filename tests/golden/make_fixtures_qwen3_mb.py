#!/usr/bin/env python3
"""Write tests/golden/qwen3_mb_reduced_seed0.json from the imported reference (Qwen3-1.7B layer geometry, batch route).

Runs ONLY in the build container, where the reference checkout is mounted at /root/reference; the fixture it
writes is plain JSON.  The reference has no batch route for the Qwen3 op set and its Qwen3 fused operations take
one row, so a batch step is that route run row by row: for every live row the imported functions
(…/qwen/qwen3__0_6b/A100/single_batch/decode_schedule/fused/operations.py: ``fused_rms_qkvproj_gemv``,
``fused_qknorm_rope_writecache``, ``fused_decode_attention``, ``fused_oproj_gemv_residual``, ``fused_mlp``,
``fused_rms_lmhead_gemv``), unchanged, on views of that row's buffers at the row's position.  Rows that have
retired follow the batch route's rule (…/llama3_2__1b/A100/single_batch/decode_schedule/fused/operations.py:218-321
on [B, H]): nothing written but zeroed ``attn_out`` / ``silu_out`` rows and logits of -1e9.

This repository's batch oracle (oracle/fused_mb_oracle.py) and its instruction VM (oracle/pyvm_mb_oracle.py, on
the MI355X scheduler's list) run the same request in lock-step.  The fused oracle must agree with the reference
bit for bit in every buffer after every layer, or nothing is written; the VM's tokens are recorded beside it.
A request of three rows at positions 70, 3 and 130, one of which reaches an end-of-sequence token on the way.
Reduced shape: 2 layers, vocabulary 2048.

usage: python tests/golden/make_fixtures_qwen3_mb.py [--steps 6]
"""
from __future__ import annotations

import argparse
import dataclasses
import importlib
import json
import sys
import types
from pathlib import Path

import torch

ROOT = Path(__file__).resolve().parents[2]
REFERENCE = Path("/root/reference")
OUT = Path(__file__).resolve().parent
Q3 = "qimeng_megakernel.models.LLM.qwen.qwen3__0_6b.A100.single_batch.decode_schedule"
LAYERS, VOCAB, SEED, ROWS, CAPACITY, PARTIALS = 2, 2048, 0, 3, 160, 8
START_POS = (70, 3, 130)
START_TOK = (7, 11, 400)
BUFFERS = ("qkv_raw", "q_post_rope", "attn_out", "silu_out", "hidden_states", "k_cache", "v_cache",
           "attn_lse_intermediates", "attn_out_intermediates")


def bits(t: torch.Tensor) -> list:
    return t.contiguous().view(torch.int16).to(torch.int32).bitwise_and(0xFFFF).tolist()


def same(a: torch.Tensor, b: torch.Tensor) -> bool:
    if a.dtype.is_floating_point:
        return bool(torch.equal(torch.nan_to_num(a.float(), neginf=-1e30), torch.nan_to_num(b.float(), neginf=-1e30)))
    return bool(torch.equal(a, b))


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--steps", type=int, default=6)
    args = ap.parse_args()
    sys.path.insert(0, str(ROOT))
    sys.path.insert(0, str(ROOT / "oracle"))
    sys.path.insert(0, str(REFERENCE))
    from __graft_entry__ import load_package

    load_package()
    from fused_mb_oracle import FusedBatchOracle
    from pyvm_mb_oracle import BatchInstructionVM
    from qimeng_megakernel_amd import synthetic
    from qimeng_megakernel_amd.decode_schedule.model_config import QWEN3_1_7B, LlamaConfig
    from qimeng_megakernel_amd.decode_schedule_mb.instructions import scheduler as my_sched
    from qimeng_megakernel_amd.decode_schedule_mb.row_state import RowState

    ops = importlib.import_module(Q3 + ".fused.operations")
    cfg = importlib.import_module(Q3 + ".model_config").Qwen3Config
    torch.set_grad_enabled(False)

    shape = dataclasses.replace(QWEN3_1_7B, num_hidden_layers=LAYERS, vocab_size=VOCAB)
    LlamaConfig.set_shape(shape)
    cfg.update_from_dict(dict(num_hidden_layers=LAYERS, hidden_size=shape.hidden_size, intermediate_size=shape.intermediate_size,
                              head_dim=shape.head_dim, num_attention_heads=shape.num_attention_heads,
                              num_key_value_heads=shape.num_key_value_heads, vocab_size=VOCAB, rms_norm_eps=shape.rms_norm_eps,
                              attn_reduction_size=shape.attn_reduction_size))
    cfg.attn_kv_block_size = shape.attn_kv_block_size
    weights = synthetic.random_weights(shape, SEED, max_positions=CAPACITY)

    def fresh(partials: int = PARTIALS):
        g = synthetic.build_batch_globals(weights, shape, CAPACITY, ROWS, "cpu", max_partials=partials)
        gen = torch.Generator().manual_seed(SEED + 1)
        g.k_cache.copy_(torch.randn(g.k_cache.shape, generator=gen).bfloat16())
        g.v_cache.copy_(torch.randn(g.v_cache.shape, generator=gen).bfloat16())
        g.position_ids.copy_(torch.tensor(START_POS, dtype=torch.int32))
        RowState.of(g)
        return g

    def row_of(g, b: int):
        """What the imported one-row functions see of row ``b``: views of its buffers, the shared weights."""
        return types.SimpleNamespace(
            hidden_states=g.hidden_states[b], position_id=int(g.position_ids[b]), qkv_raw=g.qkv_raw[b], q_post_rope=g.q_post_rope[b],
            attn_out=g.attn_out[b], k_cache=g.k_cache[:, b : b + 1], v_cache=g.v_cache[:, b : b + 1],
            attn_lse_intermediates=g.attn_lse_intermediates[b], attn_out_intermediates=g.attn_out_intermediates[b],
            silu_out=g.silu_out[b], logits=g.logits[b],
            **{n: getattr(g, n) for n in ("attn_norm_weights", "qkv_weights", "q_norm_weights", "k_norm_weights", "rope_cos", "rope_sin",
                                          "o_proj_weights", "mlp_norm_weights", "up_proj_weights", "gate_proj_weights",
                                          "down_proj_weights", "lm_head_norm_weights", "lm_head_weights")})

    ref, mine, by_vm = fresh(), fresh(), fresh(27)   # the scheduler's fan-out needs more partial slots than the fused route's 8
    oracle, vm = FusedBatchOracle(shape), BatchInstructionVM(shape)
    sched = my_sched.mi355x_scheduler(ROWS, shape)
    toks = {id(g): list(START_TOK) for g in (ref, mine, by_vm)}
    steps, eos = [], []
    for step in range(args.steps):
        for g in (ref, mine, by_vm):
            for b in range(ROWS):
                g.hidden_states[b].copy_(g.embed_tokens[toks[id(g)][b]])
        live = [b for b in range(ROWS) if bool(ref.active_mask[b])]
        for layer in range(LAYERS):
            ref.attn_out.zero_()
            ref.silu_out.zero_()
            for b in live:
                row = row_of(ref, b)
                ops.fused_rms_qkvproj_gemv(row, layer)
                ops.fused_qknorm_rope_writecache(row, layer)
                ops.fused_decode_attention(row, layer)
                ops.fused_oproj_gemv_residual(row, layer)
                ops.fused_mlp(row, layer)
            oracle.decode_layer(mine, layer)
            for name in BUFFERS:
                x, y = getattr(ref, name), getattr(mine, name)
                if name in ("qkv_raw", "q_post_rope", "attn_lse_intermediates", "attn_out_intermediates"):
                    x, y = x[live], y[live]          # retired rows keep what their last live step left
                if not same(x, y):
                    raise SystemExit(f"step {step} layer {layer}: {name} differs from the reference")
        ref.logits.fill_(-1e9)
        for b in live:
            ops.fused_rms_lmhead_gemv(row_of(ref, b))
        oracle.lm_head(mine)
        if not same(ref.logits, mine.logits):
            raise SystemExit(f"step {step}: logits differ from the reference")
        by_vm.barriers.zero_()
        vm.run(by_vm, sched.instruction_list(by_vm))
        record = {"positions": mine.position_ids.tolist(), "active": mine.active_mask.tolist()}
        for name, g in (("fused", mine), ("vm", by_vm)):
            top = torch.topk(g.logits.float(), 4, dim=-1)
            record[name] = {"tokens": g.logits.float().argmax(dim=-1).tolist(), "top_ids": top.indices.tolist(),
                            "top_bits": [bits(g.logits[b][top.indices[b]]) for b in range(ROWS)]}
        record["hidden_bits_sampled"] = [bits(mine.hidden_states[b, ::128]) for b in range(ROWS)]
        steps.append(record)
        if step == 1:   # whatever row 1 picks now becomes the end-of-sequence token: the row retires
            eos = [int(record["fused"]["tokens"][1])]
        for g in (ref, mine, by_vm):
            nxt = g.logits.float().argmax(dim=-1)
            RowState.of(g).advance(nxt, eos)
            toks[id(g)] = [int(t) for t in nxt]
    if all(steps[-1]["active"]):
        raise SystemExit("no row retired: the fixture would not cover inactive rows")
    out = {"layers": LAYERS, "vocab": VOCAB, "seed": SEED, "rows": ROWS, "kv_capacity": CAPACITY, "max_partials": PARTIALS,
           "start_positions": list(START_POS), "start_tokens": list(START_TOK), "eos_token": eos[0], "steps": steps}
    path = OUT / "qwen3_mb_reduced_seed0.json"
    path.write_text(json.dumps(out))
    print("lock-step identical for", len(steps), "steps; wrote", path, "tokens", [s["fused"]["tokens"] for s in steps],
          "vm", [s["vm"]["tokens"] for s in steps])


if __name__ == "__main__":
    main()
