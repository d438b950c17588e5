#!/usr/bin/env python3
"""Measure how far a second valid CPU evaluation of the reference sits from the golden trajectory.

Teacher-forced replay of tests/golden/llama1b_seed0.* with this repository's CPU oracle, every GEMV
evaluated as an fp32 matmul instead of a bf16 einsum: the same bf16 rounding points as the reference,
another fp32 accumulation order.  Writes tests/golden/noise_floor_llama1b_seed0.json: per-step distance
of the top-8 logits from the fixture in bf16 ulps of the top logit, and the steps where the argmax
differs, plus the deviation of the final residual stream at the recorded steps.  The GPU parity gates
are set against these numbers.

usage: python tests/golden/make_noise_floor.py [--steps 256]
"""
import argparse
import json
import sys
import time
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parents[2]
OUT = Path(__file__).resolve().parent
sys.path[:0] = [str(ROOT), str(ROOT / "oracle")]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--steps", type=int, default=256)
    args = ap.parse_args()
    from __graft_entry__ import load_package

    load_package()
    import fused_oracle as fo
    from qimeng_megakernel_amd import synthetic
    from qimeng_megakernel_amd.decode_schedule.model_config import LLAMA_3_2_1B

    torch.set_grad_enabled(False)
    meta = json.loads((OUT / "llama1b_seed0.json").read_text())
    arrays = np.load(OUT / "llama1b_seed0.npz")
    shape = LLAMA_3_2_1B
    n_prompt = meta["prompt_len"]
    weights = synthetic.random_weights(shape, meta["seed"], max_positions=n_prompt + args.steps + 1)
    g = synthetic.build_globals(weights, shape, n_prompt + args.steps + 1, "cpu")
    fo.gemv = lambda w, x: (x.float() @ w.float().t()).to(w.dtype)
    oracle = fo.FusedOracle(shape)
    seq = meta["prompt"] + meta["tokens"]
    want = torch.from_numpy(arrays["topk_bits"].astype(np.int32)).to(torch.int16).view(torch.bfloat16).float()
    dist, mismatches, hidden_dev = [], [], {}
    t0 = time.time()
    for pos in range(n_prompt + args.steps - 1):
        oracle.embed(g, seq[pos]); g.position_id = pos
        oracle.decode_step(g)
        i = pos - (n_prompt - 1)
        if i < 0:
            continue
        ids = torch.from_numpy(arrays["topk_ids"][i].astype(np.int64))
        ulp = float(2.0 ** (torch.floor(torch.log2(want[i, 0].abs())) - 7))
        dist.append(float((g.logits[ids].float() - want[i]).abs().max()) / ulp)
        if int(g.logits.argmax()) != meta["tokens"][i]:
            mismatches.append({"step": i, "margin_ulps": meta["margins"][i] / ulp})
        name = f"final_hidden_step{i - 1}"
        if name in arrays:
            ref = torch.from_numpy(arrays[name].astype(np.int32)).to(torch.int16).view(torch.bfloat16).float()
            hidden_dev[f"step{i - 1}"] = float((g.hidden_states.float() - ref).abs().max() / ref.abs().max())
        if i % 16 == 0:
            print(f"step {i}: worst so far {max(dist):.2f} ulps, {len(mismatches)} argmax differences, {time.time() - t0:.0f}s", flush=True)
            _write(args, dist, mismatches, hidden_dev)
    _write(args, dist, mismatches, hidden_dev)


def _write(args, dist, mismatches, hidden_dev):
    (OUT / "noise_floor_llama1b_seed0.json").write_text(json.dumps({
        "what": "CPU oracle with fp32-matmul GEMVs, teacher-forced on the golden tokens, vs the golden top-8 logits",
        "steps": len(dist),
        "max_ulps": max(dist),
        "mean_ulps": sum(dist) / len(dist),
        "p99_ulps": float(np.quantile(np.array(dist), 0.99)),
        "argmax_differences": mismatches,
        "final_hidden_max_diff_over_max_ref": hidden_dev,
        "per_step_max_ulps": dist,
        "torch": torch.__version__,
    }))


if __name__ == "__main__":
    main()
