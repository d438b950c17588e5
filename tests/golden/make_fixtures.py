#!/usr/bin/env python3
"""Write the golden fixtures under tests/golden/ from the imported reference.

Runs ONLY in the build container, where the reference checkout is mounted at
/root/reference; the fixtures it writes are plain data (JSON + .npz without
pickles) and are what travels.  It pins the two things no closed form pins:

1. the exact greedy token trajectory, top-k bf16 logits and sampled hidden
   states of the reference's fused decode route
   (decode_schedule/fused/layer_scheduler.py:45-56) on this repository's seeded
   synthetic Llama-3.2-1B-shaped weights (8-token prompt, KV prefilled through
   the single-token path, forced greedy continuation);
2. the reference scheduler's instruction stream at 108 SMs, word for word
   (decode_schedule/instructions/scheduler.py:164-358), as a digest plus samples.

While it runs, this repository's own oracle (oracle/fused_oracle.py) is stepped
in lock-step for the first --check-steps steps and compared bit for bit, layer
by layer, with the reference; any difference aborts before anything is written.

usage: python tests/golden/make_fixtures.py [--new-tokens 1024] [--seed 0] [--check-steps 10]
"""
from __future__ import annotations

import argparse
import hashlib
import json
import sys
import time
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parents[2]
REFERENCE = Path("/root/reference")
OUT = Path(__file__).resolve().parent
SB = "qimeng_megakernel.models.LLM.llama.llama3_2__1b.A100.single_batch.decode_schedule"

SAMPLE_STRIDE = 32          # every 32nd hidden element -> 64 samples per layer
RECORD_HIDDEN_STEPS = (0, 1, 127, 511, 1023)


def bits(t: torch.Tensor) -> np.ndarray:
    """bf16 tensor -> uint16 bit patterns (numpy has no bf16)."""
    return t.detach().contiguous().view(torch.int16).numpy().astype(np.uint16)


def checksum(t: torch.Tensor) -> int:
    return int(bits(t).astype(np.uint64).sum())


def import_reference():
    import importlib

    sys.path.insert(0, str(REFERENCE))
    ops = importlib.import_module(SB + ".fused.operations")
    layers = importlib.import_module(SB + ".fused.layer_scheduler")
    globs_mod = importlib.import_module(SB + ".globs")
    sched = importlib.import_module(SB + ".instructions.scheduler")
    cfg = importlib.import_module(SB + ".model_config")
    return ops, layers, globs_mod, sched, cfg


def scheduler_fixture(sched) -> dict:
    """Digest + samples of the reference instruction stream at 108 SMs, 16 layers."""
    sm = 108
    p = sched.pick_num_partials(sm)
    flat = []
    per_layer_counts = None
    for layer in range(16):
        groups = [
            sched.schedule_qkvproj_gemv(layer, sm),
            sched.schedule_attention_split_kv(layer, p),
            sched.schedule_attention_reduction(layer, p),
            sched.schedule_oproj_gemv(layer, sm),
            sched.schedule_upgate(layer, sm),
            sched.schedule_downproj(layer, sm),
        ]
        if per_layer_counts is None:
            per_layer_counts = [len(g) for g in groups]
        for g in groups:
            flat.extend(g)
    lm = sched.schedule_lmhead_gemv(sm)
    flat.extend(lm)
    words = [sched._serialize_and_pad(i) for i in flat]
    arr = np.asarray(words, dtype=np.int32)
    queues = sched._round_robin_assign_to_sms(list(flat), sm)
    sample_idx = [0, 1, 107, 108, 150, 212, 220, 221, 400, 500, 620, 700, len(flat) - 1]
    return {
        "sm_count": sm,
        "num_partials": p,
        "per_layer_counts": per_layer_counts,
        "lm_head_count": len(lm),
        "total": len(flat),
        "queue_len": max(len(q) for q in queues),
        "sha256_flat_int32": hashlib.sha256(arr.tobytes()).hexdigest(),
        "samples": {str(i): [int(w) for w in arr[i]] for i in sample_idx},
    }


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--new-tokens", type=int, default=1024)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--prompt-len", type=int, default=8)
    ap.add_argument("--check-steps", type=int, default=10)
    ap.add_argument("--tag", default="llama1b_seed0")
    args = ap.parse_args()

    sys.path.insert(0, str(ROOT))
    from __graft_entry__ import load_package

    pkg = load_package()
    from qimeng_megakernel_amd import synthetic
    from qimeng_megakernel_amd.decode_schedule.model_config import LLAMA_3_2_1B

    sys.path.insert(0, str(ROOT / "oracle"))
    from fused_oracle import FusedOracle

    ops, layers, globs_mod, sched, cfg = import_reference()
    torch.set_grad_enabled(False)
    shape = LLAMA_3_2_1B
    assert cfg.LlamaConfig.hidden_size == shape.hidden_size and cfg.LlamaConfig.vocab_size == shape.vocab_size

    sched_fix = scheduler_fixture(sched)
    (OUT / "reference_schedule_sm108.json").write_text(json.dumps(sched_fix, indent=1))
    print("schedule fixture:", {k: v for k, v in sched_fix.items() if k != "samples"}, flush=True)

    kv_capacity = args.prompt_len + args.new_tokens
    t0 = time.time()
    weights = synthetic.random_weights(shape, args.seed, max_positions=kv_capacity)
    prompt = synthetic.random_prompt(shape, args.seed, args.prompt_len)
    print(f"weights drawn in {time.time() - t0:.1f}s; prompt = {prompt.tolist()}", flush=True)

    ref = synthetic.build_globals(weights, shape, kv_capacity, "cpu", globals_cls=globs_mod.Globals)
    mine = synthetic.build_globals(weights, shape, kv_capacity, "cpu")
    oracle = FusedOracle(shape)

    tokens: list[int] = []
    topk_ids, topk_bits, margins = [], [], []
    hidden_samples: dict[str, np.ndarray] = {}
    hidden_sums: dict[str, list[int]] = {}
    final_hidden: dict[str, np.ndarray] = {}
    logit_samples: dict[str, np.ndarray] = {}

    def ref_step(pos: int, token: int, step_name: str | None) -> int:
        ref.hidden_states.copy_(ref.embed_tokens[token].to(ref.hidden_states.dtype))
        ref.position_id = pos
        if step_name is None:
            layers.run_fused_decode_step(ref)
        else:
            samples, sums = [], []
            for layer in range(shape.num_hidden_layers):
                ops.fused_rms_qkvproj_gemv_rope(ref, layer)
                ops.fused_decode_attention(ref, layer)
                ops.fused_oproj_gemv_residual(ref, layer)
                ops.fused_mlp(ref, layer)
                samples.append(bits(ref.hidden_states[::SAMPLE_STRIDE]))
                sums.append(checksum(ref.hidden_states))
            ops.fused_rms_lmhead_gemv(ref)
            hidden_samples[step_name] = np.stack(samples)
            hidden_sums[step_name] = sums
            final_hidden[step_name] = bits(ref.hidden_states)
            logit_samples[step_name] = bits(ref.logits[::501])
        return int(torch.argmax(ref.logits))

    def lockstep_check(pos: int, token: int, label: str) -> None:
        mine.hidden_states.copy_(mine.embed_tokens[token].to(mine.hidden_states.dtype))
        mine.position_id = pos
        oracle.decode_step(mine)
        for name in ("hidden_states", "q_post_rope", "attn_out", "silu_out", "logits"):
            if not torch.equal(getattr(mine, name), getattr(ref, name)):
                raise SystemExit(f"oracle != reference at {label}: {name}")
        if not (torch.equal(mine.k_cache, ref.k_cache) and torch.equal(mine.v_cache, ref.v_cache)):
            raise SystemExit(f"oracle != reference at {label}: kv cache")
        print(f"  lock-step {label}: oracle == reference bit for bit", flush=True)

    steps_done = 0
    t0 = time.time()
    # prefill through the single-token path
    nxt = -1
    for pos, tok in enumerate(prompt.tolist()):
        nxt = ref_step(pos, tok, None)
        if steps_done < args.check_steps:
            lockstep_check(pos, tok, f"prefill pos {pos}")
        steps_done += 1
    tokens.append(nxt)

    def record_topk() -> None:
        vals, ids = torch.topk(ref.logits.float(), 8)
        topk_ids.append(ids.numpy().astype(np.int32))
        topk_bits.append(bits(ref.logits[ids]))
        margins.append(float(vals[0] - vals[1]))

    record_topk()
    for i in range(args.new_tokens - 1):
        pos = args.prompt_len + i
        name = f"step{i}" if i in RECORD_HIDDEN_STEPS else None
        tok = tokens[-1]
        nxt = ref_step(pos, tok, name)
        if steps_done < args.check_steps:
            lockstep_check(pos, tok, f"decode step {i}")
        steps_done += 1
        tokens.append(nxt)
        record_topk()
        if i % 16 == 0:
            el = time.time() - t0
            print(f"step {i}/{args.new_tokens - 1} tok={nxt} margin={margins[-1]:.4f} elapsed={el:.0f}s", flush=True)
            # partial results survive an interrupted run
            _write(args, prompt, tokens, topk_ids, topk_bits, margins, hidden_samples, hidden_sums, final_hidden, logit_samples, partial=True)
    _write(args, prompt, tokens, topk_ids, topk_bits, margins, hidden_samples, hidden_sums, final_hidden, logit_samples, partial=False)
    print("done", flush=True)


def _write(args, prompt, tokens, topk_ids, topk_bits, margins, hidden_samples, hidden_sums, final_hidden, logit_samples, partial):
    meta = {
        "config": "Llama-3.2-1B shape, bf16 random-init N(0,0.02), norms=1, untied lm_head, rope_theta 5e5",
        "seed": args.seed,
        "prompt": prompt.tolist(),
        "prompt_len": args.prompt_len,
        "new_tokens": len(tokens),
        "complete": not partial,
        "tokens": tokens,
        "margins": margins,
        "hidden_checksums": hidden_sums,
        "sample_stride": SAMPLE_STRIDE,
        "logit_sample_stride": 501,
        "torch": torch.__version__,
        "source": "reference fused route (fused/layer_scheduler.py:45-56) imported in the build container",
    }
    (OUT / f"{args.tag}.json").write_text(json.dumps(meta))
    arrays = {
        "topk_ids": np.stack(topk_ids),
        "topk_bits": np.stack(topk_bits),
    }
    for k, v in hidden_samples.items():
        arrays[f"hidden_samples_{k}"] = v
    for k, v in final_hidden.items():
        arrays[f"final_hidden_{k}"] = v
    for k, v in logit_samples.items():
        arrays[f"logit_samples_{k}"] = v
    np.savez_compressed(OUT / f"{args.tag}.npz", **arrays)


if __name__ == "__main__":
    main()
