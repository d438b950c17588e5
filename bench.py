#!/usr/bin/env python3
"""Headline benchmark: batch-1 bf16 greedy decode, Llama-3.2-1B shape, one MI355X.

Workload (BASELINE.json configs[1], the reference's `benchmarks.llm_decode` case at
output length 1024): seeded random-init weights, 8-token random prompt, KV prefilled
through the decode kernel, then forced greedy continuation.  One "step" is one
decode step = one megakernel launch = one new token.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu-baseline] [--lengths 128,256,512,1024]

W untimed steps run as a separate short request first; then the request of the
metric's configuration is run — prompt, prefill, 1024 new tokens (contexts up to
prompt + 1023) — and exactly its LAST K decode steps are timed (all 1023 by
default; the steps before them run untimed, then the device is synchronised), the
way the reference times them (`qimeng_megakernel/models/LLM/decode.py:719-792`):
one HIP event pair per step around the kernel launch only -> kernel_tok_s (the
metric), one pair around the loop -> tok_s_gpu, perf_counter -> tok_s.  Prints
ONE JSON line.  `--lengths` adds the reference's output-length matrix
(`benchmarks/llm_decode.py:36-43, 195-254`: warm-up iterations, then the mean of
the bench iterations per length) under the key "lengths".

`roofline.achieved` = algorithmic bytes of the K timed launches (bf16 weights +
KV rows read + KV row written, see DecodeShape.step_bytes) / summed launch time.
`cpu_baseline` = the CPU oracle (a PyTorch restatement of the reference's fused
route) timed on the host cores over a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBPS = 8000.0
# HBM bytes one launch moves, from the two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE; each scaled by
# what the same counter reads for a 1 GiB copy) summarised in profiles/decode_megakernel_llama1b_hbm_counters.txt:
# 1.0080 x the algorithmic bytes over the launches this file times by default with `--steps 20` (contexts 1012..1031);
# 1.0066 over a 64-token request.  Not measured in this process.
MEASURED_TRAFFIC_OVER_ALGORITHMIC = 1.0080
# The same kernel template on the Qwen3-1.7B shape, contexts 1020..1039 (profiles/decode_megakernel_qwen3_1p7b_hbm_counters.txt).
MEASURED_TRAFFIC_OVER_ALGORITHMIC_QWEN3_1P7B = 1.0139
# The same for the batch route's kernel at batch 8 (profiles/decode_megakernel_batch_llama1b_hbm_counters.txt).
MEASURED_TRAFFIC_OVER_ALGORITHMIC_BATCH8 = 1.0244
# ... for the rows engine at 4 rows (profiles/decode_megakernel_rows_llama1b_batch4_hbm_counters.txt)
MEASURED_TRAFFIC_OVER_ALGORITHMIC_ROWS4 = 1.0175
# ... and for the MoE route's kernel (profiles/decode_megakernel_moe_qwen1p5_a2p7b_hbm_counters.txt).
MEASURED_TRAFFIC_OVER_ALGORITHMIC_MOE = 1.0111
# What `roofline.traffic` is: not a counter read in this process, but the algorithmic bytes of the timed launches times
# the ratio the counter runs of the same kernel measured (their contexts are named in the profiles/ file).
TRAFFIC_SOURCE = "constant ratio from the rocprofv3 FETCH_SIZE/WRITE_SIZE runs of this kernel (profiles/*_hbm_counters.txt) x algorithmic bytes"


def cpu_baseline(shape, weights, prompt, n_steps: int, cores: int, shape_name: str) -> dict:
    """BASELINE config 1 on the host: the prompt is prefilled through the single-token path (untimed), then
    ``n_steps`` greedy decode steps of the same seeded request are timed: a bounded sample of the configuration's 128
    (``--cpu-steps 128`` times all of them, about 80 s)."""
    import torch

    sys.path.insert(0, str(ROOT / "oracle"))
    from fused_oracle import FusedOracle  # the checker, timed as the reported CPU baseline
    from qimeng_megakernel_amd import synthetic

    torch.set_num_threads(cores)
    T = int(prompt.numel())
    g = synthetic.build_globals(weights, shape, T + n_steps + 1, "cpu")
    oracle = FusedOracle(shape)
    toks = prompt.tolist()
    for pos in range(T):      # prefill; also pages the weights in
        oracle.embed(g, toks[pos]); g.position_id = pos
        oracle.decode_step(g)
    toks.append(int(g.logits.argmax()))
    t0 = time.perf_counter()
    for pos in range(T, T + n_steps):
        oracle.embed(g, toks[pos]); g.position_id = pos
        oracle.decode_step(g)
        toks.append(int(g.logits.argmax()))
    dt = time.perf_counter() - t0
    return {
        "value": n_steps / dt,
        "unit": "tok/s",
        "cores": cores,
        "host_cpu_count": os.cpu_count(),
        "kind": "port",
        "sample": f"{n_steps} of the configuration's 128 greedy decode steps (contexts {T + 1}..{T + n_steps}) behind the {T}-token prompt of the same seeded "
                  f"{shape_name}-shaped request (the prompt prefilled through the single-token path, untimed), "
                  f"torch {torch.__version__} bf16 on {cores} threads of {os.cpu_count()} host CPUs, {dt:.1f} s",
    }


def attention_stress(contexts=(4096, 16384, 32768)) -> dict:
    """Split-KV attention at long contexts: one decode step per context on a 2-layer model of the
    Llama-3.2-1B layer geometry with the KV cache filled with ~N(0,1) rows.  The phase is timed by
    the kernel's own timeline records (100 MHz clock): from the end of the last QKV instruction of
    layer 1 to the end of its last split-KV instruction.  K/V bytes of a layer = context x KV heads
    x head_dim x 2 B x 2."""
    import dataclasses

    import numpy as np
    import torch

    from qimeng_megakernel_amd import synthetic
    from qimeng_megakernel_amd.decode_schedule import mk_kernel
    from qimeng_megakernel_amd.decode_schedule.instructions import scheduler as S
    from qimeng_megakernel_amd.decode_schedule.model_config import LLAMA_3_2_1B, LlamaConfig

    shape = dataclasses.replace(LLAMA_3_2_1B, num_hidden_layers=2, vocab_size=4096)
    LlamaConfig.set_shape(shape)
    out = {}
    for ctx in contexts:
        w = synthetic.random_weights(shape, 0, ctx)
        g = synthetic.build_globals(w, shape, ctx, "cuda:0", max_partials=32)
        g.k_cache.normal_(); g.v_cache.normal_()
        S.build(g)
        mk = mk_kernel.get_mk()
        nq, ni = g.instructions.shape[:2]
        timeline = torch.zeros(nq, ni, 8, dtype=torch.int64, device="cuda:0")
        g.position_id = ctx - 1
        for _ in range(2):
            g.hidden_states.copy_(g.embed_tokens[5])
            mk_kernel.call_mk(g, mk)
        mk.timeline = timeline
        g.hidden_states.copy_(g.embed_tokens[5])
        mk_kernel.call_mk(g, mk)
        torch.cuda.synchronize()
        mk.check()
        t = timeline.cpu().numpy().astype(np.int64)
        op, layer = t[..., 3] & 0xFF, (t[..., 3] >> 8) & 0xFFFF
        qkv_end = t[..., 2][(op == 1) & (layer == 1)].max()
        attn_end = t[..., 2][(op == 2) & (layer == 1)].max()
        us = (attn_end - qkv_end) / 100.0
        kv_bytes = ctx * shape.num_key_value_heads * shape.head_dim * 2 * 2
        out[str(ctx)] = {"partials": S.scheduler_for(g).num_partials, "phase_us": us, "GBps": kv_bytes / us / 1e3}
    return out


def phase_table(contexts=(64, 1000)) -> dict:
    """Where a decode step of the headline configuration spends its time, by phase: one step per context on the full
    Llama-3.2-1B shape with the KV cache filled with ~N(0,1) rows, timed by the kernel's own timeline records (100 MHz
    clock).  A phase lasts from the end of the previous phase's last instruction to the end of its own last one, averaged
    over layers 1..15; its bytes are the weights its instructions stream (attention: the K/V rows of the context); the
    achieved rate is bytes / duration.  The records cost the kernel 1-2 % of a step."""
    import numpy as np
    import torch

    from qimeng_megakernel_amd import synthetic
    from qimeng_megakernel_amd.decode_schedule import mk_kernel
    from qimeng_megakernel_amd.decode_schedule.instructions import scheduler as S
    from qimeng_megakernel_amd.decode_schedule.model_config import LLAMA_3_2_1B, LlamaConfig

    shape = LLAMA_3_2_1B
    LlamaConfig.set_shape(shape)
    H, F, L = shape.hidden_size, shape.intermediate_size, shape.num_hidden_layers
    g = synthetic.build_synthetic_globals(shape, seed=0, kv_capacity=1032, device=torch.device("cuda:0"))
    g.k_cache.normal_(); g.v_cache.normal_()
    S.build(g)
    mk = mk_kernel.get_mk()
    nq, ni = g.instructions.shape[:2]
    timeline = torch.zeros(nq, ni, 8, dtype=torch.int64, device="cuda:0")
    order = [(1, "qkv"), (2, "attention"), (4, "o_proj"), (5, "up_gate"), (6, "down")]
    out = {}
    for ctx in contexts:
        g.position_id = ctx
        mk.timeline = None
        for _ in range(3):
            g.hidden_states.copy_(g.embed_tokens[5])
            mk_kernel.call_mk(g, mk)
        mk.timeline = timeline
        g.hidden_states.copy_(g.embed_tokens[5])
        mk_kernel.call_mk(g, mk)
        torch.cuda.synchronize()
        mk.check()
        t = timeline.cpu().numpy().astype(np.int64)
        op, layer = t[..., 3] & 0xFF, (t[..., 3] >> 8) & 0xFFFF
        end_of = lambda o, l: t[..., 2][(op == o) & (layer == l)].max()
        nbytes = {"qkv": shape.qkv_out_dim * H * 2, "attention": (ctx + 1) * shape.num_key_value_heads * shape.head_dim * 2 * 2,
                  "o_proj": H * H * 2, "up_gate": 2 * F * H * 2, "down": H * F * 2}
        rows = {}
        for k, (o, name) in enumerate(order):
            us = []
            for l in range(1, L):
                prev = end_of(6, l - 1) if k == 0 else end_of(order[k - 1][0], l)
                us.append((end_of(o, l) - prev) / 100.0)
            d = float(np.mean(us))
            rows[name] = {"us": d, "MB": nbytes[name] / 1e6, "GBps": nbytes[name] / d / 1e3}
        layer_us = float(np.mean([(end_of(6, l) - end_of(6, l - 1)) / 100.0 for l in range(1, L)]))
        lm = op == 7
        lm_us = float((t[..., 2][lm].max() - end_of(6, L - 1)) / 100.0)
        lm_bytes = shape.vocab_size * H * 2
        rows["lm_head"] = {"us": lm_us, "MB": lm_bytes / 1e6, "GBps": lm_bytes / lm_us / 1e3}
        layer_bytes = sum(nbytes.values())
        out[str(ctx)] = {"phases": rows, "layer_us": layer_us, "layer_MB": layer_bytes / 1e6, "layer_GBps": layer_bytes / layer_us / 1e3,
                         "step_us_with_records": float((t[..., 2][op > 0].max() - t[..., 0][op > 0].min()) / 100.0)}
    mk.timeline = None
    return out


def copy_calibration(device) -> None:
    """One 1 GiB device-to-device copy: a kernel of known traffic, for scaling rocprofv3's FETCH_SIZE / WRITE_SIZE."""
    import torch

    src = torch.empty(1 << 30, dtype=torch.uint8, device=device)
    dst = torch.empty_like(src)
    dst.copy_(src)
    torch.cuda.synchronize(device)


def batch_decode(args) -> dict:
    """B rows decoded together through the batch route's kernel: same request shape as the headline
    (seeded random-init weights, one random prompt per row, greedy continuation past EOS)."""
    import dataclasses

    import torch

    from qimeng_megakernel_amd import decode_batch, synthetic
    from qimeng_megakernel_amd.decode_schedule.model_config import LLAMA_3_2_1B, QWEN3_1_7B, LlamaConfig
    from qimeng_megakernel_amd.decode_schedule_mb import mk_kernel

    B = args.batch
    if args.model == "qwen3-1.7b":
        name, kernel, shape = "Qwen3-1.7B", "decode_megakernel_batch<Qwen3_1p7B>", QWEN3_1_7B
    else:
        name, kernel = "Llama-3.2-1B", "decode_megakernel_batch<Llama1B>"
        shape = dataclasses.replace(LLAMA_3_2_1B, attn_kv_block_size=64)   # the batch route's split-KV block
    LlamaConfig.set_shape(shape)
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    new_tokens = max(args.new_tokens, args.steps + 1)
    timed = min(args.steps, new_tokens - 1)
    kv_capacity = args.prompt_len + new_tokens
    weights = synthetic.random_weights(shape, args.seed, max_positions=kv_capacity)
    prompts = torch.stack([synthetic.random_prompt(shape, args.seed + r, args.prompt_len) for r in range(B)])
    globs = synthetic.build_batch_globals(weights, shape, kv_capacity, B, device)
    # up to four rows: the batch-1 kernel's row-streaming engine (--batch-engine tiles: the batch kernel's matrix-core tiles)
    rows_engine = args.batch_engine == "rows" or (args.batch_engine == "auto" and B <= decode_batch.ROWS_ENGINE_MAX_BATCH)
    if rows_engine:
        from qimeng_megakernel_amd.decode_schedule_mb import rows_kernel

        mk = rows_kernel.get_mk()
        kernel = kernel.replace("decode_megakernel_batch<", "decode_megakernel_rows<").replace(">", "Rows>")
    else:
        mk = mk_kernel.get_mk()
    if args.copy_calibration:
        copy_calibration(device)
    if args.warmup > 0:
        decode_batch.decode(globs, prompts, min(args.warmup + 1, new_tokens), mk=mk, decode_time=False)
    globs.k_cache.zero_(); globs.v_cache.zero_()
    out = decode_batch.decode(globs, prompts, new_tokens, mk=mk, timed_steps=timed)
    t = out["timing"]
    eager_tokens = out["new_tokens"].clone()
    # the same request with the whole loop (embedding rows, kernel, argmax, row state) as one HIP graph
    globs.k_cache.zero_(); globs.v_cache.zero_()
    graphed = decode_batch.decode(globs, prompts, new_tokens, mk=mk, use_graph=True)
    traffic_ratio = None
    if args.model == "llama-3.2-1b" and B == 8 and t["engine"] == "tiles":
        traffic_ratio = MEASURED_TRAFFIC_OVER_ALGORITHMIC_BATCH8
    elif args.model == "llama-3.2-1b" and B == 4 and t["engine"] == "rows":
        traffic_ratio = MEASURED_TRAFFIC_OVER_ALGORITHMIC_ROWS4
    line = {
        "metric": "kernel_tok_s", "value": t["kernel_tok_s"], "unit": "tok/s", "n_gpus": 1, "steps": timed,
        "warmup": args.warmup, "ms_per_step": t["kernel_ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {
            "workload": f"{name}-shaped batch-{B} greedy decode, {args.prompt_len}-token prompt per row, {new_tokens} new "
                        f"tokens per row; timed: the last {timed} decode steps (context {t['first_timed_context']}.."
                        f"{t['last_timed_context']}), seeded random-init bf16 weights",
            "batch": B, "seed": args.seed, "queues": int(globs.instructions.shape[0]),
            "instructions_per_queue": int(globs.instructions.shape[1]), "engine": t["engine"],
        },
        "tok_s": t["effective_tok_s_wall"], "tok_s_gpu": t["effective_tok_s_gpu"], "kernel_tok_s": t["kernel_tok_s"],
        "tok_s_gpu_graph": graphed["timing"]["effective_tok_s_gpu"],
        "graph_tokens_equal": bool(torch.equal(graphed["new_tokens"], eager_tokens)),
        "first_tokens": out["new_tokens"][:, :4].tolist(),
        "roofline": {
            "bound": "hbm", "achieved": t["achieved_GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": t["achieved_GBps"] / HBM_PEAK_GBPS,
            # the counter runs were made on the Llama shape at batch 8 (tiles engine) and batch 4 (rows engine) only
            "traffic": (traffic_ratio * t["algorithmic_bytes"] / max(timed, 1) if traffic_ratio else None),
            "traffic_source": TRAFFIC_SOURCE if traffic_ratio else None,
            "bytes_per_launch_avg": t["algorithmic_bytes"] / max(timed, 1), "kernel": kernel,
        },
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline_batch(shape, weights, prompts, args.cpu_steps, min(os.cpu_count() or 1, 16), name)
    return line


def moe_decode(args) -> dict:
    """Greedy decode at batch 1 through the MoE route's kernel: the Qwen1.5-MoE-A2.7B shape (the reference's route) or
    the Qwen3-30B-A3B shape (BASELINE config 5: 48 layers, 128 experts of 768, renormalised top-8, no shared expert,
    32 query / 4 KV heads of 128 with the Qwen3 op set's attention; 61 GB of bf16 weights, drawn on the GPU)."""
    import dataclasses

    import torch

    from qimeng_megakernel_amd import decode_moe, synthetic
    from qimeng_megakernel_amd.decode_schedule_moe import mk_kernel
    from qimeng_megakernel_amd.decode_schedule_moe.model_config import QWEN1_5_MOE_A2_7B, QWEN3_30B_A3B, QwenMoeConfig

    a3b = args.model == "qwen3-30b-a3b"
    shape = QWEN3_30B_A3B if a3b else QWEN1_5_MOE_A2_7B
    name = "Qwen3-30B-A3B" if a3b else "Qwen1.5-MoE-A2.7B"
    QwenMoeConfig.set_shape(shape)
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    # config 5 is quoted on 512 greedy steps; the reference's own shape keeps the length the steps ask for
    new_tokens = max(args.new_tokens if args.new_tokens != 1024 else 512, args.steps + 1) if a3b else args.steps + 1
    timed = min(args.steps, new_tokens - 1)
    kv_capacity = args.prompt_len + new_tokens
    weights = synthetic.random_moe_weights(shape, args.seed, kv_capacity, device=device if a3b else "cpu")
    gen = torch.Generator().manual_seed(args.seed + 1_000_003)
    prompt = torch.randint(0, shape.vocab_size, (args.prompt_len,), generator=gen, dtype=torch.long)
    globs = synthetic.build_moe_globals(weights, shape, kv_capacity, device, max_partials=8 if a3b else 27)
    if args.batch > 1 and (args.rows_side_by_side or shape.has_shared_expert or args.batch > 4):
        return moe_decode_rows(args, shape, name, globs, kv_capacity, new_tokens, timed)
    if args.batch > 1:
        del globs
        return moe_decode_batch(args, shape, name, weights, kv_capacity, new_tokens, timed)
    mk = mk_kernel.get_mk()
    if args.copy_calibration:
        copy_calibration(device)
    if args.warmup > 0:
        decode_moe.decode(globs, prompt, min(args.warmup + 1, new_tokens), mk=mk, decode_time=False)
    globs.k_cache.zero_(); globs.v_cache.zero_()
    out = decode_moe.decode(globs, prompt, new_tokens, mk=mk, timed_steps=timed)
    t = out["timing"]
    eager_tokens = out["new_tokens"].clone()
    globs.k_cache.zero_(); globs.v_cache.zero_()
    graphed = decode_moe.decode(globs, prompt, new_tokens, mk=mk, use_graph=True, timed_steps=timed)   # the timed launches as one HIP graph
    line = {
        "metric": "kernel_tok_s", "value": t["kernel_tok_s"], "unit": "tok/s", "n_gpus": 1, "steps": timed, "warmup": args.warmup,
        "ms_per_step": t["kernel_ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"{name}-shaped batch-1 greedy decode, {args.prompt_len}-token prompt, {new_tokens} new tokens; timed: the last "
                        f"{timed} decode steps (contexts {t['first_timed_context']}..{t['last_timed_context']}), seeded random-init bf16 "
                        f"weights" + (" drawn on the GPU" if a3b else ""),
            "layers": shape.num_hidden_layers, "experts": shape.num_experts, "experts_per_token": shape.num_experts_per_tok,
            "expert_ffn": shape.moe_intermediate_size, "shared_ffn": shape.intermediate_size, "renormalised_top_k": bool(shape.norm_topk_prob),
            "q_heads": shape.num_attention_heads, "kv_heads": shape.num_key_value_heads, "head_dim": shape.head_dim, "qk_norm": bool(shape.qk_norm),
            "batch": 1, "seed": args.seed, "weight_bytes": shape.weight_bytes_per_token(),
            "queues": int(globs.instructions.shape[0]), "instructions_per_queue": int(globs.instructions.shape[1]),
        },
        "tok_s": t["effective_tok_s_wall"], "tok_s_gpu": t["effective_tok_s_gpu"], "kernel_tok_s": t["kernel_tok_s"],
        "tok_s_gpu_graph": graphed["timing"]["effective_tok_s_gpu"],
        "graph_tokens_equal": bool(torch.equal(graphed["new_tokens"], eager_tokens)),
        "first_tokens": out["new_tokens"][:8].tolist(),
        "roofline": {
            "bound": "hbm", "achieved": t["achieved_GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": t["achieved_GBps"] / HBM_PEAK_GBPS,
            # the counter runs were made on the Qwen1.5-shaped kernel only
            "traffic": None if a3b else MEASURED_TRAFFIC_OVER_ALGORITHMIC_MOE * t["algorithmic_bytes"] / max(timed, 1),
            "traffic_source": None if a3b else TRAFFIC_SOURCE,
            "bytes_per_launch_avg": t["algorithmic_bytes"] / max(timed, 1),
            "kernel": "decode_megakernel_moe<Qwen3MoeA3B>" if a3b else "decode_megakernel_moe<QwenMoeA2_7B>",
        },
    }
    if not args.no_cpu_baseline:
        sys.path.insert(0, str(ROOT / "oracle"))
        from fused_moe_oracle import FusedMoeOracle

        cores = min(os.cpu_count() or 1, 16)
        torch.set_num_threads(cores)
        if a3b:
            # 61 GB of weights do not go through host memory for a reported baseline: the fused oracle is timed on a
            # 2-layer model of the same layer geometry (its own seeded weights) plus the LM head, and the step time of
            # the 48-layer model is put together from the per-layer and the LM-head time.
            small = dataclasses.replace(shape, num_hidden_layers=2)
            w = synthetic.random_moe_weights(small, args.seed, args.cpu_steps + 1)
            g = synthetic.build_moe_globals(w, small, args.cpu_steps + 1, "cpu", max_partials=8)
            oracle = FusedMoeOracle(small)
            t_layers = t_head = 0.0
            with torch.no_grad():
                for pos in range(args.cpu_steps + 1):
                    g.hidden_states.copy_(g.embed_tokens[prompt[min(pos, len(prompt) - 1)]])
                    g.position_id = pos
                    t0 = time.perf_counter()
                    for layer in range(2):
                        oracle.decode_layer(g, layer)
                    t1 = time.perf_counter()
                    oracle.lm_head(g)
                    if pos:   # the first step pages the weights in
                        t_layers += t1 - t0
                        t_head += time.perf_counter() - t1
            per_layer, head = t_layers / (2 * args.cpu_steps), t_head / args.cpu_steps
            line["cpu_baseline"] = {
                "value": 1.0 / (shape.num_hidden_layers * per_layer + head), "unit": "tok/s", "cores": cores, "host_cpu_count": os.cpu_count(),
                "kind": "port",
                "sample": f"{args.cpu_steps} steps (contexts 2..{args.cpu_steps + 1}) of a 2-layer model of the same layer geometry through the "
                          f"fused MoE oracle: {per_layer * 1e3:.1f} ms per layer, {head * 1e3:.1f} ms for the LM head; value = 1 / (48 layers + LM head)",
            }
        else:
            g = synthetic.build_moe_globals(weights, shape, args.cpu_steps + 1, "cpu")
            oracle = FusedMoeOracle(shape)
            with torch.no_grad():
                t0 = time.perf_counter()
                for pos in range(args.cpu_steps):
                    g.hidden_states.copy_(g.embed_tokens[prompt[min(pos, len(prompt) - 1)]])
                    g.position_id = pos
                    oracle.decode_step(g)
                dt = time.perf_counter() - t0
            line["cpu_baseline"] = {"value": args.cpu_steps / dt, "unit": "tok/s", "cores": cores, "host_cpu_count": os.cpu_count(), "kind": "port",
                                    "sample": f"{args.cpu_steps} steps (contexts 1..{args.cpu_steps}) of the same workload through the fused MoE oracle"}
    return line


def moe_decode_batch(args, shape, name: str, weights, kv_capacity: int, new_tokens: int, timed: int) -> dict:
    """``--batch B`` (2..4) on a MoE shape without a shared expert: the B requests in ONE launch per step
    (qmk_decode_step_moe_rows).  Attention weights, router and LM head are read once per step, every expert once for
    all the rows that picked it; the roofline is taken on those algorithmic bytes, the distinct experts counted by
    the kernel per layer and step."""
    import torch

    from qimeng_megakernel_amd import decode_moe
    from qimeng_megakernel_amd.decode_schedule_moe import rows_kernel

    B = args.batch
    device = torch.device("cuda:0")
    globs = rows_kernel.build_rows_globals(weights, shape, kv_capacity, B, device, max_partials=8)
    gen = torch.Generator().manual_seed(args.seed + 1_000_003)
    prompts = torch.randint(0, shape.vocab_size, (B, args.prompt_len), generator=gen, dtype=torch.long)
    mk = rows_kernel.get_mk()
    if args.copy_calibration:
        copy_calibration(device)
    if args.warmup > 0:
        decode_moe.decode_batch(globs, prompts, min(args.warmup + 1, new_tokens), mk=mk, decode_time=False)
    globs.k_cache.zero_(); globs.v_cache.zero_()
    out = decode_moe.decode_batch(globs, prompts, new_tokens, mk=mk, timed_steps=timed)
    t = out["timing"]
    return {
        "metric": "kernel_tok_s", "value": t["kernel_tok_s"], "unit": "tok/s", "n_gpus": 1, "steps": timed, "warmup": args.warmup,
        "ms_per_step": t["kernel_ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"{name}-shaped greedy decode of {B} requests in one launch per step, {args.prompt_len}-token prompts, "
                        f"{new_tokens} new tokens per row; timed: the last {timed} decode steps (contexts {t['first_timed_context']}.."
                        f"{t['last_timed_context']}), seeded random-init bf16 weights drawn on the GPU",
            "layers": shape.num_hidden_layers, "experts": shape.num_experts, "experts_per_token": shape.num_experts_per_tok,
            "batch": B, "seed": args.seed, "weight_bytes_per_row": shape.weight_bytes_per_token(),
            "distinct_experts_per_layer": t["distinct_experts_per_layer"],
            "queues": int(globs.instructions.shape[0]), "instructions_per_queue": int(globs.instructions.shape[1]),
        },
        "tok_s": t["effective_tok_s_wall"], "tok_s_gpu": t["effective_tok_s_gpu"], "kernel_tok_s": t["kernel_tok_s"],
        "first_tokens": out["new_tokens"][:, :4].tolist(),
        "roofline": {
            "bound": "hbm", "achieved": t["achieved_GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": t["achieved_GBps"] / HBM_PEAK_GBPS,
            "traffic": None, "traffic_source": None, "bytes_per_launch_avg": t["algorithmic_bytes"] / max(timed, 1),
            "bytes_if_rows_alone_avg": t["moved_if_rows_alone"] / max(timed, 1),
            "kernel": "decode_megakernel_moe_rows<Qwen3MoeA3B>",
            "note": "algorithmic bytes = attention, router, LM head once + every row's KV rows + each DISTINCT expert of a layer once",
        },
        "cpu_baseline": None,
    }


def moe_decode_rows(args, shape, name: str, globs, kv_capacity: int, new_tokens: int, timed: int) -> dict:
    """``--batch B`` on the MoE route: B requests side by side on the batch-1 kernel (one launch per row and step over
    one copy of the weights).  The rows share no traffic: the bytes of a step are B times a row's."""
    import torch

    from qimeng_megakernel_amd import decode_moe

    B = args.batch
    a3b = args.model == "qwen3-30b-a3b"
    rows = decode_moe.share_weights(globs, shape, kv_capacity, B, max_partials=8 if a3b else 27)
    gen = torch.Generator().manual_seed(args.seed + 1_000_003)
    prompts = torch.randint(0, shape.vocab_size, (B, args.prompt_len), generator=gen, dtype=torch.long)
    if args.warmup > 0:
        decode_moe.decode_rows(rows, prompts, min(args.warmup + 1, new_tokens), decode_time=False)
    for g in rows:
        g.k_cache.zero_(); g.v_cache.zero_()
    out = decode_moe.decode_rows(rows, prompts, new_tokens, timed_steps=timed)
    t = out["timing"]
    return {
        "metric": "kernel_tok_s", "value": t["kernel_tok_s"], "unit": "tok/s", "n_gpus": 1, "steps": timed, "warmup": args.warmup,
        "ms_per_step": t["kernel_ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"{name}-shaped greedy decode of {B} requests side by side on the batch-1 kernel (one launch per row and step, one "
                        f"copy of the weights, no traffic shared between rows), {args.prompt_len}-token prompts, {new_tokens} new tokens "
                        f"per row; timed: the last {timed} decode steps (contexts {t['first_timed_context']}..{t['last_timed_context']}), "
                        f"seeded random-init bf16 weights" + (" drawn on the GPU" if a3b else ""),
            "layers": shape.num_hidden_layers, "experts": shape.num_experts, "experts_per_token": shape.num_experts_per_tok,
            "batch": B, "seed": args.seed, "weight_bytes_per_row": shape.weight_bytes_per_token(),
            "queues": int(globs.instructions.shape[0]), "instructions_per_queue": int(globs.instructions.shape[1]),
        },
        "tok_s": t["effective_tok_s_wall"], "tok_s_gpu": t["effective_tok_s_gpu"], "kernel_tok_s": t["kernel_tok_s"],
        "ms_per_launch": t["kernel_ms_per_launch"], "first_tokens": out["new_tokens"][:, :4].tolist(),
        "roofline": {
            "bound": "hbm", "achieved": t["achieved_GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": t["achieved_GBps"] / HBM_PEAK_GBPS,
            "traffic": None, "bytes_per_launch_avg": t["algorithmic_bytes"] / max(t["kernel_launches"], 1),
            "kernel": "decode_megakernel_moe<Qwen3MoeA3B>" if a3b else "decode_megakernel_moe<QwenMoeA2_7B>",
            "note": "bytes = every row's own weight and KV bytes: a batch kernel that read each selected expert once per step would need fewer",
        },
        "cpu_baseline": None,
    }


def cpu_baseline_batch(shape, weights, prompts, n_steps: int, cores: int, shape_name: str) -> dict:
    """The fused batch oracle on the host cores: ``n_steps`` steps of the same rows from position 0."""
    import torch

    sys.path.insert(0, str(ROOT / "oracle"))
    from fused_mb_oracle import FusedBatchOracle
    from qimeng_megakernel_amd import synthetic

    torch.set_num_threads(cores)
    B = int(prompts.shape[0])
    # the Qwen3 route's fused attention walks its partial slots in Python: the route's own 8 slots, not the kernel's fan-out
    g = synthetic.build_batch_globals(weights, shape, n_steps + 1, B, "cpu", max_partials=8 if shape.qk_norm else 27)
    oracle = FusedBatchOracle(shape)
    with torch.no_grad():
        t0 = time.perf_counter()
        for pos in range(n_steps):
            g.hidden_states.copy_(g.embed_tokens[prompts[:, min(pos, prompts.shape[1] - 1)]])
            g.position_ids.fill_(pos)
            oracle.decode_step(g)
        dt = time.perf_counter() - t0
    return {"value": B * n_steps / dt, "unit": "tok/s", "cores": cores, "kind": "port",
            "host_cpu_count": os.cpu_count(),
            "sample": f"{n_steps} steps of {B} rows (contexts 1..{n_steps}) of the {shape_name}-shaped workload through the fused batch oracle"}


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=None,
                    help="timed decode steps: the last that many of the request (default: all of them: 1023, or 511 for "
                         "--model qwen3-30b-a3b, whose configuration is quoted on 512 new tokens)")
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--prompt-len", type=int, default=8)
    ap.add_argument("--new-tokens", type=int, default=1024,
                    help="output length of the request (the metric's configuration: 1024); the last --steps of its "
                         "decode steps are timed")
    ap.add_argument("--lengths", default="",
                    help="comma-separated output lengths (the reference's matrix: 128,256,512,1024): each is run "
                         "--length-warmup-iters + --length-bench-iters times and the mean tok_s / tok_s_gpu / kernel_tok_s reported")
    ap.add_argument("--length-warmup-iters", type=int, default=2)
    ap.add_argument("--length-bench-iters", type=int, default=5)
    ap.add_argument("--cpu-steps", type=int, default=16)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--model", choices=("llama-3.2-1b", "qwen3-1.7b", "qwen1.5-moe-a2.7b", "qwen3-30b-a3b"), default="llama-3.2-1b",
                    help="layer geometry: the headline Llama-3.2-1B shape, the Qwen3-1.7B shape with the Qwen3 op set "
                         "(28 layers, per-head QK RMSNorm, tied LM head), the Qwen1.5-MoE-A2.7B shape with the MoE op set "
                         "(24 layers, 60 experts of 1408 with top-4 routing, shared expert of 5632), or the Qwen3-30B-A3B shape "
                         "(48 layers, 128 experts of 768 with renormalised top-8 routing, 32/4 heads of 128; 512 new tokens)")
    ap.add_argument("--host-sampling", action="store_true",
                    help="argmax and embedding lookup on the host between launches, as the reference's loop does "
                         "(default: inside the kernel)")
    ap.add_argument("--no-graph-run", action="store_true", help="skip the extra untimed-per-step HIP-graph run")
    ap.add_argument("--attention-stress", action="store_true",
                    help="instead of the decode request: the split-KV attention phase at contexts 4096/16384/32768 "
                         "(one JSON line, metric attention_phase_GBps)")
    ap.add_argument("--batch", type=int, default=1,
                    help="rows decoded together (2..16: the batch route's kernel, Llama-3.2-1B or Qwen3-1.7B shape; tokens/s counts all rows)")
    ap.add_argument("--batch-engine", choices=("auto", "rows", "tiles"), default="auto",
                    help="dense shapes with --batch B: 'rows' = the batch-1 kernel's row-streaming engine with every row's activation "
                         "vector (1..4 rows), 'tiles' = the batch kernel's matrix-core tiles (2..16), 'auto' = rows up to four rows")
    ap.add_argument("--rows-side-by-side", action="store_true",
                    help="MoE shapes with --batch B: one batch-1 launch per row and step (the only way for a shape with a shared "
                         "expert or more than 4 rows) instead of the B requests in one launch")
    ap.add_argument("--phase-table", action="store_true",
                    help="one decode step of the headline shape at contexts 64 and 1000 with timeline records: time, bytes and achieved GB/s per phase")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one 1 GiB device-to-device copy (a kernel of known traffic, for scaling rocprofv3 counters)")
    args = ap.parse_args()
    if args.steps is None:
        args.steps = 511 if args.model == "qwen3-30b-a3b" and args.new_tokens == 1024 else max(args.new_tokens - 1, 1)
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        raise SystemExit("bench.py: this path runs on exactly one GPU (a batch-1 decode step is one chain of "
                         "GEMVs on one vector and does not shard); run with --gpus 1")

    import torch

    from __graft_entry__ import LIBRARY, build_library, load_package

    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU")
    if not LIBRARY.is_file():
        build_library()
    load_package()
    from qimeng_megakernel_amd import decode, synthetic
    from qimeng_megakernel_amd.decode_schedule import mk_kernel
    from qimeng_megakernel_amd.decode_schedule.model_config import LLAMA_3_2_1B, QWEN3_1_7B, LlamaConfig

    if args.phase_table:
        res = phase_table()
        print(json.dumps({"metric": "phase_GBps", "unit": "GB/s", "n_gpus": 1, "higher_is_better": True, "dtype": "bf16", "data": "synthetic",
                          "config": {"workload": "Llama-3.2-1B shape, batch 1, one decode step per context, KV cache ~N(0,1); per-phase time from the kernel's timeline records"},
                          "value": res[max(res, key=int)]["layer_GBps"], "contexts": res}))
        return
    if args.attention_stress:
        res = attention_stress()
        print(json.dumps({"metric": "attention_phase_GBps", "unit": "GB/s", "n_gpus": 1, "higher_is_better": True,
                          "dtype": "bf16", "data": "synthetic",
                          "config": {"workload": "Llama-3.2-1B layer geometry, batch 1, one decode step, KV cache ~N(0,1)"},
                          "value": res[max(res, key=int)]["GBps"], "contexts": res}))
        return
    if args.model in ("qwen1.5-moe-a2.7b", "qwen3-30b-a3b"):
        if not 1 <= args.batch <= 16:
            raise SystemExit("bench.py: --batch takes 1..16 on the MoE route (rows side by side on the batch-1 kernel)")
        print(json.dumps(moe_decode(args)))
        return
    if args.batch != 1:
        if args.model not in ("llama-3.2-1b", "qwen3-1.7b") or not 2 <= args.batch <= 16:
            raise SystemExit("bench.py: --batch takes 2..16 and runs on the Llama-3.2-1B or the Qwen3-1.7B shape")
        print(json.dumps(batch_decode(args)))
        return
    shape = LLAMA_3_2_1B if args.model == "llama-3.2-1b" else QWEN3_1_7B
    model_name = "Llama-3.2-1B" if args.model == "llama-3.2-1b" else "Qwen3-1.7B"
    LlamaConfig.set_shape(shape)
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    lengths = [int(x) for x in args.lengths.split(",") if x.strip()]
    new_tokens = max(args.new_tokens, args.steps + 1)
    timed = min(args.steps, new_tokens - 1)
    kv_capacity = args.prompt_len + max([new_tokens] + lengths)
    weights = synthetic.random_weights(shape, args.seed, max_positions=kv_capacity)
    prompt = synthetic.random_prompt(shape, args.seed, args.prompt_len)
    globs = synthetic.build_globals(weights, shape, kv_capacity, device)
    mk = mk_kernel.get_mk()

    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device=device)
        dst = torch.empty_like(src)
        dst.copy_(src)                      # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize(device)
        del src, dst
    if args.warmup > 0:
        decode.decode(globs, prompt, min(args.warmup + 1, new_tokens), mk=mk, decode_time=False)
    globs.k_cache.zero_(); globs.v_cache.zero_()
    torch.cuda.synchronize(device)
    out = decode.decode(globs, prompt, new_tokens, mk=mk, decode_time=True, device_sampling=not args.host_sampling,
                        timed_steps=timed)
    torch.cuda.synchronize(device)
    t = out["timing"]
    tokens = out["new_tokens"][0].tolist()
    graph_tok_s = None
    if not args.no_graph_run and not args.host_sampling:
        # The same request once more with the timed launches as ONE HIP graph (no per-step events).
        globs.k_cache.zero_(); globs.v_cache.zero_()
        g_out = decode.decode(globs, prompt, new_tokens, mk=mk, decode_time=True, use_graph=True, timed_steps=timed)
        if g_out["new_tokens"][0].tolist() != tokens:
            raise SystemExit("bench.py: the graph replay produced different tokens than the launch loop")
        graph_tok_s = g_out["timing"]["effective_tok_s_gpu"]

    matrix = {}
    for n in lengths:   # the reference's output-length matrix: warm-up runs, then the mean over the bench runs
        samples = []
        for it in range(args.length_warmup_iters + args.length_bench_iters):
            globs.k_cache.zero_(); globs.v_cache.zero_()
            r = decode.decode(globs, prompt, n, mk=mk, decode_time=True, device_sampling=not args.host_sampling)
            if it >= args.length_warmup_iters:
                samples.append((r["timing"], r["new_tokens"][0].tolist()))
        mean = lambda key: sum(tm[key] for tm, _ in samples) / len(samples)
        matrix[f"b1_t{n}"] = {
            "max_new_tokens": n, "eos_policy": "forced_continuation", "bench_iters": len(samples), "warmup_iters": args.length_warmup_iters,
            "tok_s": mean("effective_tok_s_wall"), "tok_s_gpu": mean("effective_tok_s_gpu"), "kernel_tok_s": mean("kernel_tok_s"),
            "achieved_GBps": mean("achieved_GBps"), "hbm_frac": mean("achieved_GBps") / HBM_PEAK_GBPS,
            "greedy_rerun_match": all(tk == samples[0][1] for _, tk in samples[1:]),
        }

    golden = ROOT / "tests" / "golden" / "llama1b_seed0.json"
    match = None
    if args.model == "llama-3.2-1b" and args.seed == 0 and args.prompt_len == 8 and golden.is_file():
        want = json.loads(golden.read_text())["tokens"]
        n = min(len(want), len(tokens))
        match = next((i for i in range(n) if tokens[i] != want[i]), n)

    ctx_first, ctx_last = t["first_timed_context"], t["last_timed_context"]
    achieved = t["achieved_GBps"]
    line = {
        "metric": "kernel_tok_s",
        "value": t["kernel_tok_s"],
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": timed,
        "warmup": args.warmup,
        "ms_per_step": t["kernel_ms_per_step"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"{model_name}-shaped batch-1 greedy decode, {args.prompt_len}-token prompt, "
                        f"{new_tokens} new tokens; timed: the last {timed} decode steps (contexts {ctx_first}..{ctx_last}), "
                        f"seeded random-init bf16 weights",
            "layers": shape.num_hidden_layers, "hidden": shape.hidden_size, "ffn": shape.intermediate_size,
            "q_heads": shape.num_attention_heads, "kv_heads": shape.num_key_value_heads, "head_dim": shape.head_dim,
            "vocab": shape.vocab_size, "batch": 1, "seed": args.seed,
            "queues": int(globs.instructions.shape[0]), "instructions_per_queue": int(globs.instructions.shape[1]),
        },
        "tok_s": t["effective_tok_s_wall"],
        "tok_s_gpu": t["effective_tok_s_gpu"],
        "kernel_tok_s": t["kernel_tok_s"],
        "tok_s_gpu_graph": graph_tok_s,
        "sampling": "host" if args.host_sampling else "device",
        "golden_token_prefix_match": match,
        "roofline": {
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBPS,
            "traffic": ((MEASURED_TRAFFIC_OVER_ALGORITHMIC if args.model == "llama-3.2-1b" else MEASURED_TRAFFIC_OVER_ALGORITHMIC_QWEN3_1P7B)
                        * t["algorithmic_bytes"] / max(timed, 1)),
            "traffic_source": TRAFFIC_SOURCE,
            "bytes_per_launch_avg": t["algorithmic_bytes"] / max(timed, 1),
            "kernel": "decode_megakernel<Llama1B>" if args.model == "llama-3.2-1b" else "decode_megakernel<Qwen3_1p7B>",
        },
    }
    if matrix:
        line["lengths"] = matrix
    if not args.no_cpu_baseline:
        cores = min(os.cpu_count() or 1, 16)   # a GPU box gives one job 16 cores, whatever it reports
        line["cpu_baseline"] = cpu_baseline(shape, weights, prompt, args.cpu_steps, cores, model_name)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
