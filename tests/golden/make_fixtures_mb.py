#!/usr/bin/env python3
"""Write tests/golden/mb_reduced_seed0.json from the imported reference (batch decode route).

Runs ONLY in the build container, where the reference checkout is mounted at /root/reference; the
fixture it writes is plain JSON.  A request of three rows at different positions (70, 3, 130 — one,
two and three 64-token KV blocks), one of which reaches an end-of-sequence token on the way, is
decoded for a few steps three ways at once:

* the reference's instruction VM on the reference scheduler's instruction list
  (…/A100/multi_batch/decode_schedule/instructions/{scheduler,python_vm}.py),
* the reference's fused operations on [B, H] activations (…/single_batch/…/fused/operations.py),
* this repository's scheduler, VM and fused batch oracle,

on this repository's seeded synthetic weights (Llama-3.2-1B layer geometry, 2 layers, vocabulary
2048).  Every step the two instruction lists must serialise to the same words and every buffer
and counter must agree bit for bit between the two VMs and between the two fused routes, and the
per-row state after ``advance_decode_state`` must agree; any difference aborts before anything is
written.  The fixture keeps the digests of the instruction streams (also of the full-size
runtime template for 8 rows and 216 workers), the greedy tokens, the row state and the top-4 bf16
logits per row and step of the VM and of the fused route.

usage: python tests/golden/make_fixtures_mb.py [--steps 6]
"""
from __future__ import annotations

import argparse
import dataclasses
import hashlib
import importlib
import json
import sys
from pathlib import Path

import numpy as np
import torch

ROOT = Path(__file__).resolve().parents[2]
REFERENCE = Path("/root/reference")
OUT = Path(__file__).resolve().parent
A100 = "qimeng_megakernel.models.LLM.llama.llama3_2__1b.A100"
LAYERS, VOCAB, SEED, ROWS, CAPACITY = 2, 2048, 0, 3, 160
START_POS = (70, 3, 130)
START_TOK = (7, 11, 400)
BUFFERS = ("hidden_states", "q_post_rope", "attn_out", "silu_out", "logits", "k_cache", "v_cache")
VM_ONLY = ("attn_out_intermediates", "attn_lse_intermediates", "attn_partial_valid", "barriers",
           "attn_rms_out", "mlp_rms_out", "lm_head_rms_out")


def words(instructions) -> np.ndarray:
    return np.asarray([i.serialize() + [0] * (32 - len(i.serialize())) for i in instructions], dtype=np.int32)


def same(a: torch.Tensor, b: torch.Tensor) -> bool:
    if a.dtype.is_floating_point:   # -inf == -inf, and no NaNs are expected anywhere
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
    from qimeng_megakernel_amd.decode_schedule.model_config import LLAMA_3_2_1B, LlamaConfig
    from qimeng_megakernel_amd.decode_schedule_mb.row_state import RowState
    from qimeng_megakernel_amd.decode_schedule_mb.instructions import scheduler as my_sched

    ref_sched = importlib.import_module(A100 + ".multi_batch.decode_schedule.instructions.scheduler")
    ref_vm = importlib.import_module(A100 + ".multi_batch.decode_schedule.instructions.python_vm")
    ref_globs = importlib.import_module(A100 + ".multi_batch.decode_schedule.globs")
    ref_cfg_mb = importlib.import_module(A100 + ".multi_batch.decode_schedule.model_config").LlamaConfig
    ref_cfg_sb = importlib.import_module(A100 + ".single_batch.decode_schedule.model_config").LlamaConfig
    ref_ops = importlib.import_module(A100 + ".single_batch.decode_schedule.fused.operations")
    ref_state = importlib.import_module("qimeng_megakernel.models.LLM.decode_state")
    torch.set_grad_enabled(False)
    ref_sched._get_worker_count = lambda device: my_sched.A100_WORKERS   # no GPU here: the A100's two queues per SM

    full = dataclasses.replace(LLAMA_3_2_1B, attn_kv_block_size=ref_cfg_mb.attn_kv_block_size)
    shape = dataclasses.replace(full, num_hidden_layers=LAYERS, vocab_size=VOCAB)

    def point_reference_at(s) -> None:
        for cfg in (ref_cfg_sb, ref_cfg_mb):   # the subclass keeps attributes of its own once updated
            cfg.update_from_dict(dict(num_hidden_layers=s.num_hidden_layers, hidden_size=s.hidden_size,
                                      intermediate_size=s.intermediate_size, head_dim=s.head_dim,
                                      num_attention_heads=s.num_attention_heads, num_key_value_heads=s.num_key_value_heads,
                                      vocab_size=s.vocab_size, rms_norm_eps=s.rms_norm_eps,
                                      attn_reduction_size=s.attn_reduction_size))
        ref_cfg_mb.attn_kv_block_size = s.attn_kv_block_size

    # ---- full-size stream digests (integers only) ---------------------------------
    point_reference_at(full)
    LlamaConfig.set_shape(full)
    stub = ref_globs.Globals(hidden_states=torch.zeros(8, full.hidden_size), k_cache=torch.zeros(1, 8, 1024, 1, 1))
    ref_rt = ref_sched.build_runtime_instruction_queues(stub)
    my_rt = my_sched.reference_scheduler(8, full).runtime_queues(1024)
    ref_rt_words = np.stack([words(q) for q in ref_rt])
    my_rt_words = np.stack([words(q) for q in my_rt])
    if not np.array_equal(ref_rt_words, my_rt_words):
        raise SystemExit("full-size runtime template differs from the reference")
    full_digest = hashlib.sha256(ref_rt_words.tobytes()).hexdigest()

    # ---- the reduced request, four routes in lock-step ------------------------------
    point_reference_at(shape)
    LlamaConfig.set_shape(shape)
    weights = synthetic.random_weights(shape, SEED, max_positions=CAPACITY)

    def fresh(cls):
        g = synthetic.build_batch_globals(weights, shape, CAPACITY, ROWS, "cpu", globals_cls=cls)
        gen = torch.Generator().manual_seed(SEED + 1)
        g.k_cache.copy_(torch.randn(g.k_cache.shape, generator=gen).bfloat16())
        g.v_cache.copy_(torch.randn(g.v_cache.shape, generator=gen).bfloat16())
        g.position_ids.copy_(torch.tensor(START_POS, dtype=torch.int32))
        if cls is MyGlobals:
            RowState.of(g)
        else:
            ref_state.ensure_decode_state(g, ROWS, device=torch.device("cpu"))
        return g

    from qimeng_megakernel_amd.decode_schedule_mb.globs import Globals as MyGlobals

    routes = {"ref_vm": fresh(ref_globs.Globals), "my_vm": fresh(MyGlobals),
              "ref_fused": fresh(ref_globs.Globals), "my_fused": fresh(MyGlobals)}
    vm, fused = BatchInstructionVM(shape), FusedBatchOracle(shape)
    sched = my_sched.reference_scheduler(ROWS, shape)
    toks = {name: list(START_TOK) for name in routes}
    steps, stream_digests, eos = [], [], []
    for step in range(args.steps):
        for name, g in routes.items():
            for b in range(ROWS):
                g.hidden_states[b].copy_(g.embed_tokens[toks[name][b]])
            g.barriers.zero_()
        ref_list = ref_sched.build_instruction_list(routes["ref_vm"])
        my_list = sched.instruction_list(routes["my_vm"])
        if not np.array_equal(words(ref_list), words(my_list)):
            raise SystemExit(f"step {step}: instruction lists differ")
        stream_digests.append(hashlib.sha256(words(my_list).tobytes()).hexdigest())
        for ins in ref_list:
            ref_vm.INSTRUCTION_TO_HANDLER[type(ins)](routes["ref_vm"], ins)
        vm.run(routes["my_vm"], my_list)
        for layer in range(LAYERS):
            ref_ops.fused_rms_qkvproj_gemv_rope(routes["ref_fused"], layer)
            ref_ops.fused_decode_attention(routes["ref_fused"], layer)
            ref_ops.fused_oproj_gemv_residual(routes["ref_fused"], layer)
            ref_ops.fused_mlp(routes["ref_fused"], layer)
        ref_ops.fused_rms_lmhead_gemv(routes["ref_fused"])
        fused.decode_step(routes["my_fused"])
        for a, b, names in (("ref_vm", "my_vm", BUFFERS + VM_ONLY), ("ref_fused", "my_fused", BUFFERS)):
            for name in names:
                if not same(getattr(routes[a], name), getattr(routes[b], name)):
                    raise SystemExit(f"step {step}: {name} of {b} differs from {a}")
        record = {"positions": routes["my_vm"].position_ids.tolist(), "active": routes["my_vm"].active_mask.tolist()}
        for name in ("my_vm", "my_fused"):
            logits = routes[name].logits
            top = torch.topk(logits.float(), 4, dim=-1)
            record[name] = {"tokens": logits.float().argmax(dim=-1).tolist(), "top_ids": top.indices.tolist(),
                            "top_bits": logits.gather(1, top.indices).view(torch.int16).to(torch.int32).bitwise_and(0xFFFF).tolist()}
        record["hidden_bits_sampled"] = routes["my_vm"].hidden_states[:, ::128].contiguous().view(torch.int16).to(torch.int32).bitwise_and(0xFFFF).tolist()
        steps.append(record)
        if step == 1:   # whatever row 1 picks now becomes the end-of-sequence token: the row retires
            eos = [int(record["my_vm"]["tokens"][1])]
        for name, g in routes.items():
            nxt = g.logits.float().argmax(dim=-1)
            if name.startswith("ref"):
                ref_state.advance_decode_state(g, nxt, eos)
            else:
                RowState.of(g).advance(nxt, eos)
            toks[name] = [int(t) for t in nxt]
        for a, b in (("ref_vm", "my_vm"), ("ref_fused", "my_fused")):
            mine = RowState.of(routes[b])
            for name, got in (("position_ids", mine.position_ids), ("active_mask", mine.active_mask), ("eos_reached", mine.finished),
                              ("kv_lengths", mine.kv_lengths()), ("last_generated_tokens", mine.last_tokens)):
                if not torch.equal(getattr(routes[a], name), got):
                    raise SystemExit(f"step {step}: {name} differs after the row state advanced")
    if all(steps[-1]["active"]):
        raise SystemExit("no row retired: the fixture would not cover inactive rows")

    out = {"layers": LAYERS, "vocab": VOCAB, "seed": SEED, "rows": ROWS, "kv_capacity": CAPACITY,
           "kv_block": shape.attn_kv_block_size, "start_positions": list(START_POS), "start_tokens": list(START_TOK),
           "eos_token": eos[0], "workers": my_sched.A100_WORKERS, "steps": steps,
           "instruction_list_sha256": stream_digests,
           "full_size_runtime_template": {"rows": 8, "kv_capacity": 1024, "shape": list(ref_rt_words.shape), "sha256": full_digest}}
    (OUT / "mb_reduced_seed0.json").write_text(json.dumps(out))
    print("wrote", OUT / "mb_reduced_seed0.json", "steps", len(steps), "eos", eos, "final active", steps[-1]["active"])


if __name__ == "__main__":
    main()
