#!/usr/bin/env python3
"""Write tests/golden/moe_reduced_seed0.json from the imported reference (MoE decode route, batch 1).

Runs ONLY in the build container, where the reference checkout is mounted at /root/reference; the
fixture it writes is plain JSON.  A request is decoded greedily for a few steps four ways at once:

* the reference's instruction VM on the reference scheduler's instruction list
  (…/qwen/qwen1_5_moe_a2_7b/A100/single_batch/decode_schedule/instructions/{scheduler,python_vm}.py),
* the reference's fused operations (…/decode_schedule/fused/operations.py),
* this repository's scheduler and VM, and its fused MoE oracle,

on this repository's seeded synthetic weights (Qwen1.5-MoE layer geometry reduced to 2 layers,
vocabulary 2048, 8 experts of 256 with top-2 routing, shared expert of 1024).  Every step the two
instruction lists must serialise to the same words and every buffer and counter must agree bit
for bit between the two VMs and between the two fused routes; any difference aborts before
anything is written.  The fixture keeps the digest of the instruction stream (also of the
full-size one), per step the greedy token, the selected experts and their weights per layer, the
top-4 bf16 logits and samples of the hidden state, for the VM and for the fused route.

usage: python tests/golden/make_fixtures_moe.py [--steps 6]
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
ROUTE = "qimeng_megakernel.models.LLM.qwen.qwen1_5_moe_a2_7b.A100.single_batch.decode_schedule"
REDUCED = dict(num_hidden_layers=2, vocab_size=2048, num_experts=8, num_experts_per_tok=2, intermediate_size=1024,
               moe_intermediate_size=256)
SEED, CAPACITY, START_POS, START_TOK = 0, 96, 37, 5
BUFFERS = ("hidden_states", "q_post_rope", "attn_out", "logits", "k_cache", "v_cache", "expert_indices", "expert_weights")
VM_ONLY = ("attn_out_intermediates", "attn_lse_intermediates", "barriers", "router_logits_buf", "normed_hidden_states",
           "shared_expert_silu_out", "shared_out", "routed_silu_buffer", "routed_out_f32", "silu_out")
FUSED_ONLY = ("shared_out", "routed_out", "silu_out")


def words(instructions) -> np.ndarray:
    return np.asarray([i.serialize() + [0] * (32 - len(i.serialize())) for i in instructions], dtype=np.int32)


def same(a: torch.Tensor, b: torch.Tensor) -> bool:
    if a.dtype.is_floating_point:
        return bool(torch.equal(torch.nan_to_num(a.float(), neginf=-1e30), torch.nan_to_num(b.float(), neginf=-1e30)))
    return bool(torch.equal(a, b))


def bits(t: torch.Tensor) -> list:
    return t.contiguous().view(torch.int16).to(torch.int32).bitwise_and(0xFFFF).tolist()


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--steps", type=int, default=6)
    args = ap.parse_args()
    sys.path.insert(0, str(ROOT))
    sys.path.insert(0, str(ROOT / "oracle"))
    sys.path.insert(0, str(REFERENCE))
    from __graft_entry__ import load_package

    load_package()
    from fused_moe_oracle import FusedMoeOracle
    from pyvm_moe_oracle import MoeInstructionVM
    from qimeng_megakernel_amd import synthetic
    from qimeng_megakernel_amd.decode_schedule_moe.instructions import scheduler as my_sched
    from qimeng_megakernel_amd.decode_schedule_moe.model_config import QWEN1_5_MOE_A2_7B, QwenMoeConfig

    # The reference's modules read their constants when they are imported: the full-size stream first,
    # then the reduced shape for everything else.
    ref_cfg_mod = importlib.import_module(ROUTE + ".model_config")
    ref_cfg = ref_cfg_mod.QwenMoeConfig
    ref_sched = importlib.import_module(ROUTE + ".instructions.scheduler")
    full = QWEN1_5_MOE_A2_7B
    cpu_globs = importlib.import_module(ROUTE + ".globs").Globals()
    full_ref = ref_sched.build_instruction_list(cpu_globs)
    full_mine = my_sched.reference_scheduler(full).instruction_list()
    assert np.array_equal(words(full_ref), words(full_mine)), "full-size instruction streams differ"
    full_digest = {"layers": full.num_hidden_layers, "instructions": len(full_mine), "sha256": hashlib.sha256(words(full_mine).tobytes()).hexdigest()}

    shape = dataclasses.replace(full, **REDUCED)
    QwenMoeConfig.set_shape(shape)
    for name, value in REDUCED.items():
        setattr(ref_cfg, name, value)
    ref_cfg._recompute_derived()
    for mod in [m for m in list(sys.modules) if m.startswith(ROUTE + ".instructions") or m.startswith(ROUTE + ".fused")]:
        del sys.modules[mod]
    ref_sched = importlib.import_module(ROUTE + ".instructions.scheduler")
    ref_vm = importlib.import_module(ROUTE + ".instructions.python_vm")
    ref_ops = importlib.import_module(ROUTE + ".fused.operations")
    ref_globs_cls = importlib.import_module(ROUTE + ".globs").Globals
    ref_instruction = importlib.import_module("qimeng_megakernel.models.instruction")

    weights = synthetic.random_moe_weights(shape, SEED, CAPACITY)

    def fresh(cls=None):
        g = synthetic.build_moe_globals(weights, shape, CAPACITY, "cpu", globals_cls=cls)
        gen = torch.Generator().manual_seed(SEED + 1)
        g.k_cache.copy_(torch.randn(g.k_cache.shape, generator=gen).bfloat16())
        g.v_cache.copy_(torch.randn(g.v_cache.shape, generator=gen).bfloat16())
        return g

    routes = {"ref_vm": fresh(ref_globs_cls), "my_vm": fresh(), "ref_fused": fresh(ref_globs_cls), "my_fused": fresh()}
    my_scheduler = my_sched.reference_scheduler(shape)
    my_vm, my_fused = MoeInstructionVM(shape), FusedMoeOracle(shape)
    tokens = {name: START_TOK for name in routes}
    steps, list_digest = [], None
    with torch.no_grad():
        for step in range(args.steps):
            pos = START_POS + step
            for name, g in routes.items():
                g.position_id = pos
                g.hidden_states.copy_(g.embed_tokens[tokens[name]])
            ref_list = ref_sched.build_instruction_list(routes["ref_vm"])
            mine = my_scheduler.instruction_list()
            assert np.array_equal(words(ref_list), words(mine)), f"step {step}: instruction lists differ"
            list_digest = hashlib.sha256(words(mine).tobytes()).hexdigest()
            routes["ref_vm"].barriers.zero_(); routes["my_vm"].barriers.zero_()
            ref_instruction.run_pyvm_sequence(routes["ref_vm"], ref_list, ref_vm.INSTRUCTION_TO_HANDLER)
            my_vm.run(routes["my_vm"], mine)
            record = {"position": pos}
            experts = {"my_vm": [], "my_fused": []}
            for layer in range(shape.num_hidden_layers):
                g = routes["ref_fused"]
                ref_ops.fused_rms_qkvproj_gemv_rope(g, layer); ref_ops.fused_decode_attention(g, layer)
                ref_ops.fused_oproj_gemv_residual(g, layer); ref_ops.fused_moe_block(g, layer)
                my_fused.decode_layer(routes["my_fused"], layer)
                experts["my_fused"].append({"indices": routes["my_fused"].expert_indices.tolist(),
                                            "weights": routes["my_fused"].expert_weights.tolist()})
                assert same(g.expert_indices, routes["my_fused"].expert_indices), (step, layer)
            ref_ops.fused_rms_lmhead_gemv(routes["ref_fused"]); my_fused.lm_head(routes["my_fused"])
            for a, b, names in (("ref_vm", "my_vm", BUFFERS + VM_ONLY), ("ref_fused", "my_fused", BUFFERS + FUSED_ONLY)):
                for name in names:
                    x, y = getattr(routes[a], name), getattr(routes[b], name)
                    if name == "barriers":      # row 14 is this repository's own (per-slot counts): the reference's fourteen rows
                        x, y = x[:, :14], y[:, :14]
                    assert same(x, y), f"step {step}: {a} and {b} differ in {name}"
            for name in ("my_vm", "my_fused"):
                g = routes[name]
                top = g.logits.float().topk(4)
                record[name] = {"token": int(g.logits.float().argmax()), "top_ids": top.indices.tolist(),
                                "top_bits": bits(g.logits[top.indices]), "hidden_bits_sampled": bits(g.hidden_states[::128])}
            record["my_vm"]["last_layer_experts"] = {"indices": routes["my_vm"].expert_indices.tolist(),
                                                      "weights": routes["my_vm"].expert_weights.tolist()}
            record["my_fused"]["experts_per_layer"] = experts["my_fused"]
            steps.append(record)
            for name, g in routes.items():
                tokens[name] = int(g.logits.float().argmax())
            assert tokens["ref_vm"] == tokens["my_vm"] and tokens["ref_fused"] == tokens["my_fused"]
    out = {"shape": REDUCED, "seed": SEED, "kv_capacity": CAPACITY, "start_position": START_POS, "start_token": START_TOK,
           "queues": my_scheduler.sm_count, "num_partials": my_scheduler.num_partials,
           "instruction_list_sha256": list_digest, "instructions_per_step": len(my_scheduler.instruction_list()),
           "full_size_instruction_list": full_digest, "steps": steps}
    path = OUT / "moe_reduced_seed0.json"
    path.write_text(json.dumps(out, indent=1))
    print("wrote", path, "steps", len(steps), "tokens", [s["my_vm"]["token"] for s in steps], [s["my_fused"]["token"] for s in steps])


if __name__ == "__main__":
    main()
