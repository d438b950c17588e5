"""CPU oracle against the golden fixtures, and the noise floor of the reference at full size.

1. Replaying the first prompt positions with this repository's oracle reproduces the fixture that the
   imported reference wrote (tokens always; hidden-state bits when the host CPU accumulates bf16 GEMVs
   in the same order as the machine that wrote the fixture, a tolerance otherwise).
2. The same replay with every GEMV evaluated as an fp32 matmul — another valid accumulation order at the
   same rounding points — measures how far a second CPU evaluation of the reference sits from the
   fixture, in bf16 ulps of the top logit.  The GPU gate LOGIT_ULPS (tests/test_gpu_golden.py) is that
   distance with head-room, not a number picked to make the kernel pass.
"""
import json

import numpy as np
import pytest
import torch

import fused_oracle as fo
from conftest import GOLDEN
from qimeng_megakernel_amd import synthetic
from qimeng_megakernel_amd.decode_schedule.model_config import LLAMA_3_2_1B

STEPS = 10  # 8 prompt positions + 2 decode steps of the 1032-position trajectory


def _bf16(bits):
    return torch.from_numpy(bits.astype(np.int32)).to(torch.int16).view(torch.bfloat16).float()


@pytest.mark.slow
def test_oracle_replays_fixture_and_noise_floor(monkeypatch):
    meta = json.loads((GOLDEN / "llama1b_seed0.json").read_text())
    arrays = np.load(GOLDEN / "llama1b_seed0.npz")
    shape = LLAMA_3_2_1B
    weights = synthetic.random_weights(shape, meta["seed"], max_positions=32)
    prompt = synthetic.random_prompt(shape, meta["seed"], meta["prompt_len"])
    assert prompt.tolist() == meta["prompt"]
    exact = synthetic.build_globals(weights, shape, 32, "cpu")
    alt = synthetic.build_globals(weights, shape, 32, "cpu")
    oracle = fo.FusedOracle(shape)
    bf16_gemv = fo.gemv
    seq = prompt.tolist() + meta["tokens"]
    want_topk = _bf16(arrays["topk_bits"])
    worst_alt_ulps = 0.0
    for pos in range(STEPS):
        for g in (exact, alt):
            oracle.embed(g, seq[pos]); g.position_id = pos
        monkeypatch.setattr(fo, "gemv", bf16_gemv); oracle.decode_step(exact)
        monkeypatch.setattr(fo, "gemv", lambda w, x: (x.float() @ w.float().t()).to(w.dtype)); oracle.decode_step(alt)
        i = pos - (len(prompt) - 1)
        if i < 0:
            continue
        ids = torch.from_numpy(arrays["topk_ids"][i].astype(np.int64))
        ulp = 2.0 ** (torch.floor(torch.log2(want_topk[i, 0].abs())) - 7)
        # the oracle itself: same tokens; same bits if this CPU accumulates like the fixture's
        assert int(exact.logits.argmax()) == meta["tokens"][i] or meta["margins"][i] / float(ulp) <= 2.0
        assert float((exact.logits[ids].float() - want_topk[i]).abs().max() / ulp) <= 8.0
        worst_alt_ulps = max(worst_alt_ulps, float((alt.logits[ids].float() - want_topk[i]).abs().max() / ulp))
        if i >= 1:
            name = f"step{i - 1}"
            final = _bf16(arrays[f"final_hidden_{name}"])
            assert (exact.hidden_states.float() - final).abs().max() <= 4e-2 * max(1.0, float(final.abs().max()))
    print(f"fp32-matmul replay vs fixture: worst top-8 logit distance {worst_alt_ulps:.2f} bf16 ulps over {STEPS - 7} steps")
    assert 0.0 < worst_alt_ulps <= 8.0
