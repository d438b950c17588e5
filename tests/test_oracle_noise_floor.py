"""How far apart two valid implementations of the reference sit — the calibration of the GPU gates.

The reference fixes where values are rounded to bf16 but not the order in which a GEMV
accumulates in fp32.  Re-running the CPU oracle with its GEMVs evaluated as an fp32 matmul
(different order, same rounding points) moves individual bf16 results by one ulp; the residual
stream and the KV cache carry those flips forward.  The test records that distance on the reduced
model so that the GPU gates (2e-2 for one step from identical state, 4e-2 along a trajectory,
top-1 identical above a 2-ulp margin) are neither vacuous nor tighter than the reference itself
allows.
"""
import torch

import fused_oracle as fo
from qimeng_megakernel_amd import synthetic


def _rel(got, want):
    got, want = got.float(), want.float()
    rms = want.pow(2).mean().sqrt()
    return float(((got - want).abs() / torch.maximum(want.abs(), rms)).max())


def test_alternate_accumulation_order_distance(small_model, monkeypatch):
    shape, w, prompt = small_model
    a = synthetic.build_globals(w, shape, 96, "cpu")
    b = synthetic.build_globals(w, shape, 96, "cpu")
    oracle = fo.FusedOracle(shape)
    bf16_gemv = fo.gemv

    def fp32_gemv(weight, x):
        return (x.float() @ weight.float().t()).to(weight.dtype)

    seq = prompt.tolist()
    first_step_rel = None
    worst_logits = worst_hidden = 0.0
    clear_margin_mismatch = 0
    for pos in range(len(seq) + 24 - 1):
        for g in (a, b):
            oracle.embed(g, seq[pos]); g.position_id = pos
        monkeypatch.setattr(fo, "gemv", bf16_gemv); oracle.decode_step(a)
        monkeypatch.setattr(fo, "gemv", fp32_gemv); oracle.decode_step(b)
        if pos == 0:
            first_step_rel = max(_rel(b.logits, a.logits), _rel(b.hidden_states, a.hidden_states))
        worst_logits = max(worst_logits, _rel(b.logits, a.logits))
        worst_hidden = max(worst_hidden, _rel(b.hidden_states, a.hidden_states))
        want, got = int(a.logits.argmax()), int(b.logits.argmax())
        if pos >= len(prompt) - 1:
            seq.append(want)
            if got != want:
                top = torch.topk(a.logits.float(), 2).values
                ulp = 2.0 ** (torch.floor(torch.log2(top[0].abs())) - 7)
                clear_margin_mismatch += int((top[0] - top[1]) / ulp > 2.0)
    assert first_step_rel <= 2e-2
    assert worst_logits <= 4e-2 and worst_hidden <= 4e-2
    assert worst_logits > 2e-3            # the noise is real: a far tighter gate would reject valid runs
    assert clear_margin_mismatch == 0     # argmax only moves at near-ties
