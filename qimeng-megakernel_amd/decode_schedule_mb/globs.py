"""``Globals`` of the batch route: the single-batch tensors with a leading batch dimension, plus
per-row state (`…/A100/multi_batch/decode_schedule/globs.py:13-26`).

Shapes for batch B (Llama-3.2-1B geometry): ``hidden_states/q_post_rope/attn_out [B, 2048]``,
``silu_out [B, 8192]``, ``logits [B, V]``, ``k_cache/v_cache [L, B, S, 8, 64]``,
``attn_out_intermediates [B, 32, P, 64]``, ``attn_lse_intermediates [B, 32, P]`` (log2 domain),
``barriers [L, 10, B * 48]`` (row 1 and 2 are used per batch row).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Optional

import torch

from ..decode_schedule.globs import Globals as _SingleBatchGlobals

Tensor = torch.Tensor


@dataclass
class Globals(_SingleBatchGlobals):
    position_ids: Optional[Tensor] = None            # int32 [B]  index of the token each row decodes
    active_mask: Optional[Tensor] = None             # bool  [B]  rows that still generate
    row_state: Optional[Any] = None                  # the RowState bound to the two tensors above (row_state.py)
    eos_token_id: Optional[int] = None
    attn_partial_valid: Optional[Tensor] = None      # bool  [B, Hq, P]  which split-KV partials hold data
    attn_rms_out: Optional[Tensor] = None            # bf16  [B, H]  RMSNorm rows for the QKV GEMM
    mlp_rms_out: Optional[Tensor] = None             # bf16  [B, H]  ... for the up/gate GEMM
    lm_head_rms_out: Optional[Tensor] = None         # bf16  [B, H]  ... for the LM head
