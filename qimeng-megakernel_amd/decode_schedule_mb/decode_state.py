"""Scalar and per-row decode state (`qimeng_megakernel/models/LLM/decode_state.py:9-138`).

A request of B rows has one position and one active flag per row; a row that has produced an
end-of-sequence token stops advancing and its outputs are forced (zeros, logits -1e9) from then on.
"""
from __future__ import annotations

from typing import Any, Sequence

import torch


def batch_size(globs: Any) -> int:
    h = getattr(globs, "hidden_states", None)
    if h is None:
        raise ValueError("globs.hidden_states is required")
    return 1 if h.ndim == 1 else int(h.shape[0])


def decode_pos_id(globs: Any, row: int) -> int:
    ids = getattr(globs, "position_ids", None)
    if ids is not None:
        return int(ids[row])
    pos = getattr(globs, "position_id", None)
    return 0 if pos is None else int(pos)


def row_active(globs: Any, row: int) -> bool:
    mask = getattr(globs, "active_mask", None)
    return True if mask is None else bool(mask[row])


def kv_length(globs: Any, row: int) -> int:
    lens = getattr(globs, "kv_lengths", None)
    return int(lens[row]) if lens is not None else decode_pos_id(globs, row) + 1


def instruction_active(is_active: int, globs: Any, row: int) -> bool:
    """Instruction operand: 0 = never, 1 = always, anything else = follow the row's active flag."""
    if is_active == 0:
        return False
    if is_active == 1:
        return True
    return row_active(globs, row)


def ensure_decode_state(globs: Any, rows: int, device: torch.device) -> None:
    """Create the per-row fields a request of ``rows`` > 1 rows needs, where they are missing."""
    if rows < 2:
        return
    if getattr(globs, "active_mask", None) is None:
        globs.active_mask = torch.ones(rows, dtype=torch.bool, device=device)
    if getattr(globs, "kv_lengths", None) is None:
        ids = getattr(globs, "position_ids", None)
        if ids is not None:
            globs.kv_lengths = (ids.to(device) + 1).to(torch.long)
        else:
            pos = getattr(globs, "position_id", None)
            globs.kv_lengths = torch.full((rows,), (0 if pos is None else int(pos)) + 1, dtype=torch.long, device=device)
    if getattr(globs, "eos_reached", None) is None:
        globs.eos_reached = torch.zeros(rows, dtype=torch.bool, device=device)
    if getattr(globs, "last_generated_tokens", None) is None:
        globs.last_generated_tokens = torch.zeros(rows, dtype=torch.long, device=device)


def sync_kv_lengths(globs: Any) -> None:
    ids = getattr(globs, "position_ids", None)
    if ids is None:
        return
    if getattr(globs, "kv_lengths", None) is None or int(globs.kv_lengths.shape[0]) != int(ids.shape[0]):
        globs.kv_lengths = torch.empty(int(ids.shape[0]), dtype=torch.long, device=ids.device)
    torch.add(ids, 1, out=globs.kv_lengths)


def advance_decode_state(globs: Any, next_tokens: torch.Tensor, eos_token_ids: Sequence[int]) -> None:
    """After one step: remember the tokens, retire the rows that produced an EOS token, move the
    others one position on."""
    h = getattr(globs, "hidden_states", None)
    if h is None or h.ndim != 2 or int(h.shape[0]) < 2 or getattr(globs, "position_ids", None) is None:
        return
    device = globs.position_ids.device
    ensure_decode_state(globs, int(h.shape[0]), device)
    next_tokens = next_tokens.reshape(-1).to(device=device, dtype=torch.long)
    globs.last_generated_tokens.copy_(next_tokens)
    if isinstance(eos_token_ids, torch.Tensor) or eos_token_ids:
        eos = eos_token_ids if isinstance(eos_token_ids, torch.Tensor) else torch.tensor(list(eos_token_ids), dtype=torch.long, device=device)
        hit = (next_tokens[:, None] == eos.to(device=device, dtype=torch.long)[None, :]).any(dim=1)
    else:
        hit = torch.zeros_like(globs.active_mask)
    finished = globs.active_mask & hit
    alive = globs.active_mask & ~hit
    globs.eos_reached.logical_or_(finished)
    globs.active_mask.copy_(alive)
    globs.position_ids.add_(alive.to(globs.position_ids.dtype))
    sync_kv_lengths(globs)
