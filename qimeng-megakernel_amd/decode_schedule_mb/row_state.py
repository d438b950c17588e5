"""Where every row of a batch request stands: the position it decodes next and whether it still generates.

The kernel reads two of these tensors through ``mk(...)`` — ``position_ids`` (int32) and
``active_mask`` (bool) — and those two names are the boundary's; everything else here is this
package's.  A ``RowState`` is bound to one ``Globals`` (``RowState.of``), shares those two tensors
with it and is advanced by the host loop once per step, entirely on the device: a step never reads
anything back.  The reference keeps the same facts as loose attributes of its globals, updated by
`qimeng_megakernel/models/LLM/decode_state.py:46-138`; the rule is the same — a row that has produced
an end-of-sequence token stops advancing, stays retired, and the rows that go on move one position.
A row's KV length is always its position + 1 and is never stored.
"""
from __future__ import annotations

from typing import Any, Sequence

import torch


class RowState:
    def __init__(self, position_ids: torch.Tensor, active_mask: torch.Tensor):
        if position_ids.dtype != torch.int32 or active_mask.dtype != torch.bool or position_ids.shape != active_mask.shape:
            raise TypeError("position_ids must be int32 and active_mask bool, one element per row")
        self.position_ids = position_ids
        self.active_mask = active_mask
        self.finished = torch.zeros_like(active_mask)                    # rows retired by an end-of-sequence token
        self.last_tokens = torch.zeros_like(position_ids, dtype=torch.long)

    # ---- binding --------------------------------------------------------------
    @classmethod
    def of(cls, globs: Any) -> "RowState":
        """The state bound to ``globs``; created on first use around its ``position_ids`` / ``active_mask``
        (which are allocated here when the caller left them out: every row active, at ``position_id``)."""
        state = getattr(globs, "row_state", None)
        if isinstance(state, cls) and state.position_ids is globs.position_ids and state.active_mask is globs.active_mask:
            return state
        rows, device = rows_of(globs), globs.hidden_states.device
        if globs.position_ids is None:
            globs.position_ids = torch.full((rows,), int(getattr(globs, "position_id", None) or 0), dtype=torch.int32, device=device)
        if globs.active_mask is None:
            globs.active_mask = torch.ones(rows, dtype=torch.bool, device=device)
        state = cls(globs.position_ids, globs.active_mask)
        globs.row_state = state
        return state

    @property
    def rows(self) -> int:
        return int(self.position_ids.numel())

    # ---- the host loop --------------------------------------------------------
    def restart(self, position: int) -> None:
        """Every row active again, at ``position``: what a request starts from behind its prompt."""
        self.position_ids.fill_(position)
        self.active_mask.fill_(True)
        self.finished.zero_()

    def advance(self, next_tokens: torch.Tensor, eos: torch.Tensor | Sequence[int] | None = None) -> None:
        """One step is done and row r has produced ``next_tokens[r]``.  Rows whose token is one of ``eos``
        retire; the rows still active afterwards move on by one position."""
        tokens = next_tokens.reshape(-1).to(device=self.last_tokens.device, dtype=torch.long)
        self.last_tokens.copy_(tokens)
        if eos is not None and not isinstance(eos, torch.Tensor):
            eos = torch.tensor(list(eos), dtype=torch.long, device=tokens.device) if len(eos) else None
        if eos is not None and eos.numel():
            stopping = torch.isin(tokens, eos.to(tokens.device)).logical_and_(self.active_mask)
            self.finished.logical_or_(stopping)
            self.active_mask.logical_xor_(stopping)          # stopping rows are active rows: xor clears exactly them
        self.position_ids.add_(self.active_mask)

    def kv_lengths(self) -> torch.Tensor:
        return self.position_ids.to(torch.long) + 1

    # ---- host-side reads (scheduling a step from the present state; these synchronise) ----
    def position(self, row: int) -> int:
        return int(self.position_ids[row])

    def is_active(self, row: int) -> bool:
        return bool(self.active_mask[row])

    def follows(self, operand: int, row: int) -> bool:
        """The ``is_active`` operand of an instruction: 0 never runs, 1 always, anything else follows the row."""
        return operand == 1 or (operand != 0 and self.is_active(row))


def rows_of(globs: Any) -> int:
    """Rows of the buffers in ``globs`` (a vector is one row)."""
    hidden = globs.hidden_states
    if hidden is None:
        raise ValueError("globs.hidden_states is required")
    return int(hidden.shape[0]) if hidden.dim() > 1 else 1
