"""Host step loop of the batch ``mk`` route: B rows decoded together, each at its own position.

Counterpart of the batch branch of the reference's decode loop
(`qimeng_megakernel/models/LLM/decode.py:536-796`, per-row state `LLM/decode_state.py:46-138`):
one instruction tensor per request (the scheduler's run-time template), per step the embedding
rows of the last tokens -> ``hidden_states``, one kernel launch, ``argmax`` per row, then
``RowState.advance`` (rows that produced an EOS token retire, the others move one position on).  Timing as in the batch-1 loop: one event pair per step around the launch only.

Prefill runs the same kernel once per prompt position with every row at that position.
"""
from __future__ import annotations

import time
from typing import Any, Sequence

import torch

from .decode_schedule_mb.row_state import RowState, rows_of
from .decode_schedule_mb import mk_kernel as _mk_kernel
from .decode_schedule_mb import rows_kernel as _rows_kernel

#: up to this many rows the batch-1 kernel's row-streaming engine decodes a batch faster than the matrix-core tiles
ROWS_ENGINE_MAX_BATCH = _rows_kernel.MAX_ROWS


def _route(mk: Any, rows: int, engine: str):
    """(launcher module, mk) for ``engine``: "rows" (1..4 rows on the row-streaming engine), "tiles" (the batch kernel's
    matrix-core tiles), or "auto": what ``mk`` was made for, else rows up to four rows and tiles beyond."""
    if engine not in ("auto", "rows", "tiles"):
        raise ValueError("engine must be 'auto', 'rows' or 'tiles'")
    if engine == "auto":
        if mk is not None:
            engine = "rows" if isinstance(mk, _rows_kernel.RowsMegaKernel) else "tiles"
        else:
            engine = "rows" if rows <= ROWS_ENGINE_MAX_BATCH else "tiles"
    module = _rows_kernel if engine == "rows" else _mk_kernel
    return module, (mk or module.get_mk())


def step_bytes(shape: Any, contexts: Sequence[int]) -> int:
    """Algorithmic HBM bytes of one batch step: the weights once, per active row its context's KV
    rows read and one KV row written."""
    kv = shape.kv_bytes_per_context_token()
    return shape.weight_bytes_per_token() + sum(kv * c + kv for c in contexts)


def _embed(globs: Any, tokens: torch.Tensor) -> None:
    globs.hidden_states.copy_(globs.embed_tokens[tokens].to(globs.hidden_states.dtype))


def prefill_by_decode(globs: Any, mk: Any, prompts: torch.Tensor) -> torch.Tensor:
    """``prompts`` [B, T]: fill the KV cache one position at a time; returns the first new token of every row."""
    B, T = prompts.shape
    prompts = prompts.to(globs.hidden_states.device)
    launcher = _rows_kernel if isinstance(mk, _rows_kernel.RowsMegaKernel) else _mk_kernel
    for pos in range(T):
        _embed(globs, prompts[:, pos])
        globs.position_ids.fill_(pos)
        launcher.call_mk(globs, mk)
    return globs.logits.argmax(dim=-1)


def argmax_rows(logits: torch.Tensor) -> torch.Tensor:
    """First index of each row's maximum, in two short reductions (within runs of W columns, then over the
    runs). One long reduction per row is spread over several workgroups by torch, with a counter that a memset
    node clears, and such nodes have given wrong values on the replays of a captured graph after the first."""
    rows, vocab = logits.shape
    width = 1024
    while width > 1 and vocab % width:
        width //= 2
    if width < 32:
        return logits.argmax(dim=-1)
    best, where = logits.view(rows, vocab // width, width).max(dim=-1)
    run = best.argmax(dim=-1, keepdim=True)
    return (run * width + where.gather(1, run)).squeeze(1)


def decode(globs: Any, prompts: torch.Tensor, max_new_tokens: int, *, mk: Any = None, eos_token_ids: Sequence[int] = (),
           decode_time: bool = True, use_graph: bool = False, timed_steps: int | None = None, engine: str = "auto") -> dict[str, Any]:
    """Prefill + greedy decode of B rows to ``max_new_tokens`` tokens each (rows that hit an EOS token
    of ``eos_token_ids`` retire; with none given every row runs to the end).

    ``timed_steps``: time only the last so many decode steps of the request (the longest contexts); the steps
    before them run untimed.  Default: all of them.

    ``use_graph``: the whole decode loop (embedding rows, kernel, argmax, row state) is captured into one
    HIP graph and replayed once — the kernel reads positions and activity from device tensors, so nothing
    in a step depends on the host.  Per-step kernel times are then not available.

    ``engine``: "tiles" = the batch kernel (matrix-core tiles, 2..16 rows), "rows" = the batch-1 kernel's row-streaming
    engine with every row's activation vector (1..4 rows: `decode_schedule_mb.rows_kernel`), "auto" = what ``mk`` was
    made for, else rows up to four rows.  Both decode every active row as the batch-1 route would decode it alone."""
    from .decode import globs_shape

    device = globs.hidden_states.device
    B, T = int(prompts.shape[0]), int(prompts.shape[1])
    if B != rows_of(globs):
        raise ValueError(f"{B} prompts for buffers of {rows_of(globs)} rows")
    if T + max_new_tokens > globs.k_cache.shape[2]:
        raise ValueError("prompt_len + max_new_tokens exceeds the KV cache capacity")
    launcher, mk = _route(mk, B, engine)
    state = RowState.of(globs)
    state.restart(0)
    globs.instructions = None
    launcher.build(globs)
    out = torch.zeros(B, T + max(max_new_tokens, 1), dtype=torch.long, device=device)
    out[:, :T] = prompts.to(device)
    out[:, T] = prefill_by_decode(globs, mk, prompts)
    state.restart(T)
    ntok = max(max_new_tokens - 1, 0)
    eos = None
    if eos_token_ids:   # on the device before the loop: nothing inside a step comes from the host
        eos = torch.tensor(list(eos_token_ids), dtype=torch.long, device=device)
    timed = decode_time and not use_graph
    lead_in = 0 if timed_steps is None or use_graph else max(ntok - max(int(timed_steps), 0), 0)
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(ntok - lead_in if timed else 0)]
    loop_start, loop_end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    active_log = []

    def steps(first: int = 0, last: int = ntok) -> None:
        for i in range(first, last):
            _embed(globs, out[:, T + i])
            if events and i >= lead_in:
                events[i - lead_in][0].record()
            launcher.call_mk(globs, mk)
            if events and i >= lead_in:
                events[i - lead_in][1].record()
            nxt = argmax_rows(globs.logits) if use_graph else globs.logits.argmax(dim=-1)
            out[:, T + i + 1] = nxt
            if eos is not None:
                active_log.append(globs.active_mask.clone())
            state.advance(nxt, eos)

    graph = None
    first_token = out[:, T].clone()

    def rewind() -> None:   # the state the prefill left: what a replay of the captured loop starts from
        out[:, T] = first_token
        state.restart(T)

    if use_graph and ntok:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            steps()
        rewind()   # capturing ran nothing, but the host-side bookkeeping of the loop did
    if graph is None and lead_in:
        steps(0, lead_in)
    torch.cuda.synchronize(device)
    wall0 = time.perf_counter()
    loop_start.record()
    if graph is not None:
        graph.replay()
    else:
        steps(lead_in, ntok)
    loop_end.record()
    torch.cuda.synchronize(device)
    result: dict[str, Any] = {"generated_ids": out, "new_tokens": out[:, T:]}
    if graph is not None:
        def replay(_inputs=(eos,)) -> torch.Tensor:
            """The same request once more through the captured loop (the KV rows it wrote are simply written again).
            ``_inputs`` keeps alive what the graph reads but was allocated outside its capture."""
            rewind()
            graph.replay()
            return out[:, T:]

        result["replay"] = replay
    if decode_time and ntok:
        wall = time.perf_counter() - wall0
        gpu_s = loop_start.elapsed_time(loop_end) / 1e3
        per_step_ms = [a.elapsed_time(b) for a, b in events]
        kernel_s = sum(per_step_ms) / 1e3 if events else float("inf")
        shape = globs_shape(globs)
        if eos is not None:
            rows = [int(m.sum()) for m in active_log]
        else:
            rows = [B] * ntok
        window = range(lead_in, ntok)          # the steps between the loop's two events
        produced = sum(rows[i] for i in window)
        nbytes = sum(step_bytes(shape, [T + i + 1] * rows[i]) for i in window)
        nsteps = max(len(window), 1)
        result["timing"] = {
            "decode_wall_s": wall, "decode_gpu_s": gpu_s, "mk_kernel_gpu_s": kernel_s,
            "decode_window_new_tokens": produced,
            "effective_tok_s_wall": produced / wall, "effective_tok_s_gpu": produced / gpu_s,
            "kernel_tok_s": produced / kernel_s, "kernel_steps": len(window), "kernel_ms_per_step": kernel_s * 1e3 / nsteps,
            "algorithmic_bytes": nbytes, "achieved_GBps": nbytes / kernel_s / 1e9, "per_step_ms": per_step_ms,
            "first_timed_context": T + lead_in + 1, "last_timed_context": T + ntok,
            "engine": "rows" if launcher is _rows_kernel else "tiles",
        }
    mk.check()
    return result
