"""Host step loops of the MoE ``mk`` route: prefill-by-decode, greedy loop, timing — one request (``decode``) or
several rows side by side (``decode_rows``).

Same shape as the dense loop (``decode.py``; reference `qimeng_megakernel/models/LLM/decode.py:536-796`):
one instruction tensor per request, per step the embedding row of the last token -> ``hidden_states``,
``position_id = pos``, one kernel launch, ``argmax`` of the bf16 logits; one event pair per step around
the launch only.
"""
from __future__ import annotations

import time
from typing import Any, Sequence

import torch

from .decode_batch import argmax_rows
from .decode_schedule_moe import mk_kernel as _mk_kernel
from .decode_schedule_moe.model_config import QwenMoeConfig


def decode(globs: Any, prompt_ids: torch.Tensor, max_new_tokens: int, *, mk: Any = None, decode_time: bool = True,
           use_graph: bool = False, timed_steps: int | None = None) -> dict[str, Any]:
    """Prefill + forced greedy decode to exactly ``max_new_tokens`` tokens (no EOS stop).

    ``timed_steps``: only the last that many decode steps are timed (and captured); the steps before them run
    untimed and the device is synchronised in between.  Default: all of them.

    ``use_graph``: the loop (embedding row, kernel, argmax, token write per step) is captured into one HIP graph
    and replayed; the positions are launch arguments, so the graph belongs to this request.  The result then
    carries ``replay``, which runs the same request once more through the graph."""
    device = globs.hidden_states.device
    T = int(prompt_ids.numel())
    if T + max_new_tokens > globs.k_cache.shape[2]:
        raise ValueError("prompt_len + max_new_tokens exceeds the KV cache capacity")
    mk = mk or _mk_kernel.get_mk()
    globs.instructions = None
    _mk_kernel.build(globs, mk)
    out = torch.zeros(T + max(max_new_tokens, 1), dtype=torch.long, device=device)
    out[:T] = prompt_ids.to(device)
    for pos in range(T):
        globs.hidden_states.copy_(globs.embed_tokens[out[pos]])
        globs.position_id = pos
        _mk_kernel.call_mk(globs, mk)
    out[T] = globs.logits.argmax()
    total = max(max_new_tokens - 1, 0)
    ntok = total if timed_steps is None else max(0, min(int(timed_steps), total))
    T0 = T
    for i in range(total - ntok):   # the untimed head of the request
        globs.hidden_states.copy_(globs.embed_tokens.index_select(0, out[T + i : T + i + 1]).view(-1))
        globs.position_id = T + i
        _mk_kernel.call_mk(globs, mk)
        out[T + i + 1] = globs.logits.argmax()
    T += total - ntok
    timed = decode_time and not use_graph
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(ntok if timed else 0)]
    loop_start, loop_end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def steps() -> None:
        for i in range(ntok):
            # a one-element index tensor: indexing with a 0-d tensor would read the token back to the host
            globs.hidden_states.copy_(globs.embed_tokens.index_select(0, out[T + i : T + i + 1]).view(-1))
            globs.position_id = T + i
            if events:
                events[i][0].record()
            _mk_kernel.call_mk(globs, mk)
            if events:
                events[i][1].record()
            # under capture: two short reductions instead of one long one, whose counter a memset node would clear
            out[T + i + 1] = argmax_rows(globs.logits.view(1, -1))[0] if use_graph else globs.logits.argmax()

    graph = None
    first_token = out[T].clone()
    if use_graph and ntok:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            steps()
    torch.cuda.synchronize(device)
    wall0 = time.perf_counter()
    loop_start.record()
    if graph is not None:
        graph.replay()
    else:
        steps()
    loop_end.record()
    torch.cuda.synchronize(device)
    result: dict[str, Any] = {"generated_ids": out, "new_tokens": out[T0:]}
    if graph is not None:
        def replay() -> torch.Tensor:
            """The same request once more through the captured loop (the KV rows it wrote are written again)."""
            out[T] = first_token
            graph.replay()
            return out[T0:]

        result["replay"] = replay
    if decode_time and ntok:
        wall = time.perf_counter() - wall0
        gpu_s = loop_start.elapsed_time(loop_end) / 1e3
        per_step_ms = [a.elapsed_time(b) for a, b in events]
        kernel_s = sum(per_step_ms) / 1e3 if events else float("inf")
        shape = QwenMoeConfig.shape()
        nbytes = sum(shape.step_bytes(T + i + 1) for i in range(ntok))
        result["timing"] = {
            "decode_wall_s": wall, "decode_gpu_s": gpu_s, "mk_kernel_gpu_s": kernel_s,
            "effective_tok_s_wall": ntok / wall, "effective_tok_s_gpu": ntok / gpu_s, "kernel_tok_s": ntok / kernel_s,
            "kernel_steps": ntok, "kernel_ms_per_step": kernel_s * 1e3 / ntok, "algorithmic_bytes": nbytes,
            "first_timed_context": T + 1, "last_timed_context": T + ntok,
            "achieved_GBps": nbytes / kernel_s / 1e9, "per_step_ms": per_step_ms,
        }
    mk.check()
    return result


def share_weights(globs: Any, shape: Any, kv_capacity: int, rows: int, *, max_partials: int) -> list[Any]:
    """``rows`` sets of buffers (KV cache, activations, counters) over ONE copy of ``globs``' weights: what a batch
    of requests on the batch-1 kernel needs.  Row 0 is ``globs`` itself."""
    from . import synthetic

    weights = {name: getattr(globs, name) for name in synthetic.MOE_WEIGHT_NAMES if getattr(globs, name, None) is not None}
    weights["embed_tokens"] = globs.embed_tokens
    out = [globs]
    for _ in range(1, rows):
        out.append(synthetic.build_moe_globals(weights, shape, kv_capacity, globs.hidden_states.device, max_partials=max_partials))
    return out


def decode_rows(rows: Sequence[Any], prompts: torch.Tensor, max_new_tokens: int, *, mks: Sequence[Any] | None = None,
                decode_time: bool = True, timed_steps: int | None = None) -> dict[str, Any]:
    """Greedy decode of ``len(rows)`` requests side by side on the batch-1 kernel: every step launches the kernel
    once per row, back to back on one stream (each row has its own buffers and its own launcher, hence its own
    workspace; the weights exist once).  Nothing is shared between the rows' launches but the weights' place in
    memory: a step moves every row's weight bytes again.  The reference has no MoE route for batch sizes above
    one; its batch loop (`qimeng_megakernel/models/LLM/decode.py:536-796`) is what the step order follows.

    ``prompts`` [B, T]; ``timed_steps`` as in ``decode``.  Timing: one event pair around each launch; a step's time
    is the sum over its rows."""
    B, T = int(prompts.shape[0]), int(prompts.shape[1])
    if B != len(rows):
        raise ValueError(f"{B} prompts for {len(rows)} rows of buffers")
    device = rows[0].hidden_states.device
    if any(T + max_new_tokens > int(g.k_cache.shape[2]) for g in rows):
        raise ValueError("prompt_len + max_new_tokens exceeds the KV cache capacity")
    mks = list(mks) if mks is not None else [_mk_kernel.get_mk() for _ in rows]
    for g, mk in zip(rows, mks):
        g.instructions = None
        _mk_kernel.build(g, mk)
    out = torch.zeros(B, T + max(max_new_tokens, 1), dtype=torch.long, device=device)
    out[:, :T] = prompts.to(device)

    def step(pos: int, column: int, events: list | None) -> None:
        for r, (g, mk) in enumerate(zip(rows, mks)):
            g.hidden_states.copy_(g.embed_tokens.index_select(0, out[r, column : column + 1]).view(-1))
            g.position_id = pos
            if events is not None:
                pair = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
                pair[0].record()
            _mk_kernel.call_mk(g, mk)
            if events is not None:
                pair[1].record()
                events.append(pair)
            out[r, column + 1] = g.logits.argmax()

    for pos in range(T - 1):           # prompt positions whose prediction is not needed
        for r, (g, mk) in enumerate(zip(rows, mks)):
            g.hidden_states.copy_(g.embed_tokens.index_select(0, out[r, pos : pos + 1]).view(-1))
            g.position_id = pos
            _mk_kernel.call_mk(g, mk)
    step(T - 1, T - 1, None)           # the last prompt position predicts the first new token
    total = max(max_new_tokens - 1, 0)
    ntok = total if timed_steps is None else max(0, min(int(timed_steps), total))
    for i in range(total - ntok):
        step(T + i, T + i, None)
    first = T + total - ntok
    events: list = []
    loop_start, loop_end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize(device)
    wall0 = time.perf_counter()
    loop_start.record()
    for i in range(ntok):
        step(first + i, first + i, events if decode_time else None)
    loop_end.record()
    torch.cuda.synchronize(device)
    result: dict[str, Any] = {"generated_ids": out, "new_tokens": out[:, T:]}
    if decode_time and ntok:
        wall = time.perf_counter() - wall0
        gpu_s = loop_start.elapsed_time(loop_end) / 1e3
        launch_ms = [a.elapsed_time(b) for a, b in events]
        kernel_s = sum(launch_ms) / 1e3
        shape = QwenMoeConfig.shape()
        nbytes = B * sum(shape.step_bytes(first + i + 1) for i in range(ntok))
        result["timing"] = {
            "decode_wall_s": wall, "decode_gpu_s": gpu_s, "mk_kernel_gpu_s": kernel_s,
            "effective_tok_s_wall": B * ntok / wall, "effective_tok_s_gpu": B * ntok / gpu_s, "kernel_tok_s": B * ntok / kernel_s,
            "kernel_steps": ntok, "kernel_launches": len(launch_ms), "kernel_ms_per_step": kernel_s * 1e3 / ntok,
            "kernel_ms_per_launch": kernel_s * 1e3 / len(launch_ms), "algorithmic_bytes": nbytes,
            "first_timed_context": first + 1, "last_timed_context": first + ntok, "achieved_GBps": nbytes / kernel_s / 1e9,
        }
    for mk in mks:
        mk.check()
    return result


def decode_batch(globs: Any, prompts: torch.Tensor, max_new_tokens: int, *, mk: Any = None, decode_time: bool = True,
                 timed_steps: int | None = None, merge_in_oproj: bool = False) -> dict[str, Any]:
    """Greedy decode of ``prompts.shape[0]`` requests in ONE launch per step (``decode_schedule_moe.rows_kernel``):
    ``globs`` holds the requests' buffers with a leading row dimension over one copy of the weights.  Per step: the
    rows' embedding rows -> ``hidden_states``, their positions -> ``position_ids``, one launch, ``argmax`` per row.
    The reference has no MoE route for batch sizes above one; the step order is its batch loop's
    (`qimeng_megakernel/models/LLM/decode.py:536-796`).

    Timing: one event pair per step around the launch.  ``algorithmic_bytes`` counts what a step has to move: the
    attention weights, the router and the LM head once, each row's KV rows, and every DISTINCT expert the rows picked
    once (counted by the kernel, per layer and step); ``moved_if_rows_alone`` is what the same rows cost as B launches.
    ``merge_in_oproj``: the batch-1 stream's way of merging the split-KV partials (see ``rows_kernel.mi355x_scheduler``);
    with it a row's bits are those of the default batch-1 request, without it those of the batch-1 request whose
    stream merges by the last arrival (``MoeScheduler(merge_in_last=True)``) — the two differ by what
    ``num / den`` and ``num * (1 / den)`` differ by in the attention output."""
    from .decode_schedule_moe import rows_kernel

    B, T = int(prompts.shape[0]), int(prompts.shape[1])
    if B != int(globs.hidden_states.shape[0]):
        raise ValueError(f"{B} prompts for {int(globs.hidden_states.shape[0])} rows of buffers")
    device = globs.hidden_states.device
    if T + max_new_tokens > int(globs.k_cache.shape[3]):
        raise ValueError("prompt_len + max_new_tokens exceeds the KV cache capacity")
    mk = mk or rows_kernel.get_mk()
    globs.instructions = None
    rows_kernel.build(globs, merge_in_oproj=merge_in_oproj)
    out = torch.zeros(B, T + max(max_new_tokens, 1), dtype=torch.long, device=device)
    out[:, :T] = prompts.to(device)
    distinct = torch.zeros((), dtype=torch.int64, device=device)

    def step(column: int, events: list | None, count: bool) -> None:
        globs.hidden_states.copy_(globs.embed_tokens.index_select(0, out[:, column]))
        globs.position_ids.fill_(column)
        if events is not None:
            pair = (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
            pair[0].record()
        mk(globs)
        if events is not None:
            pair[1].record()
            events.append(pair)
        if count:
            distinct.add_(globs.distinct_experts.sum())
        if column + 1 >= T:            # a prompt position's prediction is needed only behind the last one
            out[:, column + 1] = globs.logits.argmax(dim=-1)

    for pos in range(T):
        step(pos, None, False)
    total = max(max_new_tokens - 1, 0)
    ntok = total if timed_steps is None else max(0, min(int(timed_steps), total))
    for i in range(total - ntok):
        step(T + i, None, False)
    first = T + total - ntok
    events: list = []
    loop_start, loop_end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize(device)
    wall0 = time.perf_counter()
    loop_start.record()
    for i in range(ntok):
        step(first + i, events if decode_time else None, True)
    loop_end.record()
    torch.cuda.synchronize(device)
    result: dict[str, Any] = {"generated_ids": out, "new_tokens": out[:, T:]}
    if decode_time and ntok:
        wall = time.perf_counter() - wall0
        gpu_s = loop_start.elapsed_time(loop_end) / 1e3
        launch_ms = [a.elapsed_time(b) for a, b in events]
        kernel_s = sum(launch_ms) / 1e3
        shape = QwenMoeConfig.shape()
        experts = int(distinct.item())
        expert_bytes = 3 * shape.moe_intermediate_size * shape.hidden_size * 2
        alone = sum(shape.step_bytes(first + i + 1) for i in range(ntok))            # one row's bytes per step, summed
        shared = alone - ntok * shape.num_hidden_layers * shape.num_experts_per_tok * expert_bytes
        kv = sum(shape.step_bytes(first + i + 1) - shape.weight_bytes_per_token() for i in range(ntok))   # one row's KV rows read + appended
        nbytes = shared + (B - 1) * kv + experts * expert_bytes
        result["timing"] = {
            "decode_wall_s": wall, "decode_gpu_s": gpu_s, "mk_kernel_gpu_s": kernel_s,
            "effective_tok_s_wall": B * ntok / wall, "effective_tok_s_gpu": B * ntok / gpu_s, "kernel_tok_s": B * ntok / kernel_s,
            "kernel_steps": ntok, "kernel_launches": len(launch_ms), "kernel_ms_per_step": kernel_s * 1e3 / ntok,
            "algorithmic_bytes": nbytes, "moved_if_rows_alone": B * alone,
            "distinct_experts_per_layer": experts / (ntok * shape.num_hidden_layers),
            "first_timed_context": first + 1, "last_timed_context": first + ntok, "achieved_GBps": nbytes / kernel_s / 1e9,
        }
    mk.check()
    return result
