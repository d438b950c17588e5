"""Host step loop of the ``mk`` decode route: prefill-by-decode, greedy loop, timing.

Counterpart of ``_decode_mk`` + ``FusedGenerator.generate_greedy_fast`` in the
reference (`qimeng_megakernel/models/LLM/decode.py:536-796, 1340-1435`):

* the instruction tensor is built once per request;
* per step: embedding row -> ``hidden_states``, ``position_id = pos``, one kernel
  launch, ``argmax`` of the bf16 logits written straight into the token buffer;
  nothing synchronises inside the loop;
* with ``device_sampling`` the kernel itself picks the greedy token and loads its
  embedding row (``MegaKernel.greedy_into``): the loop is then nothing but launches,
  optionally captured once into a HIP graph (``use_graph``);
* timing: one pre-allocated event pair per step around the kernel call only
  (``mk_kernel_gpu_s``), one pair around the loop (``decode_gpu_s``) and
  ``perf_counter`` (``decode_wall_s``); the first new token comes from prefill
  and is not counted (`decode.py:768-776`).

Prefill runs the same kernel once per prompt position (the reference notes this
use of the decode layer stack, `fused/layer_scheduler.py:32-36`), so the whole
request stays on the HIP path.
"""
from __future__ import annotations

import time
from typing import Any, Callable

import torch

from .decode_schedule import mk_kernel as _mk_kernel
from .decode_schedule.instructions import scheduler as _scheduler


def _embed_into_hidden(globs: Any, token_ids: torch.Tensor) -> None:
    emb = globs.embed_tokens[token_ids].to(globs.hidden_states.dtype)
    globs.hidden_states.copy_(emb.reshape(-1))


def prefill_by_decode(globs: Any, mk: Any, prompt_ids: torch.Tensor, *, sample_into: tuple[torch.Tensor, int] | None = None) -> torch.Tensor:
    """Fill the KV cache for ``prompt_ids`` one position at a time; returns the first new token (0-dim).

    With ``sample_into=(tokens, index)`` the last launch picks that token on the device, stores it
    in ``tokens.view(-1)[index]`` and leaves its embedding in ``hidden_states``."""
    if globs.instructions is None:
        _scheduler.build(globs)
    prompt_ids = prompt_ids.to(globs.hidden_states.device)
    if prompt_ids.numel() == 0:
        raise ValueError("prompt must hold at least one token")
    if prompt_ids.numel() >= globs.k_cache.shape[2]:
        raise ValueError("prompt does not fit the KV cache")
    for pos in range(prompt_ids.numel()):
        _embed_into_hidden(globs, prompt_ids[pos : pos + 1])
        globs.position_id = pos
        if sample_into is not None and pos == prompt_ids.numel() - 1:
            mk.greedy_into(_embed_table(globs), sample_into[0], sample_into[1])
        _mk_kernel.call_mk(globs, mk)
    if sample_into is not None:
        return sample_into[0].view(-1)[sample_into[1]]
    return globs.logits.argmax()


def _embed_table(globs: Any) -> torch.Tensor:
    table = globs.embed_tokens
    return table.data if isinstance(table, torch.nn.Parameter) else table


def generate_greedy_on_device(
    globs: Any,
    output_tokens: torch.Tensor,
    prompt_len: int,
    ntok: int,
    *,
    mk: Any,
    mk_step_events: list[tuple[torch.cuda.Event, torch.cuda.Event]] | None = None,
) -> int:
    """``ntok`` greedy steps with no host work between launches.

    ``hidden_states`` must already hold the embedding of ``output_tokens[0, prompt_len]`` (the
    previous launch put it there); step ``i`` writes ``output_tokens[0, prompt_len + i + 1]``."""
    table = _embed_table(globs)
    for i in range(ntok):
        pos = prompt_len + i
        globs.position_id = pos
        mk.greedy_into(table, output_tokens, pos + 1)
        if mk_step_events is not None:
            mk_step_events[i][0].record()
        _mk_kernel.call_mk(globs, mk)
        if mk_step_events is not None:
            mk_step_events[i][1].record()
    return ntok


def generate_greedy_fast(
    globs: Any,
    output_tokens: torch.Tensor,
    prompt_len: int,
    ntok: int,
    *,
    call_mk: Callable[[Any], None],
    mk_step_events: list[tuple[torch.cuda.Event, torch.cuda.Event]] | None = None,
    reset_barriers: bool = False,
) -> int:
    """``ntok`` greedy steps; ``output_tokens`` is ``[1, prompt_len + ntok + 1]`` with the first new token set."""
    events = mk_step_events
    for i in range(ntok):
        pos = prompt_len + i
        _embed_into_hidden(globs, output_tokens[:, pos])
        globs.position_id = pos
        if reset_barriers:
            globs.barriers.zero_()
        if events is not None:
            events[i][0].record()
        call_mk(globs)
        if events is not None:
            events[i][1].record()
        output_tokens[:, pos + 1] = globs.logits.argmax()
    return ntok


def decode(
    globs: Any,
    prompt_ids: torch.Tensor,
    max_new_tokens: int,
    *,
    mk: Any = None,
    decode_time: bool = True,
    device_sampling: bool = False,
    use_graph: bool = False,
    timed_steps: int | None = None,
) -> dict[str, Any]:
    """Prefill + forced greedy decode to exactly ``max_new_tokens`` tokens (no EOS stop).

    ``device_sampling``: argmax and embedding lookup run inside the kernel.  ``use_graph`` (implies
    ``device_sampling``): the decode launches are captured into one HIP graph and replayed once;
    per-step kernel times are then not available (``kernel_tok_s`` is reported as 0).
    ``timed_steps``: only the last that many decode steps of the request are timed (and captured);
    the steps before them run untimed, followed by a device synchronisation.  Default: all of them."""
    device = globs.hidden_states.device
    prompt_len = int(prompt_ids.numel())
    if prompt_len + max_new_tokens > globs.k_cache.shape[2]:
        raise ValueError("prompt_len + max_new_tokens exceeds the KV cache capacity")
    mk = mk or _mk_kernel.get_mk()
    t0 = time.perf_counter()
    _scheduler.build(globs)
    instruction_setup_wall_s = time.perf_counter() - t0

    device_sampling = device_sampling or use_graph
    output_tokens = torch.zeros(1, prompt_len + max(max_new_tokens, 1), dtype=torch.long, device=device)
    output_tokens[0, :prompt_len] = prompt_ids.to(device)
    if device_sampling:
        prefill_by_decode(globs, mk, prompt_ids, sample_into=(output_tokens, prompt_len))
    else:
        output_tokens[0, prompt_len] = prefill_by_decode(globs, mk, prompt_ids)
    total = max(max_new_tokens - 1, 0)
    ntok = total if timed_steps is None else max(0, min(int(timed_steps), total))
    lead = total - ntok
    if lead:   # the untimed head of the request
        if device_sampling:
            generate_greedy_on_device(globs, output_tokens, prompt_len, lead, mk=mk)
        else:
            generate_greedy_fast(globs, output_tokens, prompt_len, lead, call_mk=lambda g: _mk_kernel.call_mk(g, mk))
        prompt_len += lead
    graph = None
    if use_graph and ntok > 0:
        # Capture on a side stream (as torch requires); every launch carries its own position and
        # token slot, so one replay is the whole request.  The graph starts from the state the
        # prefill left: nothing it reads was produced by the capture itself.
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            generate_greedy_on_device(globs, output_tokens, prompt_len, ntok, mk=mk)

    events = None
    if decode_time:
        events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
                  for _ in range(0 if graph is not None else ntok)]
        loop_start, loop_end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize(device)
        wall0 = time.perf_counter()
        loop_start.record()
    if graph is not None:
        graph.replay()
    elif device_sampling:
        generate_greedy_on_device(globs, output_tokens, prompt_len, ntok, mk=mk, mk_step_events=events)
    else:
        generate_greedy_fast(globs, output_tokens, prompt_len, ntok, call_mk=lambda g: _mk_kernel.call_mk(g, mk),
                             mk_step_events=events)
    result: dict[str, Any] = {"generated_ids": output_tokens, "new_tokens": output_tokens[:, prompt_len - lead:]}
    if decode_time:
        loop_end.record()
        torch.cuda.synchronize(device)
        decode_wall_s = time.perf_counter() - wall0
        decode_gpu_s = loop_start.elapsed_time(loop_end) / 1e3
        per_step_ms = [a.elapsed_time(b) for a, b in events]
        mk_kernel_gpu_s = sum(per_step_ms) / 1e3
        window = ntok  # tokens produced inside the timed window
        shape = globs_shape(globs)
        step_bytes = sum(shape.step_bytes(prompt_len + i + 1) for i in range(ntok))
        result["timing"] = {
            "instruction_setup_wall_s": instruction_setup_wall_s,
            "decode_wall_s": decode_wall_s,
            "decode_gpu_s": decode_gpu_s,
            "mk_kernel_gpu_s": mk_kernel_gpu_s,
            "non_kernel_gpu_s": max(decode_gpu_s - mk_kernel_gpu_s, 0.0),
            "effective_new_tokens": total + 1,
            "first_timed_context": prompt_len + 1,
            "last_timed_context": prompt_len + ntok,
            "decode_window_new_tokens": window,
            "effective_tok_s_wall": window / decode_wall_s if window and decode_wall_s > 0 else 0.0,
            "effective_tok_s_gpu": window / decode_gpu_s if window and decode_gpu_s > 0 else 0.0,
            "kernel_tok_s": window / mk_kernel_gpu_s if window and mk_kernel_gpu_s > 0 else 0.0,
            "kernel_steps": ntok,
            "kernel_ms_per_step": (mk_kernel_gpu_s * 1e3 / ntok) if ntok else 0.0,
            "algorithmic_bytes": step_bytes,
            "achieved_GBps": (step_bytes / mk_kernel_gpu_s / 1e9) if mk_kernel_gpu_s > 0 else 0.0,
            "per_step_ms": per_step_ms,
        }
    mk.check()
    return result


def globs_shape(globs: Any):
    """The DecodeShape the tensors of ``globs`` imply (layers and vocabulary read from the tensors)."""
    import dataclasses

    from .decode_schedule.model_config import LlamaConfig

    return dataclasses.replace(
        LlamaConfig.shape(),
        num_hidden_layers=int(globs.barriers.shape[0]),
        vocab_size=int(globs.logits.shape[0]),
    )
