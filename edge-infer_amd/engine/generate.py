"""The generation loop: requests in, tokens out.

Requests are served in batches of sequences that start together: all prompts of a
batch in one step, then one token for each sequence that is still running.  A
sequence leaves its batch when it draws a stop token, reaches its length limit or
fills its cache capacity; the batch ends when its last sequence has left, its slots
are given back, and the next batch starts.  Per request the rules are those of the
reference's loop (runtime/src/inference.cpp:367-418): `max_length` counts prompt
plus generated tokens and is clipped to the capacity; a request whose limit does
not exceed its prompt produces nothing; the first token is drawn from the last
prompt row; a stop token ends the request and is not delivered.

A batch's prompts run in one step while they have at most `prompt_rows` tokens together;
beyond that they run in several steps of at most that many rows (whole prompts while they
fit, then portions), so that the step workspace, which grows with the rows of a step, stays
bounded however many long prompts start together.

The loop decides; it computes nothing.  It talks to a session through `begin`,
`step`, `end`, `capacity`, `free_tokens`, `max_batch` and to a sampler through one
call, so its decisions are tested without a GPU.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, List, Optional, Sequence

from ..cache.allocator import PAGE_TOKENS, pages_for
from ..sampling.params import SamplingParams


@dataclass
class Request:
    prompt: List[int]
    limit: int                      # total length at which the request stops
    stream: int                     # sampler stream (the request's index)
    output: List[int] = field(default_factory=list)
    slot: int = -1
    done: bool = False
    steps: int = 0                  # tokens drawn so far
    finish_reason: str = ""


def plan_batches(requests: Sequence[Request], max_batch: int, free_tokens: int) -> List[List[Request]]:
    """Consecutive requests are packed into a batch while the batch has room for one
    more sequence and the cache has pages for every sequence at its length limit."""
    batches: List[List[Request]] = []
    current: List[Request] = []
    pages_left = free_tokens // PAGE_TOKENS
    used = 0
    for request in requests:
        if request.done:
            continue
        need = pages_for(request.limit)
        if need > pages_left:
            raise ValueError(f"a request of up to {request.limit} tokens does not fit in a cache "
                             f"of {free_tokens} tokens")
        if current and (len(current) >= max_batch or used + need > pages_left):
            batches.append(current)
            current, used = [], 0
        current.append(request)
        used += need
    if current:
        batches.append(current)
    return batches


PROMPT_ROWS = 8192      # most rows of one prompt step


def prompt_steps(batch: Sequence[Request], budget: int):
    """The prompt steps of a batch: lists of (request, first token, tokens, whether the
    prompt ends here), each list at most `budget` tokens, prompts in order."""
    if budget < 1:
        raise ValueError("a prompt step needs room for at least one row")
    steps, current, room = [], [], budget
    for request in batch:
        done = 0
        while done < len(request.prompt):
            take = min(room, len(request.prompt) - done)
            current.append((request, done, take, done + take == len(request.prompt)))
            done += take
            room -= take
            if room == 0:
                steps.append(current)
                current, room = [], budget
    if current:
        steps.append(current)
    return steps


def generate(session, sampler, prompts: Sequence[Sequence[int]], *, vocab_size: int,
             max_length=None, max_new_tokens=None, params: Optional[SamplingParams] = None,
             stop_ids: Sequence[int] = (), callback: Optional[Callable[[int, int], None]] = None,
             max_batch: Optional[int] = None, first_stream: int = 0,
             prompt_rows: int = PROMPT_ROWS) -> List[List[int]]:
    """Generate for every prompt; returns the new tokens of each, in order.

    max_length (an int or one per prompt) counts prompt plus generated tokens;
    max_new_tokens counts generated ones.  `callback(index, token)` is called for
    every delivered token as it is drawn."""
    params = params or SamplingParams()
    params.validate(vocab_size)
    stop = set(int(s) for s in stop_ids)
    capacity = session.capacity
    n = len(prompts)

    def per_prompt(value):
        if value is None or isinstance(value, int):
            return [value] * n
        if len(value) != n:
            raise ValueError("one limit per prompt is needed")
        return list(value)

    lengths, news = per_prompt(max_length), per_prompt(max_new_tokens)
    requests: List[Request] = []
    for index, prompt in enumerate(prompts):
        prompt = [int(t) for t in prompt]
        if not prompt:
            raise ValueError(f"prompt {index} is empty")
        if len(prompt) > capacity:
            raise ValueError(f"prompt {index} has {len(prompt)} tokens, the capacity is {capacity}")
        for token in prompt:
            if not 0 <= token < vocab_size:
                raise ValueError(f"prompt {index} holds token id {token} outside the vocabulary")
        limit = capacity
        if lengths[index] is not None:
            limit = min(limit, int(lengths[index]))
        if news[index] is not None:
            if news[index] < 0:
                raise ValueError("max_new_tokens must not be negative")
            limit = min(limit, len(prompt) + int(news[index]))
        request = Request(prompt=prompt, limit=limit, stream=first_stream + index)
        if limit <= len(prompt):
            request.done = True
            request.finish_reason = "length"
        requests.append(request)

    batch_limit = session.max_batch if max_batch is None else min(max_batch, session.max_batch)
    for batch in plan_batches(requests, batch_limit, session.free_tokens()):
        _run_batch(session, sampler, batch, params, stop, vocab_size, callback, requests,
                   prompt_rows)
    return [request.output for request in requests]


def _deliver(request: Request, token: int, stop, vocab_size, callback, index) -> None:
    """Apply the reference's per-token rules to a freshly drawn token."""
    if not 0 <= token < vocab_size:
        raise RuntimeError(f"the sampler returned token id {token} outside the vocabulary")
    request.steps += 1
    total = len(request.prompt) + request.steps
    if token in stop:
        request.done, request.finish_reason = True, "stop"
        return
    request.output.append(token)
    if callback is not None:
        callback(index, token)
    if total >= request.limit:
        request.done, request.finish_reason = True, "length"


def _prefill(session, batch, prompt_rows):
    """Run the prompts; logits [len(batch), vocab] at each prompt's last token."""
    steps = prompt_steps(batch, prompt_rows)
    if len(steps) == 1:
        return session.step([(r.slot, r.prompt, [len(r.prompt) - 1]) for r in batch], copy=False)
    import torch
    rows = []
    for step in steps:
        logits = session.step([(r.slot, r.prompt[first:first + count], [count - 1] if last else [])
                               for r, first, count, last in step], copy=False)
        if logits.shape[0]:
            rows.append(logits.clone())     # the next step overwrites what this one returned
    return torch.cat(rows)                  # prompts end in the order of the batch


def _run_batch(session, sampler, batch, params, stop, vocab_size, callback, all_requests,
               prompt_rows=PROMPT_ROWS) -> None:
    index_of = {id(r): i for i, r in enumerate(all_requests)}
    try:
        for request in batch:
            request.slot = session.begin()
        logits = _prefill(session, batch, prompt_rows)
        active = list(batch)
        while True:
            tokens = sampler(logits, params, [r.stream for r in active],
                             [r.steps for r in active])
            for request, token in zip(active, tokens):
                _deliver(request, int(token), stop, vocab_size, callback, index_of[id(request)])
            feed = [(r, r.output[-1]) for r in active if not r.done]
            if not feed:
                break
            active = [r for r, _ in feed]
            logits = session.step([(r.slot, [token], [0]) for r, token in feed], copy=False)
    finally:
        for request in batch:
            if request.slot >= 0:
                session.end(request.slot)
                request.slot = -1
