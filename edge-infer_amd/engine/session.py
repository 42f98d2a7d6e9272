"""A session: the mutable side of generation for one model.

It owns the cache (slots, pages, fixed-size state), the workspaces and the metadata
buffers, and offers the step function: `step(entries)` runs exactly the tokens it
is given, as one batch, from what earlier steps left in the cache, and returns
float32 logits at the wanted places.  Requests are validated before anything is
written (token ids, live slots, room in the cache), so a refused step leaves the
session as it was; the reference holds the same contract, runtime/src/qwen3.cpp:405-418.
"""
from __future__ import annotations

import numbers
import os
from collections import OrderedDict
from typing import List, Optional, Sequence, Tuple

import torch

from ..cache.allocator import PAGE_TOKENS
from ..cache.storage import CacheLayout, SessionCache
from ..parts.base import StepContext, Workspace
from .batch import DeviceMeta, SeqStep, StepPlan

# EDGE_INFER_DECODE_GRAPHS=0: decode steps run eagerly instead of from HIP graphs (the
# reference has such a switch too, runtime/src/qwen3.cpp:9-12, where graphs are off unless set)
GRAPHS_SWITCH = "EDGE_INFER_DECODE_GRAPHS"
MAX_GRAPHS = 24         # captured decode steps a session keeps; the one unused for longest goes


def batch_bucket(live: int) -> int:
    """The fixed batch size a decode step of `live` sequences is padded to when it is
    captured: powers of two up to 16, multiples of 8 up to 64, then multiples of 32.  (A
    padding row costs what a live one costs: 48 sequences in a step for 64 took 4.63 ms for
    the 8B shape where the step for 48 takes 4.46.)"""
    if live <= 16:
        bucket = 1
        while bucket < live:
            bucket *= 2
        return bucket
    if live <= 64:
        return (live + 7) // 8 * 8
    return (live + 31) // 32 * 32


def context_bound(context: int, capacity: int) -> int:
    """The bound a captured decode step holds for: the next of 256, 384, 512, 768, 1024,
    1536, ... at or above the longest sequence, capped by the capacity.  Parts fix their
    launch shapes by the bound (see `StepContext.context_bound`), so finer steps mean shapes
    that fit the true lengths better, at the price of more graphs."""
    bound = 256
    while bound < context:
        bound = bound * 3 // 2 if bound & (bound - 1) == 0 else bound // 3 * 4
    return max(1, min(bound, capacity))


class _CapturedDecode:
    """A decode step of a fixed batch size, captured once as a HIP graph.  Everything
    that changes from step to step (tokens, positions, page tables, which rows are
    live) lives in its metadata buffer, which is filled before every replay."""

    def __init__(self, device):
        self.meta = DeviceMeta(device)
        self.workspace = Workspace(device)
        self.graph = None
        self.logits = None
        self.layout = None      # where the metadata sections lay when the graph was captured
        self.plan = None        # the step about to run
        self.key = None         # (batch bucket, context bound)


class Session:
    def __init__(self, model, max_tokens: int, max_seqs: Optional[int] = None,
                 max_seq_tokens: Optional[int] = None, seed: int = 0, graphs: bool = True):
        self.model = model
        self.device = model.device
        self.dtype = model.dtype
        if max_tokens < 1:
            raise ValueError("max_tokens must be positive")
        n_pages = (max_tokens + PAGE_TOKENS - 1) // PAGE_TOKENS
        if max_seqs is None:
            max_seqs = min(n_pages, 256)
        limit = model.max_positions()
        if max_seq_tokens is not None:
            if not 1 <= max_seq_tokens <= limit:
                raise ValueError(f"a sequence capacity must lie in 1..{limit}, got {max_seq_tokens}")
            limit = max_seq_tokens
        self.cache = SessionCache(CacheLayout(model.spec), max_tokens, max_seqs, self.dtype,
                                  self.device, limit)
        self.seed = int(seed)
        self._streams_used = 0
        self._sampler = None
        self.workspace = Workspace(self.device)
        self.meta = DeviceMeta(self.device)
        self.steps_run = 0
        # decode steps are replayed from HIP graphs unless the model has an operation
        # that is not safe to capture (see DecoderModel.capture_safe) or the caller or the
        # environment says no
        self.graphs = (bool(graphs) and os.environ.get(GRAPHS_SWITCH, "1") != "0"
                       and model.capture_safe())
        self._capture_rows = min(model.capture_rows(), 256) if self.graphs else 0
        self._captured: "OrderedDict[Tuple[int, int], _CapturedDecode]" = OrderedDict()
        self._graph_logits = None     # one buffer for the logits of every captured step
        self.graph_replays = 0
        self.graph_captures = 0
        # one generation or reset at a time: a callback that calls back into its own session
        # is refused, as in the reference (bindings/python/include/python_callback.hpp:16-26)
        self._busy = False
        self._unusable = False     # set for good when a failed step cannot even be waited for

    # -- slots -----------------------------------------------------------
    def begin(self) -> int:
        """Take a slot for a new sequence (length 0)."""
        self._require_usable()
        return self.cache.acquire()

    def end(self, slot: int) -> None:
        """Give a slot and everything it holds back."""
        self.cache.release(slot)

    def reset(self, trim: bool = False) -> None:
        """End every live sequence.  Allocations are kept unless `trim` is set: then the step
        workspaces and the captured graphs go too (the cache stays), which gives back what a
        single very large step made the session hold."""
        if self._busy:
            raise RuntimeError("the session is busy; wait for the current operation to finish")
        self._require_usable()
        torch.cuda.synchronize(self.device)
        self.cache.release_all()
        if trim:
            self._captured.clear()
            self._graph_logits = None
            self.workspace.clear()

    def length(self, slot: int) -> int:
        if not self.cache.slots.is_live(slot):
            raise ValueError(f"slot {slot} is not live")
        return self.cache.lengths[slot]

    @property
    def capacity(self) -> int:
        """Most tokens one sequence can hold."""
        return self.cache.max_seq_tokens

    @property
    def speculative(self) -> bool:
        """Always False (the reference's sessions say whether they draft with a second model,
        bindings/python/model_bridge.cpp:256; this library has no such sessions)."""
        return False

    @property
    def max_batch(self) -> int:
        return self.cache.n_slots

    def workspace_report(self) -> dict:
        """Bytes of the step workspaces: what is held, and for every planned shape of step
        (rows, sequences, wanted rows, decode, context bound) the arena it needs, what its
        values would need without sharing, and what sharing saves (the reference reports
        the same of its decode plan, runtime/include/qwen3.hpp:60-63)."""
        def plans(workspace):
            return {signature: {"arena_bytes": layout.arena.arena_bytes,
                                "bytes_without_sharing": layout.arena.bytes_without_sharing(),
                                "bytes_saved": layout.arena.bytes_saved(),
                                "buffers": len(layout.arena),
                                "regions": layout.arena.regions()}
                    for signature, layout in workspace._plans.items()}
        report = {"held_bytes": self.workspace.bytes(), "plans": plans(self.workspace)}
        for key, captured in self._captured.items():
            report["held_bytes"] += captured.workspace.bytes()
            report["plans"].update(plans(captured.workspace))
        return report

    def free_tokens(self) -> int:
        if not self.cache.kv_pools:
            return self.cache.n_pages * PAGE_TOKENS
        return min(pool.n_free for pool in self.cache.kv_pools) * PAGE_TOKENS

    # -- generation ----------------------------------------------------------
    def generate_batch(self, prompts, *, max_length=None, max_new_tokens=None, temperature=1.0,
                       top_p=0.9, top_k=1, seed=None, stop_ids=None, callback=None,
                       max_batch=None, first_stream=None, prompt_rows=None):
        """New tokens for every prompt (lists of ints), served in batches of prompts
        that start together.  `callback(index, token)` sees each delivered token.
        `prompt_rows`: most tokens of one prompt step (default 8,192; more prompt tokens than
        that run in several steps)."""
        from ..sampling.params import SamplingParams
        from ..sampling.sampler import Sampler
        from .generate import generate
        if self._sampler is None:
            self._sampler = Sampler(self.device)
        spec = self.model.spec
        if stop_ids is None:
            stop_ids = (spec.eos_token_id,)
        if first_stream is None:
            first_stream = self._streams_used
            self._streams_used += len(prompts)
        params = SamplingParams(temperature=float(temperature), top_p=float(top_p),
                                top_k=int(top_k), seed=self.seed if seed is None else int(seed))
        if self._busy:
            raise RuntimeError("the session is busy; wait for the current operation to finish")
        self._busy = True
        try:
            return generate(self, self._sampler, prompts, vocab_size=spec.vocab_size,
                            max_length=max_length, max_new_tokens=max_new_tokens, params=params,
                            stop_ids=stop_ids, callback=callback, max_batch=max_batch,
                            first_stream=first_stream,
                            **({} if prompt_rows is None else {"prompt_rows": int(prompt_rows)}))
        finally:
            self._busy = False

    def generate(self, input_ids, callback=None, max_length=100, temperature=1.0, top_p=0.9,
                 top_k=1, seed=None):
        """One complete fresh prompt; `max_length` counts prompt plus generated tokens;
        `callback(token)` sees every delivered token; the end-of-sequence token ends
        the request and is not delivered.  Names, meanings and defaults of the
        reference's Session.generate (bindings/python/model_bridge.cpp:248-252).
        Returns the delivered tokens."""
        wrapped = None if callback is None else (lambda index, token: callback(token))
        return self.generate_batch([list(input_ids)], max_length=max_length,
                                   temperature=temperature, top_p=top_p, top_k=top_k, seed=seed,
                                   callback=wrapped)[0]

    # -- the step function -------------------------------------------------
    def _validate(self, entries) -> List[SeqStep]:
        vocab = self.model.spec.vocab_size
        seqs: List[SeqStep] = []
        seen = set()
        if not entries:
            raise ValueError("a step needs at least one entry")
        for slot, tokens, want in entries:
            if not self.cache.slots.is_live(slot):
                raise ValueError(f"slot {slot} is not live")
            if slot in seen:
                raise ValueError(f"slot {slot} appears twice in one step")
            seen.add(slot)
            tokens = list(tokens)
            if not tokens:
                raise ValueError("an entry brings at least one token")
            for index, token in enumerate(tokens):
                if type(token) is not int:       # (the common case needs no further look)
                    if not isinstance(token, numbers.Integral) or isinstance(token, bool):
                        raise ValueError(f"token ids are integers, got {token!r}")
                    tokens[index] = token = int(token)
                if not 0 <= token < vocab:
                    raise ValueError(f"token id {token!r} is outside the vocabulary of {vocab}")
            want = list(want)
            for w in want:
                if not 0 <= w < len(tokens):
                    raise ValueError(f"wanted place {w} is outside the {len(tokens)} tokens given")
            seqs.append(SeqStep(slot=slot, start=self.cache.lengths[slot], tokens=tokens,
                                want=want))
        return seqs

    def step(self, entries: Sequence[Tuple[int, Sequence[int], Sequence[int]]],
             copy: bool = True) -> torch.Tensor:
        """entries: (slot, next tokens, wanted places among them).  Returns float32
        logits [number of wanted places, vocab] in the order of entries and places.
        With copy=False the result is a view of the session's workspace that the next
        step overwrites."""
        self._require_usable()
        seqs = self._validate(entries)
        growth = [(seq.slot, seq.start + seq.count) for seq in seqs]
        self.cache.grow(growth)                  # raises before anything changes
        saved = None
        try:
            captured = None
            if (self.graphs and batch_bucket(len(seqs)) <= self._capture_rows
                    and all(seq.count == 1 for seq in seqs)):
                captured = self._captured_for(seqs)
            if captured is None:
                plan = self._plan(seqs)
                meta, workspace = self.meta, self.workspace
            else:
                plan, meta, workspace = captured.plan, captured.meta, captured.workspace
            ctx = self._context(plan, meta, workspace, fixed_shape=captured is not None)
            if self.cache.states:
                # state of fixed size is updated in place: keep what the step may change
                saved = meta.seq_slot[:plan.n_live_seqs]
                self.cache.save_states(saved)
            logits = (self.model.forward(ctx) if captured is None
                      else self._run_captured(captured, ctx))
        except BaseException:
            self._drain_failed_step(saved)
            raise                                 # the original error
        self.cache.commit(growth)
        self.steps_run += 1
        return logits.clone() if copy else logits

    def _require_usable(self) -> None:
        if self._unusable:
            raise RuntimeError("the session is unusable after a failed GPU stream completion")

    def _drain_failed_step(self, saved_slots=None) -> None:
        """After an error in a step that may have launched work: wait for what was launched.
        The sequences keep the lengths they had: keys and values that the step wrote lie
        beyond them and are written again by the next step, and state of fixed size, which
        mixers update in place, is put back from the copy taken before the step.  So the
        session stays usable; only if the wait or the restoring itself fails is nothing known
        any more, and the session refuses every later call, as the reference's does
        (runtime/src/qwen3.cpp:126-161,374-379)."""
        try:
            torch.cuda.synchronize(self.device)
            if saved_slots is not None:
                self.cache.restore_states(saved_slots)
                torch.cuda.synchronize(self.device)
        except Exception:       # the original error is the one that is raised
            self._unusable = True

    def _plan(self, seqs, pad_seqs=None, bound=None) -> StepPlan:
        plan = StepPlan(seqs, pad_seqs=pad_seqs, context_bound=bound,
                        spare_slot=self.cache.n_slots)
        self.model.plan_step(plan)      # the parts add the sections they plan for themselves
        return plan

    def _context(self, plan, meta, workspace, fixed_shape=False):
        slots = [seq.slot for seq in plan.seqs]
        tables = [self.cache.page_rows(group, slots, plan.n_seqs)
                  for group in range(len(self.cache.kv_pages))]
        meta.upload(plan, tables)
        ctx = StepContext(dtype=self.dtype, device=self.device, n_rows=plan.n_rows,
                          n_seqs=plan.n_seqs, decode=plan.decode, meta=meta, cache=self.cache,
                          workspace=workspace, max_context=plan.max_context,
                          context_bound=plan.context_bound, fixed_shape=fixed_shape)
        ctx.sequences = plan.seqs
        return ctx

    def context_for(self, seqs: List[SeqStep]):
        """(step context, plan) for these sequences on the session's own buffers, with the
        metadata uploaded and nothing run: what a part needs to be driven on its own."""
        plan = self._plan(seqs)
        return self._context(plan, self.meta, self.workspace), plan

    def _captured_for(self, seqs: List[SeqStep]) -> _CapturedDecode:
        """The captured step for this batch: one per batch-size bucket and context bound,
        the most recently used `MAX_GRAPHS` of them.  All of them write their logits into one
        buffer of the session (the next step overwrites a step's logits anyway)."""
        bucket = batch_bucket(len(seqs))
        longest = max(seq.start + seq.count for seq in seqs)
        bound = context_bound(longest, self.capacity)
        key = (bucket, bound)
        captured = self._captured.pop(key, None)
        if captured is None:
            captured = _CapturedDecode(self.device)
            while len(self._captured) >= MAX_GRAPHS:
                self._captured.popitem(last=False)
        self._captured[key] = captured
        vocab = self.model.spec.vocab_size
        rows = batch_bucket(min(self.max_batch, self._capture_rows))
        if self._graph_logits is None or self._graph_logits.numel() < bucket * vocab:
            self._captured.clear()          # graphs hold the old buffer's address
            self._captured[key] = captured = _CapturedDecode(self.device)
            self._graph_logits = torch.empty(max(rows, bucket) * vocab, dtype=torch.float32,
                                             device=self.device)
        captured.workspace.bind("logits", self._graph_logits)
        captured.plan = self._plan(seqs, pad_seqs=bucket, bound=bound)
        captured.key = key
        return captured

    def _run_captured(self, captured: _CapturedDecode, ctx) -> torch.Tensor:
        """The first step of a (bucket, bound) pair runs eagerly on the pair's own buffers and
        is then captured; later steps only refresh the metadata and replay."""
        seqs = ctx.sequences
        layout = captured.meta.generation
        if captured.graph is not None and captured.layout != layout:
            captured.graph = None           # the metadata moved: what was captured reads stale places
        if captured.graph is None:
            try:
                logits = self.model.forward(ctx)
                torch.cuda.synchronize(self.device)
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph):
                    captured.logits = self.model.forward(ctx)
            except BaseException:
                self._captured.pop(captured.key, None)   # nothing half-made is kept
                raise
            captured.graph, captured.layout = graph, layout
            self.graph_captures += 1
        else:
            captured.graph.replay()
            self.graph_replays += 1
            logits = captured.logits
        # the captured step computes the logits of every row; hand out the wanted ones
        rows = [index for index, seq in enumerate(seqs) for _ in seq.want]
        if rows == list(range(len(seqs))):
            return logits[:len(seqs)]
        if not rows:
            return logits[:0]
        return logits[torch.tensor(rows, device=self.device)]
