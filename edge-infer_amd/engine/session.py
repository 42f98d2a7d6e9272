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
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..cache.allocator import PAGE_TOKENS
from ..cache.storage import CacheLayout, SessionCache
from ..parts.base import StepContext, Workspace
from ..parts.linear import SKINNY_ROWS
from .batch import DeviceMeta, SeqStep, StepPlan


class _Context(StepContext):
    def __init__(self, session, fixed_context=None, **kwargs):
        super().__init__(**kwargs)
        self._session = session
        self._fixed_context = fixed_context

    def decode_splits(self, n_kv_heads: int) -> int:
        """How many blocks share the key range of one (sequence, kv head) in decode:
        enough to put about two blocks on each of the 256 compute units, never more
        than there are pages.  A captured step fixes the count by the capacity (blocks
        whose share of a short sequence is empty return at once)."""
        context = self._fixed_context or self.max_context
        pages = max(1, (context + PAGE_TOKENS - 1) // PAGE_TOKENS)
        blocks = self.n_seqs * n_kv_heads
        wanted = (512 + blocks - 1) // blocks
        return max(1, min(wanted, pages, 32))

    def decode_plan(self, n_kv_heads: int, group: int = 1):
        """(slices, waves per block) for the matrix-core decode kernel.  Up to 256 (sequence,
        kv head) pairs: blocks of 16 waves, a tile of 16 keys per wave at a time, and as many
        slices of the key range as shorten a wave's walk by more than the merge kernel costs,
        while all blocks still fit the chip at once (256 compute units x 16 waves).  The
        weights are measured ones: 1.9 us for a tile a wave walks, 4.5 us for the merge and
        0.1 us for each slice it reads.  More pairs than that: blocks of 4 waves, see
        `decode_splits`."""
        context = self._fixed_context or self.max_context
        # (a block of 16 waves takes at most 4 query heads of a group: larger groups have
        # several blocks per pair)
        pairs = self.n_seqs * n_kv_heads * ((group + 3) // 4)
        if pairs > 256:
            return self.decode_splits(n_kv_heads), 4
        tiles = (context + 15) // 16
        pages = max(1, (context + PAGE_TOKENS - 1) // PAGE_TOKENS)
        best, best_cost = 1, 1.9 * ((tiles + 15) // 16)
        slices = 2
        while slices <= min(pages, 32) and pairs * 16 * slices <= 4096:
            cost = 1.9 * ((tiles + 16 * slices - 1) // (16 * slices)) + 4.5 + 0.1 * slices
            if cost < best_cost:
                best, best_cost = slices, cost
            slices *= 2
        return best, 16


class _CapturedDecode:
    """A decode step of a fixed batch size, captured once as a HIP graph.  Everything
    that changes from step to step (tokens, positions, page tables, which rows are
    live) lives in its metadata buffer, which is filled before every replay."""

    def __init__(self, device):
        self.meta = DeviceMeta(device)
        self.workspace = Workspace(device)
        self.graph = None
        self.logits = None


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
        self._item_sizes = model.attention_item_sizes()
        self.steps_run = 0
        # decode steps are replayed from HIP graphs unless the model has an operation
        # that is not safe to capture (see DecoderModel.capture_safe) or the caller or the
        # environment says no: EDGE_INFER_ENABLE_QWEN3_GRAPH=0 (the reference's switch,
        # runtime/src/qwen3.cpp:9-12, where graphs are off unless it is 1)
        self.graphs = (bool(graphs) and os.environ.get("EDGE_INFER_ENABLE_QWEN3_GRAPH", "1") != "0"
                       and model.capture_safe())
        self._captured: Dict[Tuple[int, int], _CapturedDecode] = {}
        self.graph_replays = 0
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

    def reset(self) -> None:
        """End every live sequence; allocations are kept."""
        if self._busy:
            raise RuntimeError("the session is busy; wait for the current operation to finish")
        self._require_usable()
        torch.cuda.synchronize(self.device)
        self.cache.release_all()

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
            return {signature: {"arena_bytes": layout.plan.total_bytes,
                                "unaliased_bytes": layout.plan.unaliased_bytes(),
                                "reused_bytes": layout.plan.reused_bytes(),
                                "values": len(layout.plan.allocations),
                                "slots": layout.plan.slot_count()}
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
                       max_batch=None, first_stream=None):
        """New tokens for every prompt (lists of ints), served in batches of prompts
        that start together.  `callback(index, token)` sees each delivered token."""
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
                            first_stream=first_stream)
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
                if not isinstance(token, numbers.Integral) or isinstance(token, bool):
                    raise ValueError(f"token ids are integers, got {token!r}")
                if not 0 <= token < vocab:
                    raise ValueError(f"token id {token!r} is outside the vocabulary of {vocab}")
                tokens[index] = int(token)
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
        self.cache.check_growth(growth)          # raises before anything changes
        self.cache.grow(growth)
        try:
            # batches beyond the few-rows product's reach multiply through the library, whose
            # kernels are kept out of graphs
            if (self.graphs and len(seqs) <= SKINNY_ROWS
                    and all(seq.count == 1 for seq in seqs)):
                logits = self._run_captured(seqs)
            else:
                plan = StepPlan(seqs, item_sizes=self._item_sizes)
                logits = self._run(plan, self.meta, self.workspace)
        except BaseException:
            self._drain_failed_step()
            raise                                 # the original error
        self.cache.commit(growth)
        self.steps_run += 1
        return logits.clone() if copy else logits

    def _require_usable(self) -> None:
        if self._unusable:
            raise RuntimeError("the session is unusable after a failed GPU stream completion")

    def _drain_failed_step(self) -> None:
        """After an error in a step that may have launched work: wait for what was launched.
        The sequences keep the lengths they had (what the step wrote lies beyond them and
        is written again by the next step), so the session stays usable; only if the wait
        itself fails is nothing known any more, and the session refuses every later call,
        as the reference's does (runtime/src/qwen3.cpp:126-161,374-379)."""
        try:
            torch.cuda.synchronize(self.device)
        except Exception:       # the original error is the one that is raised
            self._unusable = True

    def _context(self, plan, meta, workspace, fixed_context=None):
        slots = [seq.slot for seq in plan.seqs]
        tables = [self.cache.page_rows(group, slots, plan.n_seqs)
                  for group in range(len(self.cache.kv_pages))]
        meta.upload(plan, tables)
        ctx = _Context(self, fixed_context=fixed_context, dtype=self.dtype, device=self.device,
                       n_rows=plan.n_rows, n_seqs=plan.n_seqs, decode=plan.decode, meta=meta,
                       cache=self.cache, workspace=workspace, max_context=plan.max_context)
        ctx.sequences = plan.seqs
        return ctx

    def _run(self, plan: StepPlan, meta: DeviceMeta, workspace: Workspace) -> torch.Tensor:
        return self.model.forward(self._context(plan, meta, workspace))

    def _run_captured(self, seqs: List[SeqStep]) -> torch.Tensor:
        """A decode step through the graph of its batch-size bucket (powers of two up to
        64, then steps of 32) and context bound.  The first step of a bucket runs eagerly on the bucket's own buffers
        and is then captured; later steps only refresh the metadata and replay."""
        live = len(seqs)
        bucket = 1
        while bucket < live and bucket < 64:
            bucket *= 2
        if bucket < live:
            bucket = (live + 31) // 32 * 32
        plan = StepPlan(seqs, item_sizes=self._item_sizes, pad_seqs=bucket)
        # the launch shapes of attention depend on how long the sequences may be: a graph
        # holds for contexts up to a bound (1,024, 4,096, ... or the capacity)
        bound = 1024
        while bound < plan.max_context:
            bound *= 4
        bound = min(bound, self.capacity)
        captured = self._captured.get((bucket, bound))
        if captured is None:
            captured = self._captured[(bucket, bound)] = _CapturedDecode(self.device)
        ctx = self._context(plan, captured.meta, captured.workspace, fixed_context=bound)
        if captured.graph is None:
            try:
                logits = self.model.forward(ctx)
                torch.cuda.synchronize(self.device)
                graph = torch.cuda.CUDAGraph()
                with torch.cuda.graph(graph):
                    captured.logits = self.model.forward(ctx)
            except BaseException:
                self._captured.pop((bucket, bound), None)   # nothing half-made is kept
                raise
            captured.graph = graph
        else:
            captured.graph.replay()
            self.graph_replays += 1
            logits = captured.logits
        # the captured step computes the logits of every row; hand out the wanted ones
        wanted = [index for index, seq in enumerate(seqs) if len(seq.want) > 0]
        if len(wanted) == live:
            return logits[:live]
        if not wanted:
            return logits[:0]
        return logits[torch.tensor(wanted, device=self.device)]
