"""Row metadata of one step: built on the host, uploaded in one copy.

A step runs the tokens it is given as one packed batch of rows.  Row-wise operations
never read the metadata; position encoding, cache stores and mixers do.  All of it lives
in one int32 buffer of named sections:

  longest[1]                           most tokens any sequence holds after the step
  tokens[N] row_pos[N] row_seq[N]      per row: token id, position, index of its sequence
  want_rows[W]                         rows whose logits are wanted
  seq_slot[B] seq_start[B] seq_count[B]  per sequence: cache slot (its row in every state
                                       table), tokens held before the step, tokens brought
  pages<g>[B, width]                   per key/value group: logical page -> physical page
  ...                                  whatever the model's parts plan for themselves

The last kind is the parts' own: a part with a `plan_step(plan)` method returns
`{section name: int32 array}` (work items of its kernels, for instance) and finds them
again on the device as `ctx.meta.section(name)`.  The engine does not know what they mean.

Padding (a decode batch of fixed size with fewer live sequences) carries row_seq = -1,
want_rows = -1 and seq_count = 0: kernels skip such rows and sequences.  Its seq_slot is the
spare slot, a row that every state table has beyond the rows of the real slots and that no
sequence ever owns: a kernel may read and write it without a branch.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Mapping, Optional, Sequence, Tuple

import numpy as np
import torch


@dataclass
class SeqStep:
    slot: int
    start: int            # tokens the slot holds before the step = position of tokens[0]
    tokens: Sequence[int]
    want: Sequence[int] = ()   # indices among `tokens` whose logits are wanted
    row0: int = 0

    @property
    def count(self) -> int:
        return len(self.tokens)


class StepPlan:
    """Host-side description of a step, independent of any device.

    `context_bound`: the launch shapes of this step must hold for sequences of up to that
    many tokens (a captured step is replayed for every context up to its bound); by default
    the longest sequence of the step itself."""

    def __init__(self, seqs: List[SeqStep], pad_seqs: Optional[int] = None,
                 context_bound: Optional[int] = None, spare_slot: int = -1):
        if not seqs:
            raise ValueError("a step needs at least one sequence")
        self.seqs = seqs
        row = 0
        for seq in seqs:
            if seq.count < 1:
                raise ValueError("every sequence of a step brings at least one token")
            seq.row0 = row
            row += seq.count
        self.n_live_rows = row
        self.n_live_seqs = len(seqs)
        self.decode = all(seq.count == 1 for seq in seqs)
        if pad_seqs is not None:
            if not self.decode:
                raise ValueError("only decode steps are padded to a fixed batch")
            if pad_seqs < len(seqs):
                raise ValueError("padded batch smaller than the live batch")
        self.n_seqs = pad_seqs if pad_seqs is not None else len(seqs)
        self.n_rows = self.n_seqs if pad_seqs is not None else row
        self.padded = pad_seqs is not None
        self.max_context = max(seq.start + seq.count for seq in seqs)
        self.context_bound = self.max_context if context_bound is None else int(context_bound)
        if self.context_bound < self.max_context:
            raise ValueError("the context bound of a step is below its longest sequence")

        n = self.n_rows
        self.tokens = np.zeros(n, dtype=np.int32)
        self.row_pos = np.zeros(n, dtype=np.int32)
        self.row_seq = np.full(n, -1, dtype=np.int32)
        self.seq_slot = np.full(self.n_seqs, spare_slot, dtype=np.int32)
        self.seq_start = np.zeros(self.n_seqs, dtype=np.int32)
        self.seq_count = np.zeros(self.n_seqs, dtype=np.int32)
        want_rows: List[int] = []
        if self.decode:                  # one row a sequence: whole arrays at once
            live = len(seqs)
            starts = np.fromiter((seq.start for seq in seqs), dtype=np.int32, count=live)
            self.tokens[:live] = np.fromiter((seq.tokens[0] for seq in seqs), dtype=np.int64,
                                             count=live)
            self.row_pos[:live] = starts
            self.row_seq[:live] = np.arange(live, dtype=np.int32)
            self.seq_slot[:live] = np.fromiter((seq.slot for seq in seqs), dtype=np.int32,
                                               count=live)
            self.seq_start[:live] = starts
            self.seq_count[:live] = 1
            for seq in seqs:
                for w in seq.want:
                    if w != 0:
                        raise ValueError(f"wanted place {w} is outside the 1 token given")
                    want_rows.append(seq.row0)
        else:
            for index, seq in enumerate(seqs):
                rows = slice(seq.row0, seq.row0 + seq.count)
                self.tokens[rows] = np.asarray(seq.tokens, dtype=np.int64)
                self.row_pos[rows] = np.arange(seq.start, seq.start + seq.count)
                self.row_seq[rows] = index
                self.seq_slot[index] = seq.slot
                self.seq_start[index] = seq.start
                self.seq_count[index] = seq.count
                for w in seq.want:
                    if not 0 <= w < seq.count:
                        raise ValueError(f"wanted place {w} is outside the {seq.count} tokens given")
                    want_rows.append(seq.row0 + w)
        self.n_want_live = len(want_rows)
        if self.padded:
            # a fixed-size decode batch asks for every row; dead rows are marked -1
            want_rows = [seq.row0 for seq in seqs] + [-1] * (self.n_seqs - len(seqs))
        self.want_rows = np.asarray(want_rows, dtype=np.int32)
        self.extra: Dict[str, np.ndarray] = {}

    def add_sections(self, sections: Mapping[str, np.ndarray]) -> None:
        """Sections that a part planned for itself.  Parts of one kind may plan the same
        section; it is kept once."""
        for name, array in sections.items():
            array = np.ascontiguousarray(array, dtype=np.int32)
            held = self.extra.get(name)
            if held is not None and not np.array_equal(held, array):
                raise ValueError(f"two parts planned different contents for the section '{name}'")
            self.extra[name] = array

    def sections(self, page_tables: Sequence[np.ndarray]) -> List[Tuple[str, np.ndarray]]:
        # `longest` comes first, so that its place never depends on the batch
        out = [("longest", np.asarray([self.max_context], dtype=np.int32)),
               ("tokens", self.tokens), ("row_pos", self.row_pos), ("row_seq", self.row_seq),
               ("want_rows", self.want_rows), ("seq_slot", self.seq_slot),
               ("seq_start", self.seq_start), ("seq_count", self.seq_count)]
        for index, table in enumerate(page_tables):
            out.append((f"pages{index}", table.reshape(-1)))
        for name, array in self.extra.items():
            if any(name == taken for taken, _ in out):
                raise ValueError(f"a part planned a section under the engine's name '{name}'")
            out.append((name, array.reshape(-1)))
        return out


class DeviceMeta:
    """The metadata buffer on the device and typed views into it."""

    def __init__(self, device):
        self.device = device
        self._device_buffer: Optional[torch.Tensor] = None
        self._host_buffer: Optional[torch.Tensor] = None
        self._views: Dict[str, torch.Tensor] = {}
        self._host_sections: Dict[str, np.ndarray] = {}
        self._table_widths: List[int] = []
        self.n_seqs = 0
        self.n_want = 0
        self._copied = None
        self._shape = None            # (name, size) of every section of the last upload
        self._offsets: List[int] = []
        self._total = 0
        # counts the layouts this buffer has had: while it stays the same, every view is
        # where it was (what a captured step relies on)
        self.generation = 0

    def _reserve(self, count: int) -> None:
        if self._device_buffer is None or self._device_buffer.numel() < count:
            self._copied = None
            size = max(count, 1024)
            self._device_buffer = torch.empty(size, dtype=torch.int32, device=self.device)
            pin = self.device is not None and torch.device(self.device).type == "cuda"
            self._host_buffer = torch.empty(size, dtype=torch.int32, pin_memory=pin)

    @property
    def capacity(self) -> int:
        """int32 elements the device buffer holds (0 before the first upload)."""
        return 0 if self._device_buffer is None else self._device_buffer.numel()

    def upload(self, plan: StepPlan, page_tables: Sequence[np.ndarray]) -> None:
        sections = plan.sections(page_tables)
        shape = tuple((name, array.size) for name, array in sections)
        if shape != self._shape or self._device_buffer is None:
            # another set of sections: lay them out anew (each starts at a multiple of 4 words)
            offsets, total = [], 0
            for _, size in shape:
                offsets.append(total)
                total += (size + 3) // 4 * 4
            self._reserve(total)
            self._views = {name: self._device_buffer[offset:offset + size]
                           for (name, size), offset in zip(shape, offsets)}
            self._shape, self._offsets, self._total = shape, offsets, total
            self.generation += 1
        if self._copied is not None:
            self._copied.synchronize()   # the last upload has left the staging buffer
        host = self._host_buffer.numpy()
        for (_, array), offset in zip(sections, self._offsets):
            host[offset:offset + array.size] = array.reshape(-1)
        total = self._total
        self._device_buffer[:total].copy_(self._host_buffer[:total], non_blocking=True)
        if self._device_buffer.is_cuda:
            if self._copied is None:
                self._copied = torch.cuda.Event()
            self._copied.record()
        self._host_sections = dict(sections)
        self._table_widths = [table.shape[1] for table in page_tables]
        self.n_seqs = plan.n_seqs
        self.n_want = int(plan.want_rows.size)

    # views ------------------------------------------------------------
    def section(self, name: str) -> torch.Tensor:
        """int32 view of a named section on the device."""
        try:
            return self._views[name]
        except KeyError:
            raise KeyError(f"the step's metadata holds no section '{name}'; "
                           f"it holds {sorted(self._views)}") from None

    def host_section(self, name: str) -> np.ndarray:
        """The host's copy of a section as the last upload held it (flat int32): what a part
        planned, for checks that must not wait for the device."""
        try:
            return self._host_sections[name]
        except KeyError:
            raise KeyError(f"the step's metadata holds no section '{name}'") from None

    longest = property(lambda self: self.section("longest"))
    tokens = property(lambda self: self.section("tokens"))
    row_pos = property(lambda self: self.section("row_pos"))
    row_seq = property(lambda self: self.section("row_seq"))
    want_rows = property(lambda self: self.section("want_rows"))
    seq_slot = property(lambda self: self.section("seq_slot"))
    seq_start = property(lambda self: self.section("seq_start"))
    seq_count = property(lambda self: self.section("seq_count"))

    def page_table(self, group: int) -> torch.Tensor:
        return self.section(f"pages{group}").view(self.n_seqs, self._table_widths[group])
