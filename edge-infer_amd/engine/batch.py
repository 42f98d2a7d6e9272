"""Row metadata of one step: built on the host, uploaded in one copy.

A step runs the tokens it is given as one packed batch of rows.  Only position
encoding, cache store and attention read the metadata; every other operation is
row-wise.  All of it lives in one int32 buffer:

  longest[1] tokens[N] row_pos[N] row_seq[N] want_rows[W]
  per attention item size: item_seq[I] item_row0[I] item_npos[I]   (prefill)
  decode items: item_seq[B] item_row0[B] item_npos[B]             (decode)
  per key/value group: page_table[B, width]

Padding rows (a fixed-size decode batch with fewer live sequences) carry
row_seq = -1, want_rows = -1 and items with seq = -1: kernels skip them.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

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
    """Host-side description of a step, independent of any device."""

    def __init__(self, seqs: List[SeqStep], item_sizes: Sequence[int] = (),
                 pad_seqs: Optional[int] = None):
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

        n = self.n_rows
        self.tokens = np.zeros(n, dtype=np.int32)
        self.row_pos = np.zeros(n, dtype=np.int32)
        self.row_seq = np.full(n, -1, dtype=np.int32)
        want_rows: List[int] = []
        for index, seq in enumerate(seqs):
            rows = slice(seq.row0, seq.row0 + seq.count)
            self.tokens[rows] = np.asarray(seq.tokens, dtype=np.int64)
            self.row_pos[rows] = np.arange(seq.start, seq.start + seq.count)
            self.row_seq[rows] = index
            for w in seq.want:
                if not 0 <= w < seq.count:
                    raise ValueError(f"wanted place {w} is outside the {seq.count} tokens given")
                want_rows.append(seq.row0 + w)
        self.n_want_live = len(want_rows)
        if self.padded:
            # a fixed-size decode batch asks for every row; dead rows are marked -1
            want_rows = [seq.row0 for seq in seqs] + [-1] * (self.n_seqs - len(seqs))
        self.want_rows = np.asarray(want_rows, dtype=np.int32)
        self.item_sizes = tuple(sorted(set(item_sizes)))
        self.items: Dict[int, Tuple[np.ndarray, np.ndarray, np.ndarray]] = {}
        if not self.decode:
            for size in self.item_sizes:
                self.items[size] = self._prefill_items(size)

    def _prefill_items(self, size: int):
        """(sequence, first row, positions) of every work item, the ones with the longest
        key range first: they take longest, so they should start first."""
        items = []
        for index, seq in enumerate(self.seqs):
            for p0 in range(0, seq.count, size):
                npos = min(size, seq.count - p0)
                items.append((-(seq.start + p0 + npos), index, seq.row0 + p0, npos))
        items.sort()
        return (np.asarray([i[1] for i in items], dtype=np.int32),
                np.asarray([i[2] for i in items], dtype=np.int32),
                np.asarray([i[3] for i in items], dtype=np.int32))

    def decode_items(self):
        seq = np.full(self.n_seqs, -1, dtype=np.int32)
        seq[:self.n_live_seqs] = np.arange(self.n_live_seqs)
        row0 = np.arange(self.n_seqs, dtype=np.int32)
        npos = np.zeros(self.n_seqs, dtype=np.int32)
        npos[:self.n_live_seqs] = 1
        return seq, row0, npos

    def sections(self, page_tables: Sequence[np.ndarray]) -> List[Tuple[str, np.ndarray]]:
        # longest: the most tokens any sequence holds after this step (decode attention sizes
        # its slices by it); first, so that its place never depends on the batch
        out = [("longest", np.asarray([self.max_context], dtype=np.int32)),
               ("tokens", self.tokens), ("row_pos", self.row_pos), ("row_seq", self.row_seq),
               ("want_rows", self.want_rows)]
        if self.decode:
            seq, row0, npos = self.decode_items()
            out += [("ditem_seq", seq), ("ditem_row0", row0), ("ditem_npos", npos)]
        for size, (seq, row0, npos) in self.items.items():
            out += [(f"item{size}_seq", seq), (f"item{size}_row0", row0),
                    (f"item{size}_npos", npos)]
        for index, table in enumerate(page_tables):
            out.append((f"pages{index}", table.reshape(-1)))
        return out


class DeviceMeta:
    """The metadata buffer on the device and typed views into it."""

    def __init__(self, device):
        self.device = device
        self._device_buffer: Optional[torch.Tensor] = None
        self._host_buffer: Optional[torch.Tensor] = None
        self._views: Dict[str, torch.Tensor] = {}
        self._table_widths: List[int] = []
        self.n_seqs = 0
        self.n_want = 0
        self._copied = None

    def _reserve(self, count: int) -> None:
        if self._device_buffer is None or self._device_buffer.numel() < count:
            size = max(count, 1024)
            self._device_buffer = torch.empty(size, dtype=torch.int32, device=self.device)
            pin = self.device is not None and torch.device(self.device).type == "cuda"
            self._host_buffer = torch.empty(size, dtype=torch.int32, pin_memory=pin)

    def upload(self, plan: StepPlan, page_tables: Sequence[np.ndarray]) -> None:
        sections = plan.sections(page_tables)
        offsets, total = [], 0
        for _, array in sections:
            offsets.append(total)
            total += (array.size + 3) // 4 * 4
        self._reserve(total)
        if self._copied is not None:
            self._copied.synchronize()   # the last upload has left the staging buffer
        host = self._host_buffer.numpy()
        self._views = {}
        for (name, array), offset in zip(sections, offsets):
            host[offset:offset + array.size] = array
            self._views[name] = self._device_buffer[offset:offset + array.size]
        self._device_buffer[:total].copy_(self._host_buffer[:total], non_blocking=True)
        if self._device_buffer.is_cuda:
            self._copied = torch.cuda.Event()
            self._copied.record()
        self._table_widths = [table.shape[1] for table in page_tables]
        self.n_seqs = plan.n_seqs
        self.n_want = int(plan.want_rows.size)

    # views ------------------------------------------------------------
    @property
    def longest(self):
        return self._views["longest"]

    @property
    def tokens(self):
        return self._views["tokens"]

    @property
    def row_pos(self):
        return self._views["row_pos"]

    @property
    def row_seq(self):
        return self._views["row_seq"]

    @property
    def want_rows(self):
        return self._views["want_rows"]

    def page_table(self, group: int) -> torch.Tensor:
        return self._views[f"pages{group}"].view(self.n_seqs, self._table_widths[group])

    def decode_items(self):
        return (self._views["ditem_seq"], self._views["ditem_row0"], self._views["ditem_npos"],
                self.n_seqs)

    def prefill_items(self, size: int):
        seq = self._views[f"item{size}_seq"]
        return seq, self._views[f"item{size}_row0"], self._views[f"item{size}_npos"], seq.numel()
