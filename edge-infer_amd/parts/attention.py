"""Causal grouped-query attention over the paged key/value cache.

x -> fused q/k/v projection -> (optional) per-head RMSNorm of q and k -> rotary
encoding -> keys and values stored in the cache -> attention over the cache ->
output projection.  The order follows the reference's decoder,
runtime/include/execution/decoder.hpp:121-158.  Three separate checkpoint matrices
become one [Q + 2 KV, H] matrix when the part is built: each output element is
still the same dot product.  Each projection may have a bias
(runtime/include/models/qwen3_model.hpp:386-395: taken if the checkpoint holds it).
"""
from __future__ import annotations

import functools
import os

import numpy as np
import torch

from ..csrc import lib
from ..csrc.lib import PAGE_TOKENS
from ..weights.loader import ParamSpec
from .base import KVRequest
from .linear import Linear

# EDGE_INFER_FUSED_DECODE=0: decode steps launch the norm-rotate-store kernel of their own
# instead of letting the matrix-core decode kernel do that work
FUSED_DECODE = os.environ.get("EDGE_INFER_FUSED_DECODE", "1") != "0"


# What the matrix-core decode kernel costs, measured on an MI355X: a wave walks a tile of 16
# keys of head size 128 in 1.9 us (other head sizes in proportion: a tile's bytes are what it
# waits for); merging slices costs 4.5 us and 0.1 us a slice.
TILE_US_128, MERGE_US, MERGE_SLICE_US = 1.9, 4.5, 0.1
WAVES_A_UNIT = 16       # waves of this kernel that a compute unit holds at once
MAX_SLICES = 32
MAX_LAUNCH_PLANS = 512  # decode launch shapes a part remembers


@functools.lru_cache(maxsize=512)
def _decode_items(n_seqs: int, live: int):
    """One work item a sequence, [3, n_seqs]: sequence (-1: padding), its row, one position."""
    seq = np.full(n_seqs, -1, dtype=np.int32)
    seq[:live] = np.arange(live)
    npos = np.zeros(n_seqs, dtype=np.int32)
    npos[:live] = 1
    items = np.stack([seq, np.arange(n_seqs, dtype=np.int32), npos])
    items.setflags(write=False)
    return items


class Attention:
    @property
    def capture_safe(self):
        """Launches only this library's kernels and allocates nothing per step, as long as
        its products do."""
        return self.qkv.capture_safe and self.o.capture_safe

    @property
    def capture_rows(self):
        return min(self.qkv.capture_rows, self.o.capture_rows)

    @classmethod
    def parameters(cls, spec, hidden):
        params = {
            "q_proj.weight": ParamSpec((spec.q_width, hidden)),
            "k_proj.weight": ParamSpec((spec.kv_width, hidden)),
            "v_proj.weight": ParamSpec((spec.kv_width, hidden)),
            "o_proj.weight": ParamSpec((hidden, spec.q_width)),
            "q_proj.bias": ParamSpec((spec.q_width,), optional=True),
            "k_proj.bias": ParamSpec((spec.kv_width,), optional=True),
            "v_proj.bias": ParamSpec((spec.kv_width,), optional=True),
            "o_proj.bias": ParamSpec((hidden,), optional=True),
        }
        if spec.qk_norm:
            params["q_norm.weight"] = ParamSpec((spec.head_dim,), init="norm")
            params["k_norm.weight"] = ParamSpec((spec.head_dim,), init="norm")
        return params

    @classmethod
    def cache_request(cls, spec):
        return KVRequest(n_kv_heads=spec.n_kv_heads, head_dim=spec.head_dim, window=spec.window)

    @classmethod
    def kernel_libraries(cls, spec, dtype):
        """What this part will run, so that a model can have it compiled ahead of its first
        step."""
        group = spec.n_heads // max(1, spec.n_kv_heads)
        fast = dtype == torch.bfloat16 and lib.attention_decode_mfma_supported(spec.head_dim, group)
        return ("rope_store", "attention_mfma" if fast else "attention_generic",
                *Linear.kernel_libraries(dtype))

    @classmethod
    def check(cls, spec):
        if spec.n_heads % spec.n_kv_heads:
            raise ValueError("attention: n_heads must be a multiple of n_kv_heads")
        if spec.head_dim % 16 or not 16 <= spec.head_dim <= 256:
            raise ValueError("attention: head_dim must be a multiple of 16 between 16 and 256, "
                             f"got {spec.head_dim}")
        if spec.window is not None and spec.window < 1:
            raise ValueError("attention: a window must be at least 1")

    def __init__(self, spec, hidden, params, dtype, device, positions):
        self.check(spec)
        self.spec = spec
        self.hidden = hidden
        self.dtype = dtype
        fused = torch.cat([params["q_proj.weight"], params["k_proj.weight"],
                           params["v_proj.weight"]], dim=0)
        names = ("q_proj", "k_proj", "v_proj")
        fused_bias = None
        if any(f"{name}.bias" in params for name in names):   # absent ones count as zero
            fused_bias = torch.cat([
                params[f"{name}.bias"] if f"{name}.bias" in params
                else params[f"{name}.weight"].new_zeros(params[f"{name}.weight"].shape[0])
                for name in names])
        self.qkv = Linear(fused, dtype, device, bias=fused_bias)
        self.o = Linear(params["o_proj.weight"], dtype, device, bias=params.get("o_proj.bias"))
        self.q_norm = self.k_norm = None
        if spec.qk_norm:
            self.q_norm = params["q_norm.weight"].to(device=device, dtype=torch.float32).contiguous()
            self.k_norm = params["k_norm.weight"].to(device=device, dtype=torch.float32).contiguous()
        self.position = positions(spec.position)   # shared table object
        self.group = spec.n_heads // spec.n_kv_heads
        self.scale = spec.scale if spec.scale is not None else spec.head_dim ** -0.5
        # the matrix-core kernels take bfloat16 with head sizes 64 and 128; every other
        # case runs the generic kernel
        self.matrix_cores = (dtype == torch.bfloat16 and
                            lib.attention_decode_mfma_supported(spec.head_dim, self.group))
        self.compute_units = lib.compute_units(device)     # the chip's size, for launch plans
        self._decode_launches = {}     # (sequences, pages of context) -> decode_launch's answer

    # the number of positions of one sequence that a prefill work item covers
    def positions_per_item(self, key_ways: int = 1):
        if self.matrix_cores:          # the matrix-core prefill kernel takes the same cases
            return lib.attention_prefill_mfma_positions(self.group, key_ways)
        return lib.attention_positions_per_item(self.group) if key_ways == 1 else 0

    def prefill_key_ways(self, counts) -> int:
        """1 or 2: how many waves share the keys of a page for the same rows in the prompt
        step whose sequences bring `counts` tokens.  A step that gives every compute unit
        about one block (one prompt of 2,048 tokens of the 8B shape: 256, whose walks are 1 to
        32 pages long) takes items half as long, and with them twice the blocks, which the
        kernel then pairs, a long one with a short one; with more blocks than that the
        hardware balances them, and a wave that takes every key of a page for its rows does
        less beside its products (measured, one prompt of the 8B shape: 2,048 tokens 60
        against 71 us, 3,072 tokens 147 against 105)."""
        if not self.matrix_cores or self.positions_per_item(2) == 0:
            return 1
        size = self.positions_per_item(1)
        heads = lib.attention_prefill_mfma_heads(self.group)
        items = sum((count + size - 1) // size for count in counts)
        blocks = items * (self.group // heads) * self.spec.n_kv_heads
        return 2 if 4 * blocks <= 5 * self.compute_units else 1

    @property
    def plan_key(self):
        """Attention parts with equal keys plan the same sections."""
        return ("attention", self.positions_per_item(), self.group, self.spec.n_kv_heads)

    def _items_section(self, key_ways: int = 1):
        return f"attention.items{self.positions_per_item(key_ways)}"

    def plan_step(self, plan):
        """The work items of this step's attention kernels, as one int32 section [3, items]:
        sequence (-1: padding), first row, positions.  A prompt step cuts every sequence's
        rows into items of `positions_per_item`, the ones with the longest key range first
        (they take longest, so they start first); a decode step has one item a sequence."""
        if plan.decode:
            return {"attention.decode_items": _decode_items(plan.n_seqs, plan.n_live_seqs)}
        key_ways = self.prefill_key_ways([seq.count for seq in plan.seqs])
        size = self.positions_per_item(key_ways)
        items = []
        for index, seq in enumerate(plan.seqs):
            for p0 in range(0, seq.count, size):
                npos = min(size, seq.count - p0)
                items.append((-(seq.start + p0 + npos), index, seq.row0 + p0, npos))
        items.sort()
        return {self._items_section(key_ways): np.asarray([item[1:] for item in items],
                                                          dtype=np.int32).T.copy()}

    @staticmethod
    def _items(ctx, name):
        section = ctx.meta.section(name)
        count = section.numel() // 3
        return section[:count], section[count:2 * count], section[2 * count:], count

    def decode_launch(self, n_seqs: int, context: int):
        """(slices of the key range, waves a block, query heads of a group a block takes) of
        a decode step over `n_seqs` sequences of up to `context` tokens.  A slice is the same
        number of pages for every sequence.  A layer with a window reads at most the window's
        keys (and the rest of the page they begin in), so its slices are sized for those.

        Matrix-core kernel, up to as many (sequence, kv head) pairs as the chip has compute
        units: blocks of 16 waves, a tile of 16 keys per wave at a time, and as many slices as
        shorten a wave's walk by more than the merge kernel costs, while all blocks still fit
        the chip at once; if they then leave compute units empty, a block takes fewer heads (2
        or 1 instead of 4), as long as every block still has a unit of its own: the keys are
        fetched once more per block, from the L2, and each block has less to do per tile.  Up
        to twice as many pairs: blocks of 8 waves, no slices.  More pairs, and the generic
        kernel: blocks of 4 waves and enough slices to put about two blocks on each compute
        unit, never more than there are pages."""
        if self.spec.window is not None:
            context = min(context, self.spec.window + PAGE_TOKENS - 1)
        pages = max(1, (context + PAGE_TOKENS - 1) // PAGE_TOKENS)
        n_kv_heads = self.spec.n_kv_heads
        units = self.compute_units
        if self.matrix_cores:
            # a block of 16 waves takes at most 4 query heads of a group: larger groups have
            # several blocks per pair
            pairs = n_seqs * n_kv_heads * ((self.group + 3) // 4)
            if pairs <= units:
                tile_us = TILE_US_128 * self.spec.head_dim / 128
                tiles = (context + 15) // 16
                best, best_cost = 1, tile_us * ((tiles + 15) // 16)
                slices = 2
                while (slices <= min(pages, MAX_SLICES)
                       and pairs * 16 * slices <= units * WAVES_A_UNIT):
                    cost = (tile_us * ((tiles + 16 * slices - 1) // (16 * slices)) + MERGE_US
                            + MERGE_SLICE_US * slices)
                    if cost < best_cost:
                        best, best_cost = slices, cost
                    slices *= 2
                heads = min(4, 1 << (self.group.bit_length() - 1))
                while heads > 1:
                    blocks = n_seqs * n_kv_heads * best * -(-self.group // (heads // 2))
                    if blocks > units:
                        break
                    heads //= 2
                return best, 16, heads
            # up to twice as many pairs of at most 8 heads: blocks of 8 waves fill the chip's
            # wave slots once without slices (measured 1 to 3 % ahead of 4 waves at 32 to 64
            # sequences)
            pairs = n_seqs * n_kv_heads * ((self.group + 7) // 8)
            if pairs <= 2 * units:
                return 1, 8, 0
        blocks = n_seqs * n_kv_heads
        wanted = (2 * units + blocks - 1) // blocks
        return max(1, min(wanted, pages, MAX_SLICES)), 4, 0

    def _decode_launch_for(self, n_seqs: int, context: int):
        """`decode_launch`, remembered per (sequences, pages of context): a step that is not
        replayed from a graph asks in every layer and for every length, and the answer changes
        with the pages at most."""
        pages = (context + PAGE_TOKENS - 1) // PAGE_TOKENS
        launch = self._decode_launches.get((n_seqs, pages))
        if launch is None:
            if len(self._decode_launches) >= MAX_LAUNCH_PLANS:
                self._decode_launches.clear()
            launch = self._decode_launches[(n_seqs, pages)] = \
                self.decode_launch(n_seqs, pages * PAGE_TOKENS)
        return launch

    def forward(self, ctx, x, entry):
        spec = self.spec
        n = x.shape[0]
        meta = ctx.meta
        group_index, k_pages, v_pages = ctx.cache.kv(entry.cache)
        page_table = meta.page_table(group_index)
        qkv = self.qkv.forward(ctx, x, "attn.qkv")
        if (ctx.decode and self.matrix_cores and FUSED_DECODE and qkv.dim() == 3
                and qkv.dtype == torch.float32):
            # the decode kernel norms, rotates and stores for its rows itself: one launch less
            q = lib.DecodeProjection(qkv, self.q_norm, self.k_norm, spec.qk_norm_eps,
                                     self.position.table, entry.writes_cache)
        else:
            q = ctx.buffer("attn.q", (n, spec.q_width))
            lib.qk_norm_rope_store(
                qkv, self.q_norm, self.k_norm, spec.qk_norm_eps, self.position.table,
                meta.row_pos, meta.row_seq, page_table, q, k_pages, v_pages, spec.n_heads,
                spec.n_kv_heads, spec.head_dim, write_cache=entry.writes_cache)
        out = ctx.buffer("attn.out", (n, spec.q_width))
        part_o = part_ml = None
        if ctx.decode:
            splits, waves, heads = self._decode_launch_for(ctx.n_seqs, ctx.context_bound)
            if splits > 1:
                part_o = ctx.buffer("attn.part_o", (n * spec.n_heads * splits * spec.head_dim,),
                                    torch.float32)
                part_ml = ctx.buffer("attn.part_ml", (n * spec.n_heads * splits * 2,),
                                     torch.float32)
            if self.matrix_cores:
                lib.attention_decode_mfma(q, k_pages, v_pages, meta.row_pos, meta.row_seq,
                                          page_table, out, spec.n_heads, spec.n_kv_heads,
                                          spec.head_dim, window=spec.window, scale=self.scale,
                                          n_splits=splits, part_o=part_o, part_ml=part_ml,
                                          waves=waves, longest=meta.longest, heads=heads)
            else:
                item_seq, item_row0, item_npos, n_items = self._items(ctx, "attention.decode_items")
                lib.attention(q, k_pages, v_pages, item_seq, item_row0, item_npos, n_items,
                              meta.row_pos, meta.row_seq, page_table, out, spec.n_heads,
                              spec.n_kv_heads, spec.head_dim, window=spec.window,
                              scale=self.scale, n_splits=splits, part_o=part_o, part_ml=part_ml)
        else:
            key_ways = self.prefill_key_ways([seq.count for seq in ctx.sequences])
            section = self._items_section(key_ways)
            item_seq, item_row0, item_npos, n_items = self._items(ctx, section)
            if self.matrix_cores:
                # the largest item of the list as the host planned it: the kernel's blocks
                # hold a fixed number of rows and are told how many that must cover
                largest = ctx.notes.get(section)
                if largest is None:
                    largest = ctx.notes[section] = int(ctx.meta.host_section(section)[2 * n_items:].max())
                lib.attention_prefill_mfma(q, k_pages, v_pages, item_seq, item_row0, item_npos,
                                           n_items, meta.row_pos, page_table, out, spec.n_heads,
                                           spec.n_kv_heads, spec.head_dim, window=spec.window,
                                           scale=self.scale, key_ways=key_ways,
                                           pair_items=len({(seq.start, seq.count) for seq in ctx.sequences}) == 1,
                                           largest_item=largest)
            else:
                lib.attention(q, k_pages, v_pages, item_seq, item_row0, item_npos, n_items,
                              meta.row_pos, meta.row_seq, page_table, out, spec.n_heads,
                              spec.n_kv_heads, spec.head_dim, window=spec.window,
                              scale=self.scale)
        ctx.release(qkv, None if isinstance(q, lib.DecodeProjection) else q, part_o, part_ml)
        delta = self.o.forward(ctx, out, "attn.o")
        ctx.release(out)
        return delta
