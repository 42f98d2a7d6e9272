"""ctypes bindings of the HIP kernel libraries.

Each function takes torch tensors that live on the GPU, checks what the kernel
assumes about them (device, dtype, contiguity, sizes) and launches on torch's
current stream.  A library is loaded (and compiled, when it is not yet) the first
time one of its functions is called.  There is no other implementation behind
these functions: if a library cannot be built or loaded the call raises.
"""
from __future__ import annotations

import ctypes
import functools
import os
from ctypes import c_float, c_int, c_longlong, c_ulonglong, c_void_p
from typing import Dict, Optional

import torch

from . import build

F32, BF16 = 0, 1
_DTYPE_CODE = {torch.float32: F32, torch.bfloat16: BF16}
PAGE_TOKENS = 64

_SIGNATURES = {
    "rowwise": {
        "ei_embed_gather": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_void_p],
        "ei_add_rmsnorm": [c_void_p, c_void_p, c_int, c_int, c_longlong, c_void_p, c_void_p,
                           c_float, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
        "ei_swiglu": [c_void_p, c_int, c_int, c_longlong, c_void_p, c_int, c_int, c_int, c_int,
                      c_void_p],
        "ei_sum_slices": [c_void_p, c_int, c_longlong, c_void_p, c_longlong, c_void_p],
        "ei_bias_rows": [c_void_p, c_void_p, c_longlong, c_int, c_int, c_void_p],
    },
    "rope_store": {
        "ei_qk_norm_rope_store": [c_void_p, c_int, c_int, c_longlong, c_void_p, c_void_p, c_float,
                                  c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                  c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                  c_void_p],
    },
    "attention_generic": {
        "ei_attn_heads_per_block": [c_int],
        "ei_attn_positions_per_item": [c_int],
        "ei_attention": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int,
                         c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int,
                         c_int, c_int, c_int, c_int, c_float, c_int, c_void_p],
    },
    "attention_mfma": {
        "ei_attn_decode_mfma_supported": [c_int, c_int],
        "ei_attn_prefill_mfma_positions": [c_int],
        "ei_attention_prefill_mfma": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                      c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int,
                                      c_int, c_int, c_float, c_int, c_int, c_void_p],
        "ei_attention_decode_mfma": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                     c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                     c_int, c_int, c_float, c_int, c_int, c_int, c_void_p,
                                     c_void_p],
        "ei_attention_decode_mfma_fused": [c_void_p, c_int, c_longlong, c_void_p, c_void_p, c_float,
                                           c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                           c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int,
                                           c_int, c_int, c_int, c_int, c_float, c_int, c_int,
                                           c_int, c_void_p, c_void_p],
    },
    "gemm_f32": {
        "ei_gemm_f32": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_longlong, c_longlong,
                        c_longlong, c_void_p],
    },
    "gemm_bf16": {
        "ei_skinny_gemm_splits": [c_int, c_int, c_int, c_int],
        "ei_gemm_bf16_skinny": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                c_void_p],
        "ei_gemm_bf16_skinny_packed": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                       c_void_p],
        "ei_gemm_bf16_skinny_gated": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                      c_void_p],
    },
    "sampling": {
        "ei_argmax": [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_longlong, c_void_p],
        "ei_argmax_partial_size": [c_int, c_int],
        "ei_argmax_static": [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p],
        "ei_argmax_static_prepare": [],
        "ei_sample": [c_void_p, c_int, c_int, c_float, c_float, c_int, c_ulonglong, c_void_p,
                      c_void_p, c_void_p, c_void_p, c_void_p, c_longlong, c_void_p],
        "ei_sample_scratch_size": [c_int, c_int],
    },
    "peaks": {
        "ei_stream_read": [c_void_p, c_longlong, c_int, c_void_p, c_void_p],
        "ei_mfma_loop": [c_int, c_int, c_int, c_void_p, c_void_p],
        "ei_empty_launches": [c_int, c_int, c_void_p],
    },
}

_loaded: Dict[str, ctypes.CDLL] = {}


class KernelError(RuntimeError):
    pass


def library(name: str) -> ctypes.CDLL:
    lib = _loaded.get(name)
    if lib is not None:
        return lib
    path = build.build_library(name)
    try:
        lib = ctypes.CDLL(str(path))
    except OSError as error:
        raise KernelError(f"cannot load kernel library {path}: {error}") from error
    for symbol, argtypes in _SIGNATURES.get(name, {}).items():
        function = getattr(lib, symbol)
        function.argtypes = argtypes
        function.restype = c_int
    lib.ei_last_error.restype = ctypes.c_char_p
    _loaded[name] = lib
    return lib


def loaded_libraries():
    return sorted(_loaded)


def prepare(names) -> None:
    """Compile the kernel libraries `names` that are not built yet, at the same time.  A
    model says which ones it will need when it is made; each is still loaded at its first use."""
    build.build_libraries([name for name in names if name not in _loaded])


launches = 0        # calls of kernel entry points so far (most launch one kernel, a few two)


def _check(lib, status: int, what: str) -> None:
    global launches
    launches += 1
    if status != 0:
        message = lib.ei_last_error().decode(errors="replace")
        raise KernelError(f"{what}: {message} (status {status})")


# torch's own shortcut to the current stream's handle (no Stream object is made); a step of
# few rows launches some 300 kernels and is bound by what each launch costs the host
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


@functools.lru_cache(maxsize=None)
def _compute_units(index: int) -> int:
    return int(torch.cuda.get_device_properties(index).multi_processor_count)


def compute_units(device=None) -> int:
    """Compute units of a device (the current one by default): 256 on an MI355X.  The one
    place on the Python side where launch plans take the chip's size from."""
    if device is None:
        index = torch.cuda.current_device()
    else:
        device = torch.device(device)
        index = torch.cuda.current_device() if device.index is None else device.index
    return _compute_units(index)


def _stream() -> int:
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _gpu(tensor: torch.Tensor, name: str, dtype=None) -> int:
    if not tensor.is_cuda:
        raise KernelError(f"{name} must live on the GPU")
    if not tensor.is_contiguous():
        raise KernelError(f"{name} must be contiguous")
    if dtype is not None and tensor.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, got {tensor.dtype}")
    return tensor.data_ptr()


def _code(tensor: torch.Tensor, name: str) -> int:
    try:
        return _DTYPE_CODE[tensor.dtype]
    except KeyError:
        raise KernelError(f"{name} has unsupported dtype {tensor.dtype}") from None


def _splits(tensor: torch.Tensor, rows: int, width: int, name: str):
    """(nsplit, stride) of a [rows, width] or [nsplit, rows, width] tensor."""
    if tensor.dim() == 2 and tuple(tensor.shape) == (rows, width):
        return 1, 0
    if tensor.dim() == 3 and tuple(tensor.shape[1:]) == (rows, width):
        return tensor.shape[0], rows * width
    raise KernelError(f"{name} must be [{rows}, {width}] or [splits, {rows}, {width}], "
                      f"got {list(tensor.shape)}")


# ---------------------------------------------------------------------------
def embed_gather(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor) -> None:
    lib = library("rowwise")
    n = ids.numel()
    vocab, hidden = table.shape
    if tuple(out.shape) != (n, hidden):
        raise KernelError(f"embed_gather: out must be [{n}, {hidden}], got {list(out.shape)}")
    status = lib.ei_embed_gather(_gpu(ids, "ids", torch.int32), _gpu(table, "table"),
                                 _code(table, "table"), _gpu(out, "out", torch.float32), n,
                                 hidden, vocab, _stream())
    _check(lib, status, "embed_gather")


def add_rmsnorm(residual: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor,
                eps: float, out: torch.Tensor, rows: Optional[torch.Tensor] = None,
                write_residual: bool = True) -> None:
    """residual [R, H] float32 (+= sum of delta splits, stored back unless told not
    to); out[i] = rmsnorm(residual[rows[i] if rows else i]) * weight."""
    lib = library("rowwise")
    total_rows, hidden = residual.shape
    n = out.shape[0]
    if out.dim() != 2 or out.shape[1] != hidden:
        raise KernelError(f"add_rmsnorm: out must be [*, {hidden}], got {list(out.shape)}")
    if weight.numel() != hidden:
        raise KernelError(f"add_rmsnorm: weight must have {hidden} elements")
    if rows is None and n != total_rows:
        raise KernelError("add_rmsnorm: out and residual row counts differ")
    if rows is not None and rows.numel() != n:
        raise KernelError("add_rmsnorm: rows and out row counts differ")
    nsplit, stride, delta_ptr, delta_code = 0, 0, None, F32
    if delta is not None:
        nsplit, stride = _splits(delta, total_rows, hidden, "delta")
        delta_ptr, delta_code = _gpu(delta, "delta"), _code(delta, "delta")
    status = lib.ei_add_rmsnorm(
        _gpu(residual, "residual", torch.float32), delta_ptr, delta_code, nsplit, stride,
        None if rows is None else _gpu(rows, "rows", torch.int32),
        _gpu(weight, "weight", torch.float32), float(eps), _gpu(out, "out"), _code(out, "out"), n,
        hidden, int(write_residual), _stream())
    _check(lib, status, "add_rmsnorm")


def swiglu(gate_up: torch.Tensor, out: torch.Tensor, strip: int = 0) -> None:
    """out = silu(gate) * up of [n, 2*inter] rows (or float32 slices of them).  strip = 0:
    the gate columns come first, then the up columns; strip > 0: `strip` gate columns,
    their `strip` up columns, and so on."""
    lib = library("rowwise")
    n, inter = out.shape
    nsplit, stride = _splits(gate_up, n, 2 * inter, "gate_up")
    status = lib.ei_swiglu(_gpu(gate_up, "gate_up"), _code(gate_up, "gate_up"), nsplit, stride,
                           _gpu(out, "out"), _code(out, "out"), n, inter, int(strip), _stream())
    _check(lib, status, "swiglu")


def sum_slices(slices: torch.Tensor, out: torch.Tensor) -> None:
    """out = slices.sum(0) for float32 [s, ...] in slice order."""
    lib = library("rowwise")
    n = out.numel()
    if slices.dim() < 2 or slices[0].numel() != n:
        raise KernelError("sum_slices: out must have the shape of one slice")
    status = lib.ei_sum_slices(_gpu(slices, "slices", torch.float32), slices.shape[0], n,
                               _gpu(out, "out", torch.float32), n, _stream())
    _check(lib, status, "sum_slices")


def bias_rows(bias: torch.Tensor, out: torch.Tensor, accumulate: bool) -> None:
    """out[r, :] = bias (accumulate False) or out[r, :] + bias, float32 [rows, width]."""
    lib = library("rowwise")
    if out.dim() != 2 or bias.numel() != out.shape[1]:
        raise KernelError(f"bias_rows: bias of {bias.numel()} for rows {list(out.shape)}")
    status = lib.ei_bias_rows(_gpu(bias, "bias", torch.float32), _gpu(out, "out", torch.float32),
                              out.shape[0], out.shape[1], int(accumulate), _stream())
    _check(lib, status, "bias_rows")


def _rotated_width(rope_table, head_dim: int, what: str) -> int:
    """The width of a rotation table [positions, R]: R/2 cosines, then R/2 sines, for the
    pairs (i, i + R/2) of a head's first R <= head_dim elements; the rest pass unrotated."""
    if rope_table is None:
        return head_dim
    if rope_table.dim() != 2 or rope_table.shape[1] % 2 or not 2 <= rope_table.shape[1] <= head_dim:
        raise KernelError(f"{what}: the rotation table must be [positions, R] with R even and at "
                          f"most head_dim = {head_dim}, got {list(rope_table.shape)}")
    return rope_table.shape[1]


def qk_norm_rope_store(qkv, q_norm_w, k_norm_w, eps, rope_table, row_pos, row_seq, page_table,
                       q_out, k_pages, v_pages, n_heads, n_kv_heads, head_dim,
                       write_cache=True) -> None:
    """Per-head RMSNorm of queries and keys (weights or None), rotation by `rope_table`
    (float32 [positions, R], R <= head_dim; or None), queries to `q_out`, keys and values to
    their cache pages."""
    lib = library("rope_store")
    n = q_out.shape[0]
    width = (n_heads + 2 * n_kv_heads) * head_dim
    nsplit, stride = _splits(qkv, n, width, "qkv")
    if tuple(q_out.shape) != (n, n_heads * head_dim):
        raise KernelError("qk_norm_rope_store: q_out has the wrong shape")
    if row_pos.numel() < n or row_seq.numel() < n:
        raise KernelError("qk_norm_rope_store: row metadata shorter than the rows")
    rot_dim = _rotated_width(rope_table, head_dim, "qk_norm_rope_store")
    if write_cache:
        expect = (n_kv_heads, PAGE_TOKENS, head_dim)
        if tuple(k_pages.shape[1:]) != expect or tuple(v_pages.shape) != tuple(k_pages.shape):
            raise KernelError(f"qk_norm_rope_store: pages must be [*, {expect}]")
        if k_pages.dtype != q_out.dtype or v_pages.dtype != q_out.dtype:
            raise KernelError("qk_norm_rope_store: cache and q_out dtypes differ")
    status = lib.ei_qk_norm_rope_store(
        _gpu(qkv, "qkv"), _code(qkv, "qkv"), nsplit, stride,
        None if q_norm_w is None else _gpu(q_norm_w, "q_norm", torch.float32),
        None if k_norm_w is None else _gpu(k_norm_w, "k_norm", torch.float32), float(eps),
        None if rope_table is None else _gpu(rope_table, "rope_table", torch.float32), rot_dim,
        _gpu(row_pos, "row_pos", torch.int32), _gpu(row_seq, "row_seq", torch.int32),
        _gpu(page_table, "page_table", torch.int32), page_table.shape[-1],
        _gpu(q_out, "q_out"), _gpu(k_pages, "k_pages") if write_cache else None,
        _gpu(v_pages, "v_pages") if write_cache else None, _code(q_out, "q_out"), n, n_heads,
        n_kv_heads, head_dim, int(write_cache), _stream())
    _check(lib, status, "qk_norm_rope_store")


def attention_heads_per_block(group: int) -> int:
    return library("attention_generic").ei_attn_heads_per_block(group)


def attention_positions_per_item(group: int) -> int:
    return library("attention_generic").ei_attn_positions_per_item(group)


def attention(q, k_pages, v_pages, item_seq, item_row0, item_npos, n_items, row_pos, row_seq,
              page_table, out, n_heads, n_kv_heads, head_dim, window=None, scale=None,
              n_splits=1, part_o=None, part_ml=None) -> None:
    """Generic causal attention over the paged cache (see attention_generic.hip)."""
    lib = library("attention_generic")
    n = q.shape[0]
    if tuple(q.shape) != (n, n_heads * head_dim) or tuple(out.shape) != tuple(q.shape):
        raise KernelError("attention: q and out must be [rows, heads * head_dim]")
    expect = (n_kv_heads, PAGE_TOKENS, head_dim)
    if tuple(k_pages.shape[1:]) != expect or tuple(v_pages.shape) != tuple(k_pages.shape):
        raise KernelError(f"attention: pages must be [*, {expect}]")
    if not (q.dtype == k_pages.dtype == v_pages.dtype == out.dtype):
        raise KernelError("attention: q, cache and out dtypes differ")
    if item_seq.numel() < n_items or item_row0.numel() < n_items or item_npos.numel() < n_items:
        raise KernelError("attention: work item arrays shorter than n_items")
    if n_splits > 1:
        need_o = n * n_heads * n_splits * head_dim
        if part_o is None or part_ml is None or part_o.numel() < need_o \
                or part_ml.numel() < n * n_heads * n_splits * 2:
            raise KernelError("attention: split scratch missing or too small")
    if scale is None:
        scale = head_dim ** -0.5
    status = lib.ei_attention(
        _gpu(q, "q"), _gpu(k_pages, "k_pages"), _gpu(v_pages, "v_pages"), _code(q, "q"),
        _gpu(item_seq, "item_seq", torch.int32), _gpu(item_row0, "item_row0", torch.int32),
        _gpu(item_npos, "item_npos", torch.int32), n_items, _gpu(row_pos, "row_pos", torch.int32),
        _gpu(row_seq, "row_seq", torch.int32), _gpu(page_table, "page_table", torch.int32),
        page_table.shape[-1], _gpu(out, "out"),
        None if part_o is None else _gpu(part_o, "part_o", torch.float32),
        None if part_ml is None else _gpu(part_ml, "part_ml", torch.float32), n, n_heads,
        n_kv_heads, head_dim, int(window or 0), float(scale), n_splits, _stream())
    _check(lib, status, "attention")


MFMA_HEAD_DIMS = (64, 128)


def attention_decode_mfma_supported(head_dim: int, group: int) -> bool:
    """Whether the matrix-core attention kernels take this head size (asked without
    loading their library, so that models which do not need it never compile it)."""
    return head_dim in MFMA_HEAD_DIMS and group >= 1


def attention_prefill_mfma_heads(group: int) -> int:
    """Query heads of a kv group that one block of the matrix-core prefill kernel takes: the
    largest of 4, 2, 1 that divides the group."""
    return 4 if group % 4 == 0 else (2 if group % 2 == 0 else 1)


def attention_prefill_mfma_positions(group: int, key_ways: int = 1) -> int:
    """Positions of a sequence per work item of the matrix-core prefill kernel: a block of 8
    waves holds 4, 2 or 1 heads of a kv group, each wave 32 positions of one head; with
    `key_ways` = 2 two waves share the keys of every page for the same positions, so an item
    is half as long (0: the group has no such form)."""
    heads = attention_prefill_mfma_heads(group)
    if key_ways not in (1, 2) or heads * key_ways > 8:
        return 0
    return 32 * (8 // (heads * key_ways))


def attention_prefill_mfma(q, k_pages, v_pages, item_seq, item_row0, item_npos, n_items, row_pos,
                           page_table, out, n_heads, n_kv_heads, head_dim, window=None,
                           scale=None, key_ways=1, pair_items=True, largest_item=None) -> None:
    """bfloat16 prefill attention on the matrix cores; an item holds up to
    `attention_prefill_mfma_positions(group, key_ways)` positions of one sequence.
    pair_items: with enough items a block may take item i and then item n_items - 1 - i
    (equal work a block where the items are those of one prompt, longest first).
    largest_item: the most positions any item holds, from the host's copy of the list (the
    kernel gives a block's waves fixed rows of an item and would leave the rows of a larger
    one out); None: looked up from `item_npos` on the device, which waits for the device."""
    lib = library("attention_mfma")
    n = q.shape[0]
    capacity = attention_prefill_mfma_positions(n_heads // max(1, n_kv_heads), key_ways)
    if capacity == 0:
        raise KernelError(f"attention_prefill: no form with key_ways = {key_ways} for groups of "
                          f"{n_heads // max(1, n_kv_heads)} heads")
    if largest_item is None:
        largest_item = int(item_npos[:n_items].max().item())
    if not 0 <= int(largest_item) <= capacity:
        raise KernelError(f"attention_prefill: an item of {largest_item} positions; a block "
                          f"takes at most {capacity} with key_ways = {key_ways}")
    if tuple(q.shape) != (n, n_heads * head_dim) or tuple(out.shape) != tuple(q.shape):
        raise KernelError("attention_prefill: q and out must be [rows, heads * head_dim]")
    expect = (n_kv_heads, PAGE_TOKENS, head_dim)
    if tuple(k_pages.shape[1:]) != expect or tuple(v_pages.shape) != tuple(k_pages.shape):
        raise KernelError(f"attention_prefill: pages must be [*, {expect}]")
    if item_seq.numel() < n_items or item_row0.numel() < n_items or item_npos.numel() < n_items:
        raise KernelError("attention_prefill: work item arrays shorter than n_items")
    if scale is None:
        scale = head_dim ** -0.5
    status = lib.ei_attention_prefill_mfma(
        _gpu(q, "q", torch.bfloat16), _gpu(k_pages, "k_pages", torch.bfloat16),
        _gpu(v_pages, "v_pages", torch.bfloat16), _gpu(item_seq, "item_seq", torch.int32),
        _gpu(item_row0, "item_row0", torch.int32), _gpu(item_npos, "item_npos", torch.int32),
        n_items, _gpu(row_pos, "row_pos", torch.int32),
        _gpu(page_table, "page_table", torch.int32), page_table.shape[-1],
        _gpu(out, "out", torch.bfloat16), n_heads, n_kv_heads, head_dim, int(window or 0),
        float(scale), int(key_ways), int(bool(pair_items)), _stream())
    _check(lib, status, "attention_prefill")


class DecodeProjection:
    """What `attention_decode_mfma` needs to make queries, key and value itself: the fused
    projection as float32 partial sums [slices, rows, (heads + 2 kv heads) * head_dim], the
    per-head RMSNorm weights (float32 [head_dim], or None), their eps, the rotation table
    (float32 [positions, R] with R <= head_dim, or None), and whether the position's key and value are
    stored in the pages."""

    def __init__(self, qkv, q_norm_w, k_norm_w, eps, rope_table, write_cache):
        self.qkv, self.q_norm_w, self.k_norm_w = qkv, q_norm_w, k_norm_w
        self.eps, self.rope_table, self.write_cache = eps, rope_table, write_cache


def attention_decode_mfma(q, k_pages, v_pages, row_pos, row_seq, page_table, out, n_heads,
                          n_kv_heads, head_dim, window=None, scale=None, n_splits=1, part_o=None,
                          part_ml=None, waves=4, longest=None, heads=0) -> None:
    """bfloat16 decode attention on the matrix cores: one query row per sequence.  `waves`
    (4, 8 or 16) of a block share its key range tile by tile; more suit fewer sequences (few
    blocks), whose ranges then need fewer slices or none.  `heads` (a power of two, or 0 for
    as many as the block size allows): query heads of a kv group that one block takes; fewer
    give more, lighter blocks.  `longest` (int32 [1] on the
    device): the most tokens a sequence of the step holds; every sequence's range is then
    cut into slices of the longest one's share, so that unequal lengths give equal blocks.
    `q` is the queries [rows, heads * head_dim], or a `DecodeProjection`: the kernel then does
    the work of `qk_norm_rope_store` for its rows as well."""
    lib = library("attention_mfma")
    n = out.shape[0]
    fused = isinstance(q, DecodeProjection)
    if tuple(out.shape) != (n, n_heads * head_dim) or (not fused and tuple(q.shape) != tuple(out.shape)):
        raise KernelError("attention_decode: q and out must be [rows, heads * head_dim]")
    if fused:
        width = (n_heads + 2 * n_kv_heads) * head_dim
        if q.qkv.dim() != 3 or tuple(q.qkv.shape[1:]) != (n, width):
            raise KernelError(f"attention_decode: the projection must be [slices, {n}, {width}], "
                              f"got {list(q.qkv.shape)}")
        for name in ("q_norm_w", "k_norm_w"):
            weight = getattr(q, name)
            if weight is not None and weight.numel() != head_dim:
                raise KernelError(f"attention_decode: {name} must have {head_dim} elements")
        rot_dim = _rotated_width(q.rope_table, head_dim, "attention_decode")
    expect = (n_kv_heads, PAGE_TOKENS, head_dim)
    if tuple(k_pages.shape[1:]) != expect or tuple(v_pages.shape) != tuple(k_pages.shape):
        raise KernelError(f"attention_decode: pages must be [*, {expect}]")
    if row_pos.numel() < n or row_seq.numel() < n or page_table.shape[0] < n:
        raise KernelError("attention_decode: row metadata shorter than the rows")
    if n_splits > 1:
        if part_o is None or part_ml is None or part_o.numel() < n * n_heads * n_splits * head_dim \
                or part_ml.numel() < n * n_heads * n_splits * 2:
            raise KernelError("attention_decode: split scratch missing or too small")
    if scale is None:
        scale = head_dim ** -0.5
    if fused:
        def opt(tensor, name):
            return None if tensor is None else _gpu(tensor, name, torch.float32)
        status = lib.ei_attention_decode_mfma_fused(
            _gpu(q.qkv, "qkv", torch.float32), q.qkv.shape[0], n * width,
            opt(q.q_norm_w, "q_norm"), opt(q.k_norm_w, "k_norm"), float(q.eps),
            opt(q.rope_table, "rope_table"), rot_dim, int(bool(q.write_cache)),
            _gpu(k_pages, "k_pages", torch.bfloat16), _gpu(v_pages, "v_pages", torch.bfloat16),
            _gpu(row_pos, "row_pos", torch.int32), _gpu(row_seq, "row_seq", torch.int32),
            _gpu(page_table, "page_table", torch.int32), page_table.shape[-1],
            _gpu(out, "out", torch.bfloat16),
            None if part_o is None else _gpu(part_o, "part_o", torch.float32),
            None if part_ml is None else _gpu(part_ml, "part_ml", torch.float32), n, n_heads,
            n_kv_heads, head_dim, int(window or 0), float(scale), n_splits, int(waves),
            int(heads), None if longest is None else _gpu(longest, "longest", torch.int32),
            _stream())
        _check(lib, status, "attention_decode")
        return
    status = lib.ei_attention_decode_mfma(
        _gpu(q, "q", torch.bfloat16), _gpu(k_pages, "k_pages", torch.bfloat16),
        _gpu(v_pages, "v_pages", torch.bfloat16), _gpu(row_pos, "row_pos", torch.int32),
        _gpu(row_seq, "row_seq", torch.int32), _gpu(page_table, "page_table", torch.int32),
        page_table.shape[-1], _gpu(out, "out", torch.bfloat16),
        None if part_o is None else _gpu(part_o, "part_o", torch.float32),
        None if part_ml is None else _gpu(part_ml, "part_ml", torch.float32), n, n_heads,
        n_kv_heads, head_dim, int(window or 0), float(scale), n_splits, int(waves), int(heads),
        None if longest is None else _gpu(longest, "longest", torch.int32), _stream())
    _check(lib, status, "attention_decode")


def gemm_f32(a: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> None:
    """out[M, N] = a[M, K] . w[N, K]^T in float32."""
    lib = library("gemm_f32")
    m, k = a.shape
    n = w.shape[0]
    if w.shape[1] != k or tuple(out.shape) != (m, n):
        raise KernelError(f"gemm_f32: shapes {list(a.shape)} x {list(w.shape)}^T -> "
                          f"{list(out.shape)} do not agree")
    status = lib.ei_gemm_f32(_gpu(a, "a", torch.float32), _gpu(w, "w", torch.float32),
                             _gpu(out, "out", torch.float32), m, n, k, k, k, n, _stream())
    _check(lib, status, "gemm_f32")


def argmax_partial_size(rows: int, vocab: int) -> int:
    """float32 elements of scratch with which `argmax` searches a wide vocabulary with many
    blocks a row (0: one block a row is used anyway)."""
    return 2 * library("sampling").ei_argmax_partial_size(rows, vocab)


def argmax(logits: torch.Tensor, tokens: torch.Tensor, probabilities=None, partial=None) -> None:
    lib = library("sampling")
    rows, vocab = logits.shape
    if tokens.numel() < rows:
        raise KernelError("argmax: tokens shorter than the rows")
    status = lib.ei_argmax(_gpu(logits, "logits", torch.float32), rows, vocab,
                           _gpu(tokens, "tokens", torch.int32),
                           None if probabilities is None
                           else _gpu(probabilities, "probabilities", torch.float32),
                           None if partial is None else _gpu(partial, "partial", torch.float32),
                           0 if partial is None else partial.numel() // 2, _stream())
    _check(lib, status, "argmax")


ARGMAX_STATIC_MAX_PARTIALS = 65536


def argmax_static(logits: torch.Tensor, tokens: torch.Tensor, probabilities=None) -> None:
    """`argmax` without a buffer from the caller and without any allocation: the partial results
    of a wide vocabulary live in a device array of the library (at most 65536 pairs of row and
    chunk of 4096 logits; larger requests are refused).  Calls that overlap on one GPU race."""
    lib = library("sampling")
    rows, vocab = logits.shape
    if tokens.numel() < rows:
        raise KernelError("argmax_static: tokens shorter than the rows")
    status = lib.ei_argmax_static(_gpu(logits, "logits", torch.float32), rows, vocab,
                                  _gpu(tokens, "tokens", torch.int32),
                                  None if probabilities is None
                                  else _gpu(probabilities, "probabilities", torch.float32),
                                  _stream())
    _check(lib, status, "argmax_static")


def sample_scratch_size(rows: int, vocab: int) -> int:
    """int32 elements of zeroed scratch that `sample` takes for many blocks a row (0: none)."""
    return library("sampling").ei_sample_scratch_size(rows, vocab)


def sample(logits, temperature, top_p, top_k, seed, streams, counters, tokens,
           probabilities=None, scratch=None) -> None:
    """`scratch` (int32, zero before its first use, see `sample_scratch_size`) lets a wide
    vocabulary be searched by many blocks a row; the tokens are the same without it."""
    lib = library("sampling")
    rows, vocab = logits.shape
    if tokens.numel() < rows or streams.numel() < rows or counters.numel() < rows:
        raise KernelError("sample: per-row arrays shorter than the rows")
    status = lib.ei_sample(_gpu(logits, "logits", torch.float32), rows, vocab, float(temperature),
                           float(top_p), int(top_k), int(seed) & (2**64 - 1),
                           _gpu(streams, "streams", torch.int32),
                           _gpu(counters, "counters", torch.int32),
                           _gpu(tokens, "tokens", torch.int32),
                           None if probabilities is None
                           else _gpu(probabilities, "probabilities", torch.float32),
                           None if scratch is None else _gpu(scratch, "scratch", torch.int32),
                           0 if scratch is None else scratch.numel(), _stream())
    _check(lib, status, "sample")


# ---------------------------------------------------------------------------
def has_skinny_gemm() -> bool:
    return "gemm_bf16" in build.available_libraries()


_SKINNY_MAX_SPLITS = int(os.environ.get("EDGE_INFER_SKINNY_MAX_SPLITS", "0"))   # 0: no cap


def skinny_gemm_splits(rows: int, n: int, k: int) -> int:
    """K slices the weight-streaming product uses for [rows, k] x [n, k]^T."""
    return library("gemm_bf16").ei_skinny_gemm_splits(rows, n, k, _SKINNY_MAX_SPLITS)


# most rows for which the weight-streaming product is taken instead of the library's
SKINNY_ROWS = int(os.environ.get("EDGE_INFER_SKINNY_ROWS", "256"))
if not 1 <= SKINNY_ROWS <= 256:
    raise KernelError("EDGE_INFER_SKINNY_ROWS must lie in 1..256")


def skinny_gemm_ok(rows: int, k: int) -> bool:
    return rows <= SKINNY_ROWS and k % 8 == 0


def gemm_bf16_skinny(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> None:
    """out[s, m, n] = sum over the s-th slice of K of x[m, :] . w[n, :] (float32), for at
    most 256 rows; out.shape[0] says into how many slices K is cut."""
    lib = library("gemm_bf16")
    m, k = x.shape
    n = w.shape[0]
    if out.dim() != 3 or w.shape[1] != k or tuple(out.shape[1:]) != (m, n):
        raise KernelError(f"gemm_bf16_skinny: shapes {list(x.shape)} x {list(w.shape)}^T -> "
                          f"{list(out.shape)} do not agree")
    status = lib.ei_gemm_bf16_skinny(_gpu(x, "x", torch.bfloat16), _gpu(w, "w", torch.bfloat16),
                                     _gpu(out, "out", torch.float32), m, n, k, out.shape[0],
                                     _stream())
    _check(lib, status, "gemm_bf16_skinny")


def pack_weight(w: torch.Tensor) -> torch.Tensor:
    """The streaming copy of a bfloat16 matrix [n, k] for `gemm_bf16_skinny_packed`:
    [8*ceil(k/256), ceil(n/16), 4, 16, 8] where element (kt, strip, c, r, e) is
    w[strip*16 + r, kt*32 + c*8 + e], zero outside the matrix (k is padded to whole
    K-tiles of the kernel, 256 wide).  Made once when the weights
    are loaded; a data movement, no arithmetic."""
    if w.dtype != torch.bfloat16 or w.dim() != 2:
        raise KernelError("pack_weight: a bfloat16 matrix is expected")
    n, k = w.shape
    strips, tiles = (n + 15) // 16, 8 * ((k + 255) // 256)
    if (strips * 16, tiles * 32) != (n, k):
        padded = torch.zeros((strips * 16, tiles * 32), dtype=w.dtype, device=w.device)
        padded[:n, :k] = w
        w = padded
    return w.view(strips, 16, tiles, 4, 8).permute(2, 0, 3, 1, 4).contiguous()


def gemm_bf16_skinny_packed(x: torch.Tensor, packed: torch.Tensor, n: int,
                            out: torch.Tensor) -> None:
    """`gemm_bf16_skinny` with the weight given as `pack_weight(w)` of a matrix [n, k]."""
    lib = library("gemm_bf16")
    m, k = x.shape
    if (out.dim() != 3 or tuple(out.shape[1:]) != (m, n) or packed.dim() != 5
            or tuple(packed.shape) != (8 * ((k + 255) // 256), (n + 15) // 16, 4, 16, 8)):
        raise KernelError(f"gemm_bf16_skinny_packed: shapes {list(x.shape)} x packed "
                          f"{list(packed.shape)} (n = {n}) -> {list(out.shape)} do not agree")
    status = lib.ei_gemm_bf16_skinny_packed(_gpu(x, "x", torch.bfloat16),
                                            _gpu(packed, "packed", torch.bfloat16),
                                            _gpu(out, "out", torch.float32), m, n, k,
                                            out.shape[0], _stream())
    _check(lib, status, "gemm_bf16_skinny_packed")


GATE_STRIP = 16     # gate rows and up rows alternate in strips of this many (one MFMA tile)


def gemm_bf16_skinny_gated(x: torch.Tensor, w: torch.Tensor, n: int, act: torch.Tensor,
                           packed: bool) -> None:
    """act[m, i] = silu(x[m] . gate_i) * (x[m] . up_i) for a weight [n, k] whose rows are, in
    strips of 16, the gate rows of 16 outputs followed by their up rows; `w` is that matrix or
    (packed) its `pack_weight` copy.  For at most 256 rows; K is not sliced, so it pays where
    `skinny_gemm_splits` is 1."""
    lib = library("gemm_bf16")
    m, k = x.shape
    if tuple(act.shape) != (m, n // 2) or n % (2 * GATE_STRIP):
        raise KernelError(f"gemm_bf16_skinny_gated: {list(x.shape)} x [{n}, {k}] -> "
                          f"{list(act.shape)} do not agree")
    expect = (8 * ((k + 255) // 256), (n + 15) // 16, 4, 16, 8) if packed else (n, k)
    if tuple(w.shape) != expect:
        raise KernelError(f"gemm_bf16_skinny_gated: weight {list(w.shape)}, expected {list(expect)}")
    status = lib.ei_gemm_bf16_skinny_gated(_gpu(x, "x", torch.bfloat16), _gpu(w, "w", torch.bfloat16),
                                           _gpu(act, "act", torch.bfloat16), m, n, k, int(packed),
                                           _stream())
    _check(lib, status, "gemm_bf16_skinny_gated")


# ---------------------------------------------------------------------------
def stream_read(data: torch.Tensor, sink: torch.Tensor, blocks: int = 4096) -> None:
    """Read every byte of `data` once with a plain kernel (a yardstick for memory-bound steps)."""
    lib = library("peaks")
    nbytes = data.numel() * data.element_size()
    status = lib.ei_stream_read(_gpu(data, "data"), nbytes - nbytes % 16, int(blocks),
                                _gpu(sink, "sink", torch.int32), _stream())
    _check(lib, status, "stream_read")


MFMA_LOOP_FLOPS = 8 * 16 * 16 * 32 * 2      # per wave and iteration of `mfma_loop`


def mfma_loop(iters: int, blocks: int, sink: torch.Tensor, wide: bool = False) -> None:
    """`blocks` x 4 waves multiply bfloat16 tiles on registers: `iters` rounds of 8 products of
    16x16x32, or (wide) of 4 products of 32x32x16; `MFMA_LOOP_FLOPS` a wave and round."""
    lib = library("peaks")
    status = lib.ei_mfma_loop(int(iters), int(blocks), int(wide),
                              _gpu(sink, "sink", torch.float32), _stream())
    _check(lib, status, "mfma_loop")


def empty_launches(count: int, blocks: int = 256) -> None:
    """`count` launches of a kernel that does nothing (`blocks` blocks of one wave), one after
    the other on the current stream: the floor under a chain of that many dependent kernels."""
    lib = library("peaks")
    _check(lib, lib.ei_empty_launches(int(count), int(blocks), _stream()), "empty_launches")
