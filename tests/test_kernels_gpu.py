"""Each HIP kernel alone against its plain float64 reference, at sizes other than
the engine's tiny models (odd widths, head sizes 16..256, group ratios 1..20)."""
import math

import numpy as np
import pytest
import torch

import plain_qwen3 as plain

pytestmark = pytest.mark.gpu

DEV = "cuda"
PAGE = 64


@pytest.fixture(scope="module")
def lib():
    from edge_infer_amd.csrc import lib as kernels
    return kernels


def tol(dtype):
    return 2e-6 if dtype == torch.float32 else 1.2e-2   # bfloat16: 2^-8 relative, some slack


def close(actual, expected, dtype, scale=None):
    actual, expected = actual.double().cpu(), expected.double().cpu()
    scale = expected.abs().max().item() if scale is None else scale
    err = (actual - expected).abs().max().item()
    assert err <= tol(dtype) * max(scale, 1e-30), f"max error {err:.3e}, scale {scale:.3e}"


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embed_gather(lib, dtype):
    V, H = 381, 200
    table = torch.randn(V, H, device=DEV).to(dtype)
    ids = torch.tensor([0, 380, 17, 17, 200], dtype=torch.int32, device=DEV)
    out = torch.full((5, H), float("nan"), device=DEV)
    lib.embed_gather(ids, table, out)
    assert torch.equal(out.cpu(), plain.embedding(ids.cpu().tolist(), table.cpu()).float())


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H", [200, 4096 + 24])
def test_add_rmsnorm(lib, out_dtype, H):
    N, eps = 7, 1e-5
    residual = torch.randn(N, H, device=DEV)
    weight = (1 + 0.1 * torch.randn(H, device=DEV))
    # no delta
    out = torch.empty(N, H, device=DEV, dtype=out_dtype)
    lib.add_rmsnorm(residual, None, weight, eps, out)
    close(out, plain.rms_norm(residual.cpu(), weight.cpu(), eps), out_dtype)
    # float32 delta in three splits: residual is updated, the norm sees the sum
    delta = torch.randn(3, N, H, device=DEV)
    before = residual.clone()
    lib.add_rmsnorm(residual, delta, weight, eps, out)
    total = before.double().cpu() + delta.double().cpu().sum(0)
    close(residual, total, torch.float32)
    close(out, plain.rms_norm(total, weight.cpu(), eps), out_dtype)
    # bfloat16 delta
    if out_dtype == torch.bfloat16:
        d16 = torch.randn(N, H, device=DEV).to(torch.bfloat16)
        before = residual.clone()
        lib.add_rmsnorm(residual, d16, weight, eps, out)
        close(residual, before.double().cpu() + d16.double().cpu(), torch.float32)
    # gathered rows, one of them padding; the residual is left alone
    rows = torch.tensor([4, -1, 0], dtype=torch.int32, device=DEV)
    before = residual.clone()
    delta2 = torch.randn(1, N, H, device=DEV)
    out3 = torch.full((3, H), 7.0, device=DEV, dtype=out_dtype)
    lib.add_rmsnorm(residual, delta2, weight, eps, out3, rows=rows, write_residual=False)
    assert torch.equal(residual, before)
    expect = plain.rms_norm(before.double().cpu() + delta2[0].double().cpu(), weight.cpu(), eps)
    close(out3[0], expect[4], out_dtype)
    close(out3[2], expect[0], out_dtype)
    assert (out3[1] == 0).all()


def test_rms_norm_reference_vector_on_the_gpu(lib):
    """operators/tests/operators_cuda_bf16_contract_test.cu:235-284, float32 part (2e-6)."""
    n = 128
    x = torch.tensor([-0.8 + (i % 7) * 0.25 for i in range(n)], device=DEV).reshape(1, n)
    w = torch.tensor([0.63 + (i % 5) * 0.17 for i in range(n)], device=DEV)
    out = torch.empty(1, n, device=DEV)
    lib.add_rmsnorm(x, None, w, 1e-6, out)
    inv = 1.0 / math.sqrt(float((x.double() ** 2).sum()) / n + 1e-6)
    assert (out.double() - x.double() * inv * w.double()).abs().max().item() < 2e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("I", [200, 100, 4096 + 8])
def test_swiglu(lib, dtype, I):
    N = 5
    gate_up = torch.randn(2, N, 2 * I, device=DEV) * 3
    gate_up[0, 0, 0], gate_up[1, 0, 0] = -60.0, -28.0      # the reference's -88 tail case
    out = torch.empty(N, I, device=DEV, dtype=dtype)
    lib.swiglu(gate_up, out)
    total = gate_up.double().cpu().sum(0)
    close(out, plain.swiglu(total[:, :I], total[:, I:]), dtype)
    assert torch.isfinite(out.float()).all()
    if dtype == torch.bfloat16:
        one = gate_up[0].to(dtype).contiguous()
        lib.swiglu(one, out)
        close(out, plain.swiglu(one.double().cpu()[:, :I], one.double().cpu()[:, I:]), dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("I,strip", [(208, 16), (96, 4), (4096 + 16, 16)])
def test_swiglu_with_gate_and_up_in_strips(lib, dtype, I, strip):
    """Rows laid out as `strip` gate columns, their `strip` up columns, and so on (the
    layout the gated feed-forward gives its fused matrix)."""
    N = 3
    gate = torch.randn(2, N, I, device=DEV) * 3
    up = torch.randn(2, N, I, device=DEV)
    mixed = torch.stack([gate.reshape(2, N, I // strip, strip),
                         up.reshape(2, N, I // strip, strip)], dim=3).reshape(2, N, 2 * I)
    out = torch.empty(N, I, device=DEV, dtype=dtype)
    lib.swiglu(mixed.contiguous(), out, strip)
    close(out, plain.swiglu(gate.double().cpu().sum(0), up.double().cpu().sum(0)), dtype)
    with pytest.raises(lib.KernelError, match="divide"):
        lib.swiglu(mixed.contiguous(), out, 7)


@pytest.mark.parametrize("shape", [(1, 381, 96), (5, 64, 200), (70, 130, 33), (130, 257, 512),
                                   (8, 100, 1000), (40, 4100, 1028), (6, 77, 260), (200, 300, 264)])
def test_gemm_f32(lib, shape):
    """Few rows take the weight-streaming kernel (K in fours), many the tiled one; both sum
    every output over k in ascending order, so a row gives the same bits alone, among up to
    8 rows and among many."""
    M, N, K = shape
    a = torch.randn(M, K, device=DEV)
    w = torch.randn(N, K, device=DEV)
    out = torch.empty(M, N, device=DEV)
    lib.gemm_f32(a, w, out)
    close(out, plain.linear(a.cpu(), w.cpu()), torch.float32, scale=math.sqrt(K) * 4)
    # a row's result does not depend on its neighbours
    single = torch.empty(1, N, device=DEV)
    lib.gemm_f32(a[M // 2:M // 2 + 1].contiguous(), w, single)
    assert torch.equal(single[0], out[M // 2])
    for rows in (3, 5, 8):
        if rows <= M:
            few = torch.full((rows, N), float("nan"), device=DEV)
            lib.gemm_f32(a[:rows].contiguous(), w, few)
            assert torch.equal(few, out[:rows]), rows


# ---------------------------------------------------------------------------
def rope_table(D, theta, positions):
    angle = plain.rope_angles(list(range(positions)), D, theta)
    return torch.cat([torch.cos(angle), torch.sin(angle)], dim=1).float().to(DEV)


class PagedCache:
    """A cache with a scrambled page table, filled with NaN so that a stray read or a
    missed mask shows."""

    def __init__(self, lengths, nkv, D, dtype, seed=0, extra_pages=3):
        self.lengths = lengths
        need = [(n + PAGE - 1) // PAGE for n in lengths]
        self.n_pages = sum(need) + extra_pages
        order = np.random.RandomState(seed).permutation(self.n_pages)
        self.width = max(need) + 1
        self.table = np.full((len(lengths), self.width), -1, dtype=np.int32)
        at = 0
        for b, n in enumerate(need):
            self.table[b, :n] = order[at:at + n]
            at += n
        self.k = torch.full((self.n_pages, nkv, PAGE, D), float("nan"), device=DEV, dtype=dtype)
        self.v = torch.full((self.n_pages, nkv, PAGE, D), float("nan"), device=DEV, dtype=dtype)
        self.table_dev = torch.from_numpy(self.table).to(DEV)

    def put(self, b, k, v):
        """k, v: [len, nkv, D] for sequence b."""
        for start in range(0, k.shape[0], PAGE):
            page = self.table[b, start // PAGE]
            n = min(PAGE, k.shape[0] - start)
            self.k[page, :, :n] = k[start:start + n].transpose(0, 1).to(self.k.dtype)
            self.v[page, :, :n] = v[start:start + n].transpose(0, 1).to(self.v.dtype)

    def get(self, b, n):
        pages = self.table[b, :(n + PAGE - 1) // PAGE]
        k = torch.cat([self.k[p].transpose(0, 1) for p in pages])[:n]
        v = torch.cat([self.v[p].transpose(0, 1) for p in pages])[:n]
        return k, v


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("form", ["slices", "stored"])
@pytest.mark.parametrize("nq,nkv,D,use_norm,use_rope", [(6, 3, 48, True, True), (4, 4, 16, False, True),
                                                        (8, 1, 256, True, False), (5, 1, 128, True, True),
                                                        (3, 1, 20, True, True), (2, 2, 8, True, True)])
def test_qk_norm_rope_store(lib, dtype, form, nq, nkv, D, use_norm, use_rope):
    """Input as float32 partial sums (two slices, the decode form) or as one tensor of the
    storage type (the prefill form); head sizes that take the vector kernel (multiples of
    8, with idle lanes at 48) and one that takes the scalar kernel (20)."""
    theta, eps = 1e6, 1e-5
    lengths_before = [70, 0, 130]
    counts = [3, 5, 1]
    N = sum(counts)
    cache = PagedCache([a + c for a, c in zip(lengths_before, counts)], nkv, D, dtype, seed=1)
    sentinel_k, sentinel_v = cache.k.clone(), cache.v.clone()
    width = (nq + 2 * nkv) * D
    qkv = torch.randn(2, N, width, device=DEV)
    if form == "stored":
        qkv = qkv[0].to(dtype).unsqueeze(0)
    row_pos, row_seq = [], []
    for b, (start, count) in enumerate(zip(lengths_before, counts)):
        row_pos += list(range(start, start + count))
        row_seq += [b] * count
    row_pos[5], row_seq[5] = 0, -1         # a padding row in the middle is skipped
    pos = torch.tensor(row_pos, dtype=torch.int32, device=DEV)
    seq = torch.tensor(row_seq, dtype=torch.int32, device=DEV)
    qn = (1 + 0.1 * torch.randn(D, device=DEV)) if use_norm else None
    kn = (1 + 0.1 * torch.randn(D, device=DEV)) if use_norm else None
    table = rope_table(D, theta, 256) if use_rope else None
    q_out = torch.full((N, nq * D), float("nan"), device=DEV, dtype=dtype)
    lib.qk_norm_rope_store(qkv if form == "slices" else qkv[0], qn, kn, eps, table, pos, seq,
                           cache.table_dev, q_out, cache.k, cache.v, nq, nkv, D)
    total = qkv.double().cpu().sum(0)
    q = total[:, :nq * D].reshape(N, nq, D)
    k = total[:, nq * D:(nq + nkv) * D].reshape(N, nkv, D)
    v = total[:, (nq + nkv) * D:].reshape(N, nkv, D)
    if use_norm:
        q = plain.rms_norm(q, qn.cpu(), eps)
        k = plain.rms_norm(k, kn.cpu(), eps)
    if use_rope:
        q = plain.rope(q, row_pos, theta)
        k = plain.rope(k, row_pos, theta)
    touched_k = torch.zeros_like(cache.k, dtype=torch.bool)
    for r in range(N):
        if row_seq[r] < 0:
            assert torch.isnan(q_out[r].float()).all()
            continue
        close(q_out[r].reshape(nq, D), q[r], dtype, scale=q.abs().max().item())
        page = cache.table[row_seq[r], row_pos[r] // PAGE]
        close(cache.k[page, :, row_pos[r] % PAGE], k[r], dtype, scale=k.abs().max().item())
        close(cache.v[page, :, row_pos[r] % PAGE], v[r], dtype, scale=v.abs().max().item())
        touched_k[page, :, row_pos[r] % PAGE] = True
    # nothing else in the cache changed (NaN sentinels compare by bits)
    same_k = cache.k.view(torch.int16 if dtype == torch.bfloat16 else torch.int32) == \
        sentinel_k.view(torch.int16 if dtype == torch.bfloat16 else torch.int32)
    same_v = cache.v.view(torch.int16 if dtype == torch.bfloat16 else torch.int32) == \
        sentinel_v.view(torch.int16 if dtype == torch.bfloat16 else torch.int32)
    assert same_k[~touched_k].all() and same_v[~touched_k].all()
    assert not same_k[touched_k].any()
    # a layer that only reads another layer's cache writes nothing
    again_k = cache.k.clone()
    lib.qk_norm_rope_store(qkv, qn, kn, eps, table, pos, seq, cache.table_dev, q_out, cache.k,
                           cache.v, nq, nkv, D, write_cache=False)
    assert torch.equal(again_k.view(torch.uint8), cache.k.view(torch.uint8))


def small_angle_vector_through_the_kernel(lib, dtype):
    D = 128
    table = rope_table(D, 1e6, 21)
    basis = torch.zeros(21, 3 * D, device=DEV)
    basis[:, :D // 2] = 1.0
    cache = PagedCache([21], 1, D, dtype)
    pos = torch.arange(21, dtype=torch.int32, device=DEV)
    seq = torch.zeros(21, dtype=torch.int32, device=DEV)
    q_out = torch.empty(21, D, device=DEV, dtype=dtype)
    lib.qk_norm_rope_store(basis, None, None, 1e-6, table, pos, seq, cache.table_dev, q_out,
                           cache.k, cache.v, 1, 1, D)
    return q_out.double().cpu()


def test_rope_small_angle_reference_vector_on_the_gpu(lib):
    """operators/tests/operators_cuda_bf16_contract_test.cu:372-415."""
    out = small_angle_vector_through_the_kernel(lib, torch.float32)
    for p in range(21):
        for i in range(64):
            angle = p / (1e6 ** (2.0 * i / 128))
            assert abs(out[p, i].item() - math.cos(angle)) < 2e-6
            assert abs(out[p, i + 64].item() - math.sin(angle)) < 2e-6


# ---------------------------------------------------------------------------
def items_for(lib, starts, counts, group, per=None):
    per = per or lib.attention_positions_per_item(group)
    seq, row0, npos, row = [], [], [], 0
    for b, count in enumerate(counts):
        for p0 in range(0, count, per):
            seq.append(b)
            row0.append(row + p0)
            npos.append(min(per, count - p0))
        row += count
    as_dev = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    return as_dev(seq), as_dev(row0), as_dev(npos), len(seq)


def run_attention(lib, dtype, nq, nkv, D, starts, counts, window=None, splits=1, seed=0,
                  boost=None, kernel="generic", waves=4, longest=None, key_ways=1,
                  pair_items=True, heads=0):
    """Fill a paged cache with random keys and values, run the kernel for the last
    `counts[b]` positions of each sequence, return (kernel output, plain output)."""
    torch.manual_seed(seed)
    lengths = [s + c for s, c in zip(starts, counts)]
    cache = PagedCache(lengths, nkv, D, dtype, seed=seed)
    N = sum(counts)
    q = torch.randn(N, nq, D, device=DEV).to(dtype)
    ks, vs = [], []
    for b, n in enumerate(lengths):
        k = torch.randn(n, nkv, D, device=DEV).to(dtype)
        v = torch.randn(n, nkv, D, device=DEV).to(dtype)
        if boost is not None and boost[0] == b:
            _, key_index, row_index, factor = boost
            k[key_index] = (q[row_index, :nkv].float() * factor / D).to(dtype)
        cache.put(b, k, v)
        ks.append(k)
        vs.append(v)
    row_pos, row_seq = [], []
    for b, (s, c) in enumerate(zip(starts, counts)):
        row_pos += list(range(s, s + c))
        row_seq += [b] * c
    pos = torch.tensor(row_pos, dtype=torch.int32, device=DEV)
    seq = torch.tensor(row_seq, dtype=torch.int32, device=DEV)
    group = nq // nkv
    per = lib.attention_prefill_mfma_positions(group, key_ways) if kernel == "prefill_mfma" else None
    item_seq, item_row0, item_npos, n_items = items_for(lib, starts, counts, group, per)
    out = torch.full((N, nq * D), float("nan"), device=DEV, dtype=dtype)
    part_o = part_ml = None
    if splits > 1:
        part_o = torch.full((N * nq * splits * D,), float("nan"), device=DEV)
        part_ml = torch.full((N * nq * splits * 2,), float("nan"), device=DEV)
    if kernel == "prefill_mfma":
        lib.attention_prefill_mfma(q.reshape(N, nq * D), cache.k, cache.v, item_seq, item_row0,
                                   item_npos, n_items, pos, cache.table_dev, out, nq, nkv, D,
                                   window=window, key_ways=key_ways, pair_items=pair_items)
    elif kernel == "decode_mfma":
        lib.attention_decode_mfma(q.reshape(N, nq * D), cache.k, cache.v, pos, seq,
                                  cache.table_dev, out, nq, nkv, D, window=window,
                                  n_splits=splits, part_o=part_o, part_ml=part_ml, waves=waves,
                                  heads=heads,
                                  longest=None if longest is None else torch.tensor(
                                      [longest], dtype=torch.int32, device=DEV))
    else:
        lib.attention(q.reshape(N, nq * D), cache.k, cache.v, item_seq, item_row0, item_npos,
                      n_items, pos, seq, cache.table_dev, out, nq, nkv, D, window=window,
                      n_splits=splits, part_o=part_o, part_ml=part_ml)
    expected = torch.empty(N, nq, D, dtype=torch.float64)
    row = 0
    for b, (s, c) in enumerate(zip(starts, counts)):
        n = s + c
        full_q = torch.zeros(n, nq, D, dtype=torch.float64)
        full_q[s:] = q[row:row + c].double().cpu()
        ref = plain.attention(full_q, ks[b].double().cpu(), vs[b].double().cpu(), window=window)
        expected[row:row + c] = ref[s:]
        row += c
    return out.reshape(N, nq, D), expected


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nkv,D", [(4, 2, 16), (6, 3, 48), (8, 1, 32), (4, 4, 128),
                                      (20, 1, 64), (3, 1, 256), (32, 8, 128)])
def test_attention_prefill_unequal_sequences(lib, dtype, nq, nkv, D):
    """Whole prompts of unequal lengths (1, a page boundary, beyond one page) and a
    chunk appended to 70 cached tokens, in one launch."""
    out, expected = run_attention(lib, dtype, nq, nkv, D, starts=[0, 0, 0, 70, 0],
                                  counts=[1, 64, 131, 9, 17])
    close(out, expected, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nkv,D,splits", [(4, 2, 16, 1), (8, 1, 32, 3), (32, 8, 128, 4),
                                             (6, 3, 48, 8), (20, 1, 64, 2)])
def test_attention_decode_with_splits(lib, dtype, nq, nkv, D, splits):
    """One position per sequence; lengths around the split and page boundaries (the
    reference sweeps 1, 2, 8, 9, 16, 17, ... across its own branch thresholds,
    operators/tests/operators_cuda_attention_precision_test.cu:183)."""
    starts = [0, 1, 62, 63, 64, 127, 128, 300, 8]
    out, expected = run_attention(lib, dtype, nq, nkv, D, starts=starts, counts=[1] * len(starts),
                                  splits=splits)
    close(out, expected, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_finds_a_far_key_among_hundreds(lib, dtype):
    """One early key is made to match the last query (score ~ 25 above the rest): the
    output must be that key's value, in prefill and in split decode."""
    nq, nkv, D = 4, 2, 64
    for starts, counts, splits, row in (([0], [400], 1, 399), ([399], [1], 5, 0)):
        out, expected = run_attention(lib, dtype, nq, nkv, D, starts, counts, splits=splits,
                                      boost=(0, 3, row, 200.0), seed=4)
        close(out, expected, dtype)
        # the boosted key dominates head 0's softmax
        assert (out[row, 0].double().cpu() - expected[row, 0]).abs().max() < 0.05


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [1, 7, 64, 100])
def test_attention_window_edge(lib, dtype, window):
    """A standout key exactly at the window's edge counts; one step further it does not."""
    nq, nkv, D = 2, 1, 32
    n = 230
    for key_index in (n - window, n - window - 1):          # inside, just outside
        if key_index < 0:
            continue
        for starts, counts, splits, row in (([0], [n], 1, n - 1), ([n - 1], [1], 3, 0)):
            out, expected = run_attention(lib, dtype, nq, nkv, D, starts, counts, window=window,
                                          splits=splits, boost=(0, key_index, row, 300.0), seed=9)
            close(out, expected, dtype)


@pytest.mark.parametrize("nq,nkv,D,splits", [(32, 8, 128, 1), (32, 8, 128, 4), (8, 8, 64, 3), (64, 8, 128, 1),
                                             (6, 2, 128, 2), (20, 1, 64, 5), (16, 1, 128, 32),
                                             (2, 1, 64, 1)])
@pytest.mark.parametrize("waves", [4, 8, 16])
def test_attention_decode_on_the_matrix_cores(lib, nq, nkv, D, splits, waves):
    """The bfloat16 decode kernel: lengths around tile (16), page (64) and slice
    boundaries, group ratios that fill a head block partly, more slices than pages; blocks
    of 4, 8 and 16 waves (more waves than a short sequence has tiles)."""
    starts = [0, 1, 14, 15, 16, 62, 63, 64, 127, 128, 300, 1029, 8]
    out, expected = run_attention(lib, torch.bfloat16, nq, nkv, D, starts=starts,
                                  counts=[1] * len(starts), splits=splits, kernel="decode_mfma",
                                  waves=waves)
    close(out, expected, torch.bfloat16)


@pytest.mark.parametrize("nq,nkv,D,splits", [(32, 8, 128, 1), (32, 8, 128, 4), (6, 2, 128, 2), (16, 1, 64, 3)])
@pytest.mark.parametrize("waves,heads", [(16, 1), (16, 2), (8, 1), (8, 4), (4, 2)])
def test_attention_decode_with_fewer_heads_a_block(lib, nq, nkv, D, splits, waves, heads):
    """A block that takes fewer query heads of a group than it could (more, lighter blocks for
    steps of few sequences): the same result, also where the group is no multiple of them."""
    starts = [0, 15, 16, 63, 64, 300, 1029]
    out, expected = run_attention(lib, torch.bfloat16, nq, nkv, D, starts=starts,
                                  counts=[1] * len(starts), splits=splits, kernel="decode_mfma",
                                  waves=waves, heads=heads, seed=11)
    close(out, expected, torch.bfloat16)


def test_attention_decode_refuses_heads_a_block_that_are_no_power_of_two(lib):
    with pytest.raises(lib.KernelError, match="power of two"):
        run_attention(lib, torch.bfloat16, 8, 2, 64, starts=[5], counts=[1], kernel="decode_mfma",
                      waves=16, heads=3)


@pytest.mark.parametrize("splits,waves", [(2, 4), (5, 4), (32, 4), (3, 16)])
@pytest.mark.parametrize("longest", ["exact", "short", "long"])
def test_attention_decode_slices_of_the_longest_sequences_share(lib, splits, waves, longest):
    """Slices sized by the longest sequence (a number on the device): sequences of very
    unequal lengths, a stated length that is exact, too short (the last slice still takes
    what is left) or longer than any sequence."""
    starts = [0, 5, 63, 64, 200, 1029, 2300, 17]
    stated = {"exact": 2301, "short": 700, "long": 4000}[longest]
    out, expected = run_attention(lib, torch.bfloat16, 32, 8, 128, starts=starts,
                                  counts=[1] * len(starts), splits=splits, kernel="decode_mfma",
                                  waves=waves, longest=stated, seed=3)
    close(out, expected, torch.bfloat16)


@pytest.mark.parametrize("window", [1, 7, 64, 100])
def test_attention_decode_on_the_matrix_cores_window_and_far_key(lib, window):
    nq, nkv, D, n = 8, 2, 128, 230
    for key_index in (n - window, n - window - 1):
        out, expected = run_attention(lib, torch.bfloat16, nq, nkv, D, [n - 1], [1], window=window,
                                      splits=3, boost=(0, key_index, 0, 300.0), seed=9,
                                      kernel="decode_mfma", waves=16 if window > 7 else 4)
        close(out, expected, torch.bfloat16)
    out, expected = run_attention(lib, torch.bfloat16, nq, nkv, D, [899], [1], splits=6,
                                  boost=(0, 3, 0, 200.0), seed=4, kernel="decode_mfma")
    close(out, expected, torch.bfloat16)


@pytest.mark.parametrize("nq,nkv,D,splits,waves,slices", [
    (32, 8, 128, 1, 16, 3), (32, 8, 128, 4, 4, 1), (8, 8, 64, 1, 4, 2), (6, 2, 128, 2, 16, 5),
    (16, 2, 64, 1, 16, 2), (16, 2, 64, 3, 4, 2), (16, 1, 128, 1, 4, 4), (5, 1, 64, 2, 4, 1)])
@pytest.mark.parametrize("options", ["norm+rope", "bare", "read-only", "window"])
def test_attention_decode_from_the_projection(lib, nq, nkv, D, splits, waves, slices, options):
    """The decode kernel that norms, rotates and stores for its rows itself, against the
    separate norm-rotate-store kernel followed by the same decode kernel: the same output, the
    same keys and values in the same places of the cache and nothing else touched.  Lengths
    before the new token around tile and page boundaries; a padding row; group ratios that
    give one head block, several, and one that is not full; without norm weights and
    rotation; a run that stores nothing (it reads another run's cache); a window."""
    theta, eps = 1e4, 1e-5
    before = [0, 15, 16, 63, 64, 200, 300, 7]
    N = len(before)
    write = options != "read-only"
    window = 50 if options == "window" else None
    use = options != "bare"
    torch.manual_seed(nq + D + splits)
    caches = []
    for _ in range(2):
        cache = PagedCache([n + 1 for n in before], nkv, D, torch.bfloat16, seed=2)
        g = torch.Generator(device=DEV).manual_seed(5)
        for b, n in enumerate(before):
            total = n + (0 if write else 1)     # read-only: the position's key is there already
            if total:
                cache.put(b, torch.randn(total, nkv, D, device=DEV, generator=g),
                          torch.randn(total, nkv, D, device=DEV, generator=g))
        caches.append(cache)
    width = (nq + 2 * nkv) * D
    qkv = torch.randn(slices, N, width, device=DEV)
    row_pos, row_seq = list(before), list(range(N))
    row_seq[3] = -1                              # a padding row
    pos = torch.tensor(row_pos, dtype=torch.int32, device=DEV)
    seq = torch.tensor(row_seq, dtype=torch.int32, device=DEV)
    qn = (1 + 0.1 * torch.randn(D, device=DEV)) if use else None
    kn = (1 + 0.1 * torch.randn(D, device=DEV)) if use else None
    table = rope_table(D, theta, 512) if use else None
    longest = torch.tensor([301], dtype=torch.int32, device=DEV)
    outs = []
    for fused, cache in zip((False, True), caches):
        out = torch.full((N, nq * D), float("nan"), device=DEV, dtype=torch.bfloat16)
        part_o = part_ml = None
        if splits > 1:
            part_o = torch.full((N * nq * splits * D,), float("nan"), device=DEV)
            part_ml = torch.full((N * nq * splits * 2,), float("nan"), device=DEV)
        if fused:
            q = lib.DecodeProjection(qkv, qn, kn, eps, table, write)
        else:
            q = torch.full((N, nq * D), float("nan"), device=DEV, dtype=torch.bfloat16)
            lib.qk_norm_rope_store(qkv, qn, kn, eps, table, pos, seq, cache.table_dev, q,
                                   cache.k, cache.v, nq, nkv, D, write_cache=write)
        # the fused run also with fewer heads a block than the block could take: every block of
        # a group makes the position's key and value for itself, the first one stores them
        heads = {"window": 1, "bare": 2}.get(options, 0) if fused else 0
        lib.attention_decode_mfma(q, cache.k, cache.v, pos, seq, cache.table_dev, out, nq, nkv, D,
                                  window=window, n_splits=splits, part_o=part_o, part_ml=part_ml,
                                  waves=waves, longest=longest, heads=heads)
        outs.append(out)
    separate, fused = outs
    assert torch.isnan(fused[3].float()).all() and torch.isnan(separate[3].float()).all()
    live = [r for r in range(N) if r != 3]
    assert not torch.isnan(fused[live].float()).any()
    close(fused[live], separate[live].double().cpu(), torch.bfloat16)
    # the caches: values equal bit for bit (a copy); keys equal up to the last bit of a
    # rounding (the sum of squares is added up in another order); NaN sentinels elsewhere
    bits = lambda t: t.view(torch.int16)
    assert torch.equal(bits(caches[0].v), bits(caches[1].v))
    ka, kb = caches[0].k.float(), caches[1].k.float()
    assert torch.equal(torch.isnan(ka), torch.isnan(kb))
    there = ~torch.isnan(ka)
    assert ((ka[there] - kb[there]).abs() <= 2.0 ** -7 * ka[there].abs() + 1e-6).all()
    if write:
        for r in live:
            page = caches[1].table[row_seq[r], row_pos[r] // PAGE]
            assert not torch.isnan(kb[page, :, row_pos[r] % PAGE]).any()


@pytest.mark.parametrize("key_ways", [1, 2])
@pytest.mark.parametrize("nq,nkv,D", [(32, 8, 128), (8, 8, 64), (6, 2, 128), (5, 1, 64),
                                      (12, 3, 128), (16, 16, 64), (8, 1, 128), (2, 1, 64)])
def test_attention_prefill_on_the_matrix_cores(lib, nq, nkv, D, key_ways):
    """The bfloat16 prefill kernel: prompts of 1, 63, 64, 65 and 300 tokens, and chunks
    appended to 70 and to 640 cached tokens, in one launch; every row group with all of a
    page's keys (key_ways 1) and with two waves sharing them (2: half as many positions an
    item, the two halves merged at the end).  Probabilities are rounded to bfloat16 before the
    value product, which the bound (2^-8 of the largest value) covers."""
    assert lib.attention_prefill_mfma_positions(nq // nkv, 2) * 2 == \
        lib.attention_prefill_mfma_positions(nq // nkv, 1)
    out, expected = run_attention(lib, torch.bfloat16, nq, nkv, D,
                                  starts=[0, 0, 0, 0, 70, 0, 640],
                                  counts=[1, 64, 63, 300, 9, 65, 100], kernel="prefill_mfma",
                                  key_ways=key_ways)
    close(out, expected, torch.bfloat16)


@pytest.mark.parametrize("pair_items", [True, False])
@pytest.mark.parametrize("key_ways", [1, 2])
@pytest.mark.parametrize("counts", [[1041, 20], [1060]])
def test_attention_prefill_on_the_matrix_cores_many_blocks(lib, counts, key_ways, pair_items):
    """Enough work items (more than 512 blocks) for the kernel to give every block two of
    them, the u-th and the u-th from the end, where the caller allows it; an odd and an even
    number of items.  The same items one a block give the same result."""
    out, expected = run_attention(lib, torch.bfloat16, 64, 16, 64, starts=[0] * len(counts),
                                  counts=counts, kernel="prefill_mfma", seed=5, key_ways=key_ways,
                                  pair_items=pair_items)
    close(out, expected, torch.bfloat16)


@pytest.mark.parametrize("key_ways", [1, 2])
@pytest.mark.parametrize("window", [1, 7, 31, 33, 64, 100])
def test_attention_prefill_on_the_matrix_cores_window_and_far_key(lib, window, key_ways):
    nq, nkv, D, n = 8, 2, 128, 230
    for key_index in (n - window, n - window - 1):
        out, expected = run_attention(lib, torch.bfloat16, nq, nkv, D, [0], [n], window=window,
                                      boost=(0, key_index, n - 1, 300.0), seed=9,
                                      kernel="prefill_mfma", key_ways=key_ways)
        close(out, expected, torch.bfloat16)
    # a far key in the first half of a page and one in the second (keys 3 and 40)
    for far in (3, 40):
        out, expected = run_attention(lib, torch.bfloat16, nq, nkv, D, [0], [900],
                                      boost=(0, far, 899, 200.0), seed=4, kernel="prefill_mfma",
                                      key_ways=key_ways)
        close(out, expected, torch.bfloat16)


def test_attention_refuses_sizes_it_cannot_run(lib):
    from edge_infer_amd.csrc.lib import KernelError
    with pytest.raises(KernelError, match="multiple of 16"):
        run_attention(lib, torch.float32, 2, 1, 24, [0], [4])
    with pytest.raises(KernelError, match="multiple of 16"):
        run_attention(lib, torch.float32, 2, 1, 512, [0], [4])


# ---------------------------------------------------------------------------
def test_argmax_ties_and_nan(lib):
    rows = torch.tensor([[2, 1, 0, -1], [-3, 5, 1, 0], [0, -1, 4, 2], [1, 3, 3, 2],
                         [float("nan"), -5, -5, -7]], dtype=torch.float32, device=DEV)
    tokens = torch.empty(5, dtype=torch.int32, device=DEV)
    prob = torch.empty(5, device=DEV)
    lib.argmax(rows, tokens, prob)
    assert tokens.tolist() == [0, 1, 2, 1, 1]
    assert prob.tolist() == [1.0] * 5
    big = torch.randn(3, 151936, device=DEV)
    big[1, 150000] = 9.0
    big[1, 77] = 9.0
    tokens = torch.empty(3, dtype=torch.int32, device=DEV)
    lib.argmax(big, tokens)
    assert tokens.tolist() == [int(big[0].argmax()), 77, int(big[2].argmax())]
    # the same through many blocks a row: ties across chunks, NaN, a width that ends inside
    # a chunk, an all -inf row
    for vocab in (151936, 8193, 12288):
        big = torch.randn(5, vocab, device=DEV)
        big[1, vocab - 1] = 9.0
        big[1, 4097] = 9.0
        big[2, 5000] = float("nan")
        big[3] = float("-inf")
        big[4, vocab - 1] = 11.0
        need = lib.argmax_partial_size(5, vocab)
        assert need > 0
        partial = torch.full((need,), float("nan"), device=DEV)
        tokens = torch.full((5,), -1, dtype=torch.int32, device=DEV)
        prob = torch.zeros(5, device=DEV)
        lib.argmax(big, tokens, prob, partial)
        finite = torch.nan_to_num(big[2], nan=float("-inf"))
        assert tokens.tolist() == [int(big[0].argmax()), 4097, int(finite.argmax()), 0, vocab - 1]
        assert prob.tolist() == [1.0] * 5
        with pytest.raises(lib.KernelError, match="too small"):
            lib.argmax(big, tokens, prob, partial[:need - 2])
    assert lib.argmax_partial_size(4, 8192) == 0


def test_sample_reference_distribution(lib):
    """operators/tests/operators_cuda_sampling_test.cu:133-198: logits log{.4,.3,.2,.1}, 2048
    seeded draws for three (T, p, k): support, reported probability within 2e-5 of the
    filtered softmax, frequencies within 0.05; and every draw equals the plain sampler's."""
    logits = np.log(np.array([0.4, 0.3, 0.2, 0.1], dtype=np.float32))
    rows = 2048
    dev = torch.from_numpy(np.tile(logits, (rows, 1))).to(DEV)
    streams = torch.zeros(rows, dtype=torch.int32, device=DEV)
    counters = torch.arange(rows, dtype=torch.int32, device=DEV)
    for temperature, top_p, top_k in [(1.0, 1.0, 2), (1.0, 0.65, 4), (0.75, 0.95, 3)]:
        tokens = torch.empty(rows, dtype=torch.int32, device=DEV)
        prob = torch.empty(rows, device=DEV)
        lib.sample(dev, temperature, top_p, top_k, 1234567, streams, counters, tokens, prob)
        order, expected = plain.filtered_distribution(logits, temperature, top_p, top_k)
        table = dict(zip(order.tolist(), expected.tolist()))
        got, got_p = tokens.tolist(), prob.tolist()
        counts = {t: 0 for t in table}
        for draw, (token, p) in enumerate(zip(got, got_p)):
            assert token in table and abs(p - table[token]) < 2e-5
            counts[token] += 1
            assert token == plain.sample(logits, temperature, top_p, top_k,
                                         plain.uniform(1234567, 0, draw))
        assert max(abs(counts[t] / rows - table[t]) for t in table) < 0.05


def test_sample_large_vocabulary_matches_plain(lib):
    """Without scratch (one block a row) and with it (many blocks a row gather the pairs that
    can belong to the top k): the same tokens as the plain sampler, also where the gathered
    list overflows (thousands of ties, everything equal) or is tied beyond 1024 pairs, and
    in later calls with other row counts on the same scratch."""
    V = 151936
    g = torch.Generator().manual_seed(3)
    logits = (torch.randn(7, V, generator=g) * 2.5)
    logits[2, :5000] = 6.0                         # thousands of ties around the threshold
    logits[3, 100:104] = 30.0                      # ties at the very top
    logits[4, :] = -1.0                            # everything equal
    logits[5, 17] = float("nan")
    logits[6, 1000:3000] = 9.5                     # 2000 ties: they fit the list, not the tie table
    dev = logits.to(DEV)
    streams = torch.tensor([0, 1, 2, 3, 4, 5, 6], dtype=torch.int32, device=DEV)
    counters = torch.tensor([0, 5, 9, 1, 2, 3, 4], dtype=torch.int32, device=DEV)
    need = lib.sample_scratch_size(7, V)
    assert need > 0 and lib.sample_scratch_size(7, 5000) == 0
    scratch = torch.zeros(need, dtype=torch.int32, device=DEV)
    for temperature, top_p, top_k in [(0.8, 0.95, 50), (1.3, 1.0, 1024), (0.7, 0.5, 20),
                                      (1.0, 1.0, 3)]:
        tokens = torch.empty(7, dtype=torch.int32, device=DEV)
        lib.sample(dev, temperature, top_p, top_k, 42, streams, counters, tokens)
        wide = torch.empty(7, dtype=torch.int32, device=DEV)
        prob = torch.empty(7, device=DEV)
        lib.sample(dev, temperature, top_p, top_k, 42, streams, counters, wide, prob, scratch)
        for r in range(7):
            u = plain.uniform(42, int(streams[r]), int(counters[r]))
            expected = plain.sample(logits[r].numpy(), temperature, top_p, top_k, u)
            assert tokens[r].item() == expected, (r, temperature, top_p, top_k)
            assert wide[r].item() == expected, ("many blocks", r, temperature, top_p, top_k)
        # fewer rows on the same scratch, from the second row on
        part = torch.empty(3, dtype=torch.int32, device=DEV)
        lib.sample(dev[1:4], temperature, top_p, top_k, 42, streams[1:4], counters[1:4], part,
                   None, scratch)
        assert part.tolist() == wide[1:4].tolist()
    # every call left what must start at zero at zero (bins and counts; lists may hold anything)
    per_row = need // 7
    view = scratch.view(7, per_row)
    assert int(view[:, :4096 + 4].abs().sum().item()) == 0
    from edge_infer_amd.csrc.lib import KernelError
    with pytest.raises(KernelError, match="too small"):
        lib.sample(dev, 1.0, 1.0, 5, 42, streams, counters, tokens, None, scratch[:100])


def test_sample_refuses_bad_policies(lib):
    from edge_infer_amd.csrc.lib import KernelError
    logits = torch.zeros(1, 5000, device=DEV)
    ints = torch.zeros(1, dtype=torch.int32, device=DEV)
    for temperature, top_p, top_k in [(1.0, 0.0, 5), (1.0, 1.5, 5), (1.0, 0.9, 0), (1.0, 0.9, 1025),
                                      (0.0, 0.9, 5)]:
        with pytest.raises(KernelError):
            lib.sample(logits, temperature, top_p, top_k, 0, ints, ints, ints.clone())


# ---------------------------------------------------------------------------
@pytest.mark.parametrize("M", [1, 3, 16, 17, 33, 64, 65, 128, 129, 130, 256])
@pytest.mark.parametrize("N,K", [(381, 96), (200, 200), (96, 256), (4096, 1024), (1000, 1384),
                                 (16400, 264)])
def test_gemm_bf16_skinny(lib, M, N, K):
    """The weight-streaming product for few rows: every slice count it may choose, widths
    that are no multiple of the tile, the same row alone or among others, and more than 64
    rows (several blocks of 64 rows share each group of weight rows)."""
    torch.manual_seed(M * 7 + N)
    x = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    w = torch.randn(N, K, device=DEV).to(torch.bfloat16)
    expected = plain.linear(x.cpu(), w.cpu())
    chosen = lib.skinny_gemm_splits(M, N, K)
    tile = 256
    tiles = (K + tile - 1) // tile
    candidates = {1, chosen}
    for s in range(2, tiles + 1):            # every slice count that leaves no slice empty
        per = (tiles + s - 1) // s
        if (tiles + per - 1) // per == s:
            candidates.add(s)
    results = {}
    packed = lib.pack_weight(w)
    assert packed.shape == (8 * ((K + 255) // 256), (N + 15) // 16, 4, 16, 8)
    for splits in sorted(candidates):
        out = torch.full((splits, M, N), float("nan"), device=DEV)
        lib.gemm_bf16_skinny(x, w, out)
        err = (out.double().cpu().sum(0) - expected).abs().max().item()
        assert err <= 2e-6 * math.sqrt(K) * 16, f"splits {splits}: max error {err:.3e}"
        results[splits] = out
        # the streaming copy of the weight: the same sums in the same order
        again = torch.full((splits, M, N), float("nan"), device=DEV)
        lib.gemm_bf16_skinny_packed(x, packed, N, again)
        assert torch.equal(again, out), f"splits {splits}: packed layout differs"
    # a row gives the same bits alone as inside a batch of up to 16 rows (the same tile
    # shape and slice count, hence the same order of accumulation)
    if M <= 16 and lib.skinny_gemm_splits(1, N, K) == chosen:
        single = torch.empty((chosen, 1, N), device=DEV)
        lib.gemm_bf16_skinny(x[M // 2:M // 2 + 1].contiguous(), w, single)
        assert torch.equal(single[:, 0], results[chosen][:, M // 2])


@pytest.mark.parametrize("packed", [True, False])
@pytest.mark.parametrize("M,I,K", [(1, 48, 256), (8, 1024, 512), (16, 16, 96), (33, 2048, 256),
                                   (64, 208, 1000), (100, 2192, 256), (256, 48, 520)])
def test_gemm_bf16_skinny_gated(lib, M, I, K, packed):
    """silu(x . gate) * (x . up) written by the few-rows kernel itself, from a weight whose
    rows alternate between 16 gate rows and their 16 up rows (all of K in one slice, also
    where the plain product would cut it)."""
    torch.manual_seed(M + I)
    x = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    gate = (torch.randn(I, K, device=DEV) / math.sqrt(K) * 3).to(torch.bfloat16)
    up = (torch.randn(I, K, device=DEV) / math.sqrt(K)).to(torch.bfloat16)
    mixed = torch.stack([gate.reshape(I // 16, 16, K), up.reshape(I // 16, 16, K)],
                        dim=1).reshape(2 * I, K).contiguous()
    act = torch.full((M, I), float("nan"), device=DEV, dtype=torch.bfloat16)
    lib.gemm_bf16_skinny_gated(x, lib.pack_weight(mixed) if packed else mixed, 2 * I, act, packed)
    expected = plain.swiglu(plain.linear(x.cpu(), gate.cpu()), plain.linear(x.cpu(), up.cpu()))
    close(act, expected, torch.bfloat16)


def test_gemm_bf16_skinny_gated_refuses_what_it_cannot_run(lib):
    from edge_infer_amd.csrc.lib import KernelError
    x = torch.zeros(2, 64, device=DEV, dtype=torch.bfloat16)
    w = torch.zeros(48, 64, device=DEV, dtype=torch.bfloat16)        # 48 is no multiple of 32
    with pytest.raises(KernelError, match="do not agree"):
        lib.gemm_bf16_skinny_gated(x, w, 48, torch.empty(2, 24, device=DEV, dtype=torch.bfloat16), False)
    w = torch.zeros(64, 64, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(KernelError, match="do not agree"):            # act of the wrong width
        lib.gemm_bf16_skinny_gated(x, w, 64, torch.empty(2, 64, device=DEV, dtype=torch.bfloat16), False)


def test_gemm_bf16_skinny_refuses_what_it_cannot_run(lib):
    from edge_infer_amd.csrc.lib import KernelError
    w = torch.zeros(32, 100, device=DEV, dtype=torch.bfloat16)
    x = torch.zeros(2, 100, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(KernelError, match="multiple of 8"):
        lib.gemm_bf16_skinny(x, w, torch.empty(1, 2, 32, device=DEV))
    w = torch.zeros(32, 96, device=DEV, dtype=torch.bfloat16)
    x = torch.zeros(257, 96, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(KernelError, match="1..256"):
        lib.gemm_bf16_skinny(x, w, torch.empty(1, 257, 32, device=DEV))
    with pytest.raises(KernelError, match="do not agree"):       # packed for another n
        lib.gemm_bf16_skinny_packed(x[:2], lib.pack_weight(w), 48, torch.empty(1, 2, 48, device=DEV))


@pytest.mark.parametrize("rows,width", [(1, 7), (5, 96), (300, 1000)])
def test_bias_rows(lib, rows, width):
    g = torch.Generator().manual_seed(rows)
    bias = torch.randn(width, generator=g).cuda()
    start = torch.randn(rows, width, generator=g).cuda()
    out = start.clone()
    lib.bias_rows(bias, out, accumulate=True)
    assert torch.equal(out, start + bias)
    lib.bias_rows(bias, out, accumulate=False)
    assert torch.equal(out, bias.expand(rows, width))
    with pytest.raises(lib.KernelError):
        lib.bias_rows(bias[:-1], out, accumulate=False)


def test_sum_slices(lib):
    slices = torch.randn(5, 3, 1001, device=DEV)
    out = torch.empty(3, 1001, device=DEV)
    lib.sum_slices(slices, out)
    expected = slices[0].clone()
    for s in range(1, 5):
        expected += slices[s]
    assert torch.equal(out, expected)


# ---------------------------------------------------------------------------
# The products at the widths of real checkpoints: every (out, in) of the 8B, 32B and 0.6B
# shapes, the vocabulary of 151,936 included, at 1 to 256 rows.  The reference is a float64
# product on the GPU (the plain implementation's `linear` is the same x . W^T).
REAL_SHAPES = {
    "8b": dict(H=4096, Q=4096, KV=1024, I=12288),
    "32b": dict(H=5120, Q=8192, KV=1024, I=25600),
    "0.6b": dict(H=1024, Q=2048, KV=1024, I=3072),
}
VOCABULARY = 151936
REAL_ROWS = (1, 8, 16, 64, 256)


def real_products(shape):
    s = REAL_SHAPES[shape]
    return {"qkv": (s["Q"] + 2 * s["KV"], s["H"]), "o": (s["H"], s["Q"]),
            "gate_up": (2 * s["I"], s["H"]), "down": (s["H"], s["I"]),
            "head": (VOCABULARY, s["H"])}


@pytest.mark.parametrize("which", ["qkv", "o", "gate_up", "down", "head"])
@pytest.mark.parametrize("shape", sorted(REAL_SHAPES))
def test_gemm_bf16_skinny_at_the_widths_of_real_checkpoints(lib, shape, which):
    N, K = real_products(shape)[which]
    g = torch.Generator(device=DEV).manual_seed(N + K)
    x = torch.randn(256, K, device=DEV, generator=g).to(torch.bfloat16)
    w = torch.randn(N, K, device=DEV, generator=g).to(torch.bfloat16)
    expected = x.double() @ w.double().t()
    packed = lib.pack_weight(w)
    bound = 2e-6 * math.sqrt(K) * 16
    for M in REAL_ROWS:
        splits = lib.skinny_gemm_splits(M, N, K)
        out = torch.full((splits, M, N), float("nan"), device=DEV)
        lib.gemm_bf16_skinny_packed(x[:M], packed, N, out)
        err = (out.double().sum(0) - expected[:M]).abs().max().item()
        assert err <= bound, f"{shape} {which} {M} rows, {splits} slices: max error {err:.3e}"
        if M in (1, 64):       # the stored layout through the other entry point
            again = torch.full((splits, M, N), float("nan"), device=DEV)
            lib.gemm_bf16_skinny(x[:M], w, again)
            assert torch.equal(again, out), f"{shape} {which} {M} rows: stored layout differs"
    if which == "gate_up":
        # rows read as strips of 16 gate rows and their 16 up rows: the kernel's own activation
        pairs = expected.view(256, N // 32, 2, 16)
        gate, up = pairs[:, :, 0].reshape(256, N // 2), pairs[:, :, 1].reshape(256, N // 2)
        wanted = gate / (1 + torch.exp(-gate)) * up
        for M in (1, 8, 64, 256):
            act = torch.full((M, N // 2), float("nan"), device=DEV, dtype=torch.bfloat16)
            lib.gemm_bf16_skinny_gated(x[:M], packed, N, act, True)
            err = (act.double() - wanted[:M]).abs().max().item()
            assert err <= 1.2e-2 * wanted[:M].abs().max().item(), f"{shape} gated {M} rows: {err:.3e}"


@pytest.mark.parametrize("which", ["qkv", "o", "gate_up", "down", "head"])
@pytest.mark.parametrize("shape", sorted(REAL_SHAPES))
def test_gemm_f32_at_the_widths_of_real_checkpoints(lib, shape, which):
    N, K = real_products(shape)[which]
    g = torch.Generator(device=DEV).manual_seed(N + 3 * K)
    x = torch.randn(256, K, device=DEV, generator=g)
    w = torch.randn(N, K, device=DEV, generator=g)
    expected = x.double() @ w.double().t()
    for M in REAL_ROWS:
        out = torch.full((M, N), float("nan"), device=DEV)
        lib.gemm_f32(x[:M], w, out)
        err = (out.double() - expected[:M]).abs().max().item()
        # every output is one thread's sum over k in ascending order: K roundings of 2^-24 of
        # partial sums that grow like sqrt(k) add up to about 2^-24 K / 2.4 (one sigma)
        assert err <= 6 * 2.0 ** -24 * K, f"{shape} {which} {M} rows: max error {err:.3e}"
    del expected
    torch.cuda.empty_cache()


def test_argmax_and_sample_at_the_real_vocabulary(lib):
    rows = 64
    g = torch.Generator(device=DEV).manual_seed(9)
    logits = torch.randn(rows, VOCABULARY, device=DEV, generator=g)
    tokens = torch.empty(rows, dtype=torch.int32, device=DEV)
    partial = torch.empty(lib.argmax_partial_size(rows, VOCABULARY), device=DEV)
    lib.argmax(logits, tokens, None, partial)
    assert tokens.tolist() == logits.argmax(-1).tolist()
    static = torch.empty(rows, dtype=torch.int32, device=DEV)
    lib.argmax_static(logits, static)
    assert torch.equal(static, tokens)
