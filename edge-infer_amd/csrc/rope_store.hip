// Fused per-head q/k RMSNorm -> rotary encoding -> cache store.
//
// One wave per (row, head) over the packed projection [N, Q + 2*KV]: query heads
// are normed, rotated and written to q_out; key heads are normed, rotated and
// written to the cache page of (sequence, position); value heads are copied to
// the cache.  Sum of squares, inverse RMS, angles' sine/cosine (a float32 table)
// and the rotation are float32; one rounding to the storage type.
//
// Formulas of the reference: norm before rotation,
// runtime/include/execution/decoder.hpp:125-140; rotate-half pairs (i, i + d/2),
// x' = x cos - y sin, y' = x sin + y cos, operators/src/cuda/execution.cu:79-122;
// keys stored after norm and rotation, values raw, decoder.hpp:137-140.
//
// The rotation may cover only the first R <= D elements of a head (R = the table's width):
// pairs (i, i + R/2) for i < R/2, elements R..D-1 pass unrotated.  A lane's pair j of D/2 is
// then elements (j, j + R/2) below R/2 and (j + R/2, j + D/2) from there on, the latter with
// the identity as its rotation; with R = D this is the pair (j, j + D/2) throughout.
#include "common.h"

namespace {

constexpr int kMaxPairsPerLane = 4;  // head_dim up to 512

template <typename TI, typename TO>
__global__ void qk_norm_rope_store_kernel(
    const TI* __restrict__ qkv, int nsplit, size_t split_stride,
    const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, float eps,
    const float* __restrict__ rope_table,  // [max_pos, R]: cos[R/2] then sin[R/2]; null: none
    const int32_t* __restrict__ row_pos, const int32_t* __restrict__ row_seq,
    const int32_t* __restrict__ page_table, int table_width,
    TO* __restrict__ q_out, TO* __restrict__ k_pages, TO* __restrict__ v_pages,
    int N, int nq, int nkv, int D, int R, int write_cache) {
  const int heads = nq + 2 * nkv;
  const int wave = (blockIdx.x * blockDim.x + threadIdx.x) / EI_WAVE;
  const int lane = threadIdx.x % EI_WAVE;
  if (wave >= N * heads) return;
  const int row = wave / heads, head = wave % heads;
  const int seq = row_seq[row];
  if (seq < 0) return;  // padding row
  const bool is_q = head < nq, is_k = !is_q && head < nq + nkv;
  if (!is_q && !write_cache) return;
  const int pos = row_pos[row];
  const int half = D / 2, rhalf = R / 2;
  const size_t width = static_cast<size_t>(nq + 2 * nkv) * D;
  const TI* src = qkv + static_cast<size_t>(row) * width + static_cast<size_t>(head) * D;

  float x[kMaxPairsPerLane], y[kMaxPairsPerLane];
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < kMaxPairsPerLane; ++j) {
    const int pair = lane + j * EI_WAVE;
    x[j] = 0.f;
    y[j] = 0.f;
    if (pair < half) {
      const int i = pair < rhalf ? pair : pair + rhalf;          // the pair's first element
      const int i2 = pair < rhalf ? pair + rhalf : pair + half;  // and its second
      // slices are added in slice order, four loads per trip to memory
      for (int s0 = 0; s0 < nsplit; s0 += 4) {
        TI a[4], b[4];
#pragma unroll
        for (int u = 0; u < 4; ++u)
          if (s0 + u < nsplit) {
            a[u] = src[(s0 + u) * split_stride + i];
            b[u] = src[(s0 + u) * split_stride + i2];
          }
#pragma unroll
        for (int u = 0; u < 4; ++u)
          if (s0 + u < nsplit) {
            x[j] += ei::to_f32<TI>(a[u]);
            y[j] += ei::to_f32<TI>(b[u]);
          }
      }
      sum += x[j] * x[j] + y[j] * y[j];
    }
  }

  TO* dst;
  if (is_q) {
    dst = q_out + static_cast<size_t>(row) * nq * D + static_cast<size_t>(head) * D;
  } else {
    const int page = page_table[static_cast<size_t>(seq) * table_width + pos / EI_PAGE];
    if (page < 0) return;
    const int g = is_k ? head - nq : head - nq - nkv;
    TO* base = is_k ? k_pages : v_pages;
    dst = base + ((static_cast<size_t>(page) * nkv + g) * EI_PAGE + pos % EI_PAGE) * D;
  }

  const float* norm_w = is_q ? q_norm_w : (is_k ? k_norm_w : nullptr);
  float inv = 1.f;
  if (norm_w) {
    sum = ei::wave_sum(sum);
    inv = rsqrtf(sum / static_cast<float>(D) + eps);
  }
  const bool rotate = rope_table != nullptr && (is_q || is_k);
  const float* trig = rotate ? rope_table + static_cast<size_t>(pos) * R : nullptr;
#pragma unroll
  for (int j = 0; j < kMaxPairsPerLane; ++j) {
    const int pair = lane + j * EI_WAVE;
    if (pair < half) {
      const int i = pair < rhalf ? pair : pair + rhalf;
      const int i2 = pair < rhalf ? pair + rhalf : pair + half;
      float a = x[j], b = y[j];
      if (norm_w) {
        a = (a * inv) * norm_w[i];
        b = (b * inv) * norm_w[i2];
      }
      if (rotate && pair < rhalf) {
        const float c = trig[pair], s = trig[pair + rhalf];
        const float ra = a * c - b * s;
        const float rb = a * s + b * c;
        a = ra;
        b = rb;
      }
      dst[i] = ei::from_f32<TO>(a);
      dst[i2] = ei::from_f32<TO>(b);
    }
  }
}

// The same for head sizes (and rotated widths) that are a multiple of 2 P: G lanes (a power of
// two) share a head, each lane takes P (4 or 8) neighbouring pairs with one or two 16-byte
// accesses (one of 8 bytes for 4 bfloat16) per half, so a wave covers 64 / G heads.
template <typename TI, typename TO, int G, int P>
__device__ __forceinline__ void qk_norm_rope_store_item(
    long long item, int sub, const TI* __restrict__ qkv, int nsplit, size_t split_stride,
    const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, float eps,
    const float* __restrict__ rope_table, const int32_t* __restrict__ row_pos,
    const int32_t* __restrict__ row_seq, const int32_t* __restrict__ page_table, int table_width,
    TO* __restrict__ q_out, TO* __restrict__ k_pages, TO* __restrict__ v_pages,
    int N, int nq, int nkv, int D, int R, int write_cache) {
  using ei::VecN;
  const int heads = nq + 2 * nkv;
  const int row = static_cast<int>(item / heads), head = static_cast<int>(item % heads);
  const bool is_q = head < nq, is_k = !is_q && head < nq + nkv;
  if (!is_q && !write_cache) return;
  // The sequence and the position are asked for first and the head's elements right after,
  // before either is needed: what depends on them (the page, the angles) is then looked up
  // while the elements are on their way.  (A padding row costs its loads.)
  const int seq = row_seq[row];
  const int pos = row_pos[row];
  const int half = D / 2, rhalf = R / 2;
  const int pair0 = sub * P;                                   // the lane's first pair
  const bool active = pair0 < half;
  const bool turned = pair0 < rhalf;                           // its pairs are rotated ones
  const int i0 = turned ? pair0 : pair0 + rhalf;               // their first elements
  const int i2 = turned ? pair0 + rhalf : pair0 + half;        // and their second ones
  const size_t width = static_cast<size_t>(heads) * D;
  const TI* src = qkv + static_cast<size_t>(row) * width + static_cast<size_t>(head) * D;
  float first_a[4][P], first_b[4][P];                          // the first four slices
  if (active) {
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (u < nsplit) {
        VecN<TI, P>::load(src + u * split_stride + i0, first_a[u]);
        VecN<TI, P>::load(src + u * split_stride + i2, first_b[u]);
      }
  }
  if (seq < 0) return;  // padding row

  TO* dst;
  bool stored = true;
  if (is_q) {
    dst = q_out + static_cast<size_t>(row) * nq * D + static_cast<size_t>(head) * D;
  } else {
    const int page = page_table[static_cast<size_t>(seq) * table_width + pos / EI_PAGE];
    stored = page >= 0;
    const int g = is_k ? head - nq : head - nq - nkv;
    TO* base = is_k ? k_pages : v_pages;
    dst = base + ((static_cast<size_t>(stored ? page : 0) * nkv + g) * EI_PAGE + pos % EI_PAGE) * D;
  }
  const float* norm_w = is_q ? q_norm_w : (is_k ? k_norm_w : nullptr);
  const bool rotate = rope_table != nullptr && (is_q || is_k);

  float x[P], y[P], wx[P], wy[P], cs[P], sn[P];
#pragma unroll
  for (int i = 0; i < P; ++i) {
    x[i] = y[i] = sn[i] = 0.f;
    wx[i] = wy[i] = cs[i] = 1.f;
  }
  if (active) {
    if (norm_w) {
      VecN<float, P>::load(norm_w + i0, wx);
      VecN<float, P>::load(norm_w + i2, wy);
    }
    if (rotate && turned) {
      const float* trig = rope_table + static_cast<size_t>(pos) * R + pair0;
      VecN<float, P>::load(trig, cs);
      VecN<float, P>::load(trig + rhalf, sn);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (u < nsplit) {
#pragma unroll
        for (int i = 0; i < P; ++i) {
          x[i] += first_a[u][i];
          y[i] += first_b[u][i];
        }
      }
    for (int s0 = 4; s0 < nsplit; s0 += 4) {       // further slices in slice order, four per trip
      float a[4][P], b[4][P];
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (s0 + u < nsplit) {
          VecN<TI, P>::load(src + (s0 + u) * split_stride + i0, a[u]);
          VecN<TI, P>::load(src + (s0 + u) * split_stride + i2, b[u]);
        }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (s0 + u < nsplit) {
#pragma unroll
          for (int i = 0; i < P; ++i) {
            x[i] += a[u][i];
            y[i] += b[u][i];
          }
        }
    }
  }
  float inv = 1.f;
  if (norm_w) {
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < P; ++i) sum += x[i] * x[i] + y[i] * y[i];
#pragma unroll
    for (int offset = G / 2; offset > 0; offset >>= 1) sum += __shfl_xor(sum, offset, EI_WAVE);
    inv = rsqrtf(sum / static_cast<float>(D) + eps);
  }
  if (!active || !stored) return;
  float ox[P], oy[P];
#pragma unroll
  for (int i = 0; i < P; ++i) {
    float a = x[i], b = y[i];
    if (norm_w) {
      a = (a * inv) * wx[i];
      b = (b * inv) * wy[i];
    }
    if (rotate) {                      // (the identity for pairs beyond the rotated width)
      const float ra = a * cs[i] - b * sn[i];
      const float rb = a * sn[i] + b * cs[i];
      a = ra;
      b = rb;
    }
    ox[i] = a;
    oy[i] = b;
  }
  VecN<TO, P>::store(dst + i0, ox);
  VecN<TO, P>::store(dst + i2, oy);
}

template <typename TI, typename TO, int G, int P>
__global__ void qk_norm_rope_store_vec_kernel(
    const TI* __restrict__ qkv, int nsplit, size_t split_stride,
    const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, float eps,
    const float* __restrict__ rope_table, const int32_t* __restrict__ row_pos,
    const int32_t* __restrict__ row_seq, const int32_t* __restrict__ page_table, int table_width,
    TO* __restrict__ q_out, TO* __restrict__ k_pages, TO* __restrict__ v_pages,
    int N, int nq, int nkv, int D, int R, int write_cache) {
  const long long item = (static_cast<long long>(blockIdx.x) * blockDim.x + threadIdx.x) / G;
  const int sub = threadIdx.x % G;
  if (item >= static_cast<long long>(N) * (nq + 2 * nkv)) return;   // the same for all lanes of a group
  qk_norm_rope_store_item<TI, TO, G, P>(item, sub, qkv, nsplit, split_stride, q_norm_w, k_norm_w,
                                        eps, rope_table, row_pos, row_seq, page_table, table_width,
                                        q_out, k_pages, v_pages, N, nq, nkv, D, R, write_cache);
}

}  // namespace

// qkv: [nsplit][N, (nq + 2 nkv) * D] of in_dtype.  q_out: [N, nq * D] of out_dtype.
// k_pages / v_pages: [n_pages, nkv, 64, D] of out_dtype for this cache entry.
// page_table: int32 [n_seqs, table_width], logical page -> physical page.
extern "C" int ei_qk_norm_rope_store(
    const void* qkv, int in_dtype, int nsplit, long long split_stride, const float* q_norm_w,
    const float* k_norm_w, float eps, const float* rope_table, int rot_dim,
    const int32_t* row_pos, const int32_t* row_seq, const int32_t* page_table, int table_width,
    void* q_out, void* k_pages, void* v_pages, int out_dtype, int N, int nq, int nkv, int D,
    int write_cache, hipStream_t stream) {
  EI_REQUIRE(N > 0 && nq > 0 && nkv > 0 && D > 0, "qk_norm_rope_store: sizes must be positive");
  EI_REQUIRE(D % 2 == 0, "qk_norm_rope_store: head_dim must be even");
  EI_REQUIRE(D / 2 <= kMaxPairsPerLane * EI_WAVE, "qk_norm_rope_store: head_dim above 512");
  EI_REQUIRE(qkv && row_pos && row_seq && q_out, "qk_norm_rope_store: null pointer");
  EI_REQUIRE(!write_cache || (k_pages && v_pages && page_table && table_width > 0),
             "qk_norm_rope_store: cache pointers missing");
  EI_REQUIRE(nsplit >= 1, "qk_norm_rope_store: nsplit must be at least 1");
  // the rotated width R: the table's row length, even, at most the head size (D without a table)
  const int R = rope_table ? rot_dim : D;
  EI_REQUIRE(R >= 2 && R % 2 == 0 && R <= D,
             "qk_norm_rope_store: the rotated width must be even and at most head_dim");
  const int heads = nq + 2 * nkv;
  const int threads = 256;
  const size_t ss = static_cast<size_t>(split_stride);
  // vector kernel: P pairs a lane (8 for bfloat16 in and out where the sizes allow, else 4),
  // G = lanes a head (the power of two at or above D / 2P)
  const bool aligned = (reinterpret_cast<uintptr_t>(qkv) | reinterpret_cast<uintptr_t>(q_out) |
                        reinterpret_cast<uintptr_t>(k_pages) | reinterpret_cast<uintptr_t>(v_pages) |
                        reinterpret_cast<uintptr_t>(q_norm_w) | reinterpret_cast<uintptr_t>(k_norm_w) |
                        reinterpret_cast<uintptr_t>(rope_table)) % 16 == 0;
  if (D % 8 == 0 && R % 8 == 0 && ss % 4 == 0 && aligned) {
    const bool wide = in_dtype == EI_BF16 && out_dtype == EI_BF16 && D % 16 == 0 && R % 16 == 0 &&
                      ss % 8 == 0;
    const int per_lane = wide ? 16 : 8;            // elements of a head a lane takes
    int G = 2;
    while (G * per_lane < D) G *= 2;
    const long long items = static_cast<long long>(N) * heads;
    const long long blocks = (items * G + threads - 1) / threads;
    EI_REQUIRE(blocks < (1ll << 31), "qk_norm_rope_store: too many rows");
#define EI_ROPE_VEC(TI, TO, GG, PP)                                                               \
  qk_norm_rope_store_vec_kernel<TI, TO, GG, PP><<<static_cast<unsigned>(blocks), threads, 0, stream>>>( \
      static_cast<const TI*>(qkv), nsplit, ss, q_norm_w, k_norm_w, eps, rope_table, row_pos,      \
      row_seq, page_table, table_width, static_cast<TO*>(q_out), static_cast<TO*>(k_pages),       \
      static_cast<TO*>(v_pages), N, nq, nkv, D, R, write_cache)
#define EI_ROPE_VEC_G(TI, TO, PP)                                                                 \
  do {                                                                                            \
    if (G == 2) EI_ROPE_VEC(TI, TO, 2, PP);                                                       \
    else if (G == 4) EI_ROPE_VEC(TI, TO, 4, PP);                                                  \
    else if (G == 8) EI_ROPE_VEC(TI, TO, 8, PP);                                                  \
    else if (G == 16) EI_ROPE_VEC(TI, TO, 16, PP);                                                \
    else if (G == 32) EI_ROPE_VEC(TI, TO, 32, PP);                                                \
    else EI_ROPE_VEC(TI, TO, 64, PP);                                                             \
  } while (0)
    if (wide)
      EI_ROPE_VEC_G(bf16_t, bf16_t, 8);
    else if (in_dtype == EI_F32 && out_dtype == EI_F32)
      EI_ROPE_VEC_G(float, float, 4);
    else if (in_dtype == EI_F32 && out_dtype == EI_BF16)
      EI_ROPE_VEC_G(float, bf16_t, 4);
    else if (in_dtype == EI_BF16 && out_dtype == EI_BF16)
      EI_ROPE_VEC_G(bf16_t, bf16_t, 4);
    else
      EI_REQUIRE(false, "qk_norm_rope_store: unsupported dtype combination");
#undef EI_ROPE_VEC_G
#undef EI_ROPE_VEC
    EI_LAUNCH_CHECK();
  }
  const long long waves = static_cast<long long>(N) * heads;
  const long long blocks = (waves * EI_WAVE + threads - 1) / threads;
  EI_REQUIRE(blocks < (1ll << 31), "qk_norm_rope_store: too many rows");
#define EI_ROPE_LAUNCH(TI, TO)                                                                   \
  qk_norm_rope_store_kernel<TI, TO><<<static_cast<unsigned>(blocks), threads, 0, stream>>>(      \
      static_cast<const TI*>(qkv), nsplit, ss, q_norm_w, k_norm_w, eps, rope_table, row_pos,     \
      row_seq, page_table, table_width, static_cast<TO*>(q_out), static_cast<TO*>(k_pages),      \
      static_cast<TO*>(v_pages), N, nq, nkv, D, R, write_cache)
  if (in_dtype == EI_F32 && out_dtype == EI_F32)
    EI_ROPE_LAUNCH(float, float);
  else if (in_dtype == EI_F32 && out_dtype == EI_BF16)
    EI_ROPE_LAUNCH(float, bf16_t);
  else if (in_dtype == EI_BF16 && out_dtype == EI_BF16)
    EI_ROPE_LAUNCH(bf16_t, bf16_t);
  else
    EI_REQUIRE(false, "qk_norm_rope_store: unsupported dtype combination");
#undef EI_ROPE_LAUNCH
  EI_LAUNCH_CHECK();
}
