// Weight-streaming matrix product for few rows (decode): out[s][m][n] = partial sums of
// X[m, :] . W[n, :] over the s-th slice of K, for M <= 64 rows of X.
//
// W is a bfloat16 checkpoint matrix in its stored [N, K] layout and is read exactly once,
// straight from global memory into MFMA operand registers: with v_mfma_f32_16x16x32_bf16 a
// lane supplies 8 consecutive k of one row, and because a dot product does not care in
// which order k is visited, lane (row r, quarter c) takes the contiguous run
// k0 + c*KT/4 .. + KT/4 of its row and feeds it to successive MFMAs, eight elements at a
// time.  X (tiny) is staged through LDS once per workgroup and K-tile and read with the same
// k mapping; the next tiles of W and X are already on their way while a tile is multiplied.  A workgroup is 4 waves, each owning 16 rows of W; K may be split over
// blockIdx.y, in which case every slice writes float32 partial sums [slice, M, N] that the
// consuming kernel adds in slice order while it reads them (deterministic, no atomics, and
// no device-wide fence: the kernel boundary orders the writes before the reads).
//
// Accumulation is float32 throughout, as in the reference's cublasGemmEx call
// (operators/src/cuda/execution.cu:319-323); the sums stay float32 and the consumer rounds
// once when it stores in the storage type.
#include "common.cuh"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * EI_WAVE;
constexpr int kRowsPerBlock = kWaves * 16;
constexpr int kPackedTile = 16 * 32;      // elements of one packed tile: 16 rows x 32 k, 1 KB

// Address of the 16-byte piece that lane `lane` takes of the packed tile (kt, strip).
__device__ __forceinline__ const bf16_t* packed_piece(const bf16_t* Wp, int n_strips, int kt,
                                                      int strip, int lane) {
  return Wp + (static_cast<size_t>(kt) * n_strips + strip) * kPackedTile + lane * 8;
}

template <int MB, int KT, bool PACKED>
__global__ void __launch_bounds__(kThreads)
skinny_gemm_kernel(const bf16_t* __restrict__ W, const bf16_t* __restrict__ X,
                   float* __restrict__ out, int M, int N, int K, int k_per_split) {
  constexpr int JN = KT / 32;             // MFMA steps per K-tile
  constexpr int ROWS_X = MB * 16;
  constexpr int XS = KT + 8;              // LDS row stride in elements (16 bytes of padding)
  constexpr int CHUNKS = ROWS_X * (KT / 8);
  constexpr int XLOADS = CHUNKS / kThreads;
  static_assert(CHUNKS % kThreads == 0, "X tile must divide among the threads");
  __shared__ __attribute__((aligned(16))) bf16_t xs[ROWS_X * XS];

  const int t = threadIdx.x;
  const int wave = t / EI_WAVE, lane = t % EI_WAVE;
  const int r16 = lane & 15, c = lane >> 4;
  const int n_tile = blockIdx.x * kRowsPerBlock + wave * 16;
  const int k_begin = blockIdx.y * k_per_split;
  const int k_end = min(K, k_begin + k_per_split);
  const int n_iter = (k_end - k_begin + KT - 1) / KT;

  int w_row = n_tile + r16;
  if (w_row >= N) w_row = N - 1;          // rows past the end repeat the last one; never stored
  const int n_strips = (N + 15) / 16;
  const int strip = min(n_tile / 16, n_strips - 1);
  const bf16_t* w_ptr = PACKED ? packed_piece(W, n_strips, 0, strip, lane)
                               : W + static_cast<size_t>(w_row) * K + c * 8;
  const size_t tile_stride = static_cast<size_t>(n_strips) * kPackedTile;

  f32x4 acc[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) acc[mb] = f32x4{0.f, 0.f, 0.f, 0.f};

  bf16x8 w_a[JN], w_b[JN];
  u32x4 x_regs[XLOADS];
  const u32x4 zero4 = u32x4{0u, 0u, 0u, 0u};

  auto load_w = [&](bf16x8* dst, int kb) {
#pragma unroll
    for (int j = 0; j < JN; ++j) {
      if (PACKED) {
        // the packed copy holds whole K-tiles (zeros past K): no test, so that the loads
        // form one straight run whose arrival the compiler can count
        dst[j] = __builtin_nontemporal_load(
            reinterpret_cast<const bf16x8*>(w_ptr + (kb / 32 + j) * tile_stride));
        continue;
      }
      const int k = kb + j * 32 + c * 8;
      if (k < k_end) {
        dst[j] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(w_ptr + kb + j * 32));
      } else {
        dst[j] = __builtin_bit_cast(bf16x8, zero4);
      }
    }
  };
  auto load_x = [&](int kb) {
#pragma unroll
    for (int i = 0; i < XLOADS; ++i) {
      const int q = t + i * kThreads;
      const int row = q / (KT / 8), ch = q % (KT / 8);
      const int k = kb + ch * 8;
      x_regs[i] = (row < M && k < k_end)
                      ? *reinterpret_cast<const u32x4*>(X + static_cast<size_t>(row) * K + k)
                      : zero4;
    }
  };
  auto store_x = [&]() {
#pragma unroll
    for (int i = 0; i < XLOADS; ++i) {
      const int q = t + i * kThreads;
      const int row = q / (KT / 8), ch = q % (KT / 8);
      *reinterpret_cast<u32x4*>(&xs[row * XS + ch * 8]) = x_regs[i];
    }
  };
  auto compute = [&](const bf16x8* w) {
#pragma unroll
    for (int j = 0; j < JN; ++j) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const bf16x8 xv = *reinterpret_cast<const bf16x8*>(
            &xs[(mb * 16 + r16) * XS + j * 32 + c * 8]);
        acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[j], xv, acc[mb], 0, 0, 0);
      }
    }
  };
  // Two register sets for W alternate, so that a tile is never copied (a copy would wait
  // for its loads at once); the next tiles of W and X travel while this one is multiplied.
  if (n_iter > 0) {
    load_w(w_a, k_begin);
    load_x(k_begin);
  }
  for (int it = 0; it < n_iter; it += 2) {
    __syncthreads();                      // the previous tile of X has been read by everyone
    store_x();
    __syncthreads();
    if (it + 1 < n_iter) {
      load_w(w_b, k_begin + (it + 1) * KT);
      load_x(k_begin + (it + 1) * KT);
    }
    compute(w_a);
    if (it + 1 < n_iter) {
      __syncthreads();
      store_x();
      __syncthreads();
      if (it + 2 < n_iter) {
        load_w(w_a, k_begin + (it + 2) * KT);
        load_x(k_begin + (it + 2) * KT);
      }
      compute(w_b);
    }
  }

  // lane (c, r16) holds out[m = mb*16 + r16][n_tile + 4c + 0..3]
  float* dst = out + static_cast<size_t>(blockIdx.y) * M * N;
  const int n0 = n_tile + 4 * c;
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int m = mb * 16 + r16;
    if (m >= M) continue;
    float* p = dst + static_cast<size_t>(m) * N + n0;
    if (n0 + 3 < N && (N & 3) == 0) {
      *reinterpret_cast<f32x4*>(p) = acc[mb];
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (n0 + r < N) p[r] = acc[mb][r];
    }
  }
}

// Up to 16 rows of X and a K range of at most kPreloadK: the whole X slice is put into LDS
// once, after which the four waves stream their rows of W without meeting again.
constexpr int kPreloadK = 1024;

template <bool PACKED>
__global__ void __launch_bounds__(kThreads)
skinny_gemm_preload_kernel(const bf16_t* __restrict__ W, const bf16_t* __restrict__ X,
                           float* __restrict__ out, int M, int N, int K, int k_per_split,
                           int row_tiles) {
  constexpr int KT = 256, JN = KT / 32;
  constexpr int XS = kPreloadK + 8;
  __shared__ __attribute__((aligned(16))) bf16_t xs[16 * XS];

  const int t = threadIdx.x;
  const int wave = t / EI_WAVE, lane = t % EI_WAVE;
  const int r16 = lane & 15, c = lane >> 4;
  const int k_begin = blockIdx.y * k_per_split;
  const int k_end = min(K, k_begin + k_per_split);
  const int k_len = k_end - k_begin;                 // a multiple of 8, at most kPreloadK
  const int n_iter = (k_len + KT - 1) / KT;

  // X slice -> LDS: 16 rows (zeros past M and past the slice), 16-byte chunks, at most 8
  // per thread.  Every load is issued (from a clamped address) before the first is used.
  const u32x4 zero4 = u32x4{0u, 0u, 0u, 0u};
  const int chunks_per_row = n_iter * (KT / 8);
  constexpr int XCH = 16 * (kPreloadK / 8) / kThreads;
  u32x4 xv[XCH];
#pragma unroll
  for (int i = 0; i < XCH; ++i) {
    const int q = t + i * kThreads;
    const int row = q / chunks_per_row, k = (q % chunks_per_row) * 8;
    const bool valid = row < M && k < k_len;
    const u32x4 v = *reinterpret_cast<const u32x4*>(
        X + static_cast<size_t>(valid ? row : 0) * K + k_begin + (valid ? k : 0));
    xv[i] = valid ? v : zero4;
  }
  auto store_x = [&]() {                               // after the first loads of W are issued
#pragma unroll
    for (int i = 0; i < XCH; ++i) {
      const int q = t + i * kThreads;
      const int row = q / chunks_per_row, k = (q % chunks_per_row) * 8;
      if (row < 16) *reinterpret_cast<u32x4*>(&xs[row * XS + k]) = xv[i];
    }
  };
  const bf16_t* x_ptr = &xs[r16 * XS + c * 8];

  // The block owns `row_tiles` consecutive groups of 64 rows of W (16 per wave); the walk
  // over (group, K-tile) is one flat pipeline with two tiles of W in flight per wave.
  const int first_group = blockIdx.x * row_tiles;
  const int total = row_tiles * n_iter;
  const int n_strips = (N + 15) / 16;
  const size_t tile_stride = static_cast<size_t>(n_strips) * kPackedTile;
  auto w_pointer = [&](int group) {
    if (PACKED) {
      const int strip = min((first_group + group) * kWaves + wave, n_strips - 1);
      return packed_piece(W, n_strips, k_begin / 32, strip, lane);
    }
    int row = (first_group + group) * kRowsPerBlock + wave * 16 + r16;
    if (row >= N) row = N - 1;                        // repeats the last row; never stored
    return W + static_cast<size_t>(row) * K + k_begin + c * 8;
  };
  bf16x8 w_a[JN], w_b[JN];
  auto load_w = [&](bf16x8* dst, int step) {          // step = group * n_iter + tile
    const bf16_t* w_ptr = w_pointer(step / n_iter);
    const int kb = (step % n_iter) * KT;
#pragma unroll
    for (int j = 0; j < JN; ++j) {
      if (PACKED) {
        dst[j] = __builtin_nontemporal_load(
            reinterpret_cast<const bf16x8*>(w_ptr + (kb / 32 + j) * tile_stride));
        continue;
      }
      if (kb + j * 32 + c * 8 < k_len) {
        dst[j] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(w_ptr + kb + j * 32));
      } else {
        dst[j] = __builtin_bit_cast(bf16x8, zero4);
      }
    }
  };
  f32x4 acc0 = f32x4{0.f, 0.f, 0.f, 0.f}, acc1 = acc0;
  float* dst = out + static_cast<size_t>(blockIdx.y) * M * N;
  auto compute = [&](const bf16x8* w, int step) {
    const int kb = (step % n_iter) * KT;
#pragma unroll
    for (int j = 0; j < JN; j += 2) {
      const bf16x8 x0 = *reinterpret_cast<const bf16x8*>(x_ptr + kb + j * 32);
      const bf16x8 x1 = *reinterpret_cast<const bf16x8*>(x_ptr + kb + (j + 1) * 32);
      acc0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[j], x0, acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[j + 1], x1, acc1, 0, 0, 0);
    }
    if (step % n_iter == n_iter - 1) {                // a group of rows is complete
      const f32x4 acc = acc0 + acc1;
      acc0 = acc1 = f32x4{0.f, 0.f, 0.f, 0.f};
      const int n0 = (first_group + step / n_iter) * kRowsPerBlock + wave * 16 + 4 * c;
      if (r16 < M) {
        float* p = dst + static_cast<size_t>(r16) * N + n0;
        if (n0 + 3 < N && (N & 3) == 0) {
          *reinterpret_cast<f32x4*>(p) = acc;
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (n0 + r < N) p[r] = acc[r];
        }
      }
    }
  };
  // The loads of the steady loop are unconditional, so that on every path into a product
  // the same number of loads is outstanding and the wait before it can let the younger
  // tile stay in flight; the last two or three steps are peeled off.
  if (total == 1) {
    load_w(w_a, 0);
    store_x();
    __syncthreads();
    compute(w_a, 0);
    return;
  }
  load_w(w_a, 0);
  load_w(w_b, 1);
  store_x();
  __syncthreads();
  int step = 0;
  for (; step + 3 < total; step += 2) {
    compute(w_a, step);
    load_w(w_a, step + 2);
    compute(w_b, step + 1);
    load_w(w_b, step + 3);
  }
  compute(w_a, step);
  if (step + 2 < total) {
    load_w(w_a, step + 2);
    compute(w_b, step + 1);
    compute(w_a, step + 2);
  } else {
    compute(w_b, step + 1);
  }
}

int tile_for(int MB) { (void)MB; return 256; }

}  // namespace

// The number of K slices the kernel will use for these sizes (the caller sizes `out`).
// More slices for fewer rows: the partial sums cost M * N * 8 bytes of traffic per slice.
extern "C" int ei_skinny_gemm_splits(int M, int N, int K, int target_blocks) {
  if (M < 1 || N < 1 || K < 1) return 1;
  const int MB = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  const int KT = tile_for(MB);
  const int row_blocks = (N + kRowsPerBlock - 1) / kRowsPerBlock;
  const int k_tiles = (K + KT - 1) / KT;
  if (target_blocks <= 0) target_blocks = 512;
  int splits = (target_blocks + row_blocks - 1) / row_blocks;
  const int max_splits = MB == 1 ? 16 : (MB == 2 ? 8 : 4);
  if (splits > max_splits) splits = max_splits;
  if (MB == 1) {
    // slices of at most kPreloadK let the kernel keep its X slice in LDS
    const int need = (K + kPreloadK - 1) / kPreloadK;
    if (splits < need && need <= 16) splits = need;
  }
  if (splits > k_tiles) splits = k_tiles;
  if (splits < 1) splits = 1;
  const int tiles_per_split = (k_tiles + splits - 1) / splits;
  return (k_tiles + tiles_per_split - 1) / tiles_per_split;
}

// X: [M, K] bfloat16, W: [N, K] bfloat16, out: [splits, M, N] float32 (slice s holds the
// sums over the s-th part of K).  K must be a multiple of 8 (16-byte loads), M at most 64.
namespace {

template <bool PACKED>
int launch_skinny(const void* X, const void* W, float* out, int M, int N, int K, int splits,
                  hipStream_t stream) {
  EI_REQUIRE(M >= 1 && M <= 64, "gemm_bf16_skinny: rows must lie in 1..64");
  EI_REQUIRE(N >= 1 && K >= 8 && K % 8 == 0, "gemm_bf16_skinny: K must be a multiple of 8");
  EI_REQUIRE(X && W && out, "gemm_bf16_skinny: null pointer");

  EI_REQUIRE((reinterpret_cast<uintptr_t>(X) & 15) == 0 && (reinterpret_cast<uintptr_t>(W) & 15) == 0 &&
                 (reinterpret_cast<uintptr_t>(out) & 15) == 0,
             "gemm_bf16_skinny: pointers must be 16-byte aligned");
  const int MB = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  const int KT = tile_for(MB);
  const int k_tiles = (K + KT - 1) / KT;
  EI_REQUIRE(splits >= 1 && splits <= k_tiles, "gemm_bf16_skinny: bad slice count");
  const int tiles_per_split = (k_tiles + splits - 1) / splits;
  EI_REQUIRE((k_tiles + tiles_per_split - 1) / tiles_per_split == splits,
             "gemm_bf16_skinny: slice count leaves an empty slice");
  const int k_per_split = tiles_per_split * KT;
  const int row_blocks = (N + kRowsPerBlock - 1) / kRowsPerBlock;
  dim3 grid(row_blocks, splits);
  const bf16_t* x = static_cast<const bf16_t*>(X);
  const bf16_t* w = static_cast<const bf16_t*>(W);
  if (MB == 1 && k_per_split <= kPreloadK) {
    // fat blocks for tall matrices: several groups of 64 rows share one staged X slice,
    // as long as some 768 blocks remain
    int row_tiles = static_cast<int>(static_cast<long long>(row_blocks) * splits / 768);
    if (row_tiles < 1) row_tiles = 1;
    if (row_tiles > 8) row_tiles = 8;
    dim3 fat((row_blocks + row_tiles - 1) / row_tiles, splits);
    skinny_gemm_preload_kernel<PACKED><<<fat, kThreads, 0, stream>>>(w, x, out, M, N, K,
                                                                     k_per_split, row_tiles);
  }
  else if (MB == 1)
    skinny_gemm_kernel<1, 256, PACKED><<<grid, kThreads, 0, stream>>>(w, x, out, M, N, K, k_per_split);
  else if (MB == 2)
    skinny_gemm_kernel<2, 256, PACKED><<<grid, kThreads, 0, stream>>>(w, x, out, M, N, K, k_per_split);
  else
    skinny_gemm_kernel<4, 256, PACKED><<<grid, kThreads, 0, stream>>>(w, x, out, M, N, K, k_per_split);
  EI_LAUNCH_CHECK();
}

}  // namespace

// X: [M, K] bfloat16, W: [N, K] bfloat16, out: [splits, M, N] float32 (slice s holds the
// sums over the s-th part of K).  K must be a multiple of 8 (16-byte loads), M at most 64.
extern "C" int ei_gemm_bf16_skinny(const void* X, const void* W, float* out, int M, int N, int K,
                                   int splits, hipStream_t stream) {
  return launch_skinny<false>(X, W, out, M, N, K, splits, stream);
}

// The same product with W in the streaming layout: tiles of 16 rows x 32 k (1 KB each, rows
// past N and k past K zero, K padded to a multiple of 256 so that every K-tile of the kernel
// is whole), tile (kt, strip) at index kt * ceil(N/16) + strip, and inside a
// tile the piece of lane (c = k/8 % 4, r = row % 16) at (c * 16 + r) * 8 elements, i.e. the
// order in which a wave's lanes hold an MFMA operand.  A wave's load is then one contiguous
// kilobyte and the waves that run together read neighbouring kilobytes, which keeps every
// memory channel busy; rows of W that are 2^n bytes apart do not.
extern "C" int ei_gemm_bf16_skinny_packed(const void* X, const void* Wp, float* out, int M, int N,
                                          int K, int splits, hipStream_t stream) {
  return launch_skinny<true>(X, Wp, out, M, N, K, splits, stream);
}
