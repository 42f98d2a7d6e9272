// Weight-streaming matrix product for few rows (decode): out[s][m][n] = partial sums of
// X[m, :] . W[n, :] over the s-th slice of K, for M <= 64 rows of X.
//
// W is a bfloat16 checkpoint matrix in its stored [N, K] layout and is read exactly once,
// straight from global memory into MFMA operand registers: with v_mfma_f32_16x16x32_bf16 a
// lane supplies 8 consecutive k of one row, and because a dot product does not care in
// which order k is visited, lane (row r, quarter c) takes the contiguous run
// k0 + c*KT/4 .. + KT/4 of its row and feeds it to successive MFMAs, eight elements at a
// time.  Each row of a 16-row tile is then read in runs of KT*2 contiguous bytes.  X (tiny)
// is staged through LDS once per workgroup and K-tile, double-buffered, and read with the
// same k mapping.  A workgroup is 4 waves, each owning 16 rows of W; K may be split over
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

namespace {

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * EI_WAVE;
constexpr int kRowsPerBlock = kWaves * 16;

template <int MB, int KT>
__global__ void __launch_bounds__(kThreads)
skinny_gemm_kernel(const bf16_t* __restrict__ W, const bf16_t* __restrict__ X,
                   float* __restrict__ out, int M, int N, int K, int k_per_split) {
  constexpr int JN = KT / 32;             // MFMA steps per K-tile
  constexpr int ROWS_X = MB * 16;
  constexpr int XS = KT + 8;              // LDS row stride in elements (16 bytes of padding)
  constexpr int CHUNKS = ROWS_X * (KT / 8);
  constexpr int XLOADS = CHUNKS / kThreads;
  static_assert(CHUNKS % kThreads == 0, "X tile must divide among the threads");
  __shared__ __attribute__((aligned(16))) bf16_t xs[2][ROWS_X * XS];

  const int t = threadIdx.x;
  const int wave = t / EI_WAVE, lane = t % EI_WAVE;
  const int r16 = lane & 15, c = lane >> 4;
  const int n_tile = blockIdx.x * kRowsPerBlock + wave * 16;
  const int k_begin = blockIdx.y * k_per_split;
  const int k_end = min(K, k_begin + k_per_split);
  const int n_iter = (k_end - k_begin + KT - 1) / KT;

  int w_row = n_tile + r16;
  if (w_row >= N) w_row = N - 1;          // rows past the end repeat the last one; never stored
  const bf16_t* w_ptr = W + static_cast<size_t>(w_row) * K + c * 8;

  f32x4 acc[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) acc[mb] = f32x4{0.f, 0.f, 0.f, 0.f};

  bf16x8 w_cur[JN], w_next[JN];
  uint4 x_regs[XLOADS];
  const uint4 zero4 = uint4{0u, 0u, 0u, 0u};

  auto load_w = [&](bf16x8* dst, int kb) {
#pragma unroll
    for (int j = 0; j < JN; ++j) {
      const int k = kb + j * 32 + c * 8;
      if (k < k_end) {
        dst[j] = *reinterpret_cast<const bf16x8*>(w_ptr + kb + j * 32);
      } else {
        uint4 z = zero4;
        dst[j] = *reinterpret_cast<bf16x8*>(&z);
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
                      ? *reinterpret_cast<const uint4*>(X + static_cast<size_t>(row) * K + k)
                      : zero4;
    }
  };
  auto store_x = [&](int buf) {
#pragma unroll
    for (int i = 0; i < XLOADS; ++i) {
      const int q = t + i * kThreads;
      const int row = q / (KT / 8), ch = q % (KT / 8);
      *reinterpret_cast<uint4*>(&xs[buf][row * XS + ch * 8]) = x_regs[i];
    }
  };

  if (n_iter > 0) {
    load_w(w_cur, k_begin);
    load_x(k_begin);
    store_x(0);
  }
  __syncthreads();
  for (int it = 0; it < n_iter; ++it) {
    const int kb_next = k_begin + (it + 1) * KT;
    const bool more = it + 1 < n_iter;
    if (more) {
      load_w(w_next, kb_next);
      load_x(kb_next);
    }
    const bf16_t* xb = &xs[it & 1][0];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
#pragma unroll
      for (int j = 0; j < JN; ++j) {
        const bf16x8 xv = *reinterpret_cast<const bf16x8*>(
            xb + (mb * 16 + r16) * XS + j * 32 + c * 8);
        acc[mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_cur[j], xv, acc[mb], 0, 0, 0);
      }
    }
    if (more) {
      store_x((it + 1) & 1);
#pragma unroll
      for (int j = 0; j < JN; ++j) w_cur[j] = w_next[j];
    }
    __syncthreads();
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

int tile_for(int MB) { return MB == 4 ? 128 : 256; }

}  // namespace

// The number of K slices the kernel will use for these sizes (the caller sizes `out`).
// More slices for fewer rows: the partial sums cost M * N * 8 bytes of traffic per slice.
extern "C" int ei_skinny_gemm_splits(int M, int N, int K, int target_blocks) {
  if (M < 1 || N < 1 || K < 1) return 1;
  const int MB = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  const int KT = tile_for(MB);
  const int row_blocks = (N + kRowsPerBlock - 1) / kRowsPerBlock;
  const int k_tiles = (K + KT - 1) / KT;
  if (target_blocks <= 0) target_blocks = MB == 4 ? 512 : 1024;
  int splits = (target_blocks + row_blocks - 1) / row_blocks;
  const int max_splits = MB == 1 ? 16 : (MB == 2 ? 8 : 4);
  if (splits > max_splits) splits = max_splits;
  if (splits > k_tiles) splits = k_tiles;
  if (splits < 1) splits = 1;
  const int tiles_per_split = (k_tiles + splits - 1) / splits;
  return (k_tiles + tiles_per_split - 1) / tiles_per_split;
}

// X: [M, K] bfloat16, W: [N, K] bfloat16, out: [splits, M, N] float32 (slice s holds the
// sums over the s-th part of K).  K must be a multiple of 8 (16-byte loads), M at most 64.
extern "C" int ei_gemm_bf16_skinny(const void* X, const void* W, float* out, int M, int N, int K,
                                   int splits, hipStream_t stream) {
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
  if (MB == 1)
    skinny_gemm_kernel<1, 256><<<grid, kThreads, 0, stream>>>(w, x, out, M, N, K, k_per_split);
  else if (MB == 2)
    skinny_gemm_kernel<2, 256><<<grid, kThreads, 0, stream>>>(w, x, out, M, N, K, k_per_split);
  else
    skinny_gemm_kernel<4, 128><<<grid, kThreads, 0, stream>>>(w, x, out, M, N, K, k_per_split);
  EI_LAUNCH_CHECK();
}
