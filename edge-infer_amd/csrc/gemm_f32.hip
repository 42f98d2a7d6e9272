// True float32 matrix product C[M, N] = A[M, K] . W[N, K]^T for the 32-bit path:
// float32 inputs, float32 fused multiply-adds, no reduced-precision matrix mode.
// W is a checkpoint matrix in its stored [out, in] layout (the reference multiplies
// the same bytes through cublasGemmEx with OP_T, operators/src/cuda/execution.cu:299-324).
//
// Every output element is accumulated over k in ascending order by one thread, so a
// row's result does not depend on which other rows are in the batch, nor on which of the
// kernels below computed it: two tiled ones (64 x 64 outputs a block; 128 x 128 for many rows
// with K in fours) and the weight-streaming one for up to 8 rows (decode), which reads every
// weight row in kilobyte pieces.
#include "common.h"

namespace {

constexpr int BM = 64, BN = 64, BK = 16, TM = 4, TN = 4;

__global__ void __launch_bounds__(256)
gemm_f32_kernel(const float* __restrict__ A, const float* __restrict__ W, float* __restrict__ C,
                int M, int N, int K, long long lda, long long ldw, long long ldc) {
  __shared__ float As[BK][BM + 4];
  __shared__ float Ws[BK][BN + 4];
  const int t = threadIdx.x;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int ty = t / 16, tx = t % 16;
  float acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = 0.f;

  const int lrow = t / 4, lk = (t % 4) * 4;
  for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int k = k0 + lk + e;
      const int am = m0 + lrow, wn = n0 + lrow;
      As[lk + e][lrow] = (am < M && k < K) ? A[static_cast<size_t>(am) * lda + k] : 0.f;
      Ws[lk + e][lrow] = (wn < N && k < K) ? W[static_cast<size_t>(wn) * ldw + k] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      float a[TM], w[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = As[k][ty * TM + i];
#pragma unroll
      for (int j = 0; j < TN; ++j) w[j] = Ws[k][tx * TN + j];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + ty * TM + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + tx * TN + j;
      if (n < N) C[static_cast<size_t>(m) * ldc + n] = acc[i][j];
    }
  }
}

// Many rows (prefill): tiles of 128 x 128 outputs, 8 x 8 of them a thread (as two by two
// groups of 4 x 4, so that LDS is read in 16-byte pieces), the next K-tile on its way in
// registers while this one is multiplied.  The same sums in the same order as above.
constexpr int GM = 128, GN = 128, GK = 16, GS = GM + 4;

__global__ void __launch_bounds__(256)
gemm_f32_large_kernel(const float* __restrict__ A, const float* __restrict__ W,
                      float* __restrict__ C, int M, int N, int K, long long lda, long long ldw,
                      long long ldc) {
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  __shared__ __attribute__((aligned(16))) float As[GK * GS];
  __shared__ __attribute__((aligned(16))) float Ws[GK * GS];
  const int t = threadIdx.x, ty = t / 16, tx = t % 16;
  const int m0 = blockIdx.y * GM, n0 = blockIdx.x * GN;
  const f32x4 zero = f32x4{0.f, 0.f, 0.f, 0.f};
  float acc[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = 0.f;
  // thread -> two 16-byte pieces of each tile: row f / 4, floats 4 (f % 4) .. + 3, f = t, t + 256
  f32x4 a_next[2], w_next[2];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int f = t + 256 * i, row = f / 4, k = k0 + 4 * (f % 4);
      a_next[i] = (m0 + row < M && k < K)
                      ? *reinterpret_cast<const f32x4*>(A + static_cast<size_t>(m0 + row) * lda + k)
                      : zero;
      w_next[i] = (n0 + row < N && k < K)
                      ? *reinterpret_cast<const f32x4*>(W + static_cast<size_t>(n0 + row) * ldw + k)
                      : zero;
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += GK) {
    __syncthreads();                      // the previous tile has been read
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int f = t + 256 * i, row = f / 4, kq = 4 * (f % 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        As[(kq + e) * GS + row] = a_next[i][e];
        Ws[(kq + e) * GS + row] = w_next[i][e];
      }
    }
    __syncthreads();
    if (k0 + GK < K) fetch(k0 + GK);
#pragma unroll
    for (int k = 0; k < GK; ++k) {
      const f32x4 a0 = *reinterpret_cast<const f32x4*>(&As[k * GS + ty * 4]);
      const f32x4 a1 = *reinterpret_cast<const f32x4*>(&As[k * GS + 64 + ty * 4]);
      const f32x4 w0 = *reinterpret_cast<const f32x4*>(&Ws[k * GS + tx * 4]);
      const f32x4 w1 = *reinterpret_cast<const f32x4*>(&Ws[k * GS + 64 + tx * 4]);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          acc[i][j] = fmaf(a0[i], w0[j], acc[i][j]);
          acc[i][4 + j] = fmaf(a0[i], w1[j], acc[i][4 + j]);
          acc[4 + i][j] = fmaf(a1[i], w0[j], acc[4 + i][j]);
          acc[4 + i][4 + j] = fmaf(a1[i], w1[j], acc[4 + i][4 + j]);
        }
    }
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int m = m0 + (i / 4) * 64 + ty * 4 + i % 4;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int n = n0 + (j / 4) * 64 + tx * 4 + j % 4;
      if (n < N) C[static_cast<size_t>(m) * ldc + n] = acc[i][j];
    }
  }
}

// Up to 8 rows of A (decode).  One wave per block and 16 rows of W: the wave loads 16 x 256
// floats of W a tile (a contiguous kilobyte per row and instruction) into registers, a tile
// ahead of the one it multiplies from LDS.  Lane (n = lane % 16, g = lane / 16) sums output
// column n of rows g and g + 4 over k in ascending order with the same fused multiply-adds
// as the tiled kernel, so both give the same bits.
constexpr int FN = 16, FK = 256, FS = FK + 4;     // LDS row stride: 16-byte rows, no bank conflicts

template <int RPG>   // rows of A per lane group: 1 (M <= 4) or 2 (M <= 8)
__global__ void __launch_bounds__(EI_WAVE)
gemm_f32_few_rows_kernel(const float* __restrict__ A, const float* __restrict__ W,
                         float* __restrict__ C, int M, int N, int K, long long lda,
                         long long ldw, long long ldc) {
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  __shared__ __attribute__((aligned(16))) float Ws[FN * FS];
  __shared__ __attribute__((aligned(16))) float Xs[4 * RPG * FS];
  const int lane = threadIdx.x, n = lane % FN, g = lane / FN;
  const int n0 = blockIdx.x * FN;
  const f32x4 zero = f32x4{0.f, 0.f, 0.f, 0.f};
  f32x4 w_next[FN], x_next[4 * RPG];
  // lane takes floats 4 * lane .. + 3 of the tile of every row (rows past the end: zeros)
  auto fetch = [&](int k0) {
    const int k = k0 + 4 * lane;
#pragma unroll
    for (int i = 0; i < FN; ++i)
      w_next[i] = (n0 + i < N && k < K)
                      ? *reinterpret_cast<const f32x4*>(W + static_cast<size_t>(n0 + i) * ldw + k)
                      : zero;
#pragma unroll
    for (int m = 0; m < 4 * RPG; ++m)
      x_next[m] = (m < M && k < K)
                      ? *reinterpret_cast<const f32x4*>(A + static_cast<size_t>(m) * lda + k)
                      : zero;
  };
  float acc[RPG];
#pragma unroll
  for (int r = 0; r < RPG; ++r) acc[r] = 0.f;
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += FK) {
    __syncthreads();                      // the previous tile has been read
#pragma unroll
    for (int i = 0; i < FN; ++i) *reinterpret_cast<f32x4*>(&Ws[i * FS + 4 * lane]) = w_next[i];
#pragma unroll
    for (int m = 0; m < 4 * RPG; ++m)
      *reinterpret_cast<f32x4*>(&Xs[m * FS + 4 * lane]) = x_next[m];
    __syncthreads();
    if (k0 + FK < K) fetch(k0 + FK);      // on its way while this tile is multiplied
#pragma unroll 8
    for (int k4 = 0; k4 < FK / 4; ++k4) {
      const f32x4 w = *reinterpret_cast<const f32x4*>(&Ws[n * FS + 4 * k4]);
#pragma unroll
      for (int r = 0; r < RPG; ++r) {
        const f32x4 x = *reinterpret_cast<const f32x4*>(&Xs[(g + 4 * r) * FS + 4 * k4]);
        acc[r] = fmaf(x[0], w[0], acc[r]);
        acc[r] = fmaf(x[1], w[1], acc[r]);
        acc[r] = fmaf(x[2], w[2], acc[r]);
        acc[r] = fmaf(x[3], w[3], acc[r]);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < RPG; ++r) {
    const int m = g + 4 * r;
    if (m < M && n0 + n < N) C[static_cast<size_t>(m) * ldc + n0 + n] = acc[r];
  }
}

}  // namespace

extern "C" int ei_gemm_f32(const float* A, const float* W, float* C, int M, int N, int K,
                           long long lda, long long ldw, long long ldc, hipStream_t stream) {
  EI_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_f32: sizes must be positive");
  EI_REQUIRE(A && W && C, "gemm_f32: null pointer");
  EI_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm_f32: leading dimension too small");
  // few rows: the weight-streaming kernel (16-byte loads: K and the leading dimensions in
  // fours, pointers aligned)
  const bool fours = K % 4 == 0 && lda % 4 == 0 && ldw % 4 == 0 &&
                     ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(W)) & 15) == 0;
  if (M <= 8 && fours) {
    const unsigned blocks = static_cast<unsigned>((N + FN - 1) / FN);
    if (M <= 4)
      gemm_f32_few_rows_kernel<1><<<blocks, EI_WAVE, 0, stream>>>(A, W, C, M, N, K, lda, ldw, ldc);
    else
      gemm_f32_few_rows_kernel<2><<<blocks, EI_WAVE, 0, stream>>>(A, W, C, M, N, K, lda, ldw, ldc);
    EI_LAUNCH_CHECK();
  }
  if (M > 64 && fours) {
    const long long rows = (M + GM - 1) / GM;
    EI_REQUIRE(rows <= 65535, "gemm_f32: too many rows for one launch");
    dim3 tiles((N + GN - 1) / GN, static_cast<unsigned>(rows));
    gemm_f32_large_kernel<<<tiles, 256, 0, stream>>>(A, W, C, M, N, K, lda, ldw, ldc);
    EI_LAUNCH_CHECK();
  }
  const long long gy = (M + BM - 1) / BM;
  EI_REQUIRE(gy <= 65535, "gemm_f32: too many rows for one launch");
  dim3 grid((N + BN - 1) / BN, static_cast<unsigned>(gy));
  gemm_f32_kernel<<<grid, 256, 0, stream>>>(A, W, C, M, N, K, lda, ldw, ldc);
  EI_LAUNCH_CHECK();
}
