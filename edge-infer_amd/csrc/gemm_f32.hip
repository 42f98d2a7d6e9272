// True float32 matrix product C[M, N] = A[M, K] . W[N, K]^T for the 32-bit path:
// float32 inputs, float32 fused multiply-adds, no reduced-precision matrix mode.
// W is a checkpoint matrix in its stored [out, in] layout (the reference multiplies
// the same bytes through cublasGemmEx with OP_T, operators/src/cuda/execution.cu:299-324).
//
// Every output element is accumulated over k in ascending order by one thread, so a
// row's result does not depend on which other rows are in the batch.
#include "common.cuh"

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

}  // namespace

extern "C" int ei_gemm_f32(const float* A, const float* W, float* C, int M, int N, int K,
                           long long lda, long long ldw, long long ldc, hipStream_t stream) {
  EI_REQUIRE(M > 0 && N > 0 && K > 0, "gemm_f32: sizes must be positive");
  EI_REQUIRE(A && W && C, "gemm_f32: null pointer");
  EI_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm_f32: leading dimension too small");
  const long long gy = (M + BM - 1) / BM;
  EI_REQUIRE(gy <= 65535, "gemm_f32: too many rows for one launch");
  dim3 grid((N + BN - 1) / BN, static_cast<unsigned>(gy));
  gemm_f32_kernel<<<grid, 256, 0, stream>>>(A, W, C, M, N, K, lda, ldw, ldc);
  EI_LAUNCH_CHECK();
}
