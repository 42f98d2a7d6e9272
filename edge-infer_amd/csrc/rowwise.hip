// Row-wise kernels of the decoder step: embedding gather, fused residual-add +
// RMSNorm (optionally on gathered rows), SiLU-gate product.  The residual stream is
// float32 in both precisions; sums of squares, the inverse RMS and the products
// are float32 and the result is rounded once to the output type.
//
// Formulas: operators/src/cuda/execution.cu:67-78 (gather),
// operators/src/cuda/rms_norm_cuda.cu:19-101 (x * rsqrt(mean(x^2) + eps) * w),
// operators/src/cuda/silu_cuda.cu:44-56 (silu(gate) * up) of the reference.
#include "common.h"

namespace {

template <typename T>
__global__ void embed_gather_kernel(const int32_t* __restrict__ ids, const T* __restrict__ table,
                                    float* __restrict__ out, int H, int V) {
  const int row = blockIdx.x;
  const int id = ids[row];
  float* dst = out + static_cast<size_t>(row) * H;
  if (id < 0 || id >= V) {
    for (int i = threadIdx.x; i < H; i += blockDim.x) dst[i] = 0.f;
    return;
  }
  const T* src = table + static_cast<size_t>(id) * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) dst[i] = ei::to_f32<T>(src[i]);
}

// One block per output row.  x = residual[src] (+ sum over splits of delta[s][src]);
// optionally stored back; out[row] = x * rsqrt(mean(x^2) + eps) * weight.
template <typename TD, typename TO, bool HAS_DELTA>
__global__ void add_rmsnorm_kernel(float* __restrict__ residual, const TD* __restrict__ delta,
                                   int nsplit, size_t split_stride,
                                   const int32_t* __restrict__ rows,
                                   const float* __restrict__ weight, float eps,
                                   TO* __restrict__ out, int H, int write_residual) {
  extern __shared__ float row_values[];
  __shared__ float scratch[16];
  const int row = blockIdx.x;
  const int src = rows ? rows[row] : row;
  if (src < 0) {  // padding row of a fixed-size batch: defined output, nothing else touched
    for (int i = threadIdx.x; i < H; i += blockDim.x)
      out[static_cast<size_t>(row) * H + i] = ei::from_f32<TO>(0.f);
    return;
  }
  float* res = residual + static_cast<size_t>(src) * H;
  float sum = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float x = res[i];
    if (HAS_DELTA) {
      const TD* d = delta + static_cast<size_t>(src) * H + i;
      for (int s = 0; s < nsplit; ++s) x += ei::to_f32<TD>(d[s * split_stride]);
      if (write_residual) res[i] = x;
    }
    row_values[i] = x;
    sum += x * x;
  }
  const float total = ei::block_sum(sum, scratch);
  const float inv = rsqrtf(total / static_cast<float>(H) + eps);
  TO* dst = out + static_cast<size_t>(row) * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x)
    dst[i] = ei::from_f32<TO>((row_values[i] * inv) * weight[i]);
}

// The same for widths that are a multiple of 4: 16-byte accesses, the row kept in
// registers, up to 1024 threads a row so that few rows still have many loads in flight.
using ei::Vec4;

#ifndef EI_NORM_FEW_ROWS_THREADS
#define EI_NORM_FEW_ROWS_THREADS 1024   // threads a row when rows are few (a build-time knob)
#endif

template <typename TD, typename TO, bool HAS_DELTA, int CHUNKS>
__global__ void add_rmsnorm_vec_kernel(float* __restrict__ residual, const TD* __restrict__ delta,
                                       int nsplit, size_t split_stride,
                                       const int32_t* __restrict__ rows,
                                       const float* __restrict__ weight, float eps,
                                       TO* __restrict__ out, int H, int write_residual) {
  __shared__ float scratch[16];
  const int row = blockIdx.x;
  const int src = rows ? rows[row] : row;
  const int quads = H / 4;
  TO* dst = out + static_cast<size_t>(row) * H;
  if (src < 0) {
    const float zero[4] = {0.f, 0.f, 0.f, 0.f};
    for (int qd = threadIdx.x; qd < quads; qd += blockDim.x) Vec4<TO>::store(dst + qd * 4, zero);
    return;
  }
  float* res = residual + static_cast<size_t>(src) * H;
  float w[CHUNKS][4];                      // asked for first: it depends on nothing
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k) {
    const int qd = threadIdx.x + k * blockDim.x;
    if (qd < quads) Vec4<float>::load(weight + qd * 4, w[k]);
  }
  float x[CHUNKS][4];
  float sum = 0.f;
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k) {
    const int qd = threadIdx.x + k * blockDim.x;
    x[k][0] = x[k][1] = x[k][2] = x[k][3] = 0.f;
    if (qd < quads) {
      Vec4<float>::load(res + qd * 4, x[k]);
      if (HAS_DELTA) {
        const TD* d = delta + static_cast<size_t>(src) * H + qd * 4;
        // slices are added in slice order; eight loads are issued before the first sum so
        // that a row costs one trip to memory per eight slices
        for (int s0 = 0; s0 < nsplit; s0 += 8) {
          float v[8][4];
#pragma unroll
          for (int u = 0; u < 8; ++u)
            if (s0 + u < nsplit) Vec4<TD>::load(d + (s0 + u) * split_stride, v[u]);
#pragma unroll
          for (int u = 0; u < 8; ++u)
            if (s0 + u < nsplit) {
#pragma unroll
              for (int i = 0; i < 4; ++i) x[k][i] += v[u][i];
            }
        }
        if (write_residual) Vec4<float>::store(res + qd * 4, x[k]);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) sum += x[k][i] * x[k][i];
    }
  }
  const float total = ei::block_sum(sum, scratch);
  const float inv = rsqrtf(total / static_cast<float>(H) + eps);
#pragma unroll
  for (int k = 0; k < CHUNKS; ++k) {
    const int qd = threadIdx.x + k * blockDim.x;
    if (qd < quads) {
      float y[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) y[i] = (x[k][i] * inv) * w[k][i];
      Vec4<TO>::store(dst + qd * 4, y);
    }
  }
}

// Where gate and up of output column `col` lie in a row of 2I: the halves [gate | up]
// (strip = 0), or strips of `strip` gate columns followed by their `strip` up columns.
__device__ __forceinline__ size_t gate_column(size_t col, int strip) {
  return strip ? (col / strip) * 2 * strip + col % strip : col;
}

template <typename TI, typename TO>
__global__ void swiglu_kernel(const TI* __restrict__ gate_up, int nsplit, size_t split_stride,
                              TO* __restrict__ out, int I, size_t total, int strip) {
  const size_t start = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t step = static_cast<size_t>(gridDim.x) * blockDim.x;
  const size_t up_offset = strip ? strip : I;
  for (size_t idx = start; idx < total; idx += step) {
    const size_t row = idx / I, col = idx % I;
    const TI* g = gate_up + row * 2 * I + gate_column(col, strip);
    float gate = 0.f, up = 0.f;
    for (int s = 0; s < nsplit; ++s) {
      gate += ei::to_f32<TI>(g[s * split_stride]);
      up += ei::to_f32<TI>(g[s * split_stride + up_offset]);
    }
    out[idx] = ei::from_f32<TO>(ei::silu<TO>(gate) * up);
  }
}

// The same for I a multiple of 8: a thread takes 8 neighbouring columns of one row with
// 16-byte (bfloat16) or 2 x 16-byte (float32) accesses.
template <typename TI, typename TO>
__global__ void swiglu_vec_kernel(const TI* __restrict__ gate_up, int nsplit, size_t split_stride,
                                  TO* __restrict__ out, int I, size_t total_octets, int strip) {
  const size_t start = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t step = static_cast<size_t>(gridDim.x) * blockDim.x;
  const int octets_per_row = I / 8;
  for (size_t idx = start; idx < total_octets; idx += step) {
    const size_t row = idx / octets_per_row;
    const int col = static_cast<int>(idx % octets_per_row) * 8;
    const TI* g = gate_up + row * 2 * I + gate_column(col, strip);   // strips hold whole octets
    const size_t up_offset = strip ? strip : I;
    float gate[8], up[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) gate[i] = up[i] = 0.f;
    for (int s0 = 0; s0 < nsplit; s0 += 4) {     // four slices per trip to memory
      float a[4][4], b[4][4], c[4][4], d[4][4];
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (s0 + u < nsplit) {
          const TI* p = g + (s0 + u) * split_stride;
          Vec4<TI>::load(p, a[u]);
          Vec4<TI>::load(p + 4, b[u]);
          Vec4<TI>::load(p + up_offset, c[u]);
          Vec4<TI>::load(p + up_offset + 4, d[u]);
        }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (s0 + u < nsplit) {
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            gate[i] += a[u][i];
            gate[i + 4] += b[u][i];
            up[i] += c[u][i];
            up[i + 4] += d[u][i];
          }
        }
    }
    float y0[4], y1[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      y0[i] = ei::silu<TO>(gate[i]) * up[i];
      y1[i] = ei::silu<TO>(gate[i + 4]) * up[i + 4];
    }
    TO* dst = out + row * I + col;
    Vec4<TO>::store(dst, y0);
    Vec4<TO>::store(dst + 4, y1);
  }
}

// out[i] = sum over slices s of in[s * stride + i], in slice order.
__global__ void sum_slices_kernel(const float* __restrict__ in, int nsplit, size_t stride,
                                  float* __restrict__ out, size_t n) {
  const size_t start = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t step = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = start; i < n; i += step) {
    float total = in[i];
    for (int s = 1; s < nsplit; ++s) total += in[s * stride + i];
    out[i] = total;
  }
}

// out[r, j] = bias[j] (+ out[r, j] when `accumulate`): a bias as one more slice of a sliced
// product, or added to a finished float32 product.
// operators/src/cuda/execution.cu:61-66,307-317 of the reference (the bias initialises the
// product's accumulator).
__global__ void bias_rows_kernel(const float* __restrict__ bias, float* __restrict__ out,
                                 size_t n, int width, int accumulate) {
  const size_t start = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const size_t step = static_cast<size_t>(gridDim.x) * blockDim.x;
  for (size_t i = start; i < n; i += step) {
    const float b = bias[i % width];
    out[i] = accumulate ? out[i] + b : b;
  }
}

}  // namespace

extern "C" int ei_bias_rows(const float* bias, float* out, long long rows, int width,
                            int accumulate, hipStream_t stream) {
  EI_REQUIRE(bias && out && rows > 0 && width > 0, "bias_rows: bad arguments");
  const size_t n = static_cast<size_t>(rows) * width;
  const int threads = 256;
  size_t blocks = (n + threads - 1) / threads;
  if (blocks > ei_compute_units() * 16) blocks = ei_compute_units() * 16;
  bias_rows_kernel<<<static_cast<unsigned>(blocks), threads, 0, stream>>>(bias, out, n, width,
                                                                         accumulate);
  EI_LAUNCH_CHECK();
}

extern "C" int ei_sum_slices(const float* in, int nsplit, long long stride, float* out,
                             long long n, hipStream_t stream) {
  EI_REQUIRE(in && out && nsplit >= 1 && n > 0 && stride >= n, "sum_slices: bad arguments");
  const int threads = 256;
  long long blocks = (n + threads - 1) / threads;
  if (blocks > ei_compute_units() * 16) blocks = ei_compute_units() * 16;
  sum_slices_kernel<<<static_cast<unsigned>(blocks), threads, 0, stream>>>(
      in, nsplit, static_cast<size_t>(stride), out, static_cast<size_t>(n));
  EI_LAUNCH_CHECK();
}

extern "C" int ei_embed_gather(const int32_t* ids, const void* table, int table_dtype, float* out,
                               int N, int H, int V, hipStream_t stream) {
  EI_REQUIRE(N > 0 && H > 0 && V > 0, "embed_gather: sizes must be positive");
  EI_REQUIRE(ids && table && out, "embed_gather: null pointer");
  const int threads = H >= 1024 ? 256 : 64;
  if (table_dtype == EI_F32)
    embed_gather_kernel<float><<<N, threads, 0, stream>>>(ids, static_cast<const float*>(table),
                                                          out, H, V);
  else if (table_dtype == EI_BF16)
    embed_gather_kernel<bf16_t><<<N, threads, 0, stream>>>(ids, static_cast<const bf16_t*>(table),
                                                           out, H, V);
  else
    EI_REQUIRE(false, "embed_gather: unknown table dtype");
  EI_LAUNCH_CHECK();
}

template <typename TD, typename TO>
static void launch_add_rmsnorm(float* residual, const void* delta, int nsplit, size_t split_stride,
                               const int32_t* rows, const float* weight, float eps, void* out,
                               int N, int H, int write_residual, hipStream_t stream) {
  if (H % 4 == 0 && (!delta || split_stride % 4 == 0)) {
    const int quads = H / 4;
    // few rows: up to 1024 threads a row, so that many loads are in flight; many rows: 256
    // threads a row, so that several rows share a compute unit and overlap their phases
    const int most = N >= 512 && quads <= 4 * 256 ? 256 : EI_NORM_FEW_ROWS_THREADS;
    int threads = (quads + EI_WAVE - 1) / EI_WAVE * EI_WAVE;
    if (threads > most) threads = most;
    const int chunks = (quads + threads - 1) / threads;      // 1..4 for H <= 16384
#define EI_NORM_VEC(C)                                                                         \
  do {                                                                                         \
    if (delta)                                                                                 \
      add_rmsnorm_vec_kernel<TD, TO, true, C><<<N, threads, 0, stream>>>(                      \
          residual, static_cast<const TD*>(delta), nsplit, split_stride, rows, weight, eps,    \
          static_cast<TO*>(out), H, write_residual);                                           \
    else                                                                                       \
      add_rmsnorm_vec_kernel<TD, TO, false, C><<<N, threads, 0, stream>>>(                     \
          residual, nullptr, 0, 0, rows, weight, eps, static_cast<TO*>(out), H, 0);            \
  } while (0)
    if (chunks == 1) EI_NORM_VEC(1);
    else if (chunks == 2) EI_NORM_VEC(2);
    else EI_NORM_VEC(4);
#undef EI_NORM_VEC
    return;
  }
  const int threads = H >= 2048 ? 256 : (H >= 256 ? 128 : 64);
  const size_t lds = static_cast<size_t>(H) * sizeof(float);
  if (delta)
    add_rmsnorm_kernel<TD, TO, true><<<N, threads, lds, stream>>>(
        residual, static_cast<const TD*>(delta), nsplit, split_stride, rows, weight, eps,
        static_cast<TO*>(out), H, write_residual);
  else
    add_rmsnorm_kernel<TD, TO, false><<<N, threads, lds, stream>>>(
        residual, nullptr, 0, 0, rows, weight, eps, static_cast<TO*>(out), H, 0);
}

// residual: float32 [*, H].  delta: [nsplit][*, H] of delta_dtype or null.  rows: null
// (row r reads residual row r) or int32 [N] source rows (negative: padding).
extern "C" int ei_add_rmsnorm(float* residual, const void* delta, int delta_dtype, int nsplit,
                              long long split_stride, const int32_t* rows, const float* weight,
                              float eps, void* out, int out_dtype, int N, int H,
                              int write_residual, hipStream_t stream) {
  EI_REQUIRE(N > 0 && H > 0, "add_rmsnorm: sizes must be positive");
  EI_REQUIRE(H <= 16384, "add_rmsnorm: width above 16384 is not supported");
  EI_REQUIRE(residual && weight && out, "add_rmsnorm: null pointer");
  EI_REQUIRE(!delta || nsplit >= 1, "add_rmsnorm: nsplit must be at least 1");
  EI_REQUIRE(eps > 0.f, "add_rmsnorm: eps must be positive");
  const size_t ss = static_cast<size_t>(split_stride);
  if (delta_dtype == EI_F32 && out_dtype == EI_F32)
    launch_add_rmsnorm<float, float>(residual, delta, nsplit, ss, rows, weight, eps, out, N, H,
                                     write_residual, stream);
  else if (delta_dtype == EI_F32 && out_dtype == EI_BF16)
    launch_add_rmsnorm<float, bf16_t>(residual, delta, nsplit, ss, rows, weight, eps, out, N, H,
                                      write_residual, stream);
  else if (delta_dtype == EI_BF16 && out_dtype == EI_BF16)
    launch_add_rmsnorm<bf16_t, bf16_t>(residual, delta, nsplit, ss, rows, weight, eps, out, N, H,
                                       write_residual, stream);
  else if (delta_dtype == EI_BF16 && out_dtype == EI_F32)
    launch_add_rmsnorm<bf16_t, float>(residual, delta, nsplit, ss, rows, weight, eps, out, N, H,
                                      write_residual, stream);
  else
    EI_REQUIRE(false, "add_rmsnorm: unknown dtype");
  EI_LAUNCH_CHECK();
}

// gate_up: [nsplit][N, 2I], out: [N, I].  strip = 0: gate columns first, then up columns;
// strip > 0 (a divisor of I): `strip` gate columns, their `strip` up columns, and so on.
extern "C" int ei_swiglu(const void* gate_up, int in_dtype, int nsplit, long long split_stride,
                         void* out, int out_dtype, int N, int I, int strip, hipStream_t stream) {
  EI_REQUIRE(N > 0 && I > 0 && nsplit >= 1, "swiglu: sizes must be positive");
  EI_REQUIRE(gate_up && out, "swiglu: null pointer");
  EI_REQUIRE(strip >= 0 && (strip == 0 || I % strip == 0), "swiglu: the strip must divide the width");
  const size_t total = static_cast<size_t>(N) * I;
  const int threads = 256;
  const size_t ss = static_cast<size_t>(split_stride);
  if (I % 8 == 0 && ss % 8 == 0 && strip % 8 == 0) {
    const size_t octets = total / 8;
    size_t vblocks = (octets + threads - 1) / threads;
    if (vblocks > ei_compute_units() * 32) vblocks = ei_compute_units() * 32;
    if (in_dtype == EI_F32 && out_dtype == EI_F32)
      swiglu_vec_kernel<float, float><<<vblocks, threads, 0, stream>>>(
          static_cast<const float*>(gate_up), nsplit, ss, static_cast<float*>(out), I, octets, strip);
    else if (in_dtype == EI_F32 && out_dtype == EI_BF16)
      swiglu_vec_kernel<float, bf16_t><<<vblocks, threads, 0, stream>>>(
          static_cast<const float*>(gate_up), nsplit, ss, static_cast<bf16_t*>(out), I, octets, strip);
    else if (in_dtype == EI_BF16 && out_dtype == EI_BF16)
      swiglu_vec_kernel<bf16_t, bf16_t><<<vblocks, threads, 0, stream>>>(
          static_cast<const bf16_t*>(gate_up), nsplit, ss, static_cast<bf16_t*>(out), I, octets, strip);
    else
      EI_REQUIRE(false, "swiglu: unsupported dtype combination");
    EI_LAUNCH_CHECK();
  }
  size_t blocks = (total + threads - 1) / threads;
  if (blocks > ei_compute_units() * 32) blocks = ei_compute_units() * 32;
  if (in_dtype == EI_F32 && out_dtype == EI_F32)
    swiglu_kernel<float, float><<<blocks, threads, 0, stream>>>(
        static_cast<const float*>(gate_up), nsplit, ss, static_cast<float*>(out), I, total, strip);
  else if (in_dtype == EI_F32 && out_dtype == EI_BF16)
    swiglu_kernel<float, bf16_t><<<blocks, threads, 0, stream>>>(
        static_cast<const float*>(gate_up), nsplit, ss, static_cast<bf16_t*>(out), I, total, strip);
  else if (in_dtype == EI_BF16 && out_dtype == EI_BF16)
    swiglu_kernel<bf16_t, bf16_t><<<blocks, threads, 0, stream>>>(
        static_cast<const bf16_t*>(gate_up), nsplit, ss, static_cast<bf16_t*>(out), I, total, strip);
  else
    EI_REQUIRE(false, "swiglu: unsupported dtype combination");
  EI_LAUNCH_CHECK();
}
