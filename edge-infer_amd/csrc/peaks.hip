// Yardsticks for the measurements: how fast this GPU streams memory through a plain read
// kernel, how fast its matrix cores multiply when nothing else is asked of them, and what a
// chain of launches costs when the kernels do nothing.  The
// published peaks (8 TB/s, 2.5 PFLOP/s dense bfloat16) are what the figures are priced
// against; these kernels say how much of them any kernel can get on the machine at hand.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int kReadThreads = 256;
constexpr int kReadUnroll = 8;           // 16-byte loads a thread has in flight

// Every block walks the buffer with a grid stride, 8 loads of 16 bytes a thread at a time;
// the words are folded into one so that the loads cannot be dropped.
__global__ void __launch_bounds__(kReadThreads)
stream_read_kernel(const u32x4* __restrict__ data, long long count, uint32_t* __restrict__ sink) {
  const long long stride = static_cast<long long>(gridDim.x) * kReadThreads;
  uint32_t fold = 0;
  long long i = static_cast<long long>(blockIdx.x) * kReadThreads + threadIdx.x;
  for (; i + (kReadUnroll - 1) * stride < count; i += kReadUnroll * stride) {
    u32x4 v[kReadUnroll];
#pragma unroll
    for (int u = 0; u < kReadUnroll; ++u) v[u] = __builtin_nontemporal_load(data + i + u * stride);
#pragma unroll
    for (int u = 0; u < kReadUnroll; ++u) fold ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (; i < count; i += stride) {
    const u32x4 v = __builtin_nontemporal_load(data + i);
    fold ^= v.x ^ v.y ^ v.z ^ v.w;
  }
  if (fold == 0x9e3779b9u) sink[0] = fold;     // (practically never: the store keeps the loads)
}

// Each wave issues `iters` rounds of 8 independent 16x16x32 bfloat16 products on registers.
__global__ void __launch_bounds__(256)
mfma_loop_kernel(int iters, float* __restrict__ sink) {
  bf16x8 a, b;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    a[e] = static_cast<__bf16>(0.001f * static_cast<float>(threadIdx.x % 7 + e));
    b[e] = static_cast<__bf16>(0.002f * static_cast<float>(threadIdx.x % 5 + e));
  }
  f32x4 acc[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) acc[u] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int u = 0; u < 8; ++u)
      acc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[u], 0, 0, 0);
  }
  float total = 0.f;
#pragma unroll
  for (int u = 0; u < 8; ++u) total += acc[u][0] + acc[u][1] + acc[u][2] + acc[u][3];
  if (total == 12345.678f) sink[0] = total;
}

// The same with 32x32x16 products (32,768 flops each, 16 accumulator registers a product).
typedef float f32x16 __attribute__((ext_vector_type(16)));
__global__ void __launch_bounds__(256)
mfma_loop_wide_kernel(int iters, float* __restrict__ sink) {
  bf16x8 a, b;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    a[e] = static_cast<__bf16>(0.001f * static_cast<float>(threadIdx.x % 7 + e));
    b[e] = static_cast<__bf16>(0.002f * static_cast<float>(threadIdx.x % 5 + e));
  }
  f32x16 acc[4];
#pragma unroll
  for (int u = 0; u < 4; ++u)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[u][e] = 0.f;
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int u = 0; u < 4; ++u)
      acc[u] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[u], 0, 0, 0);
  }
  float total = 0.f;
#pragma unroll
  for (int u = 0; u < 4; ++u)
#pragma unroll
    for (int e = 0; e < 16; ++e) total += acc[u][e];
  if (total == 12345.678f) sink[0] = total;
}

// A kernel that does nothing: what a launch costs when nothing is computed.
__global__ void empty_kernel(int) {}

}  // namespace

// `count` launches of a kernel that does nothing, `blocks` blocks of one wave each, one after
// the other on `stream`: captured in a graph they are the floor under any chain of that many
// dependent kernels.
extern "C" int ei_empty_launches(int count, int blocks, hipStream_t stream) {
  EI_REQUIRE(count >= 1 && count <= 1 << 20 && blocks >= 1 && blocks <= 1 << 20,
             "empty_launches: bad sizes");
  for (int i = 0; i < count; ++i) empty_kernel<<<blocks, EI_WAVE, 0, stream>>>(i);
  EI_LAUNCH_CHECK();
}

// Reads `bytes` (a multiple of 16) from `data` once, with `blocks` blocks of 256 threads.
extern "C" int ei_stream_read(const void* data, long long bytes, int blocks, void* sink,
                              hipStream_t stream) {
  EI_REQUIRE(data && sink && bytes >= 16 && bytes % 16 == 0, "stream_read: bad buffer");
  EI_REQUIRE(blocks >= 1 && blocks <= 1 << 20, "stream_read: bad block count");
  stream_read_kernel<<<blocks, kReadThreads, 0, stream>>>(
      static_cast<const u32x4*>(data), bytes / 16, static_cast<uint32_t*>(sink));
  EI_LAUNCH_CHECK();
}

// `blocks` blocks of 4 waves each do `iters` rounds of 131,072 flops a wave: 8 products of
// 16x16x32 (wide = 0) or 4 of 32x32x16 (wide = 1).
extern "C" int ei_mfma_loop(int iters, int blocks, int wide, void* sink, hipStream_t stream) {
  EI_REQUIRE(sink && iters >= 1 && blocks >= 1 && blocks <= 1 << 20, "mfma_loop: bad sizes");
  if (wide)
    mfma_loop_wide_kernel<<<blocks, 256, 0, stream>>>(iters, static_cast<float*>(sink));
  else
    mfma_loop_kernel<<<blocks, 256, 0, stream>>>(iters, static_cast<float*>(sink));
  EI_LAUNCH_CHECK();
}
