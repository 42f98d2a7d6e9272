// Shared device helpers for the gfx950 kernels: wave64 reductions, bf16 <-> f32
// conversion (round to nearest even), typed loads/stores, launch checking.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

#define EI_WAVE 64
#define EI_PAGE 64  // tokens of one sequence that a cache page holds

// dtype codes of the C interface
#define EI_F32 0
#define EI_BF16 1

typedef uint16_t bf16_t;  // raw bfloat16 bits

namespace ei {

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
  return __uint_as_float(static_cast<uint32_t>(v) << 16);
}

// round to nearest even; NaN stays NaN (one v_cvt_pk_bf16_f32 on gfx950)
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  const __bf16 h = static_cast<__bf16>(f);
  return __builtin_bit_cast(bf16_t, h);
}

template <typename T> __device__ __forceinline__ float to_f32(T v);
template <> __device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_f32<bf16_t>(bf16_t v) { return bf16_to_f32(v); }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return f32_to_bf16(v); }

// Four neighbouring values as float: one 16-byte (float32) or 8-byte (bfloat16) access.
template <typename T> struct Vec4;
template <> struct Vec4<float> {
  static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
    const float4 x = *reinterpret_cast<const float4*>(p);
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  }
};
template <> struct Vec4<bf16_t> {
  static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[4]) {
    const uint2 x = *reinterpret_cast<const uint2*>(p);
    v[0] = __uint_as_float(x.x << 16); v[1] = __uint_as_float(x.x & 0xffff0000u);
    v[2] = __uint_as_float(x.y << 16); v[3] = __uint_as_float(x.y & 0xffff0000u);
  }
  static __device__ __forceinline__ void store(bf16_t* p, const float (&v)[4]) {
    uint2 x;
    x.x = static_cast<uint32_t>(f32_to_bf16(v[0])) | (static_cast<uint32_t>(f32_to_bf16(v[1])) << 16);
    x.y = static_cast<uint32_t>(f32_to_bf16(v[2])) | (static_cast<uint32_t>(f32_to_bf16(v[3])) << 16);
    *reinterpret_cast<uint2*>(p) = x;
  }
};

// P consecutive elements (4 or 8) of type T as floats; eight bfloat16 travel as one 16-byte
// access.
template <typename T, int P> struct VecN;
template <typename T> struct VecN<T, 4> : Vec4<T> {};
template <> struct VecN<float, 8> {
  static __device__ __forceinline__ void load(const float* p, float (&v)[8]) {
    const float4 x = *reinterpret_cast<const float4*>(p), y = *reinterpret_cast<const float4*>(p + 4);
    v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
    v[4] = y.x; v[5] = y.y; v[6] = y.z; v[7] = y.w;
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[8]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
  }
};
template <> struct VecN<bf16_t, 8> {
  static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[8]) {
    const uint4 x = *reinterpret_cast<const uint4*>(p);
    const uint32_t u[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __uint_as_float(u[i] << 16);
      v[2 * i + 1] = __uint_as_float(u[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ void store(bf16_t* p, const float (&v)[8]) {
    uint32_t u[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      u[i] = static_cast<uint32_t>(f32_to_bf16(v[2 * i])) |
             (static_cast<uint32_t>(f32_to_bf16(v[2 * i + 1])) << 16);
    *reinterpret_cast<uint4*>(p) = uint4{u[0], u[1], u[2], u[3]};
  }
};

// x / (1 + e^-x).  For a float32 result the library's exponential and a true division;
// for a bfloat16 result (8 bits of mantissa) the hardware's exp2 and reciprocal, both good
// to about one unit in the 23rd bit, which the rounding to bfloat16 swallows.
template <typename TO> __device__ __forceinline__ float silu(float x);
template <> __device__ __forceinline__ float silu<float>(float x) { return x / (1.0f + expf(-x)); }
template <> __device__ __forceinline__ float silu<bf16_t>(float x) {
  const float e = __builtin_amdgcn_exp2f(fmaxf(x, -80.f) * -1.44269504088896341f);
  return x * __builtin_amdgcn_rcpf(1.0f + e);
}

// Reductions over the four 16-lane rows of a wave (lanes l, l^16, l^32, l^48), every lane
// getting the result.  gfx950's row-swap instructions do each step in the vector ALU: with
// both operands holding x, v_permlane32_swap leaves (x of the lower half, x of the upper
// half) in all lanes of the two registers, v_permlane16_swap the same for neighbouring rows;
// a shuffle through LDS (ds_bpermute) costs an LDS round trip instead.
typedef unsigned int ei_u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float rows_max(float x) {
  ei_u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = fmaxf(__uint_as_float(r.x), __uint_as_float(r.y));
  r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r.x), __uint_as_float(r.y));
}

__device__ __forceinline__ float rows_sum(float x) {
  ei_u32x2 r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  x = __uint_as_float(r.x) + __uint_as_float(r.y);
  r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r.x) + __uint_as_float(r.y);
}

// Sum over the 64 lanes, every lane getting it.  The steps inside a row of 16 lanes are DPP
// operand modifiers of vector adds (quad permutes, then mirrors of half rows and rows), the
// two across rows are gfx950's row swaps; no step goes through LDS as a shuffle would.
__device__ __forceinline__ float wave_sum(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xb1, 0xf, 0xf, false));   // quad_perm [1,0,3,2]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4e, 0xf, 0xf, false));   // quad_perm [2,3,0,1]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, false));  // row_half_mirror
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xf, 0xf, false));  // row_mirror
  return rows_sum(v);
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int offset = EI_WAVE / 2; offset > 0; offset >>= 1)
    v = fmaxf(v, __shfl_xor(v, offset, EI_WAVE));
  return v;
}

// Sum over a block of `blockDim.x` threads (a multiple of 64, at most 1024).
// `scratch` holds at least 16 floats.  Every thread gets the total.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x / EI_WAVE, lane = threadIdx.x % EI_WAVE;
  const int waves = blockDim.x / EI_WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int i = 0; i < waves; ++i) total += scratch[i];
  return total;
}

}  // namespace ei

// Host side ---------------------------------------------------------------
// Each kernel library is one translation unit and carries its own message buffer.
#include <string.h>
static thread_local char ei_error_text[512];
static inline void ei_set_error(const char* message) {
  strncpy(ei_error_text, message, sizeof(ei_error_text) - 1);
  ei_error_text[sizeof(ei_error_text) - 1] = 0;
}
extern "C" const char* ei_last_error() { return ei_error_text; }

// Compute units of the current device, asked of the runtime once per device (256 on an
// MI355X).  Launch plans that deal blocks out to the units take the count from here.
static inline int ei_compute_units() {
  static int known[64] = {0};
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return 256;
  if (known[device] == 0) {
    int count = 0;
    if (hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess ||
        count < 1)
      count = 256;
    known[device] = count;
  }
  return known[device];
}

#define EI_REQUIRE(cond, msg)       \
  do {                              \
    if (!(cond)) {                  \
      ei_set_error(msg);            \
      return -1;                    \
    }                               \
  } while (0)

#define EI_LAUNCH_CHECK()                         \
  do {                                            \
    hipError_t e_ = hipGetLastError();            \
    if (e_ != hipSuccess) {                       \
      ei_set_error(hipGetErrorString(e_));        \
      return static_cast<int>(e_);                \
    }                                             \
    return 0;                                     \
  } while (0)
