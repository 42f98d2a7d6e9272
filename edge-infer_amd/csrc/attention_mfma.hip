// bfloat16 attention over the paged cache for head sizes 64 and 128, on the matrix cores.
//
// Decode (one query position per sequence): a block of four waves owns one
// (sequence, kv head, slice of the key range); a wave walks 16-key tiles.  Scores come from
// v_mfma_f32_16x16x32_bf16 with the key tile as the A operand (a lane loads 16 bytes of one
// key row straight from the cache page) and the group's query heads as the B operand; the
// softmax state (running maximum, sum) is float32 per head; the value product is done with
// float32 multiply-adds on value rows that are loaded fully coalesced, because it needs no
// transposed operand that way and the step is bound by memory, not arithmetic.  The four
// waves merge through LDS; slices are merged by attn_merge_kernel.
//
// Mathematics as in attention_generic.hip (operators/src/cuda/execution.cu:137-179 and
// operators/src/cuda/kernels/flash_attention_variable.cu:121-295 of the reference): keys
// t <= p (and t > p - window), scale 1/sqrt(d) or the given one, float32 softmax.
#include "common.cuh"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int kWaves = 4;
constexpr int kThreads = kWaves * EI_WAVE;
constexpr int kTile = 16;          // keys per MFMA tile
constexpr float kLowest = -1.0e30f;

__device__ __forceinline__ float bf16_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }

// GB: query heads of the kv group handled by this block (1..16).
template <int D, int GB>
__global__ void __launch_bounds__(kThreads)
attn_decode_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pages,
                   const bf16_t* __restrict__ v_pages, const int32_t* __restrict__ row_pos,
                   const int32_t* __restrict__ row_seq, const int32_t* __restrict__ page_table,
                   int table_width, bf16_t* __restrict__ out, float* __restrict__ part_o,
                   float* __restrict__ part_ml, int nq, int nkv, int head_blocks, int window,
                   float scale, int n_splits) {
  constexpr int DJ = D / 32;            // MFMA steps over the head dimension
  constexpr int LPR = D / 8;            // lanes that cover one value row with 16-byte loads
  constexpr int KPI = EI_WAVE / LPR;    // value rows per load instruction
  constexpr int VI = kTile / KPI;       // value load instructions per tile
  __shared__ float p_lds[kWaves][kTile][16];
  __shared__ float alpha_lds[kWaves][16];
  __shared__ float m_lds[kWaves][16], l_lds[kWaves][16];
  __shared__ float o_lds[kWaves][GB][D];

  const int row = blockIdx.x;                      // packed row = sequence index in decode
  const int g = blockIdx.y / head_blocks, hb = blockIdx.y % head_blocks;
  const int split = blockIdx.z;
  const int seq = row_seq[row];
  if (seq < 0) return;                             // padding row
  const int G = nq / nkv;
  const int t = threadIdx.x, wave = t / EI_WAVE, lane = t % EI_WAVE;
  const int r16 = lane & 15, c = lane >> 4;
  const int pos = row_pos[row];
  const int head0 = g * G + hb * GB;               // first query head of this block
  const int heads_here = min(GB, G - hb * GB);

  // query heads as the B operand: lane (n = r16, c) holds q[head n][j*32 + c*8 .. +8]
  bf16x8 q_reg[DJ];
#pragma unroll
  for (int j = 0; j < DJ; ++j) {
    uint4 z = uint4{0u, 0u, 0u, 0u};
    if (r16 < heads_here)
      z = *reinterpret_cast<const uint4*>(q + (static_cast<size_t>(row) * nq + head0 + r16) * D +
                                          j * 32 + c * 8);
    q_reg[j] = *reinterpret_cast<bf16x8*>(&z);
  }

  const int lo_key = window > 0 ? max(0, pos - window + 1) : 0;
  const int first_tile = lo_key / kTile, last_tile = pos / kTile;
  const int total_tiles = last_tile - first_tile + 1;
  // slices are cut at page boundaries so that they do not depend on the tile size
  const int lo_page = lo_key / EI_PAGE, hi_page = pos / EI_PAGE;
  const int pages = hi_page - lo_page + 1;
  const int per = (pages + n_splits - 1) / n_splits;
  const int tile_begin = max(first_tile, (lo_page + split * per) * (EI_PAGE / kTile));
  const int tile_end = min(last_tile + 1, (lo_page + (split + 1) * per) * (EI_PAGE / kTile));
  (void)total_tiles;

  float m_run = kLowest, l_run = 0.f;              // state of head r16 (same in all four c)
  float acc[GB][8];
#pragma unroll
  for (int h = 0; h < GB; ++h)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[h][e] = 0.f;
  const int ks = lane / LPR, dc = lane % LPR;       // value rows: key sub-index, 8-wide chunk

  for (int tile = tile_begin + wave; tile < tile_end; tile += kWaves) {
    const int key0 = tile * kTile;
    const int phys = page_table[static_cast<size_t>(seq) * table_width + key0 / EI_PAGE];
    if (phys < 0) continue;                        // released by the window: all masked
    const size_t page_base = (static_cast<size_t>(phys) * nkv + g) * EI_PAGE * D;
    const int in_page = key0 % EI_PAGE;
    // keys: A operand, lane (key r16, c) holds k[key][j*32 + c*8 .. +8]
    bf16x8 k_reg[DJ];
    const bf16_t* kp = k_pages + page_base + static_cast<size_t>(in_page + r16) * D + c * 8;
#pragma unroll
    for (int j = 0; j < DJ; ++j) k_reg[j] = *reinterpret_cast<const bf16x8*>(kp + j * 32);
    // values: lane (ks, dc) holds v[key0 + i*KPI + ks][dc*8 .. +8]
    uint4 v_reg[VI];
    const bf16_t* vp = v_pages + page_base + static_cast<size_t>(in_page + ks) * D + dc * 8;
#pragma unroll
    for (int i = 0; i < VI; ++i)
      v_reg[i] = *reinterpret_cast<const uint4*>(vp + static_cast<size_t>(i) * KPI * D);

    f32x4 s = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int j = 0; j < DJ; ++j)
      s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k_reg[j], q_reg[j], s, 0, 0, 0);
    // lane (c, n = r16) holds the scores of keys key0 + 4c + r for head n
    float sc[4];
    float tile_max = kLowest;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int key = key0 + 4 * c + r;
      const bool visible = key <= pos && key >= lo_key;
      sc[r] = visible ? s[r] * scale : -INFINITY;
      tile_max = fmaxf(tile_max, sc[r]);
    }
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, EI_WAVE));
    tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, EI_WAVE));
    const float m_new = fmaxf(m_run, tile_max);
    const float alpha = expf(m_run - m_new);
    float tile_sum = 0.f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float p = expf(sc[r] - m_new);
      p_lds[wave][4 * c + r][r16] = p;
      tile_sum += p;
    }
    tile_sum += __shfl_xor(tile_sum, 16, EI_WAVE);
    tile_sum += __shfl_xor(tile_sum, 32, EI_WAVE);
    l_run = l_run * alpha + tile_sum;
    m_run = m_new;
    if (c == 0) alpha_lds[wave][r16] = alpha;
    // the wave's own LDS rows: a wave executes in lockstep, but the compiler must not
    // move the reads above the writes
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int h = 0; h < GB; ++h) {
      const float a = alpha_lds[wave][h];
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[h][e] *= a;
    }
#pragma unroll
    for (int i = 0; i < VI; ++i) {
      const int key_local = i * KPI + ks;
      const bool live = key0 + key_local <= pos;    // later slots hold stale bytes
      const uint4 raw = live ? v_reg[i] : uint4{0u, 0u, 0u, 0u};
      float v[8];
      v[0] = bf16_lo(raw.x); v[1] = bf16_hi(raw.x); v[2] = bf16_lo(raw.y); v[3] = bf16_hi(raw.y);
      v[4] = bf16_lo(raw.z); v[5] = bf16_hi(raw.z); v[6] = bf16_lo(raw.w); v[7] = bf16_hi(raw.w);
#pragma unroll
      for (int h = 0; h < GB; ++h) {
        const float p = p_lds[wave][key_local][h];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[h][e] = fmaf(p, v[e], acc[h][e]);
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }

  // sum the partial outputs of the KPI key sub-groups inside the wave
#pragma unroll
  for (int h = 0; h < GB; ++h)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float x = acc[h][e];
#pragma unroll
      for (int offset = LPR; offset < EI_WAVE; offset <<= 1) x += __shfl_xor(x, offset, EI_WAVE);
      acc[h][e] = x;
    }
  if (c == 0) {
    m_lds[wave][r16] = m_run;
    l_lds[wave][r16] = l_run;
  }
  if (ks == 0) {
#pragma unroll
    for (int h = 0; h < GB; ++h)
#pragma unroll
      for (int e = 0; e < 8; ++e) o_lds[wave][h][dc * 8 + e] = acc[h][e];
  }
  __syncthreads();
  // merge the four waves: thread -> (head, d), strided
  for (int idx = t; idx < heads_here * D; idx += kThreads) {
    const int h = idx / D, d = idx % D;
    float m = kLowest;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) m = fmaxf(m, m_lds[w][h]);
    float l = 0.f, o = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const float f = expf(m_lds[w][h] - m);
      l += l_lds[w][h] * f;
      o += o_lds[w][h][d] * f;
    }
    const int head = head0 + h;
    if (n_splits == 1) {
      out[(static_cast<size_t>(row) * nq + head) * D + d] =
          ei::from_f32<bf16_t>(l > 0.f ? o / l : 0.f);
    } else {
      const size_t slot = (static_cast<size_t>(row) * nq + head) * n_splits + split;
      part_o[slot * D + d] = o;
      if (d == 0) {
        part_ml[slot * 2] = m;
        part_ml[slot * 2 + 1] = l;
      }
    }
  }
}

// One wave per (row, head): o = sum_s o_s e^{m_s - m} / sum_s l_s e^{m_s - m}.
__global__ void attn_merge_kernel(const float* __restrict__ part_o,
                                  const float* __restrict__ part_ml,
                                  const int32_t* __restrict__ row_seq, bf16_t* __restrict__ out,
                                  int nq, int D, int n_splits, int total) {
  const int wave = (blockIdx.x * blockDim.x + threadIdx.x) / EI_WAVE;
  const int lane = threadIdx.x % EI_WAVE;
  if (wave >= total) return;
  if (row_seq[wave / nq] < 0) return;
  const float* ml = part_ml + static_cast<size_t>(wave) * n_splits * 2;
  float m = kLowest;
  for (int s = 0; s < n_splits; ++s) m = fmaxf(m, ml[2 * s]);
  float l = 0.f;
  for (int s = 0; s < n_splits; ++s) l += ml[2 * s + 1] * expf(ml[2 * s] - m);
  const float inv = l > 0.f ? 1.f / l : 0.f;
  const float* po = part_o + static_cast<size_t>(wave) * n_splits * D;
  for (int d = lane; d < D; d += EI_WAVE) {
    float o = 0.f;
    for (int s = 0; s < n_splits; ++s) o += po[static_cast<size_t>(s) * D + d] * expf(ml[2 * s] - m);
    out[static_cast<size_t>(wave) * D + d] = ei::from_f32<bf16_t>(o * inv);
  }
}

template <int D, int GB>
void launch_decode(dim3 grid, hipStream_t stream, const bf16_t* q, const bf16_t* k,
                   const bf16_t* v, const int32_t* row_pos, const int32_t* row_seq,
                   const int32_t* page_table, int table_width, bf16_t* out, float* part_o,
                   float* part_ml, int nq, int nkv, int head_blocks, int window, float scale,
                   int n_splits) {
  attn_decode_kernel<D, GB><<<grid, kThreads, 0, stream>>>(
      q, k, v, row_pos, row_seq, page_table, table_width, out, part_o, part_ml, nq, nkv,
      head_blocks, window, scale, n_splits);
}

}  // namespace

// Whether the decode kernel of this file takes a head size and group ratio.
extern "C" int ei_attn_decode_mfma_supported(int D, int G) {
  return (D == 64 || D == 128) && G >= 1 ? 1 : 0;
}

// q, out: [rows, nq, D] bfloat16, one row per sequence (row_seq < 0: padding row);
// pages: [n_pages, nkv, 64, D]; n_splits > 1 needs part_o [rows, nq, n_splits, D] and
// part_ml [rows, nq, n_splits, 2] float32.
extern "C" int ei_attention_decode_mfma(const void* q, const void* k_pages, const void* v_pages,
                                        const int32_t* row_pos, const int32_t* row_seq,
                                        const int32_t* page_table, int table_width, void* out,
                                        float* part_o, float* part_ml, int rows, int nq, int nkv,
                                        int D, int window, float scale, int n_splits,
                                        hipStream_t stream) {
  EI_REQUIRE(rows > 0 && nq > 0 && nkv > 0 && nq % nkv == 0, "attention_decode: bad head counts");
  EI_REQUIRE(D == 64 || D == 128, "attention_decode: this kernel takes head_dim 64 or 128");
  EI_REQUIRE(q && k_pages && v_pages && row_pos && row_seq && page_table && out && table_width > 0,
             "attention_decode: null pointer");
  EI_REQUIRE(n_splits >= 1 && n_splits <= 64, "attention_decode: splits must be between 1 and 64");
  EI_REQUIRE(n_splits == 1 || (part_o && part_ml), "attention_decode: split scratch missing");
  EI_REQUIRE(window >= 0, "attention_decode: negative window");
  const int G = nq / nkv;
  const int GB = G >= 8 ? (G >= 16 ? 16 : 8) : (G >= 4 ? 4 : (G >= 2 ? 2 : 1));
  const int head_blocks = (G + GB - 1) / GB;
  EI_REQUIRE(static_cast<long long>(nkv) * head_blocks <= 65535, "attention_decode: too many heads");
  dim3 grid(rows, nkv * head_blocks, n_splits);
  const bf16_t* qq = static_cast<const bf16_t*>(q);
  const bf16_t* kk = static_cast<const bf16_t*>(k_pages);
  const bf16_t* vv = static_cast<const bf16_t*>(v_pages);
  bf16_t* oo = static_cast<bf16_t*>(out);
#define EI_DECODE(DD, GG)                                                                     \
  launch_decode<DD, GG>(grid, stream, qq, kk, vv, row_pos, row_seq, page_table, table_width,  \
                        oo, part_o, part_ml, nq, nkv, head_blocks, window, scale, n_splits)
#define EI_DECODE_G(DD)            \
  switch (GB) {                    \
    case 1: EI_DECODE(DD, 1); break;   \
    case 2: EI_DECODE(DD, 2); break;   \
    case 4: EI_DECODE(DD, 4); break;   \
    case 8: EI_DECODE(DD, 8); break;   \
    default: EI_DECODE(DD, 16); break; \
  }
  if (D == 64) {
    EI_DECODE_G(64)
  } else {
    EI_DECODE_G(128)
  }
#undef EI_DECODE_G
#undef EI_DECODE
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    ei_set_error(hipGetErrorString(e));
    return static_cast<int>(e);
  }
  if (n_splits > 1) {
    const int total = rows * nq;
    const int threads = 256;
    const int blocks = (total * EI_WAVE + threads - 1) / threads;
    attn_merge_kernel<<<blocks, threads, 0, stream>>>(part_o, part_ml, row_seq, oo, nq, D,
                                                      n_splits, total);
  }
  EI_LAUNCH_CHECK();
}
