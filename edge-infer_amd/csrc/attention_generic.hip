// Causal grouped-query attention over the paged cache, any head size that is a
// multiple of 16 up to 256, any head and group counts, float32 or bfloat16
// storage, float32 arithmetic throughout (scores, running maximum, exponentials,
// sums and the value accumulation).  One kernel serves prefill (many positions of a
// sequence) and decode (one position, the key range split over several blocks and
// merged by a second kernel).
//
// Mathematics of the reference: s_t = (q . k_t) / sqrt(d) for keys t <= p (and
// t > p - window when a window is set), streaming softmax with a running maximum,
// o = sum w_t v_t / sum w_t; query head h reads kv head h / (nq / nkv).
// operators/src/cuda/execution.cu:137-179, runtime/src/qwen.cpp:374-402,
// split merge: operators/src/cuda/kernels/gather_fa_variable.cu:14-118.
#include "common.h"

namespace {

constexpr int kRows = 16;     // query rows (positions x heads of one kv group) per block
constexpr int kThreads = 256;
constexpr float kLowest = -1.0e30f;

// Work item: `npos` consecutive packed rows starting at `row0`, all of sequence `seq`.
template <typename T>
__global__ void __launch_bounds__(kThreads)
attn_generic_kernel(const T* __restrict__ q, const T* __restrict__ k_pages,
                    const T* __restrict__ v_pages, const int32_t* __restrict__ item_seq,
                    const int32_t* __restrict__ item_row0, const int32_t* __restrict__ item_npos,
                    const int32_t* __restrict__ row_pos, const int32_t* __restrict__ page_table,
                    int table_width, T* __restrict__ out, float* __restrict__ part_o,
                    float* __restrict__ part_ml, int nq, int nkv, int D, int Gb, int head_blocks,
                    int BC, int window, float scale, int n_splits) {
  extern __shared__ float lds[];
  float* Qs = lds;                        // [kRows][D]
  float* Ks = Qs + kRows * D;             // [BC][D + 1]
  float* Vs = Ks + BC * (D + 1);          // [BC][D]
  float* Ps = Vs + BC * D;                // [kRows][BC + 1]

  const int item = blockIdx.x;
  const int g = blockIdx.y / head_blocks, hb = blockIdx.y % head_blocks;
  const int split = blockIdx.z;
  const int seq = item_seq[item];
  const int npos = item_npos[item];
  const int row0 = item_row0[item];
  const int G = nq / nkv;
  const int t = threadIdx.x;
  const int r = t / 16, cc = t % 16;
  const int pi = r / Gb, hi = r % Gb;
  const int head_in_group = hb * Gb + hi;
  const bool row_valid = seq >= 0 && pi < npos && head_in_group < G;
  const int head = g * G + head_in_group;
  const int row = row0 + pi;
  const int pos_r = row_valid ? row_pos[row] : -1;

  // query rows, pre-scaled
  for (int idx = t; idx < kRows * D; idx += kThreads) {
    const int rr = idx / D, d = idx % D;
    const int ppi = rr / Gb, hhi = hb * Gb + rr % Gb;
    float v = 0.f;
    if (seq >= 0 && ppi < npos && hhi < G)
      v = ei::to_f32<T>(q[(static_cast<size_t>(row0 + ppi) * nq + g * G + hhi) * D + d]) * scale;
    Qs[idx] = v;
  }

  float m_r = kLowest, l_r = 0.f;
  float acc[16];
#pragma unroll
  for (int k = 0; k < 16; ++k) acc[k] = 0.f;
  const int nd = D / 16;
  const int nj = BC / 16;

  if (seq >= 0 && npos > 0) {
    const int hi_key = row_pos[row0 + npos - 1];
    const int lo_key = window > 0 ? max(0, row_pos[row0] - window + 1) : 0;
    const int lo_page = lo_key / EI_PAGE, hi_page = hi_key / EI_PAGE;
    const int total_pages = hi_page - lo_page + 1;
    const int per = (total_pages + n_splits - 1) / n_splits;
    const int p_begin = lo_page + split * per;
    const int p_end = min(lo_page + (split + 1) * per, hi_page + 1);
    const int chunks_per_page = EI_PAGE / BC;
    for (int p = p_begin; p < p_end; ++p) {
      const int phys = page_table[static_cast<size_t>(seq) * table_width + p];
      if (phys < 0) continue;  // a page the window has released: every key in it is masked
      const T* kp = k_pages + (static_cast<size_t>(phys) * nkv + g) * EI_PAGE * D;
      const T* vp = v_pages + (static_cast<size_t>(phys) * nkv + g) * EI_PAGE * D;
      for (int ch = 0; ch < chunks_per_page; ++ch) {
        const int key0 = p * EI_PAGE + ch * BC;
        if (key0 > hi_key) break;
        __syncthreads();
        for (int idx = t; idx < BC * D; idx += kThreads) {
          const int c = idx / D, d = idx % D;
          const bool live = key0 + c <= hi_key;  // later slots hold stale bytes
          const size_t off = static_cast<size_t>(ch * BC + c) * D + d;
          Ks[c * (D + 1) + d] = live ? ei::to_f32<T>(kp[off]) : 0.f;
          Vs[c * D + d] = live ? ei::to_f32<T>(vp[off]) : 0.f;
        }
        __syncthreads();
        float s[4];
        float row_max = kLowest;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          s[j] = -INFINITY;
          if (j < nj) {
            const int c = cc + 16 * j;
            const int key = key0 + c;
            const bool visible = row_valid && key <= pos_r && (window <= 0 || key > pos_r - window);
            if (visible) {
              float dot = 0.f;
              const float* qr = Qs + r * D;
              const float* kr = Ks + c * (D + 1);
              for (int d = 0; d < D; ++d) dot += qr[d] * kr[d];
              s[j] = dot;
              row_max = fmaxf(row_max, dot);
            }
          }
        }
#pragma unroll
        for (int offset = 8; offset > 0; offset >>= 1)
          row_max = fmaxf(row_max, __shfl_xor(row_max, offset, 16));
        const float m_new = fmaxf(m_r, row_max);
        const float alpha = expf(m_r - m_new);
        float row_sum = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if (j < nj) {
            const float p_val = expf(s[j] - m_new);  // -inf -> 0
            Ps[r * (BC + 1) + cc + 16 * j] = p_val;
            row_sum += p_val;
          }
        }
#pragma unroll
        for (int offset = 8; offset > 0; offset >>= 1) row_sum += __shfl_xor(row_sum, offset, 16);
        l_r = l_r * alpha + row_sum;
        m_r = m_new;
        __syncthreads();
        const float* pr = Ps + r * (BC + 1);
#pragma unroll
        for (int k = 0; k < 16; ++k) {
          if (k < nd) {
            const int d = cc + 16 * k;
            float a = acc[k] * alpha;
            for (int c = 0; c < BC; ++c) a += pr[c] * Vs[c * D + d];
            acc[k] = a;
          }
        }
      }
    }
  }

  if (!row_valid) return;
  if (n_splits == 1) {
    const float inv = l_r > 0.f ? 1.f / l_r : 0.f;
    T* dst = out + (static_cast<size_t>(row) * nq + head) * D;
#pragma unroll
    for (int k = 0; k < 16; ++k)
      if (k < nd) dst[cc + 16 * k] = ei::from_f32<T>(acc[k] * inv);
  } else {
    const size_t slot = (static_cast<size_t>(row) * nq + head) * n_splits + split;
    float* dst = part_o + slot * D;
#pragma unroll
    for (int k = 0; k < 16; ++k)
      if (k < nd) dst[cc + 16 * k] = acc[k];
    if (cc == 0) {
      part_ml[slot * 2] = m_r;
      part_ml[slot * 2 + 1] = l_r;
    }
  }
}

// One wave per (row, head): o = sum_s o_s e^{m_s - m} / sum_s l_s e^{m_s - m}.
template <typename T>
__global__ void attn_merge_kernel(const float* __restrict__ part_o,
                                  const float* __restrict__ part_ml,
                                  const int32_t* __restrict__ row_seq, T* __restrict__ out, int nq,
                                  int D, int n_splits, int total) {
  const int wave = (blockIdx.x * blockDim.x + threadIdx.x) / EI_WAVE;
  const int lane = threadIdx.x % EI_WAVE;
  if (wave >= total) return;
  const int row = wave / nq;
  if (row_seq && row_seq[row] < 0) return;
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
    out[static_cast<size_t>(wave) * D + d] = ei::from_f32<T>(o * inv);
  }
}

int chunk_keys(int D) { return D <= 64 ? 64 : (D <= 128 ? 32 : 16); }

}  // namespace

// Heads of one kv group that share a block (at most 16) for a head count ratio G.
extern "C" int ei_attn_heads_per_block(int G) { return G < kRows ? G : kRows; }
// Positions of one sequence that a prefill work item holds.
extern "C" int ei_attn_positions_per_item(int G) {
  const int gb = G < kRows ? G : kRows;
  return kRows / gb;
}

// q, out: [N, nq, D]; pages: [n_pages, nkv, 64, D]; items: see the kernel.
// n_splits > 1 needs part_o [N, nq, n_splits, D] and part_ml [N, nq, n_splits, 2]
// float32 and items that hold one position each (decode); the merge follows.
extern "C" int ei_attention(const void* q, const void* k_pages, const void* v_pages, int dtype,
                            const int32_t* item_seq, const int32_t* item_row0,
                            const int32_t* item_npos, int n_items, const int32_t* row_pos,
                            const int32_t* row_seq, const int32_t* page_table, int table_width,
                            void* out, float* part_o, float* part_ml, int N, int nq, int nkv,
                            int D, int window, float scale, int n_splits, hipStream_t stream) {
  EI_REQUIRE(n_items > 0 && N > 0 && nq > 0 && nkv > 0, "attention: sizes must be positive");
  EI_REQUIRE(nq % nkv == 0, "attention: query heads must be a multiple of kv heads");
  EI_REQUIRE(D % 16 == 0 && D >= 16 && D <= 256,
             "attention: head_dim must be a multiple of 16 between 16 and 256");
  EI_REQUIRE(q && k_pages && v_pages && out && item_seq && item_row0 && item_npos && row_pos &&
                 page_table && table_width > 0,
             "attention: null pointer");
  EI_REQUIRE(n_splits >= 1 && n_splits <= 64, "attention: splits must be between 1 and 64");
  EI_REQUIRE(n_splits == 1 || (part_o && part_ml), "attention: split scratch missing");
  EI_REQUIRE(window >= 0, "attention: negative window");
  const int G = nq / nkv;
  const int Gb = G < kRows ? G : kRows;
  const int head_blocks = (G + Gb - 1) / Gb;
  const int BC = chunk_keys(D);
  const size_t lds =
      sizeof(float) * (static_cast<size_t>(kRows) * D + static_cast<size_t>(BC) * (D + 1) +
                       static_cast<size_t>(BC) * D + static_cast<size_t>(kRows) * (BC + 1));
  EI_REQUIRE(static_cast<long long>(nkv) * head_blocks <= 65535, "attention: too many heads");
  dim3 grid(n_items, nkv * head_blocks, n_splits);
  if (dtype == EI_F32) {
    attn_generic_kernel<float><<<grid, kThreads, lds, stream>>>(
        static_cast<const float*>(q), static_cast<const float*>(k_pages),
        static_cast<const float*>(v_pages), item_seq, item_row0, item_npos, row_pos, page_table,
        table_width, static_cast<float*>(out), part_o, part_ml, nq, nkv, D, Gb, head_blocks, BC,
        window, scale, n_splits);
  } else if (dtype == EI_BF16) {
    attn_generic_kernel<bf16_t><<<grid, kThreads, lds, stream>>>(
        static_cast<const bf16_t*>(q), static_cast<const bf16_t*>(k_pages),
        static_cast<const bf16_t*>(v_pages), item_seq, item_row0, item_npos, row_pos, page_table,
        table_width, static_cast<bf16_t*>(out), part_o, part_ml, nq, nkv, D, Gb, head_blocks, BC,
        window, scale, n_splits);
  } else {
    EI_REQUIRE(false, "attention: unknown dtype");
  }
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) {
    ei_set_error(hipGetErrorString(e));
    return static_cast<int>(e);
  }
  if (n_splits > 1) {
    const int total = N * nq;
    const int threads = 256;
    const int blocks = (total * EI_WAVE + threads - 1) / threads;
    if (dtype == EI_F32)
      attn_merge_kernel<float><<<blocks, threads, 0, stream>>>(
          part_o, part_ml, row_seq, static_cast<float*>(out), nq, D, n_splits, total);
    else
      attn_merge_kernel<bf16_t><<<blocks, threads, 0, stream>>>(
          part_o, part_ml, row_seq, static_cast<bf16_t*>(out), nq, D, n_splits, total);
  }
  EI_LAUNCH_CHECK();
}
