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
#include <type_traits>

#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

namespace {

constexpr int kTile = 16;          // keys per MFMA tile
constexpr float kLowest = -1.0e30f;

__device__ __forceinline__ float bf16_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }

// What a block needs to make its own queries, and the new key and value of its kv head, from
// the fused projection (PREP): the work of the separate norm-rotate-store kernel, saved as a
// launch per layer.  qkv: float32 partial sums [nsplit][rows, (nq + 2 nkv) * D], added in slice
// order; per-head RMSNorm weights (or null); the rotation table [positions, rot_dim] (cosines,
// then sines; or null; rot_dim <= D: pairs (i, i + rot_dim/2), the elements from rot_dim on
// pass unrotated, as in rope_store.hip); k_store / v_store: the cache pages to write the new key and value to (null:
// this run of the layer reads a cache that another run wrote, and has no key of its own).
// Formulas and order as in rope_store.hip (runtime/include/execution/decoder.hpp:125-140).
struct DecodePrep {
  const float* qkv;
  int nsplit;
  long long split_stride;
  const float* q_norm_w;
  const float* k_norm_w;
  float eps;
  const float* rope_table;
  int rot_dim;
  bf16_t* k_store;
  bf16_t* v_store;
};

// GB: query heads of the kv group handled by this block (1..16).  W: waves of the block, each
// taking every W-th tile of 16 keys of the block's key range: 4 where sequences and slices
// give many blocks, 8 or 16 where they give fewer (a short range then needs no slices at all).
// PREP: q is not read; the block forms its queries and the position's key and value itself
// (the block of slice 0 and head block 0 stores them; the wave that meets the position in
// its tile takes them from LDS, since the store of another block may not have landed).
template <int D, int GB, int W, bool PREP>
__global__ void __launch_bounds__(W * EI_WAVE)
attn_decode_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pages,
                   const bf16_t* __restrict__ v_pages, const int32_t* __restrict__ row_pos,
                   const int32_t* __restrict__ row_seq, const int32_t* __restrict__ page_table,
                   int table_width, bf16_t* __restrict__ out, float* __restrict__ part_o,
                   float* __restrict__ part_ml, int nq, int nkv, int head_blocks, int window,
                   float scale, int n_splits, const int32_t* __restrict__ longest,
                   DecodePrep prep) {
  constexpr int DJ = D / 32;            // MFMA steps over the head dimension
  constexpr int LPR = D / 8;            // lanes that cover one value row with 16-byte loads
  constexpr int KPI = EI_WAVE / LPR;    // value rows per load instruction
  constexpr int VI = kTile / KPI;       // value load instructions per tile
  __shared__ float p_lds[W][kTile][16];
  __shared__ float alpha_lds[W][16];
  __shared__ float m_lds[W][16], l_lds[W][16];
  __shared__ float o_lds[W][GB][D];

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

  // PREP: rows 0..GB-1 the block's query heads, row GB the new key, row GB+1 the new value,
  // normed, rotated and rounded.  A wave takes a head at a time, a lane the pair (i, i + D/2):
  // every load of a head is on its way before the first is used, and nothing but the final
  // rows goes through LDS.
  constexpr int PR = PREP ? GB + 2 : 1, FS = PREP ? D + 8 : 8;
  __shared__ __attribute__((aligned(16))) bf16_t fin_lds[PR][FS];
  const bool own_key = PREP && prep.k_store != nullptr;
  if constexpr (PREP) {
    constexpr int half = D / 2;
    static_assert(half <= EI_WAVE, "a lane holds one pair");
    const size_t width = static_cast<size_t>(nq + 2 * nkv) * D;
    const float* src = prep.qkv + static_cast<size_t>(row) * width;
    const int page_now = own_key
        ? page_table[static_cast<size_t>(seq) * table_width + pos / EI_PAGE] : -1;
    const bool active = lane < half;
    // the lane's pair: elements (i, i2), rotated if it lies within the rotated width
    const int rhalf = prep.rope_table != nullptr ? prep.rot_dim / 2 : half;
    const int pair = active ? lane : 0;
    const bool turned = pair < rhalf;
    const int i = turned ? pair : pair + rhalf;
    const int i2 = turned ? pair + rhalf : pair + half;
    for (int h = wave; h < heads_here + (own_key ? 2 : 0); h += W) {
      const int kind = h < heads_here ? 0 : (h == heads_here ? 1 : 2);   // query, key, value
      const int slot = kind == 0 ? h : GB + kind - 1;
      const int column = kind == 0 ? (head0 + h) * D
                                   : (kind == 1 ? (nq + g) * D : (nq + nkv + g) * D);
      const float* norm_w = kind == 0 ? prep.q_norm_w : (kind == 1 ? prep.k_norm_w : nullptr);
      const bool rotate = kind != 2 && prep.rope_table != nullptr && turned;
      float wx = 1.f, wy = 1.f, cs = 1.f, sn = 0.f;
      if (norm_w != nullptr) {
        wx = norm_w[i];
        wy = norm_w[i2];
      }
      if (rotate) {
        const float* trig = prep.rope_table + static_cast<size_t>(pos) * (2 * rhalf);
        cs = trig[pair];
        sn = trig[pair + rhalf];
      }
      float x = 0.f, y = 0.f;
      const float* p = src + column;
      for (int s0 = 0; s0 < prep.nsplit; s0 += 8) {       // slices in slice order, 8 per trip
        float xa[8], ya[8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (s0 + u < prep.nsplit) {
            xa[u] = p[(s0 + u) * prep.split_stride + i];
            ya[u] = p[(s0 + u) * prep.split_stride + i2];
          }
#pragma unroll
        for (int u = 0; u < 8; ++u)
          if (s0 + u < prep.nsplit) {
            x += xa[u];
            y += ya[u];
          }
      }
      if (!active) x = y = 0.f;
      float a = x, b = y;
      if (norm_w != nullptr) {
        const float sum = ei::wave_sum(x * x + y * y);
        const float inv = rsqrtf(sum / static_cast<float>(D) + prep.eps);
        a = (a * inv) * wx;
        b = (b * inv) * wy;
      }
      if (rotate) {
        const float ra = a * cs - b * sn;
        const float rb = a * sn + b * cs;
        a = ra;
        b = rb;
      }
      if (active) {
        const bf16_t a16 = ei::from_f32<bf16_t>(a), b16 = ei::from_f32<bf16_t>(b);
        fin_lds[slot][i] = a16;
        fin_lds[slot][i2] = b16;
        if (kind != 0 && hb == 0 && split == 0 && page_now >= 0) {
          bf16_t* dst = (kind == 1 ? prep.k_store : prep.v_store) +
                        ((static_cast<size_t>(page_now) * nkv + g) * EI_PAGE + pos % EI_PAGE) * D;
          dst[i] = a16;
          dst[i2] = b16;
        }
      }
    }
    __syncthreads();
  }

  // query heads as the B operand: lane (n = r16, c) holds q[head n][j*32 + c*8 .. +8]
  bf16x8 q_reg[DJ];
#pragma unroll
  for (int j = 0; j < DJ; ++j) {
    uint4 z = uint4{0u, 0u, 0u, 0u};
    if (r16 < heads_here) {
      if constexpr (PREP)
        z = *reinterpret_cast<const uint4*>(&fin_lds[r16][j * 32 + c * 8]);
      else
        z = *reinterpret_cast<const uint4*>(q + (static_cast<size_t>(row) * nq + head0 + r16) * D +
                                            j * 32 + c * 8);
    }
    q_reg[j] = *reinterpret_cast<bf16x8*>(&z);
  }

  const int lo_key = window > 0 ? max(0, pos - window + 1) : 0;
  const int first_tile = lo_key / kTile, last_tile = pos / kTile;
  const int total_tiles = last_tile - first_tile + 1;
  // slices are cut at page boundaries so that they do not depend on the tile size
  const int lo_page = lo_key / EI_PAGE, hi_page = pos / EI_PAGE;
  const int pages = hi_page - lo_page + 1;
  // A slice is the same number of pages for every sequence of the step: the longest one's
  // share (`longest`: the most tokens any sequence holds, read on the device so that a captured
  // step follows it).  Sequences of unequal lengths then give blocks of about equal work, and
  // the later slices of a short sequence are empty.  Without it (or with a window, where the
  // ranges start at different pages) every sequence is cut into n_splits equal parts.
  int per = (pages + n_splits - 1) / n_splits;
  if (longest != nullptr && window <= 0) {
    const int most_pages = (*longest + EI_PAGE - 1) / EI_PAGE;
    per = max(1, (most_pages + n_splits - 1) / n_splits);
  }
  const int tile_begin = max(first_tile, (lo_page + split * per) * (EI_PAGE / kTile));
  // (the last slice takes whatever is left, so that no key is lost should `longest` be short)
  const int tile_end = split == n_splits - 1
                           ? last_tile + 1
                           : min(last_tile + 1, (lo_page + (split + 1) * per) * (EI_PAGE / kTile));
  (void)total_tiles;

  float m_run = kLowest, l_run = 0.f;              // state of head r16 (same in all four c)
  float acc[GB][8];
#pragma unroll
  for (int h = 0; h < GB; ++h)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[h][e] = 0.f;
  const int ks = lane / LPR, dc = lane % LPR;       // value rows: key sub-index, 8-wide chunk

  // One tile of 16 keys.  OWN: the tile holds the position itself and the block has made its
  // key and value (PREP): they come from LDS.  That case has code of its own, so that in
  // every other tile the score product waits for the keys alone and not for a patch.
  auto process = [&](const int tile, auto own_tag) {
    constexpr bool OWN = decltype(own_tag)::value;
    const int key0 = tile * kTile;
    const int phys = page_table[static_cast<size_t>(seq) * table_width + key0 / EI_PAGE];
    if (phys < 0) return;                          // released by the window: all masked
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
    {
      // read once and whole lines at a time: not kept in the caches (the keys above are
      // fetched in 64-byte pieces, two instructions a line, and do better cached)
      const u32x4_t raw = __builtin_nontemporal_load(
          reinterpret_cast<const u32x4_t*>(vp + static_cast<size_t>(i) * KPI * D));
      v_reg[i] = uint4{raw.x, raw.y, raw.z, raw.w};
    }
    if constexpr (OWN) {                           // the position's own key and value
      if (key0 + r16 == pos) {
#pragma unroll
        for (int j = 0; j < DJ; ++j)
          k_reg[j] = *reinterpret_cast<const bf16x8*>(&fin_lds[GB][j * 32 + c * 8]);
      }
#pragma unroll
      for (int i = 0; i < VI; ++i)
        if (key0 + i * KPI + ks == pos)
          v_reg[i] = *reinterpret_cast<const uint4*>(&fin_lds[GB + 1][dc * 8]);
    }

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
    tile_max = ei::rows_max(tile_max);
    const float m_new = fmaxf(m_run, tile_max);
    const float alpha = expf(m_run - m_new);
    float tile_sum = 0.f;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float p = expf(sc[r] - m_new);
      p_lds[wave][4 * c + r][r16] = p;
      tile_sum += p;
    }
    tile_sum = ei::rows_sum(tile_sum);
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
  };
  for (int tile = tile_begin + wave; tile < tile_end; tile += W) {
    if (PREP && own_key && tile == last_tile)
      process(tile, std::integral_constant<bool, PREP>{});
    else
      process(tile, std::false_type{});
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
  for (int idx = t; idx < heads_here * D; idx += (W * EI_WAVE)) {
    const int h = idx / D, d = idx % D;
    float m = kLowest;
#pragma unroll
    for (int w = 0; w < W; ++w) m = fmaxf(m, m_lds[w][h]);
    float l = 0.f, o = 0.f;
#pragma unroll
    for (int w = 0; w < W; ++w) {
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

// Prefill on 32x32x16 products.  A block of eight waves owns HB query heads of one kv group
// (HB = 4, 2 or 1, the largest that divides the group) and 32 * (8 / HB) consecutive positions
// of one sequence; a wave keeps 32 rows of one head as operands in registers and walks the key
// pages of the sequence.  A page of keys and a page of values go to LDS once for the whole
// block, so the heads of a group share every byte that is fetched.  KW = 2: the eight waves are
// HB heads x half as many groups of rows x 2 halves of every page's keys; the wave of the
// second half hands its maximum, sum and output tile to the wave of the first through LDS at
// the end.  Work items are then half as long, so a short prompt gives twice the blocks, enough
// for the pairing of a long item with a short one below.  With enough blocks without it KW = 1
// is faster (what a page costs a wave beside its products is not halved).
// (A form with 16-row waves on 16x16x32 products, four waves a SIMD, was measured against this
// one: an operand read from LDS feeds half the arithmetic there and the instruction itself
// runs at a lower rate on this chip, 1.45 against 2.1 PFLOP/s in a loop of nothing else; it
// was 20 % slower from 3,000 tokens on and equal below.)
//
// Pages move from global memory straight into LDS (global_load_lds: a wave load lands as one
// kilobyte, lane l's 16 bytes at place l of it; no staging registers, no LDS stores), three
// page buffers in turn: while page p is multiplied, page p + 1 is on its way or there and page
// p + 2 is requested into the buffer that page p - 1 left at the last barrier.  One barrier a
// page says both that the next page is complete (every wave has waited for its own loads of
// it) and that this one's buffer is free.  Both pages lie in LDS row by row as in the cache,
// with the pieces of a row exchanged among themselves (below) so that operand reads meet
// every bank once; a lane fetches the piece that belongs at its place.  The slots of a
// sequence's last page beyond the item's last position hold whatever the cache held before:
// their scores are masked, and their value rows are cleared in LDS by the wave that fetched
// them (a probability of zero times a stale NaN would still be NaN).
//
// S^T = K Q^T for a block of 32 keys: A = keys (lane (key l % 32, half l / 32) reads
// k[key][16 s + 8 half .. +8] from LDS), B = the wave's queries in registers (lane (query
// l % 32, half) holds q[query][16 s + 8 half .. +8]).  The result leaves lane (query n, half h)
// with keys 8 i + 4 h + r of the block (i, r = 0..3): for a 16-key step t of the value
// product these are keys 16 t + 4 h + r and 16 t + 8 + 4 h + r, eight values that are
// exactly the lane's A operand of P, provided the values (B, lane (d column n, half h)) come
// in the same order.  They do, out of two transposing reads (ds_read_b64_tr_b16: in each 16
// lanes, lane 4 q + e receives element e of the four 8-byte pieces that lanes q, q + 4, q + 8,
// q + 12 point at): lane s of 16 points at key 4 h + s / 4 of the step (plus 8 for the second
// read) and at d columns 16 (l / 16 % 2) + 4 (s % 4) .. + 3 of the 32-wide block.  So the
// values need no transposition on their way into LDS and the probabilities never leave the
// registers.  The two lanes of a query share its running maximum (one exchange a page) and
// keep separate sums.  The output tile has lane (d column n, half h) hold queries
// 8 i + 4 h + r, so factors per query (the rescaling when a maximum moves, the final 1 / sum)
// pass through 32 floats of LDS a wave.  Softmax state is float32 (in units of log2);
// probabilities are rounded to bfloat16 for the value product (the reference's prefill kernel
// does the same, operators/src/cuda/kernels/flash_attn_prefill.cu:240).
//
// Exchange of pieces.  Keys: the 16-byte chunks of a row, chunk ^ key % 16 (64-wide heads:
// chunk ^ (key / 2) % 8), so that the 16 rows a quarter of a wave reads touch every bank once.
// Values: the 32-byte pieces of a row, piece ^ 2 (key % 4) (64-wide heads: piece ^ 2 (key / 2
// % 2)): the eight pieces that half a wave's transposing read takes (four keys, two pieces)
// then lie in eight different eighths of the banks.
// Blocks are numbered so that the blocks of one kv head fall on one XCD (the hardware deals
// consecutive workgroups round-robin to its 8 XCDs): that head's keys and values then stay
// in that XCD's L2.
constexpr int kPrefillWaves = 8;
constexpr int kPrefillThreads = kPrefillWaves * EI_WAVE;
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef short ei_s16x4 __attribute__((ext_vector_type(4)));
typedef short ei_s16x8 __attribute__((ext_vector_type(8)));
constexpr int kWideRows = 32;      // query rows of a wave
constexpr int kAhead = 3;          // LDS operand reads in flight before the product that needs the first
constexpr int kPageBuffers = 3;
// (log2) how far a row's maximum may rise above the reference point of its exponentials before
// the sums so far are rescaled to a new one: up to there the probabilities are merely larger
// than 1 (at most 2^8, which bfloat16 and the float32 sums hold as well as values below 1).
// Once the first pages are past, a page hardly ever moves any of a wave's 32 rows that far,
// where a plain running maximum moves one of them on most pages: the rescaling (64 products
// a lane and a trip through LDS) was a quarter of a page's vector work.
constexpr float kLazyRise = 8.f;

template <int D, int HB, int KW>
__global__ void __launch_bounds__(kPrefillThreads, 2)
attn_prefill_kernel(const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_pages,
                         const bf16_t* __restrict__ v_pages, const int32_t* __restrict__ item_seq,
                         const int32_t* __restrict__ item_row0,
                         const int32_t* __restrict__ item_npos, int n_items,
                         const int32_t* __restrict__ row_pos,
                         const int32_t* __restrict__ page_table, int table_width,
                         bf16_t* __restrict__ out, int nq, int nkv, int window, float scale,
                         int pair) {
  constexpr int SJ = D / 16;             // 16-wide steps over d for the scores
  constexpr int DB = D / 32;             // 32-wide output blocks over d
  constexpr int CHUNKS = D / 8;          // 16-byte chunks of a row
  constexpr int PBUF = EI_PAGE * D;      // elements of one page of keys or of values
  constexpr int NG = kPrefillWaves / (HB * KW);       // groups of 32 rows in a block
  constexpr int KBL = 2 / KW;            // blocks of 32 keys of a page that a wave takes
  // a page of keys and one of values are 2 * PBUF * 2 bytes, a wave load a kilobyte
  constexpr int LOADS = 2 * PBUF * 2 / 1024 / kPrefillWaves;   // wave loads per wave and page
  constexpr int ROWS_A_LOAD = 1024 / (2 * D);                  // rows a wave load covers
  static_assert(KW == 1 || KW == 2, "a page's keys go to one wave or to two");
  static_assert(NG >= 1, "eight waves: heads x row groups x key ways");
  static_assert(LOADS >= 2 && LOADS % 2 == 0, "a wave fetches as much of the keys as of the values");
  // buffer b: keys at b * 2 * PBUF, values PBUF further
  __shared__ __attribute__((aligned(1024))) bf16_t page_lds[kPageBuffers * 2 * PBUF];
  __shared__ __attribute__((aligned(16))) float factor_lds[kPrefillWaves][kWideRows];
  // (KW = 2) what the second wave of a (head, rows) pair hands to the first at the end: its
  // running maximum and sum per row here, its output tile in the page buffers
  __shared__ float handed_lds[KW == 2 ? kPrefillWaves / 2 : 1][2][kWideRows];
  __shared__ __attribute__((aligned(16))) float other_lds[KW == 2 ? kPrefillWaves : 1][kWideRows];
  static_assert(KW == 1 || (kPrefillWaves / 2) * (D / 32) * 16 * EI_WAVE * sizeof(float) <=
                               sizeof(bf16_t) * kPageBuffers * 2 * PBUF,
                "the handed-over output tiles fit the page buffers");

  const int G = nq / nkv;
  const int head_blocks = G / HB;
  const int units = pair ? (n_items + 1) / 2 : n_items;
  const int rests = units * head_blocks;
  int g, rest;
  {
    const int id = blockIdx.x, x = id & 7, slot = id >> 3;
    if (nkv % 8 == 0) {
      const int per = nkv / 8;
      g = x + 8 * (slot % per);
      rest = slot / per;
    } else if (8 % nkv == 0) {
      const int share = 8 / nkv;
      g = x % nkv;
      rest = slot * share + x / nkv;
    } else {
      g = id % nkv;
      rest = id / nkv;
    }
  }
  if (rest >= rests) return;
  const int unit = rest / head_blocks, hb = rest % head_blocks;
  const int t = threadIdx.x, wave = t / EI_WAVE, lane = t % EI_WAVE;
  const int n32 = lane & 31, half = lane >> 5;
  const int hw = wave % HB, pw = (wave / HB) % NG, kw = wave / (HB * NG);
  const int head = g * G + hb * HB + hw;
  // where chunk `chunk` of key row `key` lies in the row, and the same for a row of values
  auto k_place = [](int key, int chunk) {
    return CHUNKS == 16 ? (chunk ^ (key & 15)) : (chunk ^ ((key >> 1) & 7));
  };
  auto v_place = [](int key, int chunk) {
    const int piece = chunk >> 1;
    const int moved = D == 128 ? (piece ^ (2 * (key & 3))) : (piece ^ (2 * ((key >> 1) & 1)));
    return 2 * moved + (chunk & 1);
  };
  // Everything a lane needs to find its operands in a page buffer is worked out once: the
  // places of its key chunks (they differ from step to step by the exchange of chunks; key
  // blocks and buffers add constants) and of the value pieces its transposing reads point at.
  int k_read[SJ];                        // (element offsets into a page of keys)
#pragma unroll
  for (int sj = 0; sj < SJ; ++sj) k_read[sj] = n32 * D + k_place(n32, 2 * sj + half) * 8;
  int v_read[DB];                        // (element offsets into a page of values)
  {
    const int s16 = lane & 15, vkey = 4 * half + (s16 >> 2);
#pragma unroll
    for (int db = 0; db < DB; ++db)
      v_read[db] = vkey * D + v_place(vkey, 2 * (2 * db + ((lane >> 4) & 1))) * 8 + 4 * (s16 & 3);
  }
  // The wave's loads of a page: load i < LOADS / 2 brings kilobyte wave + 8 i of the keys, the
  // others the same of the values.  Lane l's 16 bytes land at place l % CHUNKS of row
  // l / CHUNKS of that kilobyte; it fetches the chunk of the row that belongs there (both
  // exchanges are their own inverses).
  int fetch_from[LOADS];                 // element offsets into the page in global memory
  int fetch_row[LOADS / 2];              // (values) the row of the page that the lane's piece belongs to
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    const int part = i % (LOADS / 2);
    const int row = (wave + kPrefillWaves * part) * ROWS_A_LOAD + lane / CHUNKS;
    const int at = lane % CHUNKS;
    fetch_from[i] = row * D + (i < LOADS / 2 ? k_place(row, at) : v_place(row, at)) * 8;
    if (i >= LOADS / 2) fetch_row[part] = row;
  }

  for (int pass = 0; pass <= pair; ++pass) {
  const int item = pass == 0 ? unit : n_items - 1 - unit;
  if (pass == 1) {
    if (item == unit) break;              // the middle item of an odd count
    __syncthreads();                      // the first item's last page has been read
  }
  const int seq = item_seq[item];
  if (seq < 0) continue;
  const int row0 = item_row0[item], npos = item_npos[item];

  // this lane's query (column n32 of S^T), its position, and the Q operand
  const int my_row = pw * kWideRows + n32;
  const bool row_valid = my_row < npos;
  const int pos_q = row_valid ? row_pos[row0 + my_row] : -1;
  bf16x8 q_reg[SJ];
#pragma unroll
  for (int sj = 0; sj < SJ; ++sj) {
    uint4 z = uint4{0u, 0u, 0u, 0u};
    if (row_valid)
      z = *reinterpret_cast<const uint4*>(
          q + (static_cast<size_t>(row0 + my_row) * nq + head) * D + sj * 16 + half * 8);
    q_reg[sj] = *reinterpret_cast<bf16x8*>(&z);
  }

  const int first_pos = row_pos[row0], last_pos = row_pos[row0 + npos - 1];
  const int lo_key = window > 0 ? max(0, first_pos - window + 1) : 0;
  const int lo_page = lo_key / EI_PAGE, hi_page = last_pos / EI_PAGE;
  const bool wave_rows_valid = pw * kWideRows + kWideRows <= npos;
  const int wave_min_pos = wave_rows_valid ? row_pos[row0 + pw * kWideRows] : -1;
  const int wave_max_pos = wave_rows_valid ? row_pos[row0 + pw * kWideRows + kWideRows - 1] : -1;
  // a wave none of whose rows exist only helps to move pages
  const bool wave_has_rows = pw * kWideRows < npos;
  const int wave_last_pos = wave_has_rows
      ? row_pos[row0 + min(npos, pw * kWideRows + kWideRows) - 1] : -1;

  const float scale_log2 = scale * 1.4426950408889634f;
  float m_run = kLowest, l_run = 0.f;     // l_run: this lane's half of the keys only
  f32x16 o_acc[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) o_acc[db][e] = 0.f;

  // Request page `page_index` of the sequence into buffer `buf` (nothing past the last page).
  // A page that the window has given back (none of its keys is visible to any row: it only
  // lies in the walk) is cleared instead, by plain stores.
  auto fetch_page = [&](int page_index, int buf) __attribute__((always_inline)) {
    if (page_index > hi_page) return;
    const int phys = page_table[static_cast<size_t>(seq) * table_width + page_index];
    bf16_t* const to = page_lds + buf * 2 * PBUF;
    if (phys < 0) {
#pragma unroll
      for (int i = 0; i < LOADS; ++i)
        *reinterpret_cast<uint4*>(to + (i / (LOADS / 2)) * PBUF +
                                  (wave + kPrefillWaves * (i % (LOADS / 2))) * 512 + lane * 8) =
            uint4{0u, 0u, 0u, 0u};
      // (the waits below count a page's loads: with none for this page, everything requested
      // before must have arrived here)
      __builtin_amdgcn_s_waitcnt(0x0F70);
      return;
    }
    const size_t base = (static_cast<size_t>(phys) * nkv + g) * EI_PAGE * D;
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const bf16_t* const from = (i < LOADS / 2 ? k_pages : v_pages) + base + fetch_from[i];
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void*)from,
          (__attribute__((address_space(3))) void*)(to + (i / (LOADS / 2)) * PBUF +
                                                    (wave + kPrefillWaves * (i % (LOADS / 2))) * 512),
          16, 0, 0);
    }
  };
  // The wave's loads of page `page_index` have arrived (all but the `younger` loads it has
  // requested since): if it is the sequence's last page, the value rows beyond the item's
  // last position are cleared, each piece by the lane that fetched it.
  auto page_arrived = [&](int page_index, int buf, auto younger_tag) __attribute__((always_inline)) {
    constexpr int younger = decltype(younger_tag)::value;
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0x0F70 | (younger & 15) | ((younger >> 4) << 14));
    if (page_index == hi_page) {
      bf16_t* const to = page_lds + buf * 2 * PBUF + PBUF;
#pragma unroll
      for (int part = 0; part < LOADS / 2; ++part)
        if (page_index * EI_PAGE + fetch_row[part] > last_pos)
          *reinterpret_cast<uint4*>(to + (wave + kPrefillWaves * part) * 512 + lane * 8) =
              uint4{0u, 0u, 0u, 0u};
    }
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
  };

  // The scores of one page from buffer `buf`, their softmax into `p_reg` (A operands of P
  // for the four 16-key steps), and the rescaling of the output so far.  MASKED: some key of
  // the page is hidden from some row of the wave (all but the last one or two pages of a
  // causal prompt need no mask).
  bf16x8 p_reg[2 * KBL];
  auto scores = [&](const int key_base, const int buf, const bool MASKED) __attribute__((always_inline)) {
    const bf16_t* const k_lds = page_lds + buf * 2 * PBUF;
    f32x16 s[KBL];
#pragma unroll
    for (int kb = 0; kb < KBL; ++kb)
#pragma unroll
      for (int e = 0; e < 16; ++e) s[kb][e] = 0.f;
#pragma unroll
    for (int sj = 0; sj < SJ; ++sj)
#pragma unroll
      for (int kb = 0; kb < KBL; ++kb) {
        const bf16x8 kf = *reinterpret_cast<const bf16x8*>(
            &k_lds[k_read[sj] + (kw * KBL + kb) * 32 * D]);
        s[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, q_reg[sj], s[kb], 0, 0, 0);
      }
    // instruction order: the operand reads from LDS run kAhead products ahead of the products
    // that take them (0x100: LDS reads, 0x008: matrix products)
    __builtin_amdgcn_sched_group_barrier(0x100, kAhead, 0);
#pragma unroll
    for (int n = 0; n < SJ * KBL; ++n) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
    }
    if (MASKED) {
      // (an empty statement the compiler may not move: it keeps this a branch, which all but
      // the last pages of a causal prompt jump over, instead of 128 predicated instructions)
      asm volatile("");
#pragma unroll
      for (int kb = 0; kb < KBL; ++kb)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int key = key_base + (kw * KBL + kb) * 32 + 8 * i + 4 * half + r;
            const bool visible = key <= pos_q && (window <= 0 || key > pos_q - window);
            if (!visible) s[kb][4 * i + r] = -INFINITY;     // (pos_q = -1: a row that is not there)
          }
    }
    float tile_max = s[0][0];
#pragma unroll
    for (int kb = 0; kb < KBL; ++kb)
#pragma unroll
      for (int e = 0; e < 16; ++e) tile_max = fmaxf(tile_max, s[kb][e]);
    {   // the other half of this query's keys sits 32 lanes away
      ei::ei_u32x2 both = __builtin_amdgcn_permlane32_swap(__float_as_uint(tile_max),
                                                           __float_as_uint(tile_max), false, false);
      tile_max = fmaxf(__uint_as_float(both.x), __uint_as_float(both.y));
    }
    // The reference point of the row's exponentials, in units of log2 (raw score * scale *
    // log2 e; the scale is positive): it follows the maximum only when that has risen by more
    // than kLazyRise.  A row with no visible key yet keeps the lowest value, not -inf, so that
    // no NaN arises.
    const float m_tile = tile_max * scale_log2;
    const float m_new = m_tile > m_run + kLazyRise ? m_tile : m_run;
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    float tile_sum = 0.f;
#pragma unroll
    for (int kb = 0; kb < KBL; ++kb)
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int e = 4 * (2 * tt + (j >> 2)) + (j & 3);
          const float p = __builtin_amdgcn_exp2f(fmaf(s[kb][e], scale_log2, -m_new));
          tile_sum += p;
          p_reg[2 * kb + tt][j] = static_cast<__bf16>(p);
        }
    l_run = l_run * alpha + tile_sum;
    m_run = m_new;
    if (__any(alpha != 1.f)) {            // the reference point of some row of this wave has moved
      if (half == 0) factor_lds[wave][n32] = alpha;
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float4 a = *reinterpret_cast<const float4*>(&factor_lds[wave][8 * i + 4 * half]);
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          o_acc[db][4 * i + 0] *= a.x;
          o_acc[db][4 * i + 1] *= a.y;
          o_acc[db][4 * i + 2] *= a.z;
          o_acc[db][4 * i + 3] *= a.w;
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }
  };
  // output += P V for the page whose probabilities are in `p_reg`, values from buffer `buf`
  auto values = [&](const int buf) __attribute__((always_inline)) {
    typedef __attribute__((address_space(3))) ei_s16x4 lds_s16x4;
    const bf16_t* const v_lds = page_lds + buf * 2 * PBUF + PBUF;
#pragma unroll
    for (int st = 0; st < 2 * KBL; ++st) {
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const bf16_t* vrow = &v_lds[v_read[db] + (kw * 2 * KBL + st) * 16 * D];
        const ei_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(vrow));
        const ei_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(vrow + 8 * D));
        const ei_s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        o_acc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
            p_reg[st], __builtin_bit_cast(bf16x8, both), o_acc[db], 0, 0, 0);
      }
    }
    __builtin_amdgcn_sched_group_barrier(0x100, 2 * kAhead, 0);      // as for the scores
#pragma unroll
    for (int n = 0; n < 2 * KBL * DB; ++n) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
  };
  // whether this wave has anything to do with a page: one that lies wholly after the wave's
  // last row (the item's later rows need it) or wholly before its window is only moved
  // (the wave's keys of a page: KBL blocks of 32 from block kw * KBL on)
  auto page_seen = [&](const int page) __attribute__((always_inline)) {
    const int key_lo = page * EI_PAGE + kw * KBL * 32, key_hi = key_lo + KBL * 32 - 1;
    return wave_has_rows && key_lo <= wave_last_pos &&
           (window <= 0 || !wave_rows_valid || key_hi > wave_min_pos - window);
  };
  auto scores_of = [&](const int page, const int buf) __attribute__((always_inline)) {
    const int key_base = page * EI_PAGE;
    const int key_lo = key_base + kw * KBL * 32, key_hi = key_lo + KBL * 32 - 1;
    const bool no_mask = wave_rows_valid && key_hi <= wave_min_pos &&
                         (window <= 0 || key_lo > wave_max_pos - window);
    scores(key_base, buf, !no_mask);
  };
  using Both = std::integral_constant<int, LOADS>;
  using None = std::integral_constant<int, 0>;
  fetch_page(lo_page, 0);
  fetch_page(lo_page + 1, 1);
  if (lo_page + 1 <= hi_page) page_arrived(lo_page, 0, Both{});
  else page_arrived(lo_page, 0, None{});
  int buf = 0;
  for (int page = lo_page; page <= hi_page; ++page) {
    const int next = buf == kPageBuffers - 1 ? 0 : buf + 1;
    fetch_page(page + 2, next == kPageBuffers - 1 ? 0 : next + 1);
    __builtin_amdgcn_sched_barrier(0);
    if (page_seen(page)) {
      scores_of(page, buf);
      values(buf);
    }
    if (page < hi_page) {
      if (page + 2 <= hi_page) page_arrived(page + 1, next, Both{});
      else page_arrived(page + 1, next, None{});
    }
    buf = next;
  }

  // 1 / sum per query through LDS; lane (d column n32, half) holds O[query 8 i + 4 half + r]
  float l_wave;
  {
    ei::ei_u32x2 both = __builtin_amdgcn_permlane32_swap(__float_as_uint(l_run),
                                                         __float_as_uint(l_run), false, false);
    l_wave = __uint_as_float(both.x) + __uint_as_float(both.y);
  }
  float own_factor = l_wave > 0.f ? 1.f / l_wave : 0.f;   // what this wave's output is scaled by
  float other_factor = 0.f;                               // and the handed-over one
  if constexpr (KW == 2) {
    // The wave of the second half of every page's keys hands its state to the wave of the
    // first: o = (o_0 2^(m_0 - m) + o_1 2^(m_1 - m)) / (l_0 2^(m_0 - m) + l_1 2^(m_1 - m)).
    float* const tile_lds = reinterpret_cast<float*>(page_lds);
    const int couple = wave % (HB * NG);
    __syncthreads();                       // every wave has read the last page
    if (kw == 1) {
#pragma unroll
      for (int db = 0; db < DB; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e)
          tile_lds[((couple * DB + db) * 16 + e) * EI_WAVE + lane] = o_acc[db][e];
      if (half == 0) {
        handed_lds[couple][0][n32] = m_run;
        handed_lds[couple][1][n32] = l_wave;
      }
    }
    __syncthreads();
    if (kw == 0) {
      const float m_other = handed_lds[couple][0][n32], l_other = handed_lds[couple][1][n32];
      const float m = fmaxf(m_run, m_other);
      const float f_own = __builtin_amdgcn_exp2f(m_run - m);
      const float f_other = __builtin_amdgcn_exp2f(m_other - m);
      const float l = l_wave * f_own + l_other * f_other;
      const float inv = l > 0.f ? 1.f / l : 0.f;
      own_factor = f_own * inv;
      other_factor = f_other * inv;
    }
  }
  if (half == 0) {
    factor_lds[wave][n32] = own_factor;
    if constexpr (KW == 2) other_lds[wave][n32] = other_factor;
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  if (kw == 0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float4 inv4 = *reinterpret_cast<const float4*>(&factor_lds[wave][8 * i + 4 * half]);
      const float inv[4] = {inv4.x, inv4.y, inv4.z, inv4.w};
      float add[4] = {0.f, 0.f, 0.f, 0.f};
      if constexpr (KW == 2) {
        const float4 add4 = *reinterpret_cast<const float4*>(&other_lds[wave][8 * i + 4 * half]);
        add[0] = add4.x; add[1] = add4.y; add[2] = add4.z; add[3] = add4.w;
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int orow = pw * kWideRows + 8 * i + 4 * half + r;
        if (orow >= npos) continue;
        bf16_t* dst = out + (static_cast<size_t>(row0 + orow) * nq + head) * D;
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          float o = o_acc[db][4 * i + r] * inv[r];
          if constexpr (KW == 2) {
            const float* const tile_lds = reinterpret_cast<const float*>(page_lds);
            o = fmaf(tile_lds[(((wave % (HB * NG)) * DB + db) * 16 + 4 * i + r) * EI_WAVE + lane],
                     add[r], o);
          }
          dst[db * 32 + n32] = ei::from_f32<bf16_t>(o);
        }
      }
    }
  }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  }  // pass
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
  // all slices of (m, l) and of this lane's outputs are fetched before anything is
  // combined: one trip to memory for up to 8 slices
  const float2* ml = reinterpret_cast<const float2*>(part_ml) + static_cast<size_t>(wave) * n_splits;
  const float* po = part_o + static_cast<size_t>(wave) * n_splits * D;
  for (int d0 = 0; d0 < D; d0 += 2 * EI_WAVE) {
    const int d = d0 + 2 * lane;
    float m = kLowest, l = 0.f, o0 = 0.f, o1 = 0.f;
    for (int s0 = 0; s0 < n_splits; s0 += 8) {
      float2 st[8], ov[8];
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (s0 + u < n_splits) {
          st[u] = ml[s0 + u];
          ov[u] = d < D ? *reinterpret_cast<const float2*>(po + static_cast<size_t>(s0 + u) * D + d)
                        : float2{0.f, 0.f};
        }
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (s0 + u < n_splits) {
          const float m_new = fmaxf(m, st[u].x);
          const float keep = expf(m - m_new), add = expf(st[u].x - m_new);
          l = l * keep + st[u].y * add;
          o0 = o0 * keep + ov[u].x * add;
          o1 = o1 * keep + ov[u].y * add;
          m = m_new;
        }
    }
    if (d < D) {
      const float inv = l > 0.f ? 1.f / l : 0.f;
      bf16_t* dst = out + static_cast<size_t>(wave) * D + d;
      dst[0] = ei::from_f32<bf16_t>(o0 * inv);
      dst[1] = ei::from_f32<bf16_t>(o1 * inv);
    }
  }
}

template <int D, int GB, bool PREP>
void launch_decode(dim3 grid, hipStream_t stream, const bf16_t* q, const bf16_t* k,
                   const bf16_t* v, const int32_t* row_pos, const int32_t* row_seq,
                   const int32_t* page_table, int table_width, bf16_t* out, float* part_o,
                   float* part_ml, int nq, int nkv, int head_blocks, int window, float scale,
                   int n_splits, int waves, const int32_t* longest, const DecodePrep& prep) {
  if constexpr (GB <= 4) {               // the caller gives 16 waves at most 4 heads a block
    if (waves == 16) {
      attn_decode_kernel<D, GB, 16, PREP><<<grid, 16 * EI_WAVE, 0, stream>>>(
          q, k, v, row_pos, row_seq, page_table, table_width, out, part_o, part_ml, nq, nkv,
          head_blocks, window, scale, n_splits, longest, prep);
      return;
    }
  }
  if constexpr (GB <= 8) {               // and 8 waves at most 8
    if (waves == 8) {
      attn_decode_kernel<D, GB, 8, PREP><<<grid, 8 * EI_WAVE, 0, stream>>>(
          q, k, v, row_pos, row_seq, page_table, table_width, out, part_o, part_ml, nq, nkv,
          head_blocks, window, scale, n_splits, longest, prep);
      return;
    }
  }
  attn_decode_kernel<D, GB, 4, PREP><<<grid, 4 * EI_WAVE, 0, stream>>>(
        q, k, v, row_pos, row_seq, page_table, table_width, out, part_o, part_ml, nq, nkv,
        head_blocks, window, scale, n_splits, longest, prep);
}

}  // namespace

// Positions of one sequence that a prefill work item of this file holds for a group ratio
// (with key_ways = 2, half as many: two waves then share the keys of every page for the same
// rows, which gives a short prompt twice the blocks).
extern "C" int ei_attn_prefill_mfma_positions(int G) {
  const int HB = G % 4 == 0 ? 4 : (G % 2 == 0 ? 2 : 1);
  return kWideRows * (kPrefillWaves / HB);
}

template <int D, int HB, int KW>
static void launch_prefill(int blocks, hipStream_t stream, const bf16_t* q, const bf16_t* k,
                                const bf16_t* v, const int32_t* item_seq,
                                const int32_t* item_row0, const int32_t* item_npos, int n_items,
                                const int32_t* row_pos, const int32_t* page_table,
                                int table_width, bf16_t* out, int nq, int nkv, int window,
                                float scale, int pair) {
  attn_prefill_kernel<D, HB, KW><<<blocks, kPrefillThreads, 0, stream>>>(
      q, k, v, item_seq, item_row0, item_npos, n_items, row_pos, page_table, table_width, out,
      nq, nkv, window, scale, pair);
}

// q, out: [N, nq, D] bfloat16; items: (sequence, first packed row, positions), each holding
// at most ei_attn_prefill_mfma_positions(nq / nkv) / key_ways positions (key_ways 1 or 2; the
// kernel does not see an item's size, so items that are too large would lose rows: the
// caller, who makes them, is bound to it).  pair_items: a block may take item i and item
// n_items - 1 - i one after the other, which pays where those sums are about equal (the
// items of one prompt, longest first) and enough blocks remain.
extern "C" int ei_attention_prefill_mfma(const void* q, const void* k_pages, const void* v_pages,
                                         const int32_t* item_seq, const int32_t* item_row0,
                                         const int32_t* item_npos, int n_items,
                                         const int32_t* row_pos, const int32_t* page_table,
                                         int table_width, void* out, int nq, int nkv, int D,
                                         int window, float scale, int key_ways, int pair_items,
                                         hipStream_t stream) {
  EI_REQUIRE(n_items > 0 && nq > 0 && nkv > 0 && nq % nkv == 0, "attention_prefill: bad sizes");
  EI_REQUIRE(D == 64 || D == 128, "attention_prefill: this kernel takes head_dim 64 or 128");
  EI_REQUIRE(q && k_pages && v_pages && item_seq && item_row0 && item_npos && row_pos &&
                 page_table && out && table_width > 0,
             "attention_prefill: null pointer");
  EI_REQUIRE(window >= 0, "attention_prefill: negative window");
  const int G = nq / nkv;
  const int HB = G % 4 == 0 ? 4 : (G % 2 == 0 ? 2 : 1);
  EI_REQUIRE(key_ways == 1 || (key_ways == 2 && HB * 2 <= kPrefillWaves),
             "attention_prefill: key_ways must be 1 or 2");
  // Enough blocks to fill the chip twice over: pair a long item with a short one per block
  // (the caller orders the items by length, longest first), so that the blocks take about
  // equally long; with fewer blocks the pairs would leave compute units empty.  One causal
  // prompt gains 2 to 3 % by it.  Prompts of unequal lengths together lose: the sums of the
  // pairs are unequal then, and blocks of one item each, started longest first wherever a
  // place is free, spread better (700 and 1,500 tokens: 65 against 90 us unpaired; 300, 900,
  // 2,000 and 4,000: 233 against 251), so their caller does not ask for pairs.
  const int pair =
      pair_items && static_cast<long long>(n_items) * (G / HB) * nkv >= 2 * ei_compute_units() ? 1 : 0;
  const long long units = pair ? (n_items + 1) / 2 : n_items;
  const long long rests = units * (G / HB);
  long long blocks;
  if (nkv % 8 == 0) blocks = rests * nkv;
  else if (8 % nkv == 0) blocks = (rests + 8 / nkv - 1) / (8 / nkv) * 8;
  else blocks = rests * nkv;
  EI_REQUIRE(blocks < (1ll << 31), "attention_prefill: too many blocks");
  const bf16_t* qq = static_cast<const bf16_t*>(q);
  const bf16_t* kk = static_cast<const bf16_t*>(k_pages);
  const bf16_t* vv = static_cast<const bf16_t*>(v_pages);
  bf16_t* oo = static_cast<bf16_t*>(out);
#define EI_PREFILL(DD, HH)                                                                    \
  do {                                                                                        \
    if (key_ways == 2)                                                                        \
      launch_prefill<DD, HH, 2>(static_cast<int>(blocks), stream, qq, kk, vv, item_seq,       \
                                item_row0, item_npos, n_items, row_pos, page_table,           \
                                table_width, oo, nq, nkv, window, scale, pair);               \
    else                                                                                      \
      launch_prefill<DD, HH, 1>(static_cast<int>(blocks), stream, qq, kk, vv, item_seq,       \
                                item_row0, item_npos, n_items, row_pos, page_table,           \
                                table_width, oo, nq, nkv, window, scale, pair);               \
  } while (0)
  if (D == 64) {
    if (HB == 4) EI_PREFILL(64, 4); else if (HB == 2) EI_PREFILL(64, 2); else EI_PREFILL(64, 1);
  } else {
    if (HB == 4) EI_PREFILL(128, 4); else if (HB == 2) EI_PREFILL(128, 2); else EI_PREFILL(128, 1);
  }
#undef EI_PREFILL
  EI_LAUNCH_CHECK();
}

// Whether the decode kernel of this file takes a head size and group ratio.
extern "C" int ei_attn_decode_mfma_supported(int D, int G) {
  return (D == 64 || D == 128) && G >= 1 ? 1 : 0;
}

static int decode_launch(const void* q, const void* k_pages, const void* v_pages,
                         const int32_t* row_pos, const int32_t* row_seq,
                         const int32_t* page_table, int table_width, void* out, float* part_o,
                         float* part_ml, int rows, int nq, int nkv, int D, int window,
                         float scale, int n_splits, int waves, int heads, const int32_t* longest,
                         const DecodePrep* prep, hipStream_t stream) {
  EI_REQUIRE(rows > 0 && nq > 0 && nkv > 0 && nq % nkv == 0, "attention_decode: bad head counts");
  EI_REQUIRE(waves == 4 || waves == 8 || waves == 16,
             "attention_decode: a block has 4, 8 or 16 waves");
  EI_REQUIRE(D == 64 || D == 128, "attention_decode: this kernel takes head_dim 64 or 128");
  EI_REQUIRE((q || prep) && k_pages && v_pages && row_pos && row_seq && page_table && out &&
                 table_width > 0,
             "attention_decode: null pointer");
  EI_REQUIRE(n_splits >= 1 && n_splits <= 64, "attention_decode: splits must be between 1 and 64");
  EI_REQUIRE(n_splits == 1 || (part_o && part_ml), "attention_decode: split scratch missing");
  EI_REQUIRE(window >= 0, "attention_decode: negative window");
  const int G = nq / nkv;
  // heads of a kv group that one block takes; blocks of 16 waves take at most 4 and blocks of
  // 8 waves at most 8 (their merge buffers grow with both), a larger group then has several
  // blocks per kv head
  int GB = G >= 8 ? (G >= 16 ? 16 : 8) : (G >= 4 ? 4 : (G >= 2 ? 2 : 1));
  if (waves == 16 && GB > 4) GB = 4;
  if (waves == 8 && GB > 8) GB = 8;
  // the caller may ask for fewer (a power of two): more, lighter blocks where the step has
  // too few of them to occupy the chip
  if (heads > 0) {
    EI_REQUIRE((heads & (heads - 1)) == 0, "attention_decode: heads a block must be a power of two");
    if (heads < GB) GB = heads;
  }
  const int head_blocks = (G + GB - 1) / GB;
  EI_REQUIRE(static_cast<long long>(nkv) * head_blocks <= 65535, "attention_decode: too many heads");
  dim3 grid(rows, nkv * head_blocks, n_splits);
  const bf16_t* qq = static_cast<const bf16_t*>(q);
  const bf16_t* kk = static_cast<const bf16_t*>(k_pages);
  const bf16_t* vv = static_cast<const bf16_t*>(v_pages);
  bf16_t* oo = static_cast<bf16_t*>(out);
  const DecodePrep none{};
#define EI_DECODE(DD, GG)                                                                     \
  do {                                                                                        \
    if (prep)                                                                                 \
      launch_decode<DD, GG, true>(grid, stream, qq, kk, vv, row_pos, row_seq, page_table,     \
                                  table_width, oo, part_o, part_ml, nq, nkv, head_blocks,     \
                                  window, scale, n_splits, waves, longest, *prep);            \
    else                                                                                      \
      launch_decode<DD, GG, false>(grid, stream, qq, kk, vv, row_pos, row_seq, page_table,    \
                                   table_width, oo, part_o, part_ml, nq, nkv, head_blocks,    \
                                   window, scale, n_splits, waves, longest, none);            \
  } while (0)
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

// q, out: [rows, nq, D] bfloat16, one row per sequence (row_seq < 0: padding row);
// pages: [n_pages, nkv, 64, D]; n_splits > 1 needs part_o [rows, nq, n_splits, D] and
// part_ml [rows, nq, n_splits, 2] float32.  longest (or null): one int32 on the device, the most
// tokens that a sequence of this step holds; slices are then that sequence's share for all.
// heads: query heads of a kv group that one block takes (a power of two; 0: as many as a
// block of `waves` waves can, 4 for 16 waves, 8 for 8, else 16); a group of more has several
// blocks.
extern "C" int ei_attention_decode_mfma(const void* q, const void* k_pages, const void* v_pages,
                                        const int32_t* row_pos, const int32_t* row_seq,
                                        const int32_t* page_table, int table_width, void* out,
                                        float* part_o, float* part_ml, int rows, int nq, int nkv,
                                        int D, int window, float scale, int n_splits,
                                        int waves, int heads, const int32_t* longest,
                                        hipStream_t stream) {
  return decode_launch(q, k_pages, v_pages, row_pos, row_seq, page_table, table_width, out,
                       part_o, part_ml, rows, nq, nkv, D, window, scale, n_splits, waves, heads,
                       longest, nullptr, stream);
}

// The same from the fused projection instead of q: qkv float32 [nsplit][rows, (nq + 2 nkv) * D]
// (partial sums, added in slice order); the kernel norms and rotates its queries itself and,
// with write_cache, also the position's key, and stores that key and the value in the pages
// (so the separate norm-rotate-store kernel is not needed for these rows).  q_norm_w, k_norm_w
// (float32 [D]) and rope_table (float32 [positions, rot_dim], rot_dim even and at most D) may
// each be null.
extern "C" int ei_attention_decode_mfma_fused(
    const float* qkv, int nsplit, long long split_stride, const float* q_norm_w,
    const float* k_norm_w, float eps, const float* rope_table, int rot_dim, int write_cache,
    void* k_pages,
    void* v_pages, const int32_t* row_pos, const int32_t* row_seq, const int32_t* page_table,
    int table_width, void* out, float* part_o, float* part_ml, int rows, int nq, int nkv, int D,
    int window, float scale, int n_splits, int waves, int heads, const int32_t* longest,
    hipStream_t stream) {
  EI_REQUIRE(qkv && nsplit >= 1 && split_stride >= 0, "attention_decode_fused: bad projection");
  EI_REQUIRE(!rope_table || (rot_dim >= 2 && rot_dim % 2 == 0 && rot_dim <= D),
             "attention_decode_fused: the rotated width must be even and at most head_dim");
  DecodePrep prep{};
  prep.qkv = qkv;
  prep.nsplit = nsplit;
  prep.split_stride = split_stride;
  prep.q_norm_w = q_norm_w;
  prep.k_norm_w = k_norm_w;
  prep.eps = eps;
  prep.rope_table = rope_table;
  prep.rot_dim = rope_table ? rot_dim : D;
  prep.k_store = write_cache ? static_cast<bf16_t*>(k_pages) : nullptr;
  prep.v_store = write_cache ? static_cast<bf16_t*>(v_pages) : nullptr;
  return decode_launch(nullptr, k_pages, v_pages, row_pos, row_seq, page_table, table_width, out,
                       part_o, part_ml, rows, nq, nkv, D, window, scale, n_splits, waves, heads,
                       longest, &prep, stream);
}
