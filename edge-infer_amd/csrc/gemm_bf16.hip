// Weight-streaming matrix product for few rows (decode): out[s][m][n] = partial sums of
// X[m, :] . W[n, :] over the s-th slice of K, for M <= 256 rows of X.
//
// W is a bfloat16 checkpoint matrix [N, K] and is read exactly once, straight from global
// memory into MFMA operand registers (v_mfma_f32_16x16x32_bf16: lane (row r, quarter c) holds
// 8 consecutive k of row r).  It is read either in its stored layout or, faster, from a copy
// packed at load time into whole MFMA tiles (see ei_gemm_bf16_skinny_packed).  X (small) is
// staged in LDS one K-tile at a time: with packed W it travels from global memory straight
// into LDS (global_load_lds, no registers), otherwise through registers.  A workgroup is 4, 6
// or 8 waves, each owning 16 rows of W (32 for more than 64 rows of X with packed W, so that
// every operand of X read from LDS feeds two products), and takes 16, 32, 64 or 128 rows of X;
// more rows go to further workgroups that share the weights through the L2 of their die.  K may be split over
// blockIdx.y, in which case every slice writes float32 partial sums [slice, M, N] that the
// consuming kernel adds in slice order while it reads them (deterministic, no atomics, and no
// device-wide fence: the kernel boundary orders the writes before the reads).  The host picks
// the waves and slices per shape.
//
// Accumulation is float32 throughout, as in the reference's cublasGemmEx call
// (operators/src/cuda/execution.cu:319-323); the sums stay float32 and the consumer rounds
// once when it stores in the storage type.
#include "common.h"

#include <type_traits>

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

namespace {

constexpr int kPackedTile = 16 * 32;      // elements of one packed tile: 16 rows x 32 k, 1 KB

// MB * 16 rows of X per workgroup, any K range.  A workgroup is WAVES waves, each owning
// STRIPS strips of 16 rows of W; X travels through LDS one K-tile (KT: 256, or 128 where two
// strips need the registers) at a time, two tiles of it alternate so that a tile costs one
// barrier.  W has two register sets that are refilled piece by piece:
// as soon as the products of one 32-wide step have read their piece, the same piece of the
// tile after next is requested, so two tiles of W per wave are always on their way.  The
// loads of the steady loop are unconditional (clamped addresses), so the number outstanding
// is the same on every path and each wait leaves the younger loads in flight.
// Few K slices: for many rows the float32 partial sums (rows x N x 4 bytes a slice, written
// in 64-byte pieces and read again by the consumer) cost more than the weights they save.
//
// GATED (one K slice only): the strips of W alternate between 16 gate rows and the 16 up rows
// that belong to them; even waves hold gate sums, their odd neighbours the up sums (with two
// strips a wave holds both), and the block writes silu(gate) * up as bfloat16 [M, N/2] to
// `gated_out` instead of any sums.
template <int MB, int WAVES, bool PACKED, bool GATED, int STRIPS, int KT>
__global__ void __launch_bounds__(WAVES * EI_WAVE)
skinny_gemm_kernel(const bf16_t* __restrict__ W, const bf16_t* __restrict__ X,
                   float* __restrict__ out, bf16_t* __restrict__ gated_out, int M, int N, int K,
                   int k_per_split, int row_groups) {
  constexpr int JN = KT / 32;             // MFMA steps per K-tile
  static_assert(KT == 256 || (KT == 128 && PACKED), "K-tiles of 256, or 128 with packed weights");
  constexpr int ROWS_X = MB * 16;
  constexpr int XS = KT;                  // LDS row stride in elements; the 16-byte chunks of a
                                          // row are stored at (chunk ^ row % 16), see store_x
  // X travels in wave loads of a kilobyte, RPL rows of the tile each: lane (half, chunk) takes
  // the 16-byte chunk `chunk` of row RPL * load + half
  constexpr int CH = KT / 8, RPL = EI_WAVE / CH;
  constexpr int PAIRS = ROWS_X / RPL;
  constexpr int XLOADS = (PAIRS + WAVES - 1) / WAVES;
  __shared__ __attribute__((aligned(16))) bf16_t xs[2][ROWS_X * XS];

  const int t = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(t / EI_WAVE), lane = t % EI_WAVE;
  const int r16 = lane & 15, c = lane >> 4;
  // More than ROWS_X rows: `row_groups` blocks share every strip group, each with ROWS_X rows
  // of X.  Block ids go round the 8 dies, so the blocks of one strip group are 8 ids apart:
  // they start together on one die and the later ones find the weights in its L2.
  int strip_block = blockIdx.x, row0 = 0;
  if (row_groups > 1) {
    row0 = (strip_block >> 3) % row_groups * ROWS_X;
    strip_block = strip_block / (8 * row_groups) * 8 + (strip_block & 7);
  }
  if (strip_block * WAVES * 16 * STRIPS >= N || row0 >= M) return;
  const int rows_here = min(ROWS_X, M - row0);
  X += static_cast<size_t>(row0) * K;
  const int n_tile = (strip_block * WAVES + wave) * 16 * STRIPS;
  const int k_begin = blockIdx.y * k_per_split;
  const int k_end = min(K, k_begin + k_per_split);
  const int n_iter = (k_end - k_begin + KT - 1) / KT;
  if (n_iter <= 0) return;

  int w_row = n_tile + r16;
  if (w_row >= N) w_row = N - 1;          // rows past the end repeat the last one; never stored
  const int n_strips = (N + 15) / 16;
  const int strip = min(n_tile / 16, n_strips - 1);
  const bf16_t* w_ptr = W + static_cast<size_t>(w_row) * K + c * 8;     // stored layout
  // packed: a base that is the same for the whole block plus a lane's 32-bit offset (the
  // loads then take a scalar address and need no address registers)
  unsigned w_lane[STRIPS];                                                                // bytes
#pragma unroll
  for (int s = 0; s < STRIPS; ++s)
    w_lane[s] = (static_cast<unsigned>(min(strip + s, n_strips - 1)) * kPackedTile + lane * 8) * 2u;
  const size_t tile_stride = static_cast<size_t>(n_strips) * kPackedTile;

  f32x4 acc[MB][STRIPS];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int s = 0; s < STRIPS; ++s) acc[mb][s] = f32x4{0.f, 0.f, 0.f, 0.f};

  bf16x8 w[2][JN][STRIPS];
  u32x4 x_regs[XLOADS];
  const u32x4 zero4 = u32x4{0u, 0u, 0u, 0u};

  auto load_w_piece = [&](int set, int tile, int j) {
    const int kb = k_begin + tile * KT;
    if (PACKED) {
      // the packed copy holds whole K-tiles (zeros past K): no test
      const bf16_t* tile = W + (kb / 32 + j) * tile_stride;
#pragma unroll
      for (int s = 0; s < STRIPS; ++s)
        w[set][j][s] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(
            reinterpret_cast<const char*>(tile) + w_lane[s]));
    } else {
      // clamped to the last piece of the slice; the matching piece of X is zero there
      const int k = min(kb + j * 32 + c * 8, k_end - 8);
      w[set][j][0] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(w_ptr + k - c * 8));
    }
  };
  // Rows past the last one repeat it (their sums are never stored), so every load is in
  // bounds and none is conditional; k past the end of the slice can only occur in its last
  // tile, where the address is clamped (and, on the register path, zeros are stored).
  // Row r keeps its 16-byte chunk g at place g ^ (r % 16), so that the operand reads (16
  // rows, quarters c and c + 1 of a 32-wide step in one access group) touch every bank once.
  const int x_half = lane / CH, x_place = lane % CH;
  unsigned x_row[XLOADS];
  int x_k[XLOADS];
#pragma unroll
  for (int i = 0; i < XLOADS; ++i) {
    const int row = RPL * min(wave + i * WAVES, PAIRS - 1) + x_half;   // surplus loads repeat the last group
    x_row[i] = static_cast<unsigned>(min(row, rows_here - 1)) * K;
    x_k[i] = (x_place ^ (row & 15)) * 8;
  }
  // packed W (zeros past K, so whatever finite X meets them counts nothing): X goes from
  // global memory straight into LDS, a wave load lands as one kilobyte at the pair's place
  auto dma_x = [&](int buf, int tile) {
    const int kb = k_begin + tile * KT;
    if constexpr (STRIPS == 2) {
      // the addresses are worked out anew at every tile (a few instructions a load) instead of
      // being kept: this form is short of registers
      int wv = wave;
      asm volatile("" : "+s"(wv));
#pragma unroll
      for (int i = 0; i < XLOADS; ++i) {
        const int pair = min(wv + i * WAVES, PAIRS - 1);
        const int row = RPL * pair + x_half;
        const unsigned k = min(kb + (x_place ^ (row & 15)) * 8, k_end - 8);
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void*)(
                X + (static_cast<unsigned>(min(row, rows_here - 1)) * K + k)),
            (__attribute__((address_space(3))) void*)(&xs[buf][pair * RPL * XS]), 16, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
      return;
    }
#pragma unroll
    for (int i = 0; i < XLOADS; ++i) {
      const int pair = min(wave + i * WAVES, PAIRS - 1);
      const unsigned k = min(kb + x_k[i], k_end - 8);
      __builtin_amdgcn_global_load_lds(
          (const __attribute__((address_space(1))) void*)(X + (x_row[i] + k)),
          (__attribute__((address_space(3))) void*)(&xs[buf][pair * RPL * XS]), 16, 0, 0);
    }
    __builtin_amdgcn_sched_barrier(0);     // the waits below count the loads issued after these
  };
  // stored layout: through registers
  auto load_x = [&](int tile) {
    const int kb = k_begin + tile * KT;
#pragma unroll
    for (int i = 0; i < XLOADS; ++i)
      x_regs[i] = *reinterpret_cast<const u32x4*>(X + (x_row[i] + min(kb + x_k[i], k_end - 8)));
  };
  // `last_tag`: the tile may be the last of the slice (k is checked)
  auto store_x = [&](int buf, int tile, auto last_tag) {
    constexpr bool check_k = decltype(last_tag)::value;
    const int kb = k_begin + tile * KT;
#pragma unroll
    for (int i = 0; i < XLOADS; ++i) {
      const int pair = wave + i * WAVES;               // the same for the whole wave
      const bool k_ok = !check_k || kb + x_k[i] < k_end;
      if (PAIRS % WAVES == 0 || pair < PAIRS)
        *reinterpret_cast<u32x4*>(&xs[buf][(RPL * pair + x_half) * XS + x_place * 8]) =
            k_ok ? x_regs[i] : zero4;
    }
  };
  // products of a tile whose W is in register set `set` and whose X is in LDS buffer `set`
  // (even tiles 0, odd tiles 1); refill >= 0: request every piece of that tile into the set
  // that is being used up.  `set` is a constant at every call, so that the sets stay registers.
  auto compute = [&](auto set_tag, auto refill_tag, int refill) {
    constexpr int set = decltype(set_tag)::value;
    constexpr bool do_refill = decltype(refill_tag)::value;
    // chunk 4j + c of row r16 lies at chunk (4j + c) ^ r16 = 4 (j ^ r16 / 4) + (c ^ r16 % 4):
    // four lane addresses (j % 4), the rest are constant offsets
    const bf16_t* x_base = &xs[set][r16 * XS + (c ^ (r16 & 3)) * 8];
    const bf16_t* x_step[4];
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) x_step[jj] = x_base + (jj ^ (r16 >> 2)) * 32;
    // a unit: one 32-wide step of W against HB row tiles of X (128 rows take two units a
    // step); the operands of the next unit are read while this one multiplies
    constexpr int HB = (STRIPS == 2 && MB == 8 && WAVES > 4) ? 2 : (MB < 4 ? MB : 4), UNITS = MB / HB;
    bf16x8 xf[2][HB];
#pragma unroll
    for (int mb = 0; mb < HB; ++mb)
      xf[0][mb] = *reinterpret_cast<const bf16x8*>(x_step[0] + mb * 16 * XS);
#pragma unroll
    for (int u = 0; u < JN * UNITS; ++u) {
      const int j = u / UNITS, h = u % UNITS;
      if (u + 1 < JN * UNITS) {
        const int jn = (u + 1) / UNITS, hn = (u + 1) % UNITS;
#pragma unroll
        for (int mb = 0; mb < HB; ++mb)
          xf[(u + 1) & 1][mb] = *reinterpret_cast<const bf16x8*>(
              x_step[jn & 3] + (hn * HB + mb) * 16 * XS + (jn & 4) * 32);
      }
      // keep this order (reads of the next unit, products, refill): left alone the
      // scheduler pairs every read with its use and gathers the refills at the end
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int mb = 0; mb < HB; ++mb)
#pragma unroll
        for (int s = 0; s < STRIPS; ++s)
          acc[h * HB + mb][s] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
              w[set][j][s], xf[u & 1][mb], acc[h * HB + mb][s], 0, 0, 0);
      if (do_refill && h == UNITS - 1) load_w_piece(set, refill, j);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  using Set0 = std::integral_constant<int, 0>;
  using Set1 = std::integral_constant<int, 1>;
  using Refill = std::true_type;
  using Last = std::false_type;

  using Inner = std::false_type;
  using MaybeLast = std::true_type;
  if constexpr (PACKED) {
    // s_waitcnt vmcnt(n): everything but the n youngest loads has arrived, i.e. the X tile
    // requested before the n pieces of W that were requested after it.  A wave waits for
    // its own part of the tile, the barrier then covers everybody's.  (No fence here: it
    // would wait for the pieces of W as well.)
    auto x_arrived = [&](auto younger_tag) {
      constexpr int younger = decltype(younger_tag)::value;
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_waitcnt(0x0F70 | (younger & 15) | ((younger >> 4) << 14));
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
    };
    using OneSet = std::integral_constant<int, JN * STRIPS>;
    using TwoSets = std::integral_constant<int, 2 * JN * STRIPS>;
    using None = std::integral_constant<int, 0>;
    dma_x(0, 0);
#pragma unroll
    for (int j = 0; j < JN; ++j) load_w_piece(0, 0, j);
    if (n_iter == 1) {
      x_arrived(OneSet{});
      compute(Set0{}, Last{}, 0);
    } else {
#pragma unroll
      for (int j = 0; j < JN; ++j) load_w_piece(1, 1, j);
      x_arrived(TwoSets{});
      int i = 0;                            // even: tile i is in set 0 and in X buffer 0
      for (; i + 3 < n_iter; i += 2) {      // tiles i + 2 and i + 3 exist
        dma_x(1, i + 1);
        compute(Set0{}, Refill{}, i + 2);
        x_arrived(OneSet{});
        dma_x(0, i + 2);
        compute(Set1{}, Refill{}, i + 3);
        x_arrived(OneSet{});
      }
      if (i + 2 < n_iter) {                 // three tiles remain
        dma_x(1, i + 1);
        compute(Set0{}, Refill{}, i + 2);
        x_arrived(OneSet{});
        dma_x(0, i + 2);
        compute(Set1{}, Last{}, 0);
        x_arrived(None{});
        compute(Set0{}, Last{}, 0);
      } else {                              // two
        dma_x(1, i + 1);
        compute(Set0{}, Last{}, 0);
        x_arrived(None{});
        compute(Set1{}, Last{}, 0);
      }
    }
  } else {
    load_x(0);
#pragma unroll
    for (int j = 0; j < JN; ++j) load_w_piece(0, 0, j);
    if (n_iter == 1) {
      store_x(0, 0, MaybeLast{});
      __syncthreads();
      compute(Set0{}, Last{}, 0);
    } else {
#pragma unroll
      for (int j = 0; j < JN; ++j) load_w_piece(1, 1, j);
      store_x(0, 0, Inner{});
      load_x(1);
      __syncthreads();
      int i = 0;                            // even: tile i is in set 0
      for (; i + 3 < n_iter; i += 2) {      // tiles i + 2 and i + 3 exist
        compute(Set0{}, Refill{}, i + 2);
        store_x(1, i + 1, Inner{});
        load_x(i + 2);
        __syncthreads();
        compute(Set1{}, Refill{}, i + 3);
        store_x(0, i + 2, Inner{});
        load_x(i + 3);
        __syncthreads();
      }
      if (i + 2 < n_iter) {                 // three tiles remain
        compute(Set0{}, Refill{}, i + 2);
        store_x(1, i + 1, Inner{});
        load_x(i + 2);
        __syncthreads();
        compute(Set1{}, Last{}, 0);
        store_x(0, i + 2, MaybeLast{});
        __syncthreads();
        compute(Set0{}, Last{}, 0);
      } else {                              // two
        compute(Set0{}, Last{}, 0);
        store_x(1, i + 1, MaybeLast{});
        __syncthreads();
        compute(Set1{}, Last{}, 0);
      }
    }
  }

  if constexpr (GATED && STRIPS == 2) {
    // the wave holds the gate sums (strip 0) and the up sums (strip 1) of its 16 outputs
    if (n_tile + 16 < N) {
      const int half = N / 2;
      const int col = n_tile / 2 + 4 * c;                       // (strip / 2) * 16 + 4c
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const int m = row0 + mb * 16 + r16;
        if (m >= M) continue;
        uint32_t packed[2];
#pragma unroll
        for (int r = 0; r < 4; r += 2) {
          const bf16_t lo = ei::f32_to_bf16(ei::silu<bf16_t>(acc[mb][0][r]) * acc[mb][1][r]);
          const bf16_t hi = ei::f32_to_bf16(ei::silu<bf16_t>(acc[mb][0][r + 1]) * acc[mb][1][r + 1]);
          packed[r / 2] = static_cast<uint32_t>(lo) | (static_cast<uint32_t>(hi) << 16);
        }
        *reinterpret_cast<uint2*>(gated_out + static_cast<size_t>(m) * half + col) =
            uint2{packed[0], packed[1]};
      }
    }
    return;
  } else if constexpr (GATED) {
    static_assert(!GATED || WAVES % 2 == 0, "gate and up strips are held by neighbouring waves");
    // up sums travel through LDS (the X tiles are done with) to the wave that holds the gates
    __syncthreads();
    f32x4* exchange = reinterpret_cast<f32x4*>(&xs[0][0]);      // WAVES/2 * MB * 64 * 16 bytes
    static_assert(sizeof(xs) >= WAVES / 2 * MB * EI_WAVE * sizeof(f32x4), "exchange fits");
    if (wave & 1) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) exchange[((wave >> 1) * MB + mb) * EI_WAVE + lane] = acc[mb][0];
    }
    __syncthreads();
    if (!(wave & 1) && n_tile + 16 < N) {
      const int half = N / 2;
      const int col = n_tile / 2 + 4 * c;                       // (strip / 2) * 16 + 4c
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const int m = row0 + mb * 16 + r16;
        if (m >= M) continue;
        const f32x4 up = exchange[((wave >> 1) * MB + mb) * EI_WAVE + lane];
        uint32_t packed[2];
#pragma unroll
        for (int r = 0; r < 4; r += 2) {
          const bf16_t lo = ei::f32_to_bf16(ei::silu<bf16_t>(acc[mb][0][r]) * up[r]);
          const bf16_t hi = ei::f32_to_bf16(ei::silu<bf16_t>(acc[mb][0][r + 1]) * up[r + 1]);
          packed[r / 2] = static_cast<uint32_t>(lo) | (static_cast<uint32_t>(hi) << 16);
        }
        *reinterpret_cast<uint2*>(gated_out + static_cast<size_t>(m) * half + col) =
            uint2{packed[0], packed[1]};
      }
    }
    return;
  }

  // lane (c, r16) holds out[m = mb*16 + r16][n_tile + 16 s + 4c + 0..3]
  float* dst = out + static_cast<size_t>(blockIdx.y) * M * N;
#pragma unroll
  for (int s = 0; s < STRIPS; ++s) {
    const int n0 = n_tile + 16 * s + 4 * c;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int m = row0 + mb * 16 + r16;
      if (m >= M) continue;
      float* p = dst + static_cast<size_t>(m) * N + n0;
      if (n0 + 3 < N && (N & 3) == 0) {
        *reinterpret_cast<f32x4*>(p) = acc[mb][s];
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if (n0 + r < N) p[r] = acc[mb][s][r];
      }
    }
  }
}

constexpr int kTile = 256;                // K-tile of the kernel
constexpr int kGroupRows = 64;            // rows of X one block takes
constexpr int kMaxRows = 256;

// Waves per block (4, 6 or 8) and what the busiest compute unit then has to do, in strips:
// `strips * splits` strip-slices are dealt out in blocks of `waves` strips.  Up to two blocks
// per unit all run at once, so the unit with the most blocks sets the time; many more blocks
// than that even out.  Every block also costs a start (about 3 strip-tiles).  Near ties go
// to the larger block, which shares a tile of X among more waves.  `row_groups` blocks work
// on every strip group (more rows of X than one block takes).
int tile_kernel_waves(int n_strips, int splits, int row_groups, double tiles_per_slice,
                      double* cost_out) {
  const int kComputeUnits = ei_compute_units();
  int best = 8;
  double best_cost = 1e30;
  for (int waves = 8; waves >= 4; waves -= 2) {
    const double blocks = static_cast<double>((n_strips + waves - 1) / waves) * splits * row_groups;
    const double per_unit = blocks <= 2 * kComputeUnits
                                ? static_cast<double>((static_cast<long long>(blocks) + kComputeUnits - 1) / kComputeUnits)
                                : blocks / kComputeUnits + 0.25;
    const double cost = per_unit * (waves * tiles_per_slice + 3.0);
    if (cost < best_cost * 0.97) {          // a smaller block must be clearly better
      best_cost = cost;
      best = waves;
    }
  }
  if (cost_out) *cost_out = best_cost;
  return best;
}

// How a row count is served with packed weights: 16-row tiles of X a block, strips of W a
// wave, width of a K-tile.  Up to 64 rows the product is bound by memory and a wave owns one
// strip.  Beyond, a product per kilobyte read from LDS is twice what LDS delivers, so a wave
// owns two strips and every operand of X feeds two products: 65 to 128 rows as two blocks of
// 64 rows for each group of strips, more as two blocks of 128 (the slices are planned for
// that).  Except for 65 to 128 rows of a matrix with at least four strips for every wave
// slot of the chip's first round (gate_up, the head): there one block of 128 rows with one
// strip a wave reads the weights once, which weighs more (measured in the decode step: 46
// against 49 us for gate_up of the 8B shape, 266 against 305 for its head).  The stored
// layout keeps one strip and blocks of 64 rows.
struct TileMode {
  int mb, strips, kt;
};

TileMode packed_mode(int M, int N) {
  if (M > 128) return TileMode{8, 2, 128};
  if (M > kGroupRows && (N + 15) / 16 >= 4 * ei_compute_units()) return TileMode{8, 1, 256};
  if (M > kGroupRows) return TileMode{4, 2, 128};
  return TileMode{M <= 16 ? 1 : (M <= 32 ? 2 : 4), 1, 256};
}

bool valid_slice_count(int k_tiles, int splits) {
  if (splits < 1 || splits > k_tiles) return false;
  const int per = (k_tiles + splits - 1) / splits;
  return (k_tiles + per - 1) / per == splits;
}

}  // namespace

// The number of K slices the kernel will use for these sizes (the caller sizes `out`): the
// count that leaves the busiest compute unit the least to do, where a slice's partial sums
// (rows * N * 4 bytes, written in small pieces and read again by the consumer) are priced at
// 2.5 times their size.  `max_splits` > 0 caps it.
extern "C" int ei_skinny_gemm_splits(int M, int N, int K, int max_splits) {
  if (M < 1 || N < 1 || K < 1) return 1;
  const int k_tiles = (K + kTile - 1) / kTile;
  const int n_strips = (N + 15) / 16;
  if (max_splits <= 0 || max_splits > 16) max_splits = 16;
  const int kComputeUnits = ei_compute_units();
  int best = 1;
  double best_cost = 1e30;
  for (int splits = 1; splits <= max_splits && splits <= k_tiles; ++splits) {
    if (!valid_slice_count(k_tiles, splits)) continue;
    const double tiles = static_cast<double>((k_tiles + splits - 1) / splits);
    double cost = 0.0;                                   // in strip-tiles (8 KB of W) per unit
    const TileMode mode = packed_mode(M, N);
    tile_kernel_waves((n_strips + mode.strips - 1) / mode.strips, splits,
                      (M + mode.mb * 16 - 1) / (mode.mb * 16), mode.strips * tiles, &cost);
    cost += 2.5 * splits * static_cast<double>(M) * N * 4.0 / kComputeUnits / 8192.0;
    if (cost < best_cost - 1e-9) {
      best_cost = cost;
      best = splits;
    }
  }
  return best;
}

namespace {

template <int MB, bool PACKED, bool GATED, int STRIPS, int KT = 256>
void launch_tile_kernel(const bf16_t* w, const bf16_t* x, float* out, bf16_t* gated_out, int M,
                        int N, int K, int k_per_split, int splits, hipStream_t stream) {
  const int n_strips = ((N + 15) / 16 + STRIPS - 1) / STRIPS;     // what a wave owns
  const int row_groups = (M + MB * 16 - 1) / (MB * 16);
  const int waves = tile_kernel_waves(n_strips, splits, row_groups,
                                      STRIPS * k_per_split / static_cast<double>(kTile), nullptr);
  int strip_blocks = (n_strips + waves - 1) / waves;
  if (row_groups > 1) strip_blocks = (strip_blocks + 7) / 8 * 8;   // whole rounds of the dies
  dim3 grid(strip_blocks * row_groups, splits);
  if (waves == 4)
    skinny_gemm_kernel<MB, 4, PACKED, GATED, STRIPS, KT><<<grid, 4 * EI_WAVE, 0, stream>>>(
        w, x, out, gated_out, M, N, K, k_per_split, row_groups);
  else if (waves == 6)
    skinny_gemm_kernel<MB, 6, PACKED, GATED, STRIPS, KT><<<grid, 6 * EI_WAVE, 0, stream>>>(
        w, x, out, gated_out, M, N, K, k_per_split, row_groups);
  else
    skinny_gemm_kernel<MB, 8, PACKED, GATED, STRIPS, KT><<<grid, 8 * EI_WAVE, 0, stream>>>(
        w, x, out, gated_out, M, N, K, k_per_split, row_groups);
}

template <bool PACKED, bool GATED>
int launch_skinny(const void* X, const void* W, float* out, void* gated_out, int M, int N, int K,
                  int splits, hipStream_t stream) {
  EI_REQUIRE(M >= 1 && M <= kMaxRows, "gemm_bf16_skinny: rows must lie in 1..256");
  EI_REQUIRE(N >= 1 && K >= 8 && K % 8 == 0, "gemm_bf16_skinny: K must be a multiple of 8");
  EI_REQUIRE(X && W && (GATED ? gated_out != nullptr : out != nullptr), "gemm_bf16_skinny: null pointer");

  EI_REQUIRE((reinterpret_cast<uintptr_t>(X) & 15) == 0 && (reinterpret_cast<uintptr_t>(W) & 15) == 0 &&
                 (reinterpret_cast<uintptr_t>(out) & 15) == 0 &&
                 (reinterpret_cast<uintptr_t>(gated_out) & 15) == 0,
             "gemm_bf16_skinny: pointers must be 16-byte aligned");
  if (GATED) {
    EI_REQUIRE(splits == 1, "gemm_bf16_skinny_gated: K cannot be sliced");
    EI_REQUIRE(N % 32 == 0, "gemm_bf16_skinny_gated: N must be a multiple of 32 (gate and up strips)");
  }
  const TileMode mode = PACKED ? packed_mode(M, N) : TileMode{M <= 16 ? 1 : (M <= 32 ? 2 : 4), 1, 256};
  const int MB = mode.mb;
  const int k_tiles = (K + kTile - 1) / kTile;
  EI_REQUIRE(splits >= 1 && splits <= k_tiles, "gemm_bf16_skinny: bad slice count");
  EI_REQUIRE(valid_slice_count(k_tiles, splits), "gemm_bf16_skinny: slice count leaves an empty slice");
  const int k_per_split = (k_tiles + splits - 1) / splits * kTile;
  const bf16_t* x = static_cast<const bf16_t*>(X);
  const bf16_t* w = static_cast<const bf16_t*>(W);
  bf16_t* g = static_cast<bf16_t*>(gated_out);
  if (mode.strips == 2) {
    if constexpr (PACKED) {
      if (MB == 4)
        launch_tile_kernel<4, PACKED, GATED, 2, 128>(w, x, out, g, M, N, K, k_per_split, splits, stream);
      else
        launch_tile_kernel<8, PACKED, GATED, 2, 128>(w, x, out, g, M, N, K, k_per_split, splits, stream);
    }
  } else if (MB == 1) {
    launch_tile_kernel<1, PACKED, GATED, 1>(w, x, out, g, M, N, K, k_per_split, splits, stream);
  } else if (MB == 2) {
    launch_tile_kernel<2, PACKED, GATED, 1>(w, x, out, g, M, N, K, k_per_split, splits, stream);
  } else if (MB == 4) {
    launch_tile_kernel<4, PACKED, GATED, 1>(w, x, out, g, M, N, K, k_per_split, splits, stream);
  } else {
    if constexpr (PACKED)
      launch_tile_kernel<8, PACKED, GATED, 1>(w, x, out, g, M, N, K, k_per_split, splits, stream);
  }
  EI_LAUNCH_CHECK();
}

}  // namespace

// X: [M, K] bfloat16, W: [N, K] bfloat16, out: [splits, M, N] float32 (slice s holds the
// sums over the s-th part of K).  K must be a multiple of 8 (16-byte loads), M at most 256
// (beyond 64 rows several blocks share the weights through the L2 of their die).
extern "C" int ei_gemm_bf16_skinny(const void* X, const void* W, float* out, int M, int N, int K,
                                   int splits, hipStream_t stream) {
  return launch_skinny<false, false>(X, W, out, nullptr, M, N, K, splits, stream);
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
  return launch_skinny<true, false>(X, Wp, out, nullptr, M, N, K, splits, stream);
}

// Gated feed-forward in one pass: W [N, K] holds, in strips of 16 rows, the gate rows of 16
// outputs followed by their up rows (N = 2 * outputs, a multiple of 32); act [M, N/2]
// bfloat16 = silu(X . gate^T) * (X . up^T).  All of K in one slice.  `packed`: W is in the
// streaming layout of ei_gemm_bf16_skinny_packed.
extern "C" int ei_gemm_bf16_skinny_gated(const void* X, const void* W, void* act, int M, int N,
                                         int K, int packed, hipStream_t stream) {
  if (packed) return launch_skinny<true, true>(X, W, nullptr, act, M, N, K, 1, stream);
  return launch_skinny<false, true>(X, W, nullptr, act, M, N, K, 1, stream);
}
