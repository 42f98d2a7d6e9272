// Sampling from float32 logits, one block per row of the batch.
//
// Greedy: argmax, ties to the lowest index.  Stochastic, in the reference's order
// (operators/src/cuda/execution.cu:193-234, 455-498): z = logit / temperature
// (NaN -> -inf); the k = min(top_k, V) largest, sorted descending with ties to the
// lower index; e_i = exp(z_i - z_0); the shortest prefix whose mass reaches
// top_p * total, at least one element and including the one that crosses; a uniform
// u in (0, 1]; the first kept element whose cumulative mass reaches u * retained.
// Instead of sorting the whole vocabulary the k-th largest value is found by a radix
// select and only the k candidates are sorted.  The uniform number comes from a
// counter-based generator keyed by (seed, request stream, step counter), so a
// request draws the same numbers alone or in any batch.
#include "common.h"
#include "sampling_static.h"

#include <atomic>

namespace {

constexpr int kThreads = 1024;
constexpr int kMaxTopK = 1024;

__device__ __forceinline__ uint32_t sortable_key(float z) {
  const uint32_t u = __float_as_uint(z);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);  // ascending in z
}

__device__ __forceinline__ float key_value(uint32_t key) {
  const uint32_t u = (key & 0x80000000u) ? (key & 0x7fffffffu) : ~key;
  return __uint_as_float(u);
}

__device__ __forceinline__ float scaled_logit(float logit, float temperature, bool scale) {
  if (isnan(logit)) return -INFINITY;
  return scale ? logit / temperature : logit;
}

// splitmix64 finalizer of seed + golden * (stream * 2^32 + counter + 1); (0, 1].
__device__ __forceinline__ float uniform_draw(uint64_t seed, uint32_t stream, uint32_t counter) {
  uint64_t z = seed + 0x9E3779B97F4A7C15ull *
                          ((static_cast<uint64_t>(stream) << 32) + counter + 1ull);
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  z ^= z >> 31;
  return (static_cast<float>(z >> 40) + 1.0f) * (1.0f / 16777216.0f);
}

__global__ void __launch_bounds__(kThreads)
argmax_kernel(const float* __restrict__ logits, int V, int32_t* __restrict__ tokens,
              float* __restrict__ probabilities) {
  __shared__ float best_value[kThreads / EI_WAVE];
  __shared__ int best_index[kThreads / EI_WAVE];
  const float* row = logits + static_cast<size_t>(blockIdx.x) * V;
  float value = -INFINITY;
  int index = 0x7fffffff;
  for (int i = threadIdx.x; i < V; i += kThreads) {
    const float z = scaled_logit(row[i], 1.f, false);
    if (z > value || (z == value && i < index)) {
      value = z;
      index = i;
    }
  }
#pragma unroll
  for (int offset = EI_WAVE / 2; offset > 0; offset >>= 1) {
    const float other_value = __shfl_xor(value, offset, EI_WAVE);
    const int other_index = __shfl_xor(index, offset, EI_WAVE);
    if (other_value > value || (other_value == value && other_index < index)) {
      value = other_value;
      index = other_index;
    }
  }
  const int wave = threadIdx.x / EI_WAVE, lane = threadIdx.x % EI_WAVE;
  if (lane == 0) {
    best_value[wave] = value;
    best_index[wave] = index;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kThreads / EI_WAVE; ++w) {
      if (best_value[w] > value || (best_value[w] == value && best_index[w] < index)) {
        value = best_value[w];
        index = best_index[w];
      }
    }
    tokens[blockIdx.x] = index == 0x7fffffff ? 0 : index;
    if (probabilities) probabilities[blockIdx.x] = 1.f;
  }
}

// Wide vocabularies, two steps: every block finds the best of one chunk of a row, then one
// wave a row picks the best chunk.  The same order (larger value, then lower index) as above.
constexpr int kArgmaxThreads = 256;
constexpr int kArgmaxChunk = 4096;

__device__ __forceinline__ void keep_better(float& value, int& index, float other_value,
                                            int other_index) {
  if (other_value > value || (other_value == value && other_index < index)) {
    value = other_value;
    index = other_index;
  }
}

__global__ void __launch_bounds__(kArgmaxThreads)
argmax_chunks_kernel(const float* __restrict__ logits, int V, float2* __restrict__ partial) {
  __shared__ float best_value[kArgmaxThreads / EI_WAVE];
  __shared__ int best_index[kArgmaxThreads / EI_WAVE];
  const float* row = logits + static_cast<size_t>(blockIdx.y) * V;
  const int begin = blockIdx.x * kArgmaxChunk;
  const int end = min(V, begin + kArgmaxChunk);
  float value = -INFINITY;
  int index = 0x7fffffff;
  constexpr int kPerThread = kArgmaxChunk / kArgmaxThreads;
  float z[kPerThread];
#pragma unroll
  for (int j = 0; j < kPerThread; ++j) {          // all loads first
    const int i = begin + threadIdx.x + j * kArgmaxThreads;
    z[j] = i < end ? row[i] : -INFINITY;
  }
#pragma unroll
  for (int j = 0; j < kPerThread; ++j) {
    const int i = begin + threadIdx.x + j * kArgmaxThreads;
    if (i < end) keep_better(value, index, scaled_logit(z[j], 1.f, false), i);
  }
#pragma unroll
  for (int offset = EI_WAVE / 2; offset > 0; offset >>= 1)
    keep_better(value, index, __shfl_xor(value, offset, EI_WAVE), __shfl_xor(index, offset, EI_WAVE));
  const int wave = threadIdx.x / EI_WAVE, lane = threadIdx.x % EI_WAVE;
  if (lane == 0) {
    best_value[wave] = value;
    best_index[wave] = index;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < kArgmaxThreads / EI_WAVE; ++w)
      keep_better(value, index, best_value[w], best_index[w]);
    partial[static_cast<size_t>(blockIdx.y) * gridDim.x + blockIdx.x] =
        make_float2(value, __int_as_float(index));
  }
}

__global__ void __launch_bounds__(EI_WAVE)
argmax_merge_kernel(const float2* __restrict__ partial, int chunks, int32_t* __restrict__ tokens,
                    float* __restrict__ probabilities) {
  const float2* mine = partial + static_cast<size_t>(blockIdx.x) * chunks;
  float value = -INFINITY;
  int index = 0x7fffffff;
  for (int c = threadIdx.x; c < chunks; c += EI_WAVE)
    keep_better(value, index, mine[c].x, __float_as_int(mine[c].y));
#pragma unroll
  for (int offset = EI_WAVE / 2; offset > 0; offset >>= 1)
    keep_better(value, index, __shfl_xor(value, offset, EI_WAVE), __shfl_xor(index, offset, EI_WAVE));
  if (threadIdx.x == 0) {
    tokens[blockIdx.x] = index == 0x7fffffff ? 0 : index;
    if (probabilities) probabilities[blockIdx.x] = 1.f;
  }
}

// For the first 256 threads of a block, each holding the count of its bin (thread t: bin t):
// the counts of all higher bins added up (an exclusive suffix sum).  `wave_totals`: four
// words of shared memory; every thread of the block calls this (it synchronizes).
__device__ __forceinline__ unsigned count_above(unsigned own, unsigned* wave_totals) {
  const int t = threadIdx.x, lane = t % EI_WAVE, wave = t / EI_WAVE;
  unsigned inclusive = own;
#pragma unroll
  for (int offset = 1; offset < EI_WAVE; offset <<= 1) {
    const unsigned other = __shfl_down(inclusive, offset, EI_WAVE);
    if (lane + offset < EI_WAVE) inclusive += other;
  }
  if (lane == 0 && wave < 256 / EI_WAVE) wave_totals[wave] = inclusive;
  __syncthreads();
  unsigned above = inclusive - own;
  for (int w = wave + 1; w < 256 / EI_WAVE; ++w) above += wave_totals[w];
  return above;
}

struct SampleShared {
  unsigned histogram[256];
  unsigned long long candidates[kMaxTopK];  // (key << 32) | ~index
  int equal_index[kMaxTopK];
  unsigned select_prefix, select_remaining, n_taken, n_equal_taken, n_equal_seen;
  unsigned wave_totals[4];
};

// Where the (key, vocabulary index) pairs of a row come from: the row itself, or a list of
// the pairs that can belong to the top k, gathered beforehand in any order.
template <bool LIST>
struct Source {
  const float* row;
  float temperature;
  const unsigned long long* list;
  int n;
  __device__ __forceinline__ uint32_t key(int i) const {
    return LIST ? static_cast<uint32_t>(list[i] >> 32)
                : sortable_key(scaled_logit(row[i], temperature, true));
  }
  __device__ __forceinline__ int index(int i) const {
    return LIST ? static_cast<int>(~static_cast<uint32_t>(list[i] & 0xffffffffull)) : i;
  }
};

// One block samples one row from `source` (n >= k pairs).  False (nothing written): a list
// with more than 1024 pairs tied at the k-th value, which needs the row in index order.
template <bool LIST>
__device__ bool sample_row(const Source<LIST>& source, int k, float top_p, uint64_t seed,
                           uint32_t stream, uint32_t counter, int32_t* token, float* probability,
                           SampleShared& sh) {
  unsigned (&histogram)[256] = sh.histogram;
  unsigned long long (&candidates)[kMaxTopK] = sh.candidates;
  int (&equal_index)[kMaxTopK] = sh.equal_index;
  unsigned& select_prefix = sh.select_prefix;
  unsigned& select_remaining = sh.select_remaining;
  unsigned& n_taken = sh.n_taken;
  unsigned& n_equal_taken = sh.n_equal_taken;
  unsigned& n_equal_seen = sh.n_equal_seen;
  const int t = threadIdx.x;
  const int V = source.n;

  // radix select of the k-th largest key, eight bits at a time from the top
  if (t == 0) {
    select_prefix = 0u;
    select_remaining = static_cast<unsigned>(k);
  }
  unsigned mask = 0u;
  for (int shift = 24; shift >= 0; shift -= 8) {
    if (t < 256) histogram[t] = 0u;
    __syncthreads();
    const unsigned prefix = select_prefix;
    for (int i = t; i < V; i += kThreads) {
      const uint32_t key = source.key(i);
      if ((key & mask) == prefix) atomicAdd(&histogram[(key >> shift) & 0xffu], 1u);
    }
    __syncthreads();
    {
      // the highest bin that, together with the bins above it, holds the keys still wanted
      const unsigned remaining = select_remaining;
      const unsigned own = t < 256 ? histogram[t] : 0u;
      const unsigned above = count_above(own, sh.wave_totals);
      __syncthreads();                      // everybody has read select_remaining
      if (t < 256 && above < remaining && above + own >= remaining) {
        select_remaining = remaining - above;
        select_prefix = prefix | (static_cast<unsigned>(t) << shift);
      }
    }
    mask |= 0xffu << shift;
    __syncthreads();
  }
  const uint32_t kth = select_prefix;
  const unsigned need_equal = select_remaining;  // how many keys equal to kth belong to the top k
  if (t == 0) {
    n_taken = 0u;
    n_equal_taken = 0u;
    n_equal_seen = 0u;
  }
  __syncthreads();
  // keys above the k-th: all of them, in any order (the sort below orders them);
  // keys equal to it are listed aside
  for (int i = t; i < V; i += kThreads) {
    const uint32_t key = source.key(i);
    if (key > kth) {
      const unsigned at = atomicAdd(&n_taken, 1u);
      candidates[at] = (static_cast<unsigned long long>(key) << 32) |
                       (~static_cast<uint32_t>(source.index(i)));
    } else if (key == kth) {
      const unsigned at = atomicAdd(&n_equal_seen, 1u);
      if (at < kMaxTopK) equal_index[at] = source.index(i);
    }
  }
  __syncthreads();
  const unsigned base = n_taken;  // == k - need_equal
  if (n_equal_seen <= kMaxTopK) {
    // few ties: the `need_equal` lowest indices by counting smaller ones
    const unsigned count = n_equal_seen;
    if (static_cast<unsigned>(t) < count) {
      const int mine = equal_index[t];
      unsigned rank = 0u;
      for (unsigned j = 0; j < count; ++j) rank += equal_index[j] < mine;
      if (rank < need_equal)
        candidates[base + rank] =
            (static_cast<unsigned long long>(kth) << 32) | (~static_cast<uint32_t>(mine));
    }
  } else if (LIST) {
    return false;                           // the same for every thread: n_equal_seen is shared
  } else {
    // many ties: walk the vocabulary in index order until enough are found
    for (int start = 0; start < V; start += kThreads) {
      if (n_equal_taken >= need_equal) break;
      const int i = start + t;
      const bool equal = i < V && source.key(i) == kth;
      const unsigned long long ballot = __ballot(equal);
      const int lane = t % EI_WAVE, wave = t / EI_WAVE;
      const unsigned in_wave = __popcll(ballot & ((1ull << lane) - 1ull));
      __syncthreads();
      if (lane == 0) histogram[wave] = __popcll(ballot);
      __syncthreads();
      unsigned before = 0u;
      for (int w = 0; w < wave; ++w) before += histogram[w];
      unsigned total = 0u;
      for (int w = 0; w < kThreads / EI_WAVE; ++w) total += histogram[w];
      const unsigned already = n_equal_taken;
      if (equal) {
        const unsigned rank = already + before + in_wave;
        if (rank < need_equal)
          candidates[base + rank] =
              (static_cast<unsigned long long>(kth) << 32) | (~static_cast<uint32_t>(i));
      }
      __syncthreads();
      if (t == 0) n_equal_taken = already + total;
      __syncthreads();
    }
  }
  __syncthreads();
  // pad to a power of two and sort descending (bitonic)
  int padded = 1;
  while (padded < k) padded <<= 1;
  for (int i = k + t; i < padded; i += kThreads) candidates[i] = 0ull;
  __syncthreads();
  for (int size = 2; size <= padded; size <<= 1) {
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      for (int i = t; i < padded; i += kThreads) {
        const int partner = i ^ stride;
        if (partner > i) {
          const bool descending = (i & size) == 0;
          const unsigned long long a = candidates[i], b = candidates[partner];
          if ((a < b) == descending) {
            candidates[i] = b;
            candidates[partner] = a;
          }
        }
      }
      __syncthreads();
    }
  }
  // masses in parallel, their sums by one thread in index order (the order of the sums is
  // part of the result: the draw compares against them)
  const float z0 = key_value(static_cast<uint32_t>(candidates[0] >> 32));
  float* mass = reinterpret_cast<float*>(equal_index);      // the tie table is done with
  static_assert(kMaxTopK <= kThreads, "one thread a candidate");
  if (t < k) mass[t] = expf(key_value(static_cast<uint32_t>(candidates[t] >> 32)) - z0);
  __syncthreads();
  if (t == 0) {
    const int first = static_cast<int>(~static_cast<uint32_t>(candidates[0] & 0xffffffffull));
    if (!isfinite(z0)) {
      *token = first;
      if (probability) *probability = 1.f;
      return true;
    }
    float total = 0.f;
    for (int i = 0; i < k; ++i) total += mass[i];
    const float threshold = top_p * total;
    float retained = 0.f;
    int kept = 0;
    do {
      retained += mass[kept];
      ++kept;
    } while (kept < k && retained < threshold);
    const float u = uniform_draw(seed, stream, counter);
    const float target = u * retained;
    float cumulative = 0.f;
    int selected = kept - 1;
    for (int i = 0; i < kept; ++i) {
      cumulative += mass[i];
      if (cumulative >= target) {
        selected = i;
        break;
      }
    }
    *token = static_cast<int>(~static_cast<uint32_t>(candidates[selected] & 0xffffffffull));
    if (probability) *probability = mass[selected] / retained;
  }
  return true;
}

__global__ void __launch_bounds__(kThreads)
sample_kernel(const float* __restrict__ logits, int V, float temperature, float top_p, int top_k,
              uint64_t seed, const int32_t* __restrict__ streams,
              const int32_t* __restrict__ counters, int32_t* __restrict__ tokens,
              float* __restrict__ probabilities) {
  __shared__ SampleShared sh;
  const int r = blockIdx.x;
  const Source<false> whole{logits + static_cast<size_t>(r) * V, temperature, nullptr, V};
  sample_row<false>(whole, top_k < V ? top_k : V, top_p, seed, static_cast<uint32_t>(streams[r]),
                    static_cast<uint32_t>(counters[r]), tokens + r,
                    probabilities ? probabilities + r : nullptr, sh);
}

// Wide vocabularies in three steps, the first two with many blocks a row.
// (1) counts of the rows' keys by their upper 12 bits (sign, exponent, three bits of the
//     fraction), summed over the blocks of a row in `bins` [rows, 4096];
// (2) every block finds the bin T that holds the k-th largest key and appends its keys from
//     bins >= T to the row's list (fewer than k pairs above T, plus whatever shares T);
// (3) one block a row samples from the list exactly as sample_kernel does from the row, or
//     from the row itself if the list overflowed or is tied beyond reach; it then clears the
//     row's bins and count, which therefore start at zero in every call once they did in
//     the first.
constexpr int kBins = 4096, kBinShift = 20;
constexpr int kChunk = 4096, kChunkThreads = 256;
// a row's scratch, in 4-byte units: its bins, its count (4 units, which keeps the list
// 8-byte aligned) and its list of up to kListCapacity pairs; a row's place does not depend
// on how many rows a call has
constexpr int kListCapacity = 4096;
constexpr long long kScratchPerRow = kBins + 4 + 2ll * kListCapacity;
__device__ __forceinline__ unsigned* row_bins(unsigned* scratch, int r) {
  return scratch + static_cast<size_t>(r) * kScratchPerRow;
}
__device__ __forceinline__ unsigned* row_count(unsigned* scratch, int r) {
  return row_bins(scratch, r) + kBins;
}
__device__ __forceinline__ unsigned long long* row_list(unsigned* scratch, int r) {
  return reinterpret_cast<unsigned long long*>(row_bins(scratch, r) + kBins + 4);
}

__global__ void __launch_bounds__(kChunkThreads)
sample_count_kernel(const float* __restrict__ logits, int V, float temperature,
                    unsigned* __restrict__ scratch) {
  __shared__ unsigned local[kBins];
  const int t = threadIdx.x, r = blockIdx.y;
  for (int b = t; b < kBins; b += kChunkThreads) local[b] = 0u;
  __syncthreads();
  const float* row = logits + static_cast<size_t>(r) * V;
  const int begin = blockIdx.x * kChunk, end = min(V, begin + kChunk);
  for (int i = begin + t; i < end; i += kChunkThreads)
    atomicAdd(&local[sortable_key(scaled_logit(row[i], temperature, true)) >> kBinShift], 1u);
  __syncthreads();
  for (int b = t; b < kBins; b += kChunkThreads)
    if (local[b]) atomicAdd(&row_bins(scratch, r)[b], local[b]);
}

__global__ void __launch_bounds__(kChunkThreads)
sample_gather_kernel(const float* __restrict__ logits, int V, float temperature, int k,
                     unsigned* __restrict__ scratch) {
  static_assert(kChunkThreads == 256, "count_above works on 256 counts");
  __shared__ unsigned partial[4];
  __shared__ unsigned long long mine[kChunk];
  __shared__ unsigned threshold_bin, n_mine, base;
  const int t = threadIdx.x, r = blockIdx.y;
  constexpr int per = kBins / kChunkThreads;
  const unsigned* bins = row_bins(scratch, r);
  unsigned own[per], sum = 0u;
#pragma unroll
  for (int j = 0; j < per; ++j) {
    own[j] = bins[t * per + j];
    sum += own[j];
  }
  if (t == 0) n_mine = 0u;
  unsigned above = count_above(sum, partial);   // keys in the bins of the threads after this one
  if (above < static_cast<unsigned>(k) && above + sum >= static_cast<unsigned>(k)) {
    int bin = per - 1;                      // exactly one thread gets here (k <= V = all keys)
#pragma unroll
    for (; bin > 0; --bin) {
      if (above + own[bin] >= static_cast<unsigned>(k)) break;
      above += own[bin];
    }
    threshold_bin = static_cast<unsigned>(t * per + bin);
  }
  __syncthreads();
  const unsigned first_bin = threshold_bin;
  const float* row = logits + static_cast<size_t>(r) * V;
  const int begin = blockIdx.x * kChunk, end = min(V, begin + kChunk);
  for (int i = begin + t; i < end; i += kChunkThreads) {
    const uint32_t key = sortable_key(scaled_logit(row[i], temperature, true));
    if ((key >> kBinShift) >= first_bin)
      mine[atomicAdd(&n_mine, 1u)] =
          (static_cast<unsigned long long>(key) << 32) | (~static_cast<uint32_t>(i));
  }
  __syncthreads();
  const unsigned count = n_mine;
  if (t == 0) base = count ? atomicAdd(row_count(scratch, r), count) : 0u;
  __syncthreads();
  unsigned long long* list = row_list(scratch, r);
  for (unsigned j = t; j < count; j += kChunkThreads)
    if (base + j < static_cast<unsigned>(kListCapacity)) list[base + j] = mine[j];
}

__global__ void __launch_bounds__(kThreads)
sample_list_kernel(const float* __restrict__ logits, int V, float temperature, float top_p,
                   int top_k, uint64_t seed, const int32_t* __restrict__ streams,
                   const int32_t* __restrict__ counters, int32_t* __restrict__ tokens,
                   float* __restrict__ probabilities, unsigned* __restrict__ scratch) {
  __shared__ SampleShared sh;
  const int r = blockIdx.x, t = threadIdx.x;
  const int k = top_k < V ? top_k : V;
  const unsigned listed = *row_count(scratch, r);
  const uint32_t stream = static_cast<uint32_t>(streams[r]);
  const uint32_t counter = static_cast<uint32_t>(counters[r]);
  float* probability = probabilities ? probabilities + r : nullptr;
  bool done = false;
  if (listed <= static_cast<unsigned>(kListCapacity)) {
    const Source<true> list{nullptr, temperature, row_list(scratch, r), static_cast<int>(listed)};
    done = sample_row<true>(list, k, top_p, seed, stream, counter, tokens + r, probability, sh);
  }
  if (!done) {
    __syncthreads();
    const Source<false> whole{logits + static_cast<size_t>(r) * V, temperature, nullptr, V};
    sample_row<false>(whole, k, top_p, seed, stream, counter, tokens + r, probability, sh);
  }
  __syncthreads();                          // every thread has read the count
  for (int b = t; b < kBins; b += kThreads) row_bins(scratch, r)[b] = 0u;
  if (t == 0) *row_count(scratch, r) = 0u;
}


}  // namespace

// Elements of `partial` (float2) that ei_argmax wants for these sizes; 0: it needs none.
extern "C" int ei_argmax_partial_size(int rows, int V) {
  if (rows < 1 || V <= 2 * kArgmaxChunk) return 0;
  const long long size = static_cast<long long>(rows) * ((V + kArgmaxChunk - 1) / kArgmaxChunk);
  return size < (1ll << 30) ? static_cast<int>(size) : 0;
}

// `partial` (float2 [rows, chunks], or null) lets a wide vocabulary be searched by many
// blocks a row; without it one block takes a row.  The result is the same either way.
extern "C" int ei_argmax(const float* logits, int rows, int V, int32_t* tokens,
                         float* probabilities, void* partial, long long partial_size,
                         hipStream_t stream) {
  EI_REQUIRE(rows > 0 && V > 0, "argmax: sizes must be positive");
  EI_REQUIRE(logits && tokens, "argmax: null pointer");
  const int want = ei_argmax_partial_size(rows, V);
  if (partial && want > 0) {
    EI_REQUIRE(partial_size >= want, "argmax: the partial buffer is too small");
    const int chunks = (V + kArgmaxChunk - 1) / kArgmaxChunk;
    argmax_chunks_kernel<<<dim3(chunks, rows), kArgmaxThreads, 0, stream>>>(
        logits, V, static_cast<float2*>(partial));
    argmax_merge_kernel<<<rows, EI_WAVE, 0, stream>>>(static_cast<const float2*>(partial), chunks,
                                                      tokens, probabilities);
    EI_LAUNCH_CHECK();
  }
  argmax_kernel<<<rows, kThreads, 0, stream>>>(logits, V, tokens, probabilities);
  EI_LAUNCH_CHECK();
}

// The partial results of ei_argmax_static: one copy on every GPU, at an address of its own
// there.  Host code never passes this name to a kernel (on the host it is a stand-in, not a
// device address); it asks the runtime for the address once per device and uses that.
static __device__ __align__(256) float2 argmax_static_scratch[EI_ARGMAX_STATIC_MAX_PARTIALS];

constexpr int kStaticDevices = 64;
static std::atomic<float2*> argmax_static_address[kStaticDevices];

// The array's address on the current device: looked up once per device (with that device
// current) and kept.  The lookup may load the library's code on the device, which a stream
// that is being captured does not allow, so it is never started from a call under capture.
static int argmax_static_resolve(float2** out, bool capturing) {
  int device = -1;
  hipError_t status = hipGetDevice(&device);
  if (status != hipSuccess) {
    ei_set_error(hipGetErrorString(status));
    return static_cast<int>(status);
  }
  EI_REQUIRE(device >= 0 && device < kStaticDevices, "argmax_static: device index out of range");
  float2* partial = argmax_static_address[device].load(std::memory_order_acquire);
  if (partial == nullptr) {
    EI_REQUIRE(!capturing, "argmax_static: the first call on a device cannot run under stream "
                           "capture; call ei_argmax_static_prepare() on that device before");
    void* address = nullptr;
    status = hipGetSymbolAddress(&address, HIP_SYMBOL(argmax_static_scratch));
    if (status != hipSuccess) {
      ei_set_error(hipGetErrorString(status));
      return static_cast<int>(status);
    }
    EI_REQUIRE(address != nullptr, "argmax_static: the static buffer has no device address");
    partial = static_cast<float2*>(address);
    argmax_static_address[device].store(partial, std::memory_order_release);
  }
  *out = partial;
  return 0;
}

// See sampling_static.h.
extern "C" int ei_argmax_static_prepare() {
  float2* partial = nullptr;
  return argmax_static_resolve(&partial, false);
}

// See sampling_static.h.  Nothing is allocated, by this call or by the lookup.
extern "C" int ei_argmax_static(const float* logits, int rows, int V, int32_t* tokens,
                                float* probabilities, hipStream_t stream) {
  EI_REQUIRE(rows > 0 && V > 0, "argmax_static: sizes must be positive");
  EI_REQUIRE(logits && tokens, "argmax_static: null pointer");
  const long long chunks = (static_cast<long long>(V) + kArgmaxChunk - 1) / kArgmaxChunk;
  if (V <= 2 * kArgmaxChunk) {          // one block a row: no partial results
    argmax_kernel<<<rows, kThreads, 0, stream>>>(logits, V, tokens, probabilities);
    EI_LAUNCH_CHECK();
  }
  EI_REQUIRE(static_cast<long long>(rows) * chunks <= EI_ARGMAX_STATIC_MAX_PARTIALS,
             "argmax_static: rows * ceil(V / 4096) exceeds the 65536 partial results that the "
             "library's static buffer holds");
  hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &capture) != hipSuccess) capture = hipStreamCaptureStatusNone;
  float2* partial = nullptr;
  const int resolved = argmax_static_resolve(&partial, capture != hipStreamCaptureStatusNone);
  if (resolved != 0) return resolved;
  argmax_chunks_kernel<<<dim3(static_cast<unsigned>(chunks), rows), kArgmaxThreads, 0, stream>>>(
      logits, V, partial);
  argmax_merge_kernel<<<rows, EI_WAVE, 0, stream>>>(partial, static_cast<int>(chunks), tokens,
                                                    probabilities);
  EI_LAUNCH_CHECK();
}

// Scratch that ei_sample wants for a wide vocabulary, in 4-byte units (0: it needs none).
// It must be zero before its first use; every call leaves the bins and counts of its rows
// zero again, and a row's part lies at the same place whatever the number of rows.
constexpr int kWideVocabulary = 4 * kChunk;

extern "C" int ei_sample_scratch_size(int rows, int V) {
  if (rows < 1 || V <= kWideVocabulary) return 0;
  const long long size = rows * kScratchPerRow;
  return size < (1ll << 30) ? static_cast<int>(size) : 0;
}

// temperature > 0, 0 < top_p <= 1, 1 <= min(top_k, V) <= 1024.  `scratch` (uint32
// [scratch_size], or null): see ei_sample_scratch_size; the tokens are the same with or
// without it.
extern "C" int ei_sample(const float* logits, int rows, int V, float temperature, float top_p,
                         int top_k, unsigned long long seed, const int32_t* streams,
                         const int32_t* counters, int32_t* tokens, float* probabilities,
                         void* scratch, long long scratch_size, hipStream_t stream) {
  EI_REQUIRE(rows > 0 && V > 0, "sample: sizes must be positive");
  EI_REQUIRE(logits && tokens && streams && counters, "sample: null pointer");
  EI_REQUIRE(temperature > 0.f && temperature < 3.0e38f, "sample: temperature must be positive");
  EI_REQUIRE(top_p > 0.f && top_p <= 1.f, "sample: top_p must lie in (0, 1]");
  EI_REQUIRE(top_k >= 1 && (top_k < V ? top_k : V) <= kMaxTopK,
             "sample: min(top_k, vocabulary) must lie in 1..1024");
  const int want = ei_sample_scratch_size(rows, V);
  if (scratch && want > 0) {
    EI_REQUIRE(scratch_size >= want, "sample: the scratch buffer is too small");
    EI_REQUIRE((reinterpret_cast<uintptr_t>(scratch) & 7) == 0, "sample: scratch must be 8-byte aligned");
    unsigned* words = static_cast<unsigned*>(scratch);
    const dim3 grid((V + kChunk - 1) / kChunk, rows);
    sample_count_kernel<<<grid, kChunkThreads, 0, stream>>>(logits, V, temperature, words);
    sample_gather_kernel<<<grid, kChunkThreads, 0, stream>>>(logits, V, temperature,
                                                            top_k < V ? top_k : V, words);
    sample_list_kernel<<<rows, kThreads, 0, stream>>>(logits, V, temperature, top_p, top_k, seed,
                                                      streams, counters, tokens, probabilities,
                                                      words);
    EI_LAUNCH_CHECK();
  }
  sample_kernel<<<rows, kThreads, 0, stream>>>(logits, V, temperature, top_p, top_k, seed,
                                               streams, counters, tokens, probabilities);
  EI_LAUNCH_CHECK();
}
