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
#include "common.cuh"

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

__global__ void __launch_bounds__(kThreads)
sample_kernel(const float* __restrict__ logits, int V, float temperature, float top_p, int top_k,
              uint64_t seed, const int32_t* __restrict__ streams,
              const int32_t* __restrict__ counters, int32_t* __restrict__ tokens,
              float* __restrict__ probabilities) {
  __shared__ unsigned histogram[256];
  __shared__ unsigned long long candidates[kMaxTopK];  // (key << 32) | ~index
  __shared__ int equal_index[kMaxTopK];
  __shared__ unsigned select_prefix, select_remaining, n_taken, n_equal_taken, n_equal_seen;
  const int t = threadIdx.x;
  const float* row = logits + static_cast<size_t>(blockIdx.x) * V;
  const int k = top_k < V ? top_k : V;

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
      const uint32_t key = sortable_key(scaled_logit(row[i], temperature, true));
      if ((key & mask) == prefix) atomicAdd(&histogram[(key >> shift) & 0xffu], 1u);
    }
    __syncthreads();
    if (t == 0) {
      unsigned remaining = select_remaining, above = 0u;
      int bin = 255;
      for (; bin > 0; --bin) {
        if (above + histogram[bin] >= remaining) break;
        above += histogram[bin];
      }
      select_remaining = remaining - above;
      select_prefix = prefix | (static_cast<unsigned>(bin) << shift);
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
    const uint32_t key = sortable_key(scaled_logit(row[i], temperature, true));
    if (key > kth) {
      const unsigned at = atomicAdd(&n_taken, 1u);
      candidates[at] = (static_cast<unsigned long long>(key) << 32) | (~static_cast<uint32_t>(i));
    } else if (key == kth) {
      const unsigned at = atomicAdd(&n_equal_seen, 1u);
      if (at < kMaxTopK) equal_index[at] = i;
    }
  }
  __syncthreads();
  const unsigned base = n_taken;  // == k - need_equal
  if (n_equal_seen <= kMaxTopK) {
    // few ties: the `need_equal` lowest indices by counting smaller ones
    const unsigned count = n_equal_seen;
    if (t < count) {
      const int mine = equal_index[t];
      unsigned rank = 0u;
      for (unsigned j = 0; j < count; ++j) rank += equal_index[j] < mine;
      if (rank < need_equal)
        candidates[base + rank] =
            (static_cast<unsigned long long>(kth) << 32) | (~static_cast<uint32_t>(mine));
    }
  } else {
    // many ties: walk the vocabulary in index order until enough are found
    for (int start = 0; start < V; start += kThreads) {
      if (n_equal_taken >= need_equal) break;
      const int i = start + t;
      const bool equal =
          i < V && sortable_key(scaled_logit(row[i], temperature, true)) == kth;
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
  if (t == 0) {
    const float z0 = key_value(static_cast<uint32_t>(candidates[0] >> 32));
    const int first = static_cast<int>(~static_cast<uint32_t>(candidates[0] & 0xffffffffull));
    if (!isfinite(z0)) {
      tokens[blockIdx.x] = first;
      if (probabilities) probabilities[blockIdx.x] = 1.f;
      return;
    }
    float total = 0.f;
    for (int i = 0; i < k; ++i)
      total += expf(key_value(static_cast<uint32_t>(candidates[i] >> 32)) - z0);
    const float threshold = top_p * total;
    float retained = 0.f;
    int kept = 0;
    do {
      retained += expf(key_value(static_cast<uint32_t>(candidates[kept] >> 32)) - z0);
      ++kept;
    } while (kept < k && retained < threshold);
    const float u = uniform_draw(seed, static_cast<uint32_t>(streams[blockIdx.x]),
                                 static_cast<uint32_t>(counters[blockIdx.x]));
    const float target = u * retained;
    float cumulative = 0.f;
    int selected = kept - 1;
    for (int i = 0; i < kept; ++i) {
      cumulative += expf(key_value(static_cast<uint32_t>(candidates[i] >> 32)) - z0);
      if (cumulative >= target) {
        selected = i;
        break;
      }
    }
    tokens[blockIdx.x] =
        static_cast<int>(~static_cast<uint32_t>(candidates[selected] & 0xffffffffull));
    if (probabilities)
      probabilities[blockIdx.x] =
          expf(key_value(static_cast<uint32_t>(candidates[selected] >> 32)) - z0) / retained;
  }
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

// temperature > 0, 0 < top_p <= 1, 1 <= min(top_k, V) <= 1024.
extern "C" int ei_sample(const float* logits, int rows, int V, float temperature, float top_p,
                         int top_k, unsigned long long seed, const int32_t* streams,
                         const int32_t* counters, int32_t* tokens, float* probabilities,
                         hipStream_t stream) {
  EI_REQUIRE(rows > 0 && V > 0, "sample: sizes must be positive");
  EI_REQUIRE(logits && tokens && streams && counters, "sample: null pointer");
  EI_REQUIRE(temperature > 0.f && temperature < 3.0e38f, "sample: temperature must be positive");
  EI_REQUIRE(top_p > 0.f && top_p <= 1.f, "sample: top_p must lie in (0, 1]");
  EI_REQUIRE(top_k >= 1 && (top_k < V ? top_k : V) <= kMaxTopK,
             "sample: min(top_k, vocabulary) must lie in 1..1024");
  sample_kernel<<<rows, kThreads, 0, stream>>>(logits, V, temperature, top_p, top_k, seed,
                                               streams, counters, tokens, probabilities);
  EI_LAUNCH_CHECK();
}
