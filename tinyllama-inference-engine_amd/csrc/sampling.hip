// Sampling on the device: one block per row of float logits.
//
// reference: GreedySample (src/operators.cpp:166-175): first index of the maximum, non-finite
// logits are an error; Engine::Sample (app/server.cpp:237-277): temperature <= 0 is greedy, else
// w_i = exp((l_i - max) / T), the tokens are sorted by w descending, the shortest prefix whose
// share of the total reaches top_p is kept (the one that crosses it included), and a token is
// drawn from the kept ones in proportion to w.
//
// Here the kept set is found without sorting: the weight of the last kept token is the largest
// threshold t with sum{w_i >= t} >= top_p * total, found by bisection on the bit pattern of the
// logit (32 passes over the row).  Tokens that tie with that threshold are all kept.  The draw
// walks the kept tokens in index order, which gives the same distribution as walking them in
// sorted order.  The uniform number comes from a counter-based hash of (seed, counter), so it does
// not depend on what else is in the batch; the caller passes the request's seed and the index of
// the token being generated.
#include "common.h"

namespace tlie {

__device__ __forceinline__ uint32_t order_key(float v) {
  // monotonic map float -> uint32 (larger float, larger key)
  const uint32_t bits = __float_as_uint(v);
  return (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);
}

__device__ __forceinline__ uint64_t splitmix64(uint64_t x) {
  x += 0x9E3779B97F4A7C15ull;
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
  return x ^ (x >> 31);
}

// uniform in [0, 1) with 24 bits, from (seed, counter)
__device__ __forceinline__ float uniform01(uint64_t seed, uint64_t counter) {
  const uint64_t h = splitmix64(splitmix64(seed) ^ (counter * 0xD1342543DE82EF95ull + 1));
  return static_cast<float>(h >> 40) * (1.0f / 16777216.0f);
}

constexpr int kSampleThreads = 1024;

// f(index, value) for every element of the row, spread over the block's threads; a thread meets its
// indices in rising order.  Rows that start on a 16-byte boundary are read four elements at a time.
template <typename F>
__device__ __forceinline__ void scan_row(const float* __restrict__ row, int vocab, int tid, F f) {
  int done = 0;
  if ((reinterpret_cast<uintptr_t>(row) & 15) == 0) {
    const int chunks = vocab >> 2;
    for (int c = tid; c < chunks; c += kSampleThreads) {
      const float4 v = reinterpret_cast<const float4*>(row)[c];
      f(4 * c, v.x), f(4 * c + 1, v.y), f(4 * c + 2, v.z), f(4 * c + 3, v.w);
    }
    done = chunks << 2;
  }
  for (int i = done + tid; i < vocab; i += kSampleThreads) f(i, row[i]);
}

// out[r] = sampled token, or -1 when the row holds a NaN or an infinity.
__global__ void __launch_bounds__(kSampleThreads)
sample_kernel(const float* __restrict__ logits, int vocab, const float* __restrict__ temperature,
              const float* __restrict__ top_p, const long long* __restrict__ seed,
              const long long* __restrict__ counter, int* __restrict__ out) {
  __shared__ float scratch[16];
  __shared__ int iscratch[16];
  __shared__ float segment_sum[kSampleThreads];
  __shared__ int chosen;
  const int r = blockIdx.x, tid = threadIdx.x;
  const float* row = logits + static_cast<size_t>(r) * vocab;

  // maximum, its first index, and finiteness
  float best = -INFINITY;
  int best_index = 0x7fffffff;
  int bad = 0;
  scan_row(row, vocab, tid, [&](int i, float v) {
    if (!isfinite(v)) bad = 1;
    if (v > best) { best = v; best_index = i; }     // a thread meets its indices in rising order
  });
  const float row_max = block_max(best, scratch);
  const int any_bad = __syncthreads_or(bad);
  // first index among the threads that hold the maximum
  int candidate = (best == row_max) ? best_index : 0x7fffffff;
  for (int offset = kWave / 2; offset > 0; offset >>= 1) candidate = min(candidate, __shfl_xor(candidate, offset, kWave));
  if ((tid & (kWave - 1)) == 0) iscratch[tid / kWave] = candidate;
  __syncthreads();
  int arg_max = 0x7fffffff;
  for (int w = 0; w < kSampleThreads / kWave; ++w) arg_max = min(arg_max, iscratch[w]);
  if (any_bad) {
    if (tid == 0) out[r] = -1;
    return;
  }
  const float temp = temperature ? temperature[r] : 0.f;
  if (!(temp > 0.f)) {
    if (tid == 0) out[r] = arg_max;
    return;
  }
  const float inv_temp = 1.f / temp;
  const float p_keep = top_p ? top_p[r] : 1.f;

  float local = 0.f;
  scan_row(row, vocab, tid, [&](int, float v) { local += expf((v - row_max) * inv_temp); });
  const float total = block_sum(local, scratch);

  uint32_t threshold = 0;        // keep every token whose key is >= threshold
  if (p_keep < 1.f) {
    const float target = p_keep * total;
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t trial = threshold | (1u << bit);
      float mass = 0.f;
      scan_row(row, vocab, tid, [&](int, float v) {
        if (order_key(v) >= trial) mass += expf((v - row_max) * inv_temp);
      });
      mass = block_sum(mass, scratch);
      if (mass >= target) threshold = trial;
    }
  }

  // kept weights summed per contiguous segment of the vocabulary, then a walk in index order
  const int segment = (vocab + kSampleThreads - 1) / kSampleThreads;
  const int first = tid * segment, last = min(vocab, first + segment);
  float mine = 0.f;
  for (int i = first; i < last; ++i) {
    const float v = row[i];
    if (order_key(v) >= threshold) mine += expf((v - row_max) * inv_temp);
  }
  segment_sum[tid] = mine;
  if (tid == 0) chosen = -1;
  __syncthreads();
  if (tid == 0) {
    float kept_total = 0.f;
    for (int s = 0; s < kSampleThreads; ++s) kept_total += segment_sum[s];
    const float u = uniform01(static_cast<uint64_t>(seed ? seed[r] : 0), static_cast<uint64_t>(counter ? counter[r] : 0));
    const float goal = u * kept_total;
    float cursor = 0.f;
    int owner = -1;
    for (int s = 0; s < kSampleThreads; ++s) {
      if (segment_sum[s] > 0.f) {
        owner = s;                               // the last segment with kept weight is the fallback
        if (goal <= cursor + segment_sum[s]) break;
        cursor += segment_sum[s];
      }
    }
    // walk the owning segment
    int token = arg_max;
    if (owner >= 0) {
      const int begin = owner * segment, end = min(vocab, begin + segment);
      for (int i = begin; i < end; ++i) {
        const float v = row[i];
        if (order_key(v) >= threshold) {
          token = i;
          cursor += expf((v - row_max) * inv_temp);
          if (goal <= cursor) break;
        }
      }
    }
    chosen = token;
  }
  __syncthreads();
  if (tid == 0) out[r] = chosen;
}

}  // namespace tlie

using namespace tlie;

// temperature, top_p, seed, counter: arrays of `rows` entries, or null (greedy for every row).
// tokens[i] = sampled[source[i]] where source[i] >= 0: a decode step whose tokens are the last step's
// samples takes them on the device, before the host has read them.  A sample of -1 (the row's logits
// held a NaN or an infinity; the host raises numerical_error when it reads it) becomes token 0 here,
// and a value beyond the vocabulary is clamped to its last entry: the step that is already on its way
// must not index the embedding table outside its rows.
__global__ void feed_tokens_kernel(int* __restrict__ tokens, const int* __restrict__ source,
                                   const int* __restrict__ sampled, int count, int vocab) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < count && source[i] >= 0) tokens[i] = min(max(sampled[source[i]], 0), vocab - 1);
}

extern "C" int tlie_feed_tokens(int* tokens, const int* source, const int* sampled, int count, int vocab, void* stream) {
  if (count <= 0 || vocab <= 0) return kBadArgument;
  hipLaunchKernelGGL(feed_tokens_kernel, dim3((count + 63) / 64), dim3(64), 0, (hipStream_t)stream, tokens, source,
                     sampled, count, vocab);
  return launch_status();
}

extern "C" int tlie_sample(const float* logits, int rows, int vocab, const float* temperature, const float* top_p,
                           const long long* seed, const long long* counter, int* out, void* stream) {
  if (rows <= 0 || vocab <= 0) return kBadArgument;
  hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(kSampleThreads), 0, (hipStream_t)stream, logits, vocab,
                     temperature, top_p, seed, counter, out);
  return launch_status();
}
