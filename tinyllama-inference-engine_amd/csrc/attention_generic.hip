// Paged causal grouped-query attention, the plain kernel: any storage type, any head size up to
// the block size, any number of tokens per sequence.  It is the whole 32-bit path's attention and
// the fallback of the bfloat16 path for sizes the tiled kernels refuse.
//
// reference: AttentionDecodeKernel (src/cuda/kernels.cu:147-196): one block per query head,
// scores = (q . k) * rsqrt(d) over positions 0..pos, max, exp, sum, normalise, then one thread
// per output dimension sums p * v serially.  That kernel keeps all scores of the context in
// shared memory and serves one token; this one walks the context in chunks of 64, 128 or 256 keys
// (the least that holds the head size) with running maxima and sums (so the context length is
// unbounded), serves every token of a step in one launch, finds keys through the block table, and
// optionally limits the keys to a window.  Chunks start at multiples of their size counted from
// position 0, so the order of the sums for a given (sequence, position) never depends on how the
// step was cut.
#include "common.h"

namespace tlie {

// q: [tokens][nq][d]; cache: [pages][2][nkv][page_size * d], keys [row][dim], values [dim][row];
// out: [tokens][nq][d].
// token_seq[t]: row of the block table; positions[t]: absolute position of the token.
// window <= 0: all keys 0..pos; otherwise keys pos-window+1..pos.
// A workgroup of 256 threads serves one (token, head).  Its threads form 256 / CHUNK groups of
// CHUNK threads (CHUNK >= d); chunk c of the context (keys c * CHUNK ..) belongs to group
// c % groups, and every group keeps a running maximum, sum and output of its own over its chunks,
// in the order of their index; at the end the groups' results are put together in the order of
// the groups.  Which keys meet in which sum, and in which order, depends on the positions alone.
template <typename T, int CHUNK>
__global__ void __launch_bounds__(256)
attention_generic_kernel(const T* __restrict__ q, const T* __restrict__ cache, const int* __restrict__ block_table,
                         int max_blocks, const int* __restrict__ token_seq, const int* __restrict__ positions,
                         T* __restrict__ out, int nq, int nkv, int d, int page_size, int window, float scale) {
  constexpr int kGroups = 256 / CHUNK, kWavesPerGroup = CHUNK / 64;
  extern __shared__ float lds[];
  float* q_row = lds;                              // d
  float* prob = q_row + d;                         // 256: a group's probabilities of its current chunk
  float* wave_part = prob + 256;                   // 4: one value per wave, for the reductions within a group
  float* group_stat = wave_part + 4;               // kGroups x 2: maximum, sum
  float* group_out = group_stat + 2 * kGroups;     // kGroups x d
  const int t = blockIdx.x, h = blockIdx.y;
  const int group = threadIdx.x / CHUNK, place = threadIdx.x % CHUNK;       // place: key of the chunk, then dim of the output
  const int wave = threadIdx.x / 64, first_wave = group * kWavesPerGroup;
  const int kv_head = h / (nq / nkv);
  const int pos = positions[t];
  const int* pages = block_table + static_cast<size_t>(token_seq[t]) * max_blocks;
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const size_t page_stride = static_cast<size_t>(2) * nkv * page_size * d;
  const size_t head_offset = static_cast<size_t>(kv_head) * page_size * d;
  const size_t v_offset = static_cast<size_t>(nkv) * page_size * d;

  for (int i = threadIdx.x; i < d; i += 256) q_row[i] = to_float(q[(static_cast<size_t>(t) * nq + h) * d + i]);
  __syncthreads();

  // the reductions over a group: over each of its waves by shuffles, then over its waves through LDS
  // (every thread of the workgroup takes part in every call: the barriers are the workgroup's)
  auto over_group = [&](float value, bool maximum) {
    value = maximum ? wave_max(value) : wave_sum(value);
    if (kWavesPerGroup == 1) return value;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) wave_part[wave] = value;
    __syncthreads();
    float total = wave_part[first_wave];
    for (int w = 1; w < kWavesPerGroup; ++w) total = maximum ? fmaxf(total, wave_part[first_wave + w]) : total + wave_part[first_wave + w];
    return total;
  };

  float running_max = -INFINITY, running_sum = 0.f, acc = 0.f;
  constexpr int kRound = CHUNK * kGroups;          // keys all groups take in one turn of the loop
  for (int base = (lo / kRound) * kRound; base <= pos; base += kRound) {
    const int start = base + group * CHUNK;        // (a group whose chunk lies outside lo..pos goes along with nothing to add)
    const int j = start + place;
    const bool valid = j >= lo && j <= pos;
    float score = -INFINITY;
    if (valid) {
      const T* key = cache + static_cast<size_t>(pages[j / page_size]) * page_stride + head_offset +
                     static_cast<size_t>(j % page_size) * d;
      float dot = 0.f;
      for (int i = 0; i < d; ++i) dot += q_row[i] * to_float(key[i]);
      score = dot * scale;
    }
    const float new_max = fmaxf(running_max, over_group(score, true));
    const float p = valid ? expf(score - new_max) : 0.f;
    prob[threadIdx.x] = p;
    const float chunk_sum = over_group(p, false);
    __syncthreads();                               // prob[] is written
    // nothing seen yet (new_max = -inf): nothing to rescale, nothing to add
    const float alpha = new_max == -INFINITY ? 1.f : expf(running_max - new_max);   // 0 when this chunk is the group's first with keys
    running_sum = running_sum * alpha + chunk_sum;
    running_max = new_max;
    if (place < d) {
      acc *= alpha;
      const int first = max(0, lo - start), last = min(CHUNK, pos - start + 1);
      for (int jj = first; jj < last; ++jj) {
        const int key_pos = start + jj;
        const T* value = cache + static_cast<size_t>(pages[key_pos / page_size]) * page_stride + v_offset + head_offset +
                         static_cast<size_t>(place) * page_size + key_pos % page_size;
        acc += prob[group * CHUNK + jj] * to_float(*value);
      }
    }
    __syncthreads();                               // prob[] is read
  }
  // the groups' results into one, in the order of the groups
  if (place == 0) group_stat[2 * group] = running_max, group_stat[2 * group + 1] = running_sum;
  if (place < d) group_out[group * d + place] = acc;
  __syncthreads();
  if (threadIdx.x < d) {
    float top = -INFINITY;
    for (int g = 0; g < kGroups; ++g) top = fmaxf(top, group_stat[2 * g]);
    float total = 0.f, result = 0.f;
    for (int g = 0; g < kGroups; ++g) {
      const float m = group_stat[2 * g];
      if (m == -INFINITY) continue;                // a group that saw no key
      const float w = expf(m - top);
      total += w * group_stat[2 * g + 1];
      result += w * group_out[g * d + threadIdx.x];
    }
    out[(static_cast<size_t>(t) * nq + h) * d + threadIdx.x] = from_float<T>(result / total);
  }
}

}  // namespace tlie

using namespace tlie;

extern "C" int tlie_attention_generic(const void* q, const void* cache, int dtype, const int* block_table,
                                      int max_blocks, const int* token_seq, const int* positions, void* out,
                                      int tokens, int nq, int nkv, int d, int page_size, int window, float scale,
                                      void* stream) {
  if (tokens <= 0 || nq <= 0 || nkv <= 0 || nq % nkv != 0 || d <= 0 || d > 256 || page_size <= 0 || max_blocks <= 0)
    return kBadArgument;
  const int chunk = d <= 64 ? 64 : (d <= 128 ? 128 : 256);
  const int groups = 256 / chunk;
  const size_t lds = (static_cast<size_t>(d) + 256 + 4 + 2 * groups + static_cast<size_t>(groups) * d) * sizeof(float);
  hipStream_t s = (hipStream_t)stream;
#define TLIE_LAUNCH(T, CHUNK)                                                                                         \
  hipLaunchKernelGGL((attention_generic_kernel<T, CHUNK>), dim3(tokens, nq), dim3(256), lds, s, (const T*)q,           \
                     (const T*)cache, block_table, max_blocks, token_seq, positions, (T*)out, nq, nkv, d, page_size,   \
                     window, scale)
  if (dtype == kF32) {
    if (chunk == 64) TLIE_LAUNCH(float, 64); else if (chunk == 128) TLIE_LAUNCH(float, 128); else TLIE_LAUNCH(float, 256);
  } else if (dtype == kBF16) {
    if (chunk == 64) TLIE_LAUNCH(bf16, 64); else if (chunk == 128) TLIE_LAUNCH(bf16, 128); else TLIE_LAUNCH(bf16, 256);
  }
  else
    return kBadArgument;
#undef TLIE_LAUNCH
  return launch_status();
}
