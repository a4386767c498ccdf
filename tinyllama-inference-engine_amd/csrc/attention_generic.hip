// Paged causal grouped-query attention, the plain kernel: any storage type, any head size up to
// the block size, any number of tokens per sequence.  It is the whole 32-bit path's attention and
// the fallback of the bfloat16 path for sizes the tiled kernels refuse.
//
// reference: AttentionDecodeKernel (src/cuda/kernels.cu:147-196): one block per query head,
// scores = (q . k) * rsqrt(d) over positions 0..pos, max, exp, sum, normalise, then one thread
// per output dimension sums p * v serially.  That kernel keeps all scores of the context in
// shared memory and serves one token; this one walks the context in chunks of one block width
// with a running maximum and sum (so the context length is unbounded), serves every token of a
// step in one launch, finds keys through the block table, and optionally limits the keys to a
// window.  Chunks start at multiples of the block width counted from position 0, so the order of
// the sums for a given (sequence, position) never depends on how the step was cut.
#include "common.h"

namespace tlie {

// q: [tokens][nq][d]; cache: [pages][2][nkv][page_size * d], keys [row][dim], values [dim][row];
// out: [tokens][nq][d].
// token_seq[t]: row of the block table; positions[t]: absolute position of the token.
// window <= 0: all keys 0..pos; otherwise keys pos-window+1..pos.
template <typename T>
__global__ void attention_generic_kernel(const T* __restrict__ q, const T* __restrict__ cache,
                                         const int* __restrict__ block_table, int max_blocks,
                                         const int* __restrict__ token_seq, const int* __restrict__ positions,
                                         T* __restrict__ out, int nq, int nkv, int d, int page_size, int window,
                                         float scale) {
  extern __shared__ float lds[];
  float* q_row = lds;                    // d
  float* prob = q_row + d;               // blockDim.x
  float* scratch = prob + blockDim.x;    // 16
  const int t = blockIdx.x, h = blockIdx.y;
  const int kv_head = h / (nq / nkv);
  const int pos = positions[t];
  const int* pages = block_table + static_cast<size_t>(token_seq[t]) * max_blocks;
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int chunk = blockDim.x;
  const size_t page_stride = static_cast<size_t>(2) * nkv * page_size * d;
  const size_t head_offset = static_cast<size_t>(kv_head) * page_size * d;
  const size_t v_offset = static_cast<size_t>(nkv) * page_size * d;

  for (int i = threadIdx.x; i < d; i += blockDim.x) q_row[i] = to_float(q[(static_cast<size_t>(t) * nq + h) * d + i]);
  __syncthreads();

  float running_max = -INFINITY, running_sum = 0.f, acc = 0.f;
  for (int start = (lo / chunk) * chunk; start <= pos; start += chunk) {
    const int j = start + threadIdx.x;
    const bool valid = j >= lo && j <= pos;
    float score = -INFINITY;
    if (valid) {
      const T* key = cache + static_cast<size_t>(pages[j / page_size]) * page_stride + head_offset +
                     static_cast<size_t>(j % page_size) * d;
      float dot = 0.f;
      for (int i = 0; i < d; ++i) dot += q_row[i] * to_float(key[i]);
      score = dot * scale;
    }
    const float new_max = fmaxf(running_max, block_max(score, scratch));
    const float p = valid ? expf(score - new_max) : 0.f;
    prob[threadIdx.x] = p;
    const float chunk_sum = block_sum(p, scratch);     // also orders the prob[] writes before the reads below
    const float alpha = expf(running_max - new_max);   // 0 on the first chunk (running_max = -inf)
    running_sum = running_sum * alpha + chunk_sum;
    running_max = new_max;
    if (threadIdx.x < d) {
      acc *= alpha;
      const int last = min(chunk, pos - start + 1);
      for (int jj = max(0, lo - start); jj < last; ++jj) {
        const int key_pos = start + jj;
        const T* value = cache + static_cast<size_t>(pages[key_pos / page_size]) * page_stride + v_offset + head_offset +
                         static_cast<size_t>(threadIdx.x) * page_size + key_pos % page_size;
        acc += prob[jj] * to_float(*value);
      }
    }
    __syncthreads();
  }
  if (threadIdx.x < d) out[(static_cast<size_t>(t) * nq + h) * d + threadIdx.x] = from_float<T>(acc / running_sum);
}

}  // namespace tlie

using namespace tlie;

extern "C" int tlie_attention_generic(const void* q, const void* cache, int dtype, const int* block_table,
                                      int max_blocks, const int* token_seq, const int* positions, void* out,
                                      int tokens, int nq, int nkv, int d, int page_size, int window, float scale,
                                      void* stream) {
  if (tokens <= 0 || nq <= 0 || nkv <= 0 || nq % nkv != 0 || d <= 0 || d > 256 || page_size <= 0 || max_blocks <= 0)
    return kBadArgument;
  const int threads = d <= 64 ? 64 : (d <= 128 ? 128 : 256);
  const size_t lds = (static_cast<size_t>(d) + threads + 16) * sizeof(float);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == kF32)
    hipLaunchKernelGGL(attention_generic_kernel<float>, dim3(tokens, nq), dim3(threads), lds, s, (const float*)q,
                       (const float*)cache, block_table, max_blocks, token_seq, positions, (float*)out, nq, nkv, d,
                       page_size, window, scale);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(attention_generic_kernel<bf16>, dim3(tokens, nq), dim3(threads), lds, s, (const bf16*)q,
                       (const bf16*)cache, block_table, max_blocks, token_seq, positions, (bf16*)out, nq, nkv, d,
                       page_size, window, scale);
  else
    return kBadArgument;
  return launch_status();
}
