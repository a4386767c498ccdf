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

#include <type_traits>

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
// seq_start (or null) with min_tokens: the step's cumulative token counts per sequence; tokens of
// sequences that bring min_tokens tokens or more are then left to the tiled kernel below, which
// is launched beside this one for the same step and leaves the others to this one.
template <typename T, int CHUNK>
__global__ void __launch_bounds__(256)
attention_generic_kernel(const T* __restrict__ q, const T* __restrict__ cache, const int* __restrict__ block_table,
                         int max_blocks, const int* __restrict__ token_seq, const int* __restrict__ positions,
                         T* __restrict__ out, int nq, int nkv, int d, int page_size, int window, float scale,
                         const int* __restrict__ seq_start, int min_tokens) {
  constexpr int kGroups = 256 / CHUNK, kWavesPerGroup = CHUNK / 64;
  if (seq_start != nullptr) {                      // (the same for the whole workgroup)
    const int seq = token_seq[blockIdx.x];
    if (seq_start[seq + 1] - seq_start[seq] >= min_tokens) return;
  }
  extern __shared__ __attribute__((aligned(16))) float lds[];
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
  // whole 16-byte loads of keys and values where everything is a multiple of four floats
  const bool wide = (d & 3) == 0 && (page_size & 3) == 0 && (reinterpret_cast<uintptr_t>(cache) & 15) == 0;

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
      int i = 0;
      if (std::is_same<T, float>::value && wide) {
        // (four dims a load; the additions stay in the order of the dims)
#pragma unroll 4
        for (; i + 4 <= d; i += 4) {
          const float4 kv = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(key) + i);
          const float4 qv = *reinterpret_cast<const float4*>(q_row + i);
          dot += qv.x * kv.x;
          dot += qv.y * kv.y;
          dot += qv.z * kv.z;
          dot += qv.w * kv.w;
        }
      }
      for (; i < d; ++i) dot += q_row[i] * to_float(key[i]);
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
      int jj = first;
      if (std::is_same<T, float>::value && wide) {
        // (four keys a load where they lie on one page, four to a boundary: chunks start at multiples of
        // 64 and pages hold a multiple of four rows; the additions stay in the order of the keys)
        for (; jj < last && (jj & 3) != 0; ++jj) {
          const int key_pos = start + jj;
          const T* value = cache + static_cast<size_t>(pages[key_pos / page_size]) * page_stride + v_offset + head_offset +
                           static_cast<size_t>(place) * page_size + key_pos % page_size;
          acc += prob[group * CHUNK + jj] * to_float(*value);
        }
#pragma unroll 4
        for (; jj + 4 <= last; jj += 4) {
          const int key_pos = start + jj;
          const float* value = reinterpret_cast<const float*>(cache) + static_cast<size_t>(pages[key_pos / page_size]) * page_stride +
                               v_offset + head_offset + static_cast<size_t>(place) * page_size + key_pos % page_size;
          const float4 vv = *reinterpret_cast<const float4*>(value);
          const float4 pv = *reinterpret_cast<const float4*>(prob + group * CHUNK + jj);
          acc += pv.x * vv.x;
          acc += pv.y * vv.y;
          acc += pv.z * vv.z;
          acc += pv.w * vv.w;
        }
      }
      for (; jj < last; ++jj) {
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

// The same attention for steps that bring several tokens of a sequence (prompt portions): a
// workgroup serves up to 32 columns, a column being a (token, query head) pair, of up to 32 / heads
// consecutive tokens of the step and the heads of one kv head (or 32 of them), and brings every
// chunk of 64 keys and values through LDS once for all of them, where the kernel above reads
// each key and value again for every column (a prompt of 2048 tokens: 34 GB of cache traffic a layer).
//
// The arithmetic of a column is the kernel's above, operation for operation: chunk c of the context
// belongs to running state c % 4 (there: to thread group c % 4), a chunk's scores are 64 dot products
// summed in the order of the dims, its maximum and sum are the same reductions over a wave, the
// values are added in the order of the keys, and the four states meet in the same order at the end.
// A column therefore gets the same bits from either kernel, and a step may take whichever is faster.
// Head sizes up to 64.  Tokens of a workgroup that belong to different sequences are served one
// run of equal sequences after the other.
constexpr int kTiledCols = 32, kTiledWaves = 8, kTiledSlots = kTiledCols / kTiledWaves;     // columns a workgroup, its waves, columns a wave
template <typename T>
__global__ void __launch_bounds__(64 * kTiledWaves)
attention_generic_tiled_kernel(const T* __restrict__ q, const T* __restrict__ cache, const int* __restrict__ block_table,
                               int max_blocks, const int* __restrict__ token_seq, const int* __restrict__ positions,
                               T* __restrict__ out, int tokens, int nq, int nkv, int d, int page_size, int window, float scale,
                               int tokens_per_block, int heads_per_block, const int* __restrict__ seq_start, int min_tokens) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  // rows of a multiple of 4 floats, so that four values are one LDS read, plus 4: a wave's lanes, each
  // on a row of its own, then spread over the banks
  const int k_stride = (d + 3) / 4 * 4 + 4, q_stride = (d + 3) / 4 * 4;
  constexpr int kValueStride = 68;
  float* k_tile = lds;                             // [64 keys][k_stride]
  float* v_tile = k_tile + 64 * k_stride;          // [d][68]
  float* q_tile = v_tile + d * kValueStride;       // [32 columns][q_stride]
  float* prob = q_tile + kTiledCols * q_stride;    // [waves][4 columns][64 keys]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int G = nq / nkv, kv_head = blockIdx.y;
  const int tok0 = blockIdx.x * tokens_per_block, head0 = blockIdx.z * heads_per_block;
  const int ntok = min(tokens_per_block, tokens - tok0), nheads = min(heads_per_block, G - head0);
  const int ncols = ntok * nheads;                 // column c = (token c / nheads, head c % nheads)
  const size_t page_stride = static_cast<size_t>(2) * nkv * page_size * d;
  const size_t head_offset = static_cast<size_t>(kv_head) * page_size * d;
  const size_t v_offset = static_cast<size_t>(nkv) * page_size * d;

  for (int e = threadIdx.x; e < ncols * d; e += 64 * kTiledWaves) {
    const int c = e / d, i = e - c * d;
    q_tile[c * q_stride + i] = to_float(q[(static_cast<size_t>(tok0 + c / nheads) * nq + kv_head * G + head0 + c % nheads) * d + i]);
  }
  // this wave's columns: slot s is column wave + kTiledWaves * s
  int col_pos[kTiledSlots], col_lo[kTiledSlots], col_tok[kTiledSlots];     // col_tok: the column's token among the workgroup's, or -1
#pragma unroll
  for (int s = 0; s < kTiledSlots; ++s) {
    const int c = wave + kTiledWaves * s;
    bool live = c < ncols;
    if (live && seq_start != nullptr) {            // a token of a sequence that brings few tokens is the other kernel's
      const int seq = token_seq[tok0 + c / nheads];
      live = seq_start[seq + 1] - seq_start[seq] >= min_tokens;
    }
    col_tok[s] = live ? c / nheads : -1;
    col_pos[s] = live ? positions[tok0 + col_tok[s]] : -1;
    col_lo[s] = live && window > 0 ? max(0, col_pos[s] - window + 1) : 0;
  }
  float run_max[4][kTiledSlots], run_sum[4][kTiledSlots], acc[4][kTiledSlots];
#pragma unroll
  for (int g = 0; g < 4; ++g)
#pragma unroll
    for (int s = 0; s < kTiledSlots; ++s) run_max[g][s] = -INFINITY, run_sum[g][s] = 0.f, acc[g][s] = 0.f;

  // runs of tokens of one sequence, in the order of the tokens (a column belongs to the run its token
  // lies in: a sequence may come twice among a workgroup's tokens, when a recorded step pads its
  // tokens with tokens of its first sequence)
  int run_first = 0;
  while (run_first < ntok) {                       // (the same for every thread: the barriers below are the workgroup's)
    const int seq = token_seq[tok0 + run_first];
    int run_end = run_first + 1;
    while (run_end < ntok && token_seq[tok0 + run_end] == seq) ++run_end;
    if (seq_start != nullptr && seq_start[seq + 1] - seq_start[seq] < min_tokens) {   // (the same for every thread)
      run_first = run_end;
      continue;
    }
    // the keys the run's columns see: from the least lower bound to the last token's position
    int hi = -1, lo = 1 << 30;
    for (int t = run_first; t < run_end; ++t) {
      const int pos = positions[tok0 + t];
      hi = max(hi, pos);
      lo = min(lo, window > 0 ? max(0, pos - window + 1) : 0);
    }
    const int* pages = block_table + static_cast<size_t>(seq) * max_blocks;
    for (int base = (lo / 256) * 256; base <= hi; base += 256) {
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int start = base + g * 64;
        if (start > hi) break;                     // (uniform)
        __syncthreads();                           // the tiles of the chunk before have been read
        for (int e = threadIdx.x; e < 64 * d; e += 64 * kTiledWaves) {
          const int r = e / d, i = e - r * d, j = start + r;
          if (j <= hi && j >= lo)
            k_tile[r * k_stride + i] = to_float(cache[static_cast<size_t>(pages[j / page_size]) * page_stride + head_offset +
                                                      static_cast<size_t>(j % page_size) * d + i]);
        }
        for (int e = threadIdx.x; e < 64 * d; e += 64 * kTiledWaves) {
          const int dim = e >> 6, r = e & 63, j = start + r;
          if (j <= hi && j >= lo)
            v_tile[dim * kValueStride + r] = to_float(cache[static_cast<size_t>(pages[j / page_size]) * page_stride + v_offset + head_offset +
                                                  static_cast<size_t>(dim) * page_size + j % page_size]);
        }
        __syncthreads();
        // four columns at a time: their dot products share each read of a key, and the chains of
        // additions of one column wait for each other less
#pragma unroll
        for (int b = 0; b < kTiledSlots / 4; ++b) {
          bool any = false;
#pragma unroll
          for (int u = 0; u < 4; ++u)
            any |= col_tok[b * 4 + u] >= run_first && col_tok[b * 4 + u] < run_end && col_pos[b * 4 + u] >= start && col_lo[b * 4 + u] < start + 64;
          if (!any) continue;                      // (uniform over the wave: the columns are the wave's)
          const int j = start + lane;
          float dot[4] = {0.f, 0.f, 0.f, 0.f};
          const float* key = k_tile + lane * k_stride;
          const float* query[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) query[u] = q_tile + min(wave + kTiledWaves * (b * 4 + u), kTiledCols - 1) * q_stride;
          // (four dims a read; the additions of a column stay in the order of the dims)
          int i = 0;
#pragma unroll 4
          for (; i + 4 <= d; i += 4) {
            const float4 kv = *reinterpret_cast<const float4*>(key + i);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              const float4 qv = *reinterpret_cast<const float4*>(query[u] + i);
              dot[u] += qv.x * kv.x;
              dot[u] += qv.y * kv.y;
              dot[u] += qv.z * kv.z;
              dot[u] += qv.w * kv.w;
            }
          }
          for (; i < d; ++i) {
            const float kv = key[i];
#pragma unroll
            for (int u = 0; u < 4; ++u) dot[u] += query[u][i] * kv;
          }
          float* my_prob = prob + (wave * 4) * 64;
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const int s = b * 4 + u;
            const bool column = col_tok[s] >= run_first && col_tok[s] < run_end && col_pos[s] >= start && col_lo[s] < start + 64;   // a chunk without keys changes nothing
            if (!column) continue;                 // (uniform over the wave)
            const bool valid = j >= col_lo[s] && j <= col_pos[s];
            const float score = valid ? dot[u] * scale : -INFINITY;
            const float new_max = fmaxf(run_max[g][s], wave_max(score));
            const float p = valid ? expf(score - new_max) : 0.f;
            my_prob[u * 64 + lane] = p;
            const float chunk_sum = wave_sum(p);
            const float alpha = new_max == -INFINITY ? 1.f : expf(run_max[g][s] - new_max);
            run_sum[g][s] = run_sum[g][s] * alpha + chunk_sum;
            run_max[g][s] = new_max;
            acc[g][s] *= alpha;
          }
          // what one lane wrote to prob above, another lane of the wave reads below: the writes are
          // ordered before the reads for the compiler and the memory model (no instruction on this hardware,
          // where a wave's LDS operations complete in order)
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
          __builtin_amdgcn_wave_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
          if (lane < d) {
            const float* value = v_tile + lane * kValueStride;
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              const int s = b * 4 + u;
              const bool column = col_tok[s] >= run_first && col_tok[s] < run_end && col_pos[s] >= start && col_lo[s] < start + 64;
              if (!column) continue;
              const int first = max(0, col_lo[s] - start), last = min(64, col_pos[s] - start + 1);
              float sum = acc[g][s];
              const float* weight = my_prob + u * 64;
              int jj = first;
              for (; jj < last && (jj & 3) != 0; ++jj) sum += weight[jj] * value[jj];
#pragma unroll 4
              for (; jj + 4 <= last; jj += 4) {           // (four keys a read; the additions stay in the order of the keys)
                const float4 pv = *reinterpret_cast<const float4*>(weight + jj), vv = *reinterpret_cast<const float4*>(value + jj);
                sum += pv.x * vv.x;
                sum += pv.y * vv.y;
                sum += pv.z * vv.z;
                sum += pv.w * vv.w;
              }
              for (; jj < last; ++jj) sum += weight[jj] * value[jj];
              acc[g][s] = sum;
            }
          }
        }
      }
    }
    run_first = run_end;
  }
  // the four states of a column into one, in their order
  if (lane < d) {
#pragma unroll
    for (int s = 0; s < kTiledSlots; ++s) {
      const int c = wave + kTiledWaves * s;
      if (c >= ncols || col_tok[s] < 0) continue;
      float top = -INFINITY;
#pragma unroll
      for (int g = 0; g < 4; ++g) top = fmaxf(top, run_max[g][s]);
      float total = 0.f, result = 0.f;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const float m = run_max[g][s];
        if (m == -INFINITY) continue;
        const float w = expf(m - top);
        total += w * run_sum[g][s];
        result += w * acc[g][s];
      }
      out[(static_cast<size_t>(tok0 + c / nheads) * nq + kv_head * G + head0 + c % nheads) * d + lane] = from_float<T>(result / total);
    }
  }
}

}  // namespace tlie

using namespace tlie;

extern "C" int tlie_attention_generic(const void* q, const void* cache, int dtype, const int* block_table,
                                      int max_blocks, const int* token_seq, const int* positions, void* out,
                                      int tokens, int nq, int nkv, int d, int page_size, int window, float scale,
                                      int tiled, const int* seq_start, int min_tokens, void* stream) {
  // tiled 0: the kernel of one (token, head) a workgroup; 1: the kernel that shares keys among a
  // sequence's tokens (head sizes up to 64); 2: both, each token served by one of them: the second
  // takes the sequences that bring min_tokens tokens or more (seq_start: int32 [sequences + 1], the
  // step's cumulative token counts), the first the others.  A token gets the same bits from either.
  if (tokens <= 0 || nq <= 0 || nkv <= 0 || nq % nkv != 0 || d <= 0 || d > 256 || page_size <= 0 || max_blocks <= 0)
    return kBadArgument;
  if (tiled < 0 || tiled > 2 || (tiled == 2 && (seq_start == nullptr || min_tokens < 1))) return kBadArgument;
  if (dtype != kF32 && dtype != kBF16) return kBadArgument;
  if (d > 64) tiled = 0;
  const int* select = tiled == 2 ? seq_start : nullptr;
  if (tiled) {
    // (the same bits as the kernel below, for steps whose sequences bring several tokens each)
    const int G = nq / nkv;
    const int heads_per_block = G < kTiledCols ? G : kTiledCols;
    const int tokens_per_block = kTiledCols / heads_per_block;
    const dim3 grid((tokens + tokens_per_block - 1) / tokens_per_block, nkv, (G + heads_per_block - 1) / heads_per_block);
    const size_t rounded = (static_cast<size_t>(d) + 3) / 4 * 4;
    const size_t bytes = (64 * (rounded + 4) + static_cast<size_t>(d) * 68 + kTiledCols * rounded + kTiledWaves * 4 * 64) * sizeof(float);
    if (dtype == kF32)
      hipLaunchKernelGGL((attention_generic_tiled_kernel<float>), grid, dim3(64 * kTiledWaves), bytes, (hipStream_t)stream, (const float*)q,
                         (const float*)cache, block_table, max_blocks, token_seq, positions, (float*)out, tokens, nq, nkv, d,
                         page_size, window, scale, tokens_per_block, heads_per_block, select, min_tokens);
    else
      hipLaunchKernelGGL((attention_generic_tiled_kernel<bf16>), grid, dim3(64 * kTiledWaves), bytes, (hipStream_t)stream, (const bf16*)q,
                         (const bf16*)cache, block_table, max_blocks, token_seq, positions, (bf16*)out, tokens, nq, nkv, d,
                         page_size, window, scale, tokens_per_block, heads_per_block, select, min_tokens);
    const int status = launch_status();
    if (status != kOk || tiled == 1) return status;
  }
  const int chunk = d <= 64 ? 64 : (d <= 128 ? 128 : 256);
  const int groups = 256 / chunk;
  const size_t lds = (static_cast<size_t>(d) + 256 + 4 + 2 * groups + static_cast<size_t>(groups) * d) * sizeof(float);
  hipStream_t s = (hipStream_t)stream;
#define TLIE_LAUNCH(T, CHUNK)                                                                                         \
  hipLaunchKernelGGL((attention_generic_kernel<T, CHUNK>), dim3(tokens, nq), dim3(256), lds, s, (const T*)q,           \
                     (const T*)cache, block_table, max_blocks, token_seq, positions, (T*)out, nq, nkv, d, page_size,   \
                     window, scale, select, min_tokens)
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
