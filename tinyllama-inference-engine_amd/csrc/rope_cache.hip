// Rotary positions on q and k, and the write of k and v into the paged cache, in one pass over
// the fused qkv projection's output.
//
// reference: RopeKernel (src/cuda/kernels.cu:86-115) rotates the pair (i, i + d/2) of every head
// by angle = float(position) * theta^(-2i/d), sine and cosine in float; KvUpdateKernel
// (kernels.cu:137-145) then copies the rotated key and the value to the cache row of the
// position.  Here all tokens of a step go in one launch, positions come from an array, the
// frequencies from a table made once per model, and the cache row is found through the slot map.
// A block serves a few heads of one token: it first forms the token's d/2 sines and cosines once
// (not once per head), then every thread sums its element's partial results, trades it with its
// rotation partner through LDS, and writes q or the cache.
#include "common.h"

namespace tlie {

// qkv: [nsplit][tokens][(nq + 2 nkv) * d], columns ordered q heads | k heads | v heads.
// q_out: [tokens][nq * d].  cache: [pages][2][nkv][page_size * d]: keys at index 0 as [row][dim],
// values at index 1 transposed, [dim][row] (the attention kernels read 4 consecutive rows of one dim).
// slot_map[t] = page * page_size + row of token t, or -1: nothing is written for that token.
// rot_dim <= d, even: dimensions from rot_dim on are copied unrotated.  inv_freq may be null
// (no rotation at all).  paired: within a q or k head the input's columns are stored with the two
// elements of a rotation pair side by side (element i at 2i, element i + rot_dim/2 at 2i + 1), as
// the product of few rows wants its weight's rows; outputs are in natural order either way.
// blockDim.x = heads_per_block * d; grid = (tokens, ceil(heads / heads_per_block)).
template <typename D, typename A>
__global__ void rope_cache_kernel(const D* __restrict__ qkv, int nsplit, size_t split_stride,
                                  const int* __restrict__ positions, const int* __restrict__ slot_map,
                                  const float* __restrict__ inv_freq, int rot_dim, A* __restrict__ q_out,
                                  A* __restrict__ cache, int nq, int nkv, int d, int page_size, int paired) {
  extern __shared__ float lds[];
  float* cosines = lds;                  // rot_dim / 2
  float* sines = cosines + rot_dim / 2;  // rot_dim / 2
  float* values = sines + rot_dim / 2;   // blockDim.x
  const int t = blockIdx.x;
  const int heads = nq + 2 * nkv;
  const int width = heads * d;
  const int half = rot_dim / 2;
  if (inv_freq != nullptr) {
    const float pos = static_cast<float>(positions[t]);
    for (int i = threadIdx.x; i < half; i += blockDim.x) sincosf(pos * inv_freq[i], &sines[i], &cosines[i]);
  }
  const int local_head = threadIdx.x / d, e = threadIdx.x % d;
  const int head = blockIdx.y * (blockDim.x / d) + local_head;
  const bool live = head < heads;
  float mine = 0.f;
  int column = e;
  if (paired && head < nq + nkv && e < rot_dim) column = e < half ? 2 * e : 2 * (e - half) + 1;
  if (live) mine = sum_splits(qkv + static_cast<size_t>(t) * width + head * d + column, nsplit, split_stride);
  values[threadIdx.x] = mine;
  __syncthreads();
  if (!live) return;
  float result = mine;
  if (inv_freq != nullptr && head < nq + nkv && e < rot_dim) {
    if (e < half) {
      result = mine * cosines[e] - values[threadIdx.x + half] * sines[e];
    } else {
      result = mine * cosines[e - half] + values[threadIdx.x - half] * sines[e - half];
    }
  }
  if (head < nq) {
    q_out[static_cast<size_t>(t) * nq * d + head * d + e] = from_float<A>(result);
    return;
  }
  const int slot = slot_map[t];
  if (slot < 0) return;
  const size_t head_stride = static_cast<size_t>(page_size) * d;
  A* page = cache + static_cast<size_t>(slot / page_size) * 2 * nkv * head_stride;
  const int row = slot % page_size;
  if (head < nq + nkv) {
    page[(head - nq) * head_stride + static_cast<size_t>(row) * d + e] = from_float<A>(result);
  } else {
    // value head (head - nq - nkv) lies after the nkv key heads: at head offset (head - nq), transposed
    page[(head - nq) * head_stride + static_cast<size_t>(e) * page_size + row] = from_float<A>(result);
  }
}

// The same for one summand with eight input columns a thread (16-byte loads): d % 8 == 0 and, where
// there is rotation, paired columns and rot_dim % 8 == 0, so that a thread holds four whole pairs.
// One block a token; blockDim.x covers (nq + 2 nkv) * d / 8 groups, or loops.
template <typename D, typename A>
__global__ void rope_cache_wide_kernel(const D* __restrict__ qkv, const int* __restrict__ positions,
                                       const int* __restrict__ slot_map, const float* __restrict__ inv_freq,
                                       int rot_dim, A* __restrict__ q_out, A* __restrict__ cache, int nq, int nkv,
                                       int d, int page_size) {
  extern __shared__ float lds[];
  const int half = rot_dim / 2;
  float* cosines = lds;                  // half
  float* sines = cosines + half;         // half
  const int t = blockIdx.x;
  const int heads = nq + 2 * nkv, per_head = d / 8;
  const int slot = slot_map[t];
  // this thread's first eight columns are asked for before the angles are made: their way from memory
  // is then hidden behind the sines and cosines (and the barrier after them)
  float first_v[8];
  const bool first_live = static_cast<int>(threadIdx.x) < heads * per_head;
  if (first_live)
    load8(qkv + (static_cast<size_t>(t) * heads + threadIdx.x / per_head) * d + (threadIdx.x % per_head) * 8, first_v);
  if (inv_freq != nullptr) {
    const float pos = static_cast<float>(positions[t]);
    for (int i = threadIdx.x; i < half; i += blockDim.x) sincosf(pos * inv_freq[i], &sines[i], &cosines[i]);
    __syncthreads();
  }
  const size_t head_stride = static_cast<size_t>(page_size) * d;
  A* page = cache + static_cast<size_t>(slot < 0 ? 0 : slot / page_size) * 2 * nkv * head_stride;
  const int row = slot < 0 ? 0 : slot % page_size;
  for (int g = threadIdx.x; g < heads * per_head; g += blockDim.x) {
    const int head = g / per_head, c = (g % per_head) * 8;
    if (head >= nq && slot < 0) continue;
    float v[8];
    if (g == static_cast<int>(threadIdx.x)) {
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = first_v[j];
    } else {
      load8(qkv + (static_cast<size_t>(t) * heads + head) * d + c, v);
    }
    if (head >= nq + nkv) {
      // a value head: after the nkv key heads of the page, transposed
      A* out = page + (head - nq) * head_stride + static_cast<size_t>(c) * page_size + row;
#pragma unroll
      for (int j = 0; j < 8; ++j) out[static_cast<size_t>(j) * page_size] = from_float<A>(v[j]);
      continue;
    }
    A* out = head < nq ? q_out + (static_cast<size_t>(t) * nq + head) * d
                       : page + (head - nq) * head_stride + static_cast<size_t>(row) * d;
    if (inv_freq != nullptr && c < rot_dim) {
      const int first = c / 2;           // v[2j], v[2j + 1] = elements first + j and first + j + half
      float lo[4], hi[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float cs = cosines[first + j], sn = sines[first + j];
        lo[j] = v[2 * j] * cs - v[2 * j + 1] * sn;
        hi[j] = v[2 * j + 1] * cs + v[2 * j] * sn;
      }
      store4(out + first, lo[0], lo[1], lo[2], lo[3]);
      store4(out + half + first, hi[0], hi[1], hi[2], hi[3]);
    } else {
      store8(out + c, v);
    }
  }
}

}  // namespace tlie

using namespace tlie;

extern "C" int tlie_rope_cache(const void* qkv, int in_dtype, int nsplit, long long split_stride,
                               const int* positions, const int* slot_map, const float* inv_freq, int rot_dim,
                               void* q_out, void* cache, int act_dtype, int tokens, int nq, int nkv, int d,
                               int page_size, int paired, void* stream) {
  if (tokens <= 0 || nq <= 0 || nkv <= 0 || d <= 0 || d > 1024 || page_size <= 0 || nsplit < 1) return kBadArgument;
  if (rot_dim < 0 || rot_dim > d || rot_dim % 2 != 0) return kBadArgument;
  const int heads = nq + 2 * nkv;
  hipStream_t s = (hipStream_t)stream;
  const bool aligned = ((reinterpret_cast<uintptr_t>(qkv) | reinterpret_cast<uintptr_t>(q_out) |
                         reinterpret_cast<uintptr_t>(cache)) & 31) == 0;
  if (nsplit == 1 && (d & 7) == 0 && aligned && (inv_freq == nullptr || (paired && (rot_dim & 7) == 0))) {
    const int groups = heads * d / 8;
    const int wide = groups >= 1024 ? 1024 : (groups + 63) / 64 * 64;
    const size_t wide_lds = static_cast<size_t>(rot_dim) * sizeof(float);
#define TLIE_WIDE(DC, D, AC, A)                                                                              \
  if (in_dtype == DC && act_dtype == AC) {                                                                   \
    hipLaunchKernelGGL((rope_cache_wide_kernel<D, A>), dim3(tokens), dim3(wide), wide_lds, s, (const D*)qkv,   \
                       positions, slot_map, inv_freq, rot_dim, (A*)q_out, (A*)cache, nq, nkv, d, page_size);  \
    return launch_status();                                                                                  \
  }
    TLIE_WIDE(kF32, float, kF32, float)
    TLIE_WIDE(kF32, float, kBF16, bf16)
    TLIE_WIDE(kBF16, bf16, kBF16, bf16)
#undef TLIE_WIDE
    return kBadArgument;
  }
  int heads_per_block = 256 / d;
  if (heads_per_block < 1) heads_per_block = 1;
  if (heads_per_block > heads) heads_per_block = heads;
  const int threads = heads_per_block * d;
  const dim3 grid(tokens, (heads + heads_per_block - 1) / heads_per_block);
  if (grid.y > 65535) return kBadArgument;
  const size_t lds = (static_cast<size_t>(rot_dim) + threads) * sizeof(float);
#define TLIE_CASE(DC, D, AC, A)                                                                              \
  if (in_dtype == DC && act_dtype == AC) {                                                                   \
    hipLaunchKernelGGL((rope_cache_kernel<D, A>), grid, dim3(threads), lds, s, (const D*)qkv, nsplit,         \
                       (size_t)split_stride, positions, slot_map, inv_freq, rot_dim, (A*)q_out, (A*)cache, nq, \
                       nkv, d, page_size, paired);                                                           \
    return launch_status();                                                                                  \
  }
  TLIE_CASE(kF32, float, kF32, float)
  TLIE_CASE(kF32, float, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kBF16, bf16)
#undef TLIE_CASE
  return kBadArgument;
}
