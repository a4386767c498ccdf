// Rotary positions on q and k, and the write of k and v into the paged cache, in one pass over
// the fused qkv projection's output.
//
// reference: RopeKernel (src/cuda/kernels.cu:86-115) rotates the pair (i, i + d/2) of every head
// by angle = float(position) * theta^(-2i/d), sine and cosine in float; KvUpdateKernel
// (kernels.cu:137-145) then copies the rotated key and the value to the cache row of the
// position.  Here all tokens of a step go in one launch, positions come from an array, the
// frequencies from a table made once per model, and the cache row is found through the slot map.
#include "common.h"

namespace tlie {

// qkv: [nsplit][tokens][(nq + 2 nkv) * d], columns ordered q heads | k heads | v heads.
// q_out: [tokens][nq * d].  cache: [pages][2][nkv][page_size * d]: keys at index 0 as [row][dim],
// values at index 1 transposed, [dim][row] (the attention kernels read 4 consecutive rows of one dim).
// slot_map[t] = page * page_size + row of token t, or -1: nothing is written for that token.
// rot_dim <= d, even: dimensions from rot_dim on are copied unrotated.  inv_freq may be null
// (no rotation at all).
template <typename D, typename A>
__global__ void rope_cache_kernel(const D* __restrict__ qkv, int nsplit, size_t split_stride,
                                  const int* __restrict__ positions, const int* __restrict__ slot_map,
                                  const float* __restrict__ inv_freq, int rot_dim, A* __restrict__ q_out,
                                  A* __restrict__ cache, int nq, int nkv, int d, int page_size) {
  const int t = blockIdx.x;
  const int width = (nq + 2 * nkv) * d;
  const D* row = qkv + static_cast<size_t>(t) * width;
  const float pos = static_cast<float>(positions[t]);
  const int slot = slot_map[t];
  const int half = rot_dim / 2;
  const size_t page_stride = static_cast<size_t>(2) * nkv * page_size * d;
  A* cache_row = nullptr;
  if (slot >= 0) cache_row = cache + static_cast<size_t>(slot / page_size) * page_stride + static_cast<size_t>(slot % page_size) * d;
  const size_t head_stride = static_cast<size_t>(page_size) * d;

  auto value = [&](int column) {
    float v = 0.f;
    for (int s = 0; s < nsplit; ++s) v += to_float(row[s * split_stride + column]);
    return v;
  };

  // q and k heads: one work item per (head, i) with i < d/2 covers elements i and i + d/2 when
  // both are unrotated, or the rotated pair (i, i + half) when i < half.
  const int rotated_heads = nq + nkv;
  const int items = rotated_heads * d;
  for (int item = threadIdx.x; item < items; item += blockDim.x) {
    const int head = item / d, e = item % d;
    float result;
    if (inv_freq != nullptr && e < rot_dim) {
      const int i = e < half ? e : e - half;
      const float angle = pos * inv_freq[i];
      float sine, cosine;
      sincosf(angle, &sine, &cosine);
      const float first = value(head * d + i), second = value(head * d + i + half);
      result = e < half ? first * cosine - second * sine : second * cosine + first * sine;
    } else {
      result = value(head * d + e);
    }
    if (head < nq) {
      q_out[static_cast<size_t>(t) * nq * d + head * d + e] = from_float<A>(result);
    } else if (cache_row) {
      cache_row[(head - nq) * head_stride + e] = from_float<A>(result);
    }
  }
  if (slot >= 0) {
    A* v_page = cache + static_cast<size_t>(slot / page_size) * page_stride + static_cast<size_t>(nkv) * head_stride +
                slot % page_size;
    for (int item = threadIdx.x; item < nkv * d; item += blockDim.x) {
      const int head = item / d, e = item % d;
      v_page[head * head_stride + static_cast<size_t>(e) * page_size] = from_float<A>(value((nq + nkv + head) * d + e));
    }
  }
}

}  // namespace tlie

using namespace tlie;

extern "C" int tlie_rope_cache(const void* qkv, int in_dtype, int nsplit, long long split_stride,
                               const int* positions, const int* slot_map, const float* inv_freq, int rot_dim,
                               void* q_out, void* cache, int act_dtype, int tokens, int nq, int nkv, int d,
                               int page_size, void* stream) {
  if (tokens <= 0 || nq <= 0 || nkv <= 0 || d <= 0 || page_size <= 0 || nsplit < 1) return kBadArgument;
  if (rot_dim < 0 || rot_dim > d || rot_dim % 2 != 0) return kBadArgument;
  const int threads = (nq + nkv) * d >= 1024 ? 256 : 64;
  hipStream_t s = (hipStream_t)stream;
#define TLIE_CASE(DC, D, AC, A)                                                                              \
  if (in_dtype == DC && act_dtype == AC) {                                                                   \
    hipLaunchKernelGGL((rope_cache_kernel<D, A>), dim3(tokens), dim3(threads), 0, s, (const D*)qkv, nsplit,   \
                       (size_t)split_stride, positions, slot_map, inv_freq, rot_dim, (A*)q_out, (A*)cache, nq, \
                       nkv, d, page_size);                                                                   \
    return launch_status();                                                                                  \
  }
  TLIE_CASE(kF32, float, kF32, float)
  TLIE_CASE(kF32, float, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kBF16, bf16)
#undef TLIE_CASE
  return kBadArgument;
}
