// Paged causal grouped-query attention on the matrix cores, bfloat16 storage, 32-bit softmax.
// One kernel serves prompt portions, single decoded tokens and mixed steps.
//
// reference: AttentionDecodeKernel (src/cuda/kernels.cu:147-196) serves one token of one
// sequence, one block per query head: every head of a group reads its kv head's keys and values
// again, the scores of the whole context sit in shared memory, and P.V is a serial loop per
// output dimension.  The arithmetic is kept (score = (q . k) * rsqrt(d), softmax with the maximum
// subtracted, sum of p * v, all in float); the organisation is new:
//
//  * A wave owns 16 "columns": consecutive (token, query head) pairs of one sequence that share
//    one kv head.  For a decode step these are the group's heads of the one token; for a prompt
//    portion, the heads of several tokens.  Keys and values are read once per wave for all 16.
//  * Scores are computed transposed, S^T = K . Q^T, with v_mfma_f32_16x16x32_bf16: operand A is
//    16 keys x 32 dims straight from the cache page (a key's dims are contiguous), operand B is Q.
//    The result leaves each lane with 4 keys of one column, so the softmax statistics of a column
//    are a reduction over 4 registers and 4 lane groups, and the probabilities are already laid out
//    as operand B of the second product, O^T = V^T . P^T.  Nothing passes through LDS.
//  * Values are cached transposed ([dim][row in page]), so operand A of the second product, 4
//    consecutive keys of one dim, is one 8-byte load.
//  * Keys are walked in blocks of 32 that start at multiples of 32 from position 0, with a running
//    maximum and sum: the context length is unbounded and the order of the sums for a (sequence,
//    position) does not depend on how the step was cut.
//  * With nsplit > 1 the keys are cut into nsplit parts of split_len positions handled by
//    different waves (a decode step of few sequences would otherwise leave most of the chip idle);
//    each writes an unnormalised partial result with its maximum and sum, and a second kernel
//    merges them.  The parts are fixed ranges of positions, so a wave can fetch its first keys
//    before it knows how long the sequence is: the position, the block table and the keys are not
//    three loads in a row.
#include "common.h"

namespace tlie {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

union Pack8 {
  uint4 u;
  uint2 h[2];
  uint16_t e[8];
  bf16x8 v;
};

__device__ __forceinline__ uint16_t float_to_bf16_bits(float v) {
  // round to nearest even; the inputs here are finite probabilities in [0, 1]
  uint32_t bits = __float_as_uint(v);
  bits += 0x7fffu + ((bits >> 16) & 1u);
  return static_cast<uint16_t>(bits >> 16);
}

// tiles[i] = (sequence row of the block table, index of the sequence's first token in this step,
//             number of its tokens in this step, first column of the tile)
// column c of a sequence = (token c / G of its tokens in this step, head c % G of the group).
// tiles == nullptr: a decode step, token i is the one token of sequence i; the tile index is
// sequence * ceil(G / 16) + tile of the group.
// DT = head_dim / 16.
template <int DT>
__global__ void __launch_bounds__(64)
attention_mfma_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ cache,
                      const int* __restrict__ block_table, int max_blocks, const int4* __restrict__ tiles,
                      const int* __restrict__ positions, uint16_t* __restrict__ out, float* __restrict__ part_o,
                      float* __restrict__ part_ml, int nsplit, int split_len, int nq, int nkv, int page_size,
                      int window, float scale) {
  constexpr int D = DT * 16;
  constexpr int KS = (DT + 1) / 2;                 // 32-wide k steps of the first product
  const int lane = threadIdx.x, col = lane & 15, grp = lane >> 4;
  const int kvh = blockIdx.y, split = blockIdx.z;
  const int G = nq / nkv;
  int seq, tok0, ntok, col0;
  if (tiles != nullptr) {
    const int4 tile = tiles[blockIdx.x];
    seq = tile.x, tok0 = tile.y, ntok = tile.z, col0 = tile.w;
  } else {
    const int per_seq = (G + 15) / 16;
    seq = tok0 = blockIdx.x / per_seq, ntok = 1, col0 = (blockIdx.x % per_seq) * 16;
  }
  const int pos0 = positions[tok0];
  const int ncols = ntok * G;
  const int c = col0 + col;
  const bool valid_col = c < ncols;
  const int tok = tok0 + (valid_col ? c / G : 0);
  const int head = kvh * G + (valid_col ? c % G : 0);
  const int pos_col = valid_col ? pos0 + c / G : -1;
  const int lo_col = window > 0 ? max(0, pos_col - window + 1) : 0;

  // the tile's key range, and this split's part of it
  const int last_col = min(col0 + 15, ncols - 1);
  const int tile_hi = pos0 + last_col / G + 1;
  const int tile_lo = window > 0 ? max(0, pos0 + col0 / G - window + 1) : 0;
  const int split_lo = nsplit > 1 ? split * split_len : 0;
  const int range_lo = max(tile_lo, split_lo);
  const int range_hi = nsplit > 1 ? min(tile_hi, split_lo + split_len) : tile_hi;
  const int key_limit = max_blocks * page_size - 1;      // the last position the block table has an entry for

  const int* pages = block_table + static_cast<size_t>(seq) * max_blocks;
  const size_t page_stride = static_cast<size_t>(2) * nkv * page_size * D;
  const uint16_t* k_base = cache + static_cast<size_t>(kvh) * page_size * D;
  const uint16_t* v_base = cache + static_cast<size_t>(nkv) * page_size * D + static_cast<size_t>(kvh) * page_size * D;

  // Q as operand B: lane (col, grp) holds dims ks*32 + grp*8 .. +8 of its column
  Pack8 qreg[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int dim = ks * 32 + grp * 8;
    qreg[ks].u = make_uint4(0, 0, 0, 0);
    if (valid_col && dim < D) qreg[ks].u = *reinterpret_cast<const uint4*>(q + (static_cast<size_t>(tok) * nq + head) * D + dim);
  }

  float running_max = -INFINITY, running_sum = 0.f;
  floatx4 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) o[dt] = floatx4{0.f, 0.f, 0.f, 0.f};

  // A block of 32 keys in registers: operand A of the first product (2 tiles of 16 keys) and of the
  // second (per 16 dims, 2 x 4 consecutive keys).  Rows outside the range are read all the same,
  // from whatever page the block table names there (absent entries name page 0), and masked or
  // zeroed when used; so the addresses do not depend on the sequence's length.
  struct KeyBlock {
    Pack8 k[2][KS];
    uint2 v[DT][2];
  };
  auto load_block = [&](int kb, KeyBlock& block) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int key = min(kb + t * 16 + col, key_limit);
      const uint16_t* k_row = k_base + static_cast<size_t>(pages[key / page_size]) * page_stride +
                              static_cast<size_t>(key % page_size) * D;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int dim = ks * 32 + grp * 8;
        block.k[t][ks].u = dim < D ? *reinterpret_cast<const uint4*>(k_row + dim) : make_uint4(0, 0, 0, 0);
      }
    }
    // slot i < 4 of group grp is key kb + grp*4 + i, slot i >= 4 is key kb + 16 + grp*4 + (i - 4)
    const int clamp_a = min(kb + grp * 4, key_limit & ~3);
    const int clamp_b = min(kb + 16 + grp * 4, key_limit & ~3);
    const uint16_t* v_a = v_base + static_cast<size_t>(pages[clamp_a / page_size]) * page_stride + clamp_a % page_size;
    const uint16_t* v_b = v_base + static_cast<size_t>(pages[clamp_b / page_size]) * page_stride + clamp_b % page_size;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const size_t dim = dt * 16 + col;
      block.v[dt][0] = *reinterpret_cast<const uint2*>(v_a + dim * page_size);
      block.v[dt][1] = *reinterpret_cast<const uint2*>(v_b + dim * page_size);
    }
  };

  // without a window the first block's place is known before the position is: (split_lo & ~31)
  const int first_block = (window > 0 ? range_lo : split_lo) & ~31;
  KeyBlock next;
  load_block(first_block, next);
  for (int kb = first_block; kb < range_hi; kb += 32) {
    KeyBlock block = next;
    if (kb + 32 < range_hi) load_block(kb + 32, next);     // in flight while this block is worked on
    // ---- S^T = K . Q^T for 2 x 16 keys -------------------------------------------------------
    floatx4 s[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      s[t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        s[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(block.k[t][ks].v, qreg[ks].v, s[t], 0, 0, 0);
    }
    // ---- mask, scale, running softmax: s[t][j] is key kb + t*16 + grp*4 + j of column `col` ------
    float block_max = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int key = kb + t * 16 + grp * 4 + j;
        const bool ok = key >= range_lo && key < range_hi && key <= pos_col && key >= lo_col;
        s[t][j] = ok ? s[t][j] * scale : -INFINITY;
        block_max = fmaxf(block_max, s[t][j]);
      }
    block_max = fmaxf(block_max, __shfl_xor(block_max, 16, 64));
    block_max = fmaxf(block_max, __shfl_xor(block_max, 32, 64));
    const float new_max = fmaxf(running_max, block_max);
    float alpha = 1.f, block_sum = 0.f;
    Pack8 p;
    if (new_max == -INFINITY) {
      p.u = make_uint4(0, 0, 0, 0);                    // nothing visible to this column yet
    } else {
      alpha = expf(running_max - new_max);             // 0 while running_max is -inf
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float e = expf(s[t][j] - new_max);     // 0 for masked keys
          block_sum += e;
          p.e[t * 4 + j] = float_to_bf16_bits(e);
        }
    }
    block_sum += __shfl_xor(block_sum, 16, 64);
    block_sum += __shfl_xor(block_sum, 32, 64);
    running_sum = running_sum * alpha + block_sum;
    running_max = new_max;

    // ---- O^T = O^T * alpha + V^T . P^T ---------------------------------------------------------
    const bool ragged = kb < range_lo || kb + 32 > range_hi;
    const int key_a = kb + grp * 4, key_b = kb + 16 + grp * 4;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      Pack8 a;
      a.h[0] = block.v[dt][0];
      a.h[1] = block.v[dt][1];
      if (ragged) {
        // rows outside the range may hold anything (another request's values, or none ever
        // written): zero them, so that 0 * NaN cannot arise
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (key_a + i < range_lo || key_a + i >= range_hi) a.e[i] = 0;
          if (key_b + i < range_lo || key_b + i >= range_hi) a.e[4 + i] = 0;
        }
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) o[dt][j] *= alpha;
      o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, p.v, o[dt], 0, 0, 0);
    }
  }

  // o[dt][j] is dim dt*16 + grp*4 + j of column `col`
  if (!valid_col) return;
  if (nsplit == 1) {
    const float inv = 1.f / running_sum;
    uint16_t* o_row = out + (static_cast<size_t>(tok) * nq + head) * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      uint2 packed;
      packed.x = static_cast<uint32_t>(__bfloat16_as_ushort(__float2bfloat16(o[dt][0] * inv))) |
                 (static_cast<uint32_t>(__bfloat16_as_ushort(__float2bfloat16(o[dt][1] * inv))) << 16);
      packed.y = static_cast<uint32_t>(__bfloat16_as_ushort(__float2bfloat16(o[dt][2] * inv))) |
                 (static_cast<uint32_t>(__bfloat16_as_ushort(__float2bfloat16(o[dt][3] * inv))) << 16);
      *reinterpret_cast<uint2*>(o_row + dt * 16 + grp * 4) = packed;
    }
  } else {
    const size_t slot = (static_cast<size_t>(tok) * nq + head) * nsplit + split;
    float* po = part_o + slot * D;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
      *reinterpret_cast<float4*>(po + dt * 16 + grp * 4) = make_float4(o[dt][0], o[dt][1], o[dt][2], o[dt][3]);
    if (grp == 0) {
      part_ml[slot * 2] = running_max;
      part_ml[slot * 2 + 1] = running_sum;
    }
  }
}

// out[t][h][:] = sum_p w_p O_p / sum_p w_p l_p with w_p = exp(m_p - max m).  One wave per (token, head);
// the weights are formed once, by the lanes, and kept in LDS.
__global__ void __launch_bounds__(64)
attention_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                       uint16_t* __restrict__ out, int nsplit, int d) {
  extern __shared__ float weight[];                  // nsplit
  const size_t row = blockIdx.x;                     // token * nq + head
  const float* ml = part_ml + row * nsplit * 2;
  const int lane = threadIdx.x;
  float top = -INFINITY;
  for (int p = lane; p < nsplit; p += 64) top = fmaxf(top, ml[p * 2]);
  top = wave_max(top);
  float total = 0.f;
  for (int p = lane; p < nsplit; p += 64) {
    const float m = ml[p * 2];
    const float w = m == -INFINITY ? 0.f : expf(m - top);
    weight[p] = w;
    total += w * ml[p * 2 + 1];
  }
  total = wave_sum(total);
  __syncthreads();
  const float inv = 1.f / total;
  for (int i = lane; i < d; i += 64) {
    const float* column = part_o + row * nsplit * d + i;
    float a = 0.f, b = 0.f;
    int p = 0;
    for (; p + 1 < nsplit; p += 2) {
      a += weight[p] * column[static_cast<size_t>(p) * d];
      b += weight[p + 1] * column[static_cast<size_t>(p + 1) * d];
    }
    if (p < nsplit) a += weight[p] * column[static_cast<size_t>(p) * d];
    out[row * d + i] = __bfloat16_as_ushort(__float2bfloat16((a + b) * inv));
  }
}

template <int DT>
static int launch_attention(const void* q, const void* cache, const int* block_table, int max_blocks, const void* tiles,
                            int num_tiles, const int* positions, void* out, float* part_o, float* part_ml, int nsplit,
                            int split_len, int nq, int nkv, int page_size, int window, float scale, hipStream_t stream) {
  hipLaunchKernelGGL(attention_mfma_kernel<DT>, dim3(num_tiles, nkv, nsplit), dim3(64), 0, stream, (const uint16_t*)q,
                     (const uint16_t*)cache, block_table, max_blocks, (const int4*)tiles, positions, (uint16_t*)out, part_o,
                     part_ml, nsplit, split_len, nq, nkv, page_size, window, scale);
  return launch_status();
}

}  // namespace tlie

using namespace tlie;

// q, out: bfloat16 [tokens, nq, d]; cache: bfloat16 [pages, 2, nkv, page_size * d] (keys [row][dim], values [dim][row]).
// tiles: int32 [num_tiles, 4], or null for a decode step (then num_tiles = tokens * ceil(G / 16)).
// part_o: float [tokens * nq * nsplit * d], part_ml: float [tokens * nq * nsplit * 2] (both only when nsplit > 1);
// split_len: positions per part, a multiple of 32, nsplit * split_len >= the longest sequence.
// d % 16 == 0, d <= 256, page_size % 4 == 0.
extern "C" int tlie_attention_mfma(const void* q, const void* cache, const int* block_table, int max_blocks,
                                   const void* tiles, int num_tiles, const int* positions, void* out, float* part_o,
                                   float* part_ml, int nsplit, int split_len, int tokens, int nq, int nkv, int d,
                                   int page_size, int window, float scale, void* stream) {
  if (num_tiles <= 0 || tokens <= 0 || nq <= 0 || nkv <= 0 || nq % nkv != 0 || d <= 0 || d > 256 || d % 16 != 0 ||
      page_size < 4 || page_size % 4 != 0 || max_blocks <= 0 || nsplit < 1 || nsplit > 65535 || nkv > 65535)
    return kBadArgument;
  if (nsplit > 1 && (part_o == nullptr || part_ml == nullptr || split_len <= 0 || split_len % 32 != 0)) return kBadArgument;
  if (tiles == nullptr && num_tiles != tokens * ((nq / nkv + 15) / 16)) return kBadArgument;
  hipStream_t s = (hipStream_t)stream;
  int status = kBadArgument;
#define TLIE_CASE(DT)                                                                                                  \
  case DT:                                                                                                             \
    status = launch_attention<DT>(q, cache, block_table, max_blocks, tiles, num_tiles, positions, out, part_o, part_ml, \
                                  nsplit, split_len, nq, nkv, page_size, window, scale, s);                            \
    break;
  switch (d / 16) {
    TLIE_CASE(1) TLIE_CASE(2) TLIE_CASE(3) TLIE_CASE(4) TLIE_CASE(5) TLIE_CASE(6) TLIE_CASE(7) TLIE_CASE(8)
    TLIE_CASE(9) TLIE_CASE(10) TLIE_CASE(11) TLIE_CASE(12) TLIE_CASE(13) TLIE_CASE(14) TLIE_CASE(15) TLIE_CASE(16)
  }
#undef TLIE_CASE
  if (status != kOk || nsplit == 1) return status;
  hipLaunchKernelGGL(attention_merge_kernel, dim3(tokens * nq), dim3(64), nsplit * sizeof(float), s, part_o, part_ml,
                     (uint16_t*)out, nsplit, d);
  return launch_status();
}
