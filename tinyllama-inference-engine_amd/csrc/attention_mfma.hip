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
//    consecutive keys of one dim, is one 8-byte load.  Pages hold at least 16 rows, so the 16 keys
//    of half a block share a page: page numbers are scalar loads and a lane's addresses are a
//    scalar base plus a constant.
//  * Keys are walked in blocks of 32 that start at multiples of 32 from position 0, with a running
//    maximum and sum: the context length is unbounded and the order of the sums for a (sequence,
//    position) does not depend on how the step was cut.
//  * A decode step of few sequences has few tiles, so the keys of a tile are shared out.  First
//    among the waves of a workgroup (up to 16): wave w takes the blocks w, w + W, ... and the
//    waves' results are merged through LDS, so the kernel still writes final results.  Then, for
//    long contexts, among nsplit workgroups of split_len positions each, which write unnormalised
//    partial results with their maxima and sums for a second kernel to merge.  The parts are fixed ranges of positions, so a wave can fetch its first keys
//    before it knows how long the sequence is: the position, the block table and the keys are not
//    three loads in a row.
#include "common.h"
#include "no_alloc.h"

#include <mutex>
#include <type_traits>

namespace tlie {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;


union Pack8 {
  uint4 u;
  uint2 h[2];
  uint32_t w[4];
  uint16_t e[8];
  bf16x8 v;
};

// Reductions over the four lane groups of a column (lanes l, l ^ 16, l ^ 32, l ^ 48) with the
// gfx950 row and half swaps: v_permlane16_swap exchanges the odd 16-lane rows of one operand with
// the even rows of the other, v_permlane32_swap the upper half with the lower; with both operands
// the same value, the two results hold a lane's own value and its partner's.
typedef __attribute__((__vector_size__(2 * sizeof(unsigned)))) unsigned uintx2;
__device__ __forceinline__ float groups_max(float v) {
  uintx2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
  r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float groups_sum(float v) {
  uintx2 r = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(r[0]) + __uint_as_float(r[1]);
  r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// The larger of two scores (no NaN, none above 3e38) as the median of them and 3e38: one
// instruction, where fmaxf first makes sure that its operands are no signalling NaNs (an
// instruction each for values that come from the matrix cores).
__device__ __forceinline__ float larger(float a, float b) { return __builtin_amdgcn_fmed3f(a, b, 3.0e38f); }

// tiles[i] = (sequence row of the block table, index of the sequence's first token in this step,
//             number of its tokens in this step, first column of the tile)
// column c of a sequence = (token c / G of its tokens in this step, head c % G of the group).
// tiles == nullptr: a decode step, token i is the one token of sequence i; the tile index is
// sequence * ceil(G / 16) + tile of the group.
// DT = head_dim / 16.  CT = groups of 16 columns per wave: a tile has 16 * CT columns, and every
// key and value the wave loads serves all of them (prompt portions take CT = 1 or 2, decode steps 1;
// 4 fit the registers for head sizes up to 64 and measured slower).
// A workgroup has at most 8 waves, and at most 1024 / (16 * CT * DT): their merge fits LDS, and
// every wave may use 256 registers;
// head sizes above 128 need more registers still and get 4 waves at most.
constexpr int attention_max_waves(int dt, int ct) {
  const int fit = 1024 / (16 * ct * dt), cap = dt * ct > 8 ? 4 : 8;
  return fit > cap ? cap : (fit < 1 ? 1 : fit);
}

// SHARED: the waves of a workgroup do not share a tile's keys but take 16 * CT columns each of a
// tile of 16 * CT * waves columns, and every block of keys and values is brought once, through LDS,
// for all of them (prompt portions: the tiles of neighbouring tokens read the same keys, and read
// each on its own they are bound by the L2's bandwidth, not by their arithmetic).  These kernels
// wait more than they compute (a block's chain of loads, products, maxima and exponentials is
// longer than what a wave can issue meanwhile), so for head sizes up to 64 the compiler is asked to
// stay within the registers of 4 waves a SIMD with one column group and 3 with two, where it would
// take those of 3 and 2 (a prompt of 2048 tokens 53 -> 51 us, of 4096 158 -> 150).
template <int DT, int CT, bool SHARED>
__global__ void __launch_bounds__(SHARED ? 512 : 64 * attention_max_waves(DT, CT), (SHARED && DT <= 4) ? (CT == 1 ? 4 : 3) : 1)
attention_mfma_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ cache,
                      const int* __restrict__ block_table, int max_blocks, const int4* __restrict__ tiles,
                      const int* __restrict__ positions, uint16_t* __restrict__ out, float* __restrict__ part_o,
                      float* __restrict__ part_ml, int nsplit, int split_len, int nq, int nkv, int page_size,
                      int window, float scale_log2, int round_size) {
  constexpr int D = DT * 16;
  constexpr int KS = (DT + 1) / 2;                 // 32-wide k steps of the first product
  const int lane = threadIdx.x & 63, col = lane & 15, grp = lane >> 4;
  const int wave = threadIdx.x >> 6, waves = blockDim.x >> 6;     // waves that share the tile's keys
  // Which (tile, kv head) this workgroup takes.  The tiles come sorted, longest first, and all kv
  // heads of a tile are equally long.  Workgroups start in the order of their index, one round of
  // round_size (the number of CUs) after the other; the rounds run through the sorted list forwards
  // and backwards in turn, so that a CU that got a long tile in one round gets a short one in the
  // next: when the whole grid is resident at once (a prompt of a few thousand tokens) the CUs then
  // finish together, where equal partners would leave half of them idle half of the time.
  int tile_index = blockIdx.x, kvh = blockIdx.y;
  if (tiles != nullptr && round_size > 0) {
    const int total = gridDim.x * gridDim.y, linear = blockIdx.y * gridDim.x + blockIdx.x;
    const int round = linear / round_size, place = linear - round * round_size;
    const int in_round = min(round_size, total - round * round_size);
    const int item = round * round_size + ((round & 1) ? in_round - 1 - place : place);
    tile_index = item / static_cast<int>(gridDim.y), kvh = item - tile_index * static_cast<int>(gridDim.y);
  }
  const int split = blockIdx.z;
  // whether a lane's 8 dims of k step ks exist: always, unless the head size is an odd multiple of 16
  auto has_dims = [&](int ks) { return DT % 2 == 0 || ks < KS - 1 || grp < 2; };
  const int G = nq / nkv;
  int seq, tok0, ntok, col0;
  if (tiles != nullptr) {
    const int4 tile = tiles[tile_index];
    seq = tile.x, tok0 = tile.y, ntok = tile.z, col0 = tile.w;
    if (ntok <= 0) return;                       // a list of fixed size ends in tiles without tokens (the same for the whole workgroup)
  } else {
    const int per_seq = (G + 16 * CT - 1) / (16 * CT);
    seq = tok0 = blockIdx.x / per_seq, ntok = 1, col0 = (blockIdx.x % per_seq) * 16 * CT;
  }
  // everything about the tile is the same for all lanes: keep it in scalar registers, so that the
  // conditions on it below are branches of the wave and not masks over its lanes
  seq = __builtin_amdgcn_readfirstlane(seq), tok0 = __builtin_amdgcn_readfirstlane(tok0);
  ntok = __builtin_amdgcn_readfirstlane(ntok), col0 = __builtin_amdgcn_readfirstlane(col0);
  const int pos0 = __builtin_amdgcn_readfirstlane(positions[tok0]);
  const int ncols = ntok * G;
  const int group_col0 = col0;                                   // the workgroup's first column
  if (SHARED) col0 += __builtin_amdgcn_readfirstlane(wave) * 16 * CT;
  const bool wave_active = col0 < ncols;                         // (a shared tile's last waves may have no column)
  bool valid_col[CT];
  int tok[CT], head[CT], pos_col[CT], lo_col[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int c = col0 + ct * 16 + col;
    valid_col[ct] = c < ncols;
    tok[ct] = tok0 + (valid_col[ct] ? c / G : 0);
    head[ct] = kvh * G + (valid_col[ct] ? c % G : 0);
    pos_col[ct] = valid_col[ct] ? pos0 + c / G : -1;
    lo_col[ct] = window > 0 ? max(0, pos_col[ct] - window + 1) : 0;
  }

  // the tile's key range, and this split's part of it
  const int last_col = min(col0 + 16 * CT - 1, ncols - 1);
  const int tile_hi = pos0 + last_col / G + 1;
  const int tile_lo = window > 0 ? max(0, pos0 + col0 / G - window + 1) : 0;
  const int split_lo = nsplit > 1 ? split * split_len : 0;
  const int range_lo = __builtin_amdgcn_readfirstlane(wave_active ? max(tile_lo, split_lo) : 0);
  const int range_hi = __builtin_amdgcn_readfirstlane(wave_active ? (nsplit > 1 ? min(tile_hi, split_lo + split_len) : tile_hi) : 0);

  // Pages hold a power of two of rows, at least 16, and blocks of 32 keys start at multiples of 32:
  // each half of a block (16 keys) lies on one page, the same for every lane.  So the page numbers
  // are scalars, and a lane's addresses are a scalar base plus an offset that never changes.
  const int page_shift = 31 - __clz(page_size), page_mask = page_size - 1;
  const int* pages = block_table + static_cast<size_t>(seq) * max_blocks;
  // For the walk that brings blocks through LDS: the wave keeps 128 consecutive entries of the
  // sequence's block table in two registers, one entry a lane each, loaded before it walks the
  // blocks they cover, and reads page numbers from there, so that a block asked for ahead of its
  // turn does not wait for a page number to come back from memory first.
  int table_first = 0, table_low = 0, table_high = 0;
  auto load_table = [&](int first_index) {
    table_first = first_index;
    table_low = pages[min(first_index + lane, max_blocks - 1)];
    table_high = pages[min(first_index + 64 + lane, max_blocks - 1)];
  };
  auto page_of = [&](int index) -> int {                   // index: the same for every lane, within the window
    const int place = __builtin_amdgcn_readfirstlane(index - table_first);
    const int low = __builtin_amdgcn_readlane(table_low, place & 63);
    const int high = __builtin_amdgcn_readlane(table_high, place & 63);
    return place < 64 ? low : high;                        // (all scalar: a select, not a mask)
  };
  const int table_span = 128 << page_shift;                // keys that one window covers
  const size_t page_stride = static_cast<size_t>(2) * nkv * page_size * D;
  const uint16_t* k_base = cache + static_cast<size_t>(kvh) * page_size * D;
  const uint16_t* v_base = k_base + static_cast<size_t>(nkv) * page_size * D;
  const int k_lane = col * D + grp * 8;                    // operand A of the first product: key `col`, dims grp*8..
  const int v_lane = (col << page_shift) + grp * 4;        // operand A of the second: dim `col`, keys grp*4..

  // Q as operand B: lane (col, grp) holds dims ks*32 + grp*8 .. +8 of its column
  Pack8 qreg[CT][KS];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct)
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int dim = ks * 32 + grp * 8;
      qreg[ct][ks].u = make_uint4(0, 0, 0, 0);
      if (valid_col[ct] && has_dims(ks))
        qreg[ct][ks].u = *reinterpret_cast<const uint4*>(q + (static_cast<size_t>(tok[ct]) * nq + head[ct]) * D + dim);
    }

  // The softmax runs in base 2: scores are scaled by scale * log2(e) and exponentiated with exp2
  // (one instruction); the result is the same function of the scores.
  float running_max[CT], running_sum[CT];
  floatx4 o[CT][DT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    running_max[ct] = -INFINITY, running_sum[ct] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[ct][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  }

  // A block of 32 keys in registers: operand A of the first product (2 halves of 16 keys) and of
  // the second (per 16 dims, 2 x 4 consecutive keys).  Rows outside the range are read all the
  // same, from whatever page the block table names there (absent entries name page 0; past the
  // table, its last entry), and masked or zeroed when used; so the addresses do not depend on the
  // sequence's length and a block can be fetched before its turn.
  struct KeyBlock {
    Pack8 k[2][KS];
    uint2 v[DT][2];
  };
  auto load_block = [&](int kb, KeyBlock& block) {
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int first = kb + t * 16;
      const int page = __builtin_amdgcn_readfirstlane(pages[min(first >> page_shift, max_blocks - 1)]);
      const uint16_t* k_half = k_base + static_cast<size_t>(page) * page_stride + (first & page_mask) * D;
      const uint16_t* v_half = v_base + static_cast<size_t>(page) * page_stride + (first & page_mask);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        block.k[t][ks].u = has_dims(ks) ? *reinterpret_cast<const uint4*>(k_half + k_lane + ks * 32) : make_uint4(0, 0, 0, 0);
      // slot i < 4 of group grp is key kb + grp*4 + i, slot i >= 4 is key kb + 16 + grp*4 + (i - 4)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
        block.v[dt][t] = *reinterpret_cast<const uint2*>(v_half + v_lane + ((dt * 16) << page_shift));
    }
  };

  // masked_tag: whether any key of the block is hidden from any column of the tile (the range's
  // ends, the causal diagonal, the window's edge); the many blocks in between take the other copy
  // of this code, which has no comparisons in it
  auto work_block = [&](int kb, KeyBlock& block, auto masked_tag) {
    constexpr bool kMasked = decltype(masked_tag)::value;
    const bool ragged = kMasked && (kb < range_lo || kb + 32 > range_hi);
    if (ragged) {
      // rows outside the range may hold anything (another request's values, or none ever
      // written): zero them, so that 0 * NaN cannot arise
      const int key_a = kb + grp * 4, key_b = kb + 16 + grp * 4;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        Pack8 a;
        a.h[0] = block.v[dt][0];
        a.h[1] = block.v[dt][1];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (key_a + i < range_lo || key_a + i >= range_hi) a.e[i] = 0;
          if (key_b + i < range_lo || key_b + i >= range_hi) a.e[4 + i] = 0;
        }
        block.v[dt][0] = a.h[0];
        block.v[dt][1] = a.h[1];
      }
    }
    // The steps below run over all the wave's column groups one step at a time, not one group at
    // a time: the groups do not depend on each other, and a wave issues in order.
    // ---- S^T = K . Q^T for 2 x 16 keys ---------------------------------------------------------
    floatx4 s[CT][2];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        s[ct][t] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
          s[ct][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(block.k[t][ks].v, qreg[ct][ks].v, s[ct][t], 0, 0, 0);
      }
    // ---- mask; each lane's maximum over its 8 keys of a column (the scale goes into the exponent's
    // multiply-add): s[ct][t][j] is key kb + t*16 + grp*4 + j of the column -------------------------
    float lane_max[CT];
    bool exceeds = false;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      if (kMasked) {
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int key = kb + t * 16 + grp * 4 + j;
            const bool ok = key >= range_lo && key < range_hi && key <= pos_col[ct] && key >= lo_col[ct];
            s[ct][t][j] = ok ? s[ct][t][j] : -INFINITY;
          }
      }
      lane_max[ct] = larger(larger(larger(s[ct][0][0], s[ct][0][1]), larger(s[ct][0][2], s[ct][0][3])),
                            larger(larger(s[ct][1][0], s[ct][1][1]), larger(s[ct][1][2], s[ct][1][3]))) * scale_log2;   // the scale is positive
      exceeds = exceeds || lane_max[ct] > running_max[ct];
    }
    // ---- running softmax.  The running maximum of a column is shared by its four lane groups, and
    // moves only when a block holds a larger score: rare once the first blocks have passed, so the
    // reduction across the groups, and the rescaling of what has been summed so far, sit behind a
    // branch of the whole wave.  Each group keeps the sum of its own keys; the groups' sums are
    // added once, after the last block. ---------------------------------------------------------
    if (__builtin_amdgcn_ballot_w64(exceeds) != 0) {
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) {
        const float new_max = fmaxf(running_max[ct], groups_max(lane_max[ct]));
        const float alpha = new_max == -INFINITY ? 1.f : __builtin_amdgcn_exp2f(running_max[ct] - new_max);   // 0 while the running maximum is -inf
        running_max[ct] = new_max;
        running_sum[ct] *= alpha;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
          for (int j = 0; j < 4; ++j) o[ct][dt][j] *= alpha;
      }
    }
    Pack8 p[CT];
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      if (kMasked && running_max[ct] == -INFINITY) {
        p[ct].u = make_uint4(0, 0, 0, 0);              // nothing visible to this column yet
      } else {
        float e[8];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int j = 0; j < 4; ++j) e[t * 4 + j] = __builtin_amdgcn_exp2f(fmaf(s[ct][t][j], scale_log2, -running_max[ct]));   // 0 for masked keys
        running_sum[ct] += ((e[0] + e[1]) + (e[2] + e[3])) + ((e[4] + e[5]) + (e[6] + e[7]));
#pragma unroll
        for (int i = 0; i < 4; ++i) p[ct].w[i] = pack_bf16(e[2 * i], e[2 * i + 1]);
      }
    }
    // ---- O^T += V^T . P^T -------------------------------------------------------------------------
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      Pack8 a;
      a.h[0] = block.v[dt][0];
      a.h[1] = block.v[dt][1];
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) o[ct][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, p[ct].v, o[ct][dt], 0, 0, 0);
    }
  };

  // A ring of blocks: while one is worked on, the others are on their way: four with one column
  // group a wave and a head size up to 64 (a decode step lives on the loads it has in flight:
  // inside whole decode steps of the TinyLlama shape four measured 1.5% faster than two at batch
  // 1, 8 and 64), two otherwise, the registers hold no more.  The ring's first loads are made
  // before the sequence's length is known (without a window the first block's place is
  // split_lo & ~31 whatever the position), so some may lie past the range: they are safe (see
  // above) and unused.
  constexpr int NB = (CT == 1 && DT <= 4) ? 4 : 2;
  const int first_block = ((window > 0 ? range_lo : split_lo) & ~31) + 32 * wave;
  const int stride = 32 * waves;
  // a block that every column of the tile sees whole: inside the range, below the first column's
  // position, inside the last column's window
  const int open_lo = __builtin_amdgcn_readfirstlane(max((range_lo + 31) & ~31, window > 0 ? tile_hi - window : 0));
  const int open_hi = __builtin_amdgcn_readfirstlane(min(range_hi, pos0 + col0 / G + 1) & ~31);
  auto work = [&](int kb, KeyBlock& block) {
    if (kb >= open_lo && kb + 32 <= open_hi)
      work_block(kb, block, std::false_type{});
    else
      work_block(kb, block, std::true_type{});
  };
  if constexpr (SHARED) {
    // ---- every block once for the whole workgroup, through LDS ------------------------------------
    // keys as [key][D + 8] (the padding spreads a strip's 16 rows over the banks), values as
    // [dim][32 + 4]; two buffers in turn, so that one barrier a block is enough: a wave writes
    // buffer b of block i + 1 only after the barrier of block i, which every wave reaches only
    // after it has read buffer b for block i - 1.
    constexpr int kKeyStride = D + 8, kValueStride = 36;
    __shared__ __attribute__((aligned(16))) uint16_t lds_k[2][32 * kKeyStride];
    __shared__ __attribute__((aligned(16))) uint16_t lds_v[2][D * kValueStride];
    constexpr int kPieces = 32 * D / 8;                  // 16-byte pieces of a block of keys; of its values as well
    constexpr int kStage = (kPieces + 255) / 256;        // pieces a thread brings (a workgroup has 256 or 512 threads)
    const int group_last = min(group_col0 + 16 * CT * waves - 1, ncols - 1);
    const int group_hi = pos0 + group_last / G + 1;
    const int group_lo = window > 0 ? max(0, pos0 + group_col0 / G - window + 1) : 0;
    const int all_lo = max(group_lo, split_lo);
    const int all_hi = nsplit > 1 ? min(group_hi, split_lo + split_len) : group_hi;
    // Blocks are asked for kAhead blocks before their turn and wait in registers: a workgroup walks
    // its blocks one after the other, and the longest tile's walk is what a prompt step waits for.
    constexpr int kAhead = DT <= 4 ? 4 : 2;                // (larger heads: the registers hold no more)
    typedef uint32_t Piece __attribute__((ext_vector_type(4)));     // a native vector: it stays in registers
    Piece staged_k[kAhead][kStage], staged_v[kAhead][kStage];
    // where a thread's pieces lie within a half block's page rows: fixed for the whole walk, so that a
    // block's addresses are two scalar bases (one per half, from its page numbers) plus these
    int key_place[kStage], value_place[kStage];
    bool key_second[kStage], value_second[kStage];
#pragma unroll
    for (int j = 0; j < kStage; ++j) {
      // (threads beyond the block's pieces load the last piece again and do not store it: a load
      // under a condition would hide from the compiler how many loads are on their way)
      const int piece = min(static_cast<int>(threadIdx.x + j * blockDim.x), kPieces - 1);
      const int key = piece / (D / 8), chunk = piece % (D / 8);
      key_second[j] = key >= 16;
      key_place[j] = (key & 15) * D + chunk * 8;
      const int half = piece / (2 * D), rest = piece % (2 * D), dim = rest >> 1, part = rest & 1;
      value_second[j] = half != 0;
      value_place[j] = (dim << page_shift) + part * 8;
    }
    auto bring = [&](int kb, Piece (&keys)[kStage], Piece (&values)[kStage]) {
      // (a block starts at a multiple of 32 and a page holds at least 16 rows: each half's 16 keys are
      // consecutive rows of one page)
      const size_t page_a = static_cast<size_t>(page_of(kb >> page_shift)) * page_stride;
      const size_t page_b = static_cast<size_t>(page_of((kb + 16) >> page_shift)) * page_stride;
      const int row_a = kb & page_mask, row_b = (kb + 16) & page_mask;
      const uint16_t* keys_a = k_base + page_a + row_a * D;
      const uint16_t* keys_b = k_base + page_b + row_b * D;
      const uint16_t* values_a = v_base + page_a + row_a;
      const uint16_t* values_b = v_base + page_b + row_b;
#pragma unroll
      for (int j = 0; j < kStage; ++j) {
        keys[j] = *reinterpret_cast<const Piece*>((key_second[j] ? keys_b : keys_a) + key_place[j]);
        values[j] = *reinterpret_cast<const Piece*>((value_second[j] ? values_b : values_a) + value_place[j]);
      }
    };
    auto put = [&](int buffer, const Piece (&keys)[kStage], const Piece (&values)[kStage]) {
#pragma unroll
      for (int j = 0; j < kStage; ++j) {
        const int piece = threadIdx.x + j * blockDim.x;
        if (piece < kPieces) {
          const int key = piece / (D / 8), chunk = piece % (D / 8);
          *reinterpret_cast<Piece*>(lds_k[buffer] + key * kKeyStride + chunk * 8) = keys[j];
          const int half = piece / (2 * D), rest = piece % (2 * D), dim = rest >> 1, part = rest & 1;
          uint2* place = reinterpret_cast<uint2*>(lds_v[buffer] + dim * kValueStride + half * 16 + part * 8);
          place[0] = make_uint2(values[j].x, values[j].y);
          place[1] = make_uint2(values[j].z, values[j].w);
        }
      }
    };
    auto take = [&](int buffer, KeyBlock& block) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks)
          block.k[t][ks].u = has_dims(ks) ? *reinterpret_cast<const uint4*>(lds_k[buffer] + (t * 16 + col) * kKeyStride + ks * 32 + grp * 8)
                                          : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
          block.v[dt][t] = *reinterpret_cast<const uint2*>(lds_v[buffer] + (dt * 16 + col) * kValueStride + t * 16 + grp * 4);
      }
    };
    // One turn of the ring, for a place in it that is known when the code is compiled (so that the
    // waiting blocks stay in registers).  Every turn asks for a block and stores one, whether or
    // not a block is left (past the last one it asks for the last one again): the number of loads
    // on their way is then the same on every path, and a turn waits for its own block only.
    auto turn = [&](auto place, int mine, int last) {
      constexpr int j = decltype(place)::value;
      put(j & 1, staged_k[j], staged_v[j]);
      __syncthreads();
      bring(min(mine + 32 * kAhead, last), staged_k[j], staged_v[j]);
      if (mine <= last && mine + 32 > range_lo && mine < range_hi) {
        KeyBlock block;
        take(j & 1, block);
        work(mine, block);
      }
    };
    for (int begin = all_lo & ~31; begin < all_hi; begin += table_span) {
      load_table(begin >> page_shift);
      const int last = (min(all_hi, begin + table_span) - 1) & ~31;      // the window's last block of the range
      bring(begin, staged_k[0], staged_v[0]);
      bring(min(begin + 32, last), staged_k[1], staged_v[1]);
      if constexpr (kAhead == 4) {
        bring(min(begin + 64, last), staged_k[2], staged_v[2]);
        bring(min(begin + 96, last), staged_k[3], staged_v[3]);
      }
      for (int kb = begin; kb <= last; kb += 32 * kAhead) {
        turn(std::integral_constant<int, 0>{}, kb, last);
        turn(std::integral_constant<int, 1>{}, kb + 32, last);
        if constexpr (kAhead == 4) {
          turn(std::integral_constant<int, 2>{}, kb + 64, last);
          turn(std::integral_constant<int, 3>{}, kb + 96, last);
        }
      }
      __syncthreads();                                       // (the next window's first block reuses buffer 0)
    }
  } else {
  KeyBlock ring[NB];
#pragma unroll
  for (int j = 0; j < NB; ++j) load_block(first_block + j * stride, ring[j]);
  for (int kb = first_block; kb < range_hi; kb += NB * stride) {
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const int mine = kb + j * stride;
      if (mine >= range_hi) break;
      work(mine, ring[j]);
      // (a ring of two keeps asking past the range: the unconditional load measured 1.5% faster in
      // prompt steps; a ring of four asks only inside the range, which measured 2% faster in decode steps)
      if (NB == 2 || mine + NB * stride < range_hi) load_block(mine + NB * stride, ring[j]);
    }
  }
  }
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) running_sum[ct] = groups_sum(running_sum[ct]);

  if (!SHARED && waves > 1) {
    // ---- the waves' results into one, through LDS -------------------------------------------------
    extern __shared__ float lds[];
    float* stats = lds;                                  // [waves][CT][16][2]: maximum, sum
    float* slots = lds + waves * CT * 32;                // [waves / 2][CT * DT][64][4]
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
      if (grp == 0) {
        stats[((wave * CT + ct) * 16 + col) * 2] = running_max[ct];
        stats[((wave * CT + ct) * 16 + col) * 2 + 1] = running_sum[ct];
      }
    __syncthreads();
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      float top = -INFINITY;
      for (int w = 0; w < waves; ++w) top = fmaxf(top, stats[((w * CT + ct) * 16 + col) * 2]);
      float total = 0.f;
      for (int w = 0; w < waves; ++w) {
        const float m = stats[((w * CT + ct) * 16 + col) * 2];
        if (m != -INFINITY) total += __builtin_amdgcn_exp2f(m - top) * stats[((w * CT + ct) * 16 + col) * 2 + 1];
      }
      const float mine = running_max[ct] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(running_max[ct] - top);
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int j = 0; j < 4; ++j) o[ct][dt][j] *= mine;
      running_max[ct] = top;
      running_sum[ct] = total;
    }
    // all results are now on the same scale: add them pairwise, the upper half of the waves handing
    // theirs to the lower half, until wave 0 holds the sum
    for (int half = waves >> 1; half >= 1; half >>= 1) {
      __syncthreads();
      if (wave >= half && wave < 2 * half) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
          for (int dt = 0; dt < DT; ++dt)
            *reinterpret_cast<float4*>(slots + (((wave - half) * CT * DT + ct * DT + dt) * 64 + lane) * 4) =
                make_float4(o[ct][dt][0], o[ct][dt][1], o[ct][dt][2], o[ct][dt][3]);
      }
      __syncthreads();
      if (wave < half) {
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) {
            const float4 other = *reinterpret_cast<const float4*>(slots + ((wave * CT * DT + ct * DT + dt) * 64 + lane) * 4);
            o[ct][dt][0] += other.x, o[ct][dt][1] += other.y, o[ct][dt][2] += other.z, o[ct][dt][3] += other.w;
          }
      }
    }
    if (wave != 0) return;
  }

  // o[ct][dt][j] is dim dt*16 + grp*4 + j of the column; maxima and sums are in base 2
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    if (!valid_col[ct]) continue;
    if (nsplit == 1) {
      const float inv = 1.f / running_sum[ct];
      uint16_t* o_row = out + (static_cast<size_t>(tok[ct]) * nq + head[ct]) * D;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        uint2 packed;
        packed.x = static_cast<uint32_t>(__bfloat16_as_ushort(__float2bfloat16(o[ct][dt][0] * inv))) |
                   (static_cast<uint32_t>(__bfloat16_as_ushort(__float2bfloat16(o[ct][dt][1] * inv))) << 16);
        packed.y = static_cast<uint32_t>(__bfloat16_as_ushort(__float2bfloat16(o[ct][dt][2] * inv))) |
                   (static_cast<uint32_t>(__bfloat16_as_ushort(__float2bfloat16(o[ct][dt][3] * inv))) << 16);
        *reinterpret_cast<uint2*>(o_row + dt * 16 + grp * 4) = packed;
      }
    } else {
      const size_t slot = (static_cast<size_t>(tok[ct]) * nq + head[ct]) * nsplit + split;
      float* po = part_o + slot * D;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
        *reinterpret_cast<float4*>(po + dt * 16 + grp * 4) =
            make_float4(o[ct][dt][0], o[ct][dt][1], o[ct][dt][2], o[ct][dt][3]);
      if (grp == 0) {
        part_ml[slot * 2] = running_max[ct];
        part_ml[slot * 2 + 1] = running_sum[ct];
      }
    }
  }
}

// out[t][h][:] = sum_p w_p O_p / sum_p w_p l_p with w_p = 2^(m_p - max m) (the maxima are in base 2).  One wave per (token, head);
// the weights are formed once, by the lanes, and kept in LDS.
__global__ void __launch_bounds__(64)
attention_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                       uint16_t* __restrict__ out, int nsplit, int d) {
  extern __shared__ float weight[];                  // nsplit
  const size_t row = blockIdx.x;                     // token * nq + head
  const float* ml = part_ml + row * nsplit * 2;
  const int lane = threadIdx.x;
  // Up to 16 parts and a head size up to 64 (a lane, a dim): the lane asks for its parts of O together
  // with the maxima and sums, so that the kernel waits for memory once, not twice in a row.
  constexpr int kParts = 16;
  const bool ahead = nsplit <= kParts && d <= 64;
  float early[kParts];
  if (ahead) {
    const float* column = part_o + row * nsplit * d + min(lane, d - 1);
#pragma unroll
    for (int p = 0; p < kParts; ++p)
      if (p < nsplit) early[p] = column[static_cast<size_t>(p) * d];      // (a branch of the whole wave)
  }
  float top = -INFINITY;
  for (int p = lane; p < nsplit; p += 64) top = fmaxf(top, ml[p * 2]);
  top = wave_max(top);
  float total = 0.f;
  for (int p = lane; p < nsplit; p += 64) {
    const float m = ml[p * 2];
    const float w = m == -INFINITY ? 0.f : exp2f(m - top);
    weight[p] = w;
    total += w * ml[p * 2 + 1];
  }
  total = wave_sum(total);
  __syncthreads();
  const float inv = 1.f / total;
  if (ahead) {
    float a = 0.f, b = 0.f;                                // (the same order of additions as below)
#pragma unroll
    for (int p = 0; p < kParts; p += 2) {
      if (p + 1 < nsplit) {
        a += weight[p] * early[p];
        b += weight[p + 1] * early[p + 1];
      } else if (p < nsplit) {
        a += weight[p] * early[p];
      }
    }
    if (lane < d) out[row * d + lane] = __bfloat16_as_ushort(__float2bfloat16((a + b) * inv));
    return;
  }
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

// the number of CUs of the current device (asked once per device)
static int compute_units() {
  static int cached[64] = {};
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return 0;
  if (cached[device] == 0) {
    int count = 0;
    if (hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) return 0;
    cached[device] = count;
  }
  return cached[device];
}

template <int DT, int CT, bool SHARED = false>
static int launch_attention(const void* q, const void* cache, const int* block_table, int max_blocks, const void* tiles,
                            int num_tiles, const int* positions, void* out, float* part_o, float* part_ml, int nsplit,
                            int split_len, int nq, int nkv, int page_size, int window, float scale, int waves,
                            hipStream_t stream) {
  const float scale_log2 = scale * 1.4426950408889634f;
  // LDS for merging the waves: their maxima and sums, and half as many slots as waves for the results
  const size_t lds = !SHARED && waves > 1 ? (static_cast<size_t>(waves) * CT * 32 + static_cast<size_t>(waves / 2) * CT * DT * 256) * sizeof(float) : 0;
  if (lds > 64 * 1024) return kBadArgument;
  hipLaunchKernelGGL((attention_mfma_kernel<DT, CT, SHARED>), dim3(num_tiles, nkv, nsplit), dim3(64 * waves), lds, stream, (const uint16_t*)q,
                     (const uint16_t*)cache, block_table, max_blocks, (const int4*)tiles, positions, (uint16_t*)out, part_o,
                     part_ml, nsplit, split_len, nq, nkv, page_size, window, scale_log2, compute_units());
  return launch_status();
}

}  // namespace tlie

using namespace tlie;

// q, out: bfloat16 [tokens, nq, d]; cache: bfloat16 [pages, 2, nkv, page_size * d] (keys [row][dim], values [dim][row]).
// tiles: int32 [num_tiles, 4] with 16 * col_tiles columns each, or null for a decode step (then
// col_tiles = 1 and num_tiles = tokens * ceil(G / 16)).
// part_o: float [tokens * nq * nsplit * d], part_ml: float [tokens * nq * nsplit * 2] (both only when nsplit > 1);
// split_len: positions per part, a multiple of 32, nsplit * split_len >= the longest sequence.
// d % 16 == 0, d <= 256, page_size a power of two >= 16; col_tiles 1, or 4 for d <= 64, or 2 for d <= 128.
// shared != 0 (prompt portions, col_tiles 1 or 2, d <= 128, 4 or 8 waves): tiles have 16 * col_tiles * waves columns, every wave
// takes 16 * col_tiles of them, and keys and values reach the waves through LDS.  Otherwise:
// waves: 1, 2, 4 or 8 waves of a workgroup share a tile's keys; waves * col_tiles * d <= 1024 (their merge's LDS), and
// at most 4 when col_tiles * d > 128.
static int attention_entry(const void* q, const void* cache, const int* block_table, int max_blocks,
                           const void* tiles, int num_tiles, int col_tiles, const int* positions, void* out,
                           float* part_o, float* part_ml, int nsplit, int split_len, int tokens, int nq, int nkv,
                           int d, int page_size, int window, float scale, int waves, int shared, void* stream) {
  if (num_tiles <= 0 || tokens <= 0 || nq <= 0 || nkv <= 0 || nq % nkv != 0 || d <= 0 || d > 256 || d % 16 != 0 ||
      page_size < 16 || (page_size & (page_size - 1)) != 0 || max_blocks <= 0 || nsplit < 1 || nsplit > 65535 || nkv > 65535)
    return kBadArgument;
  if (nsplit > 1 && (part_o == nullptr || part_ml == nullptr || split_len <= 0 || split_len % 32 != 0)) return kBadArgument;
  if (col_tiles != 1 && !(col_tiles == 4 && d <= 64) && !(col_tiles == 2 && d <= 128)) return kBadArgument;
  if (shared) {
    // the waves take columns of their own: tiles of 16 * col_tiles * waves columns, 4 or 8 waves
    if (tiles == nullptr || (col_tiles != 2 && col_tiles != 1) || d > 128 || (waves != 4 && waves != 8)) return kBadArgument;
  } else if (waves < 1 || (waves & (waves - 1)) != 0 || waves > attention_max_waves(d / 16, col_tiles)) {
    return kBadArgument;
  }
  if (tiles == nullptr && (col_tiles != 1 || num_tiles != tokens * ((nq / nkv + 15) / 16))) return kBadArgument;
  if (!(scale > 0.f)) return kBadArgument;     // the maximum is taken before the scores are scaled
  hipStream_t s = (hipStream_t)stream;
  int status = kBadArgument;
#define TLIE_ARGS q, cache, block_table, max_blocks, tiles, num_tiles, positions, out, part_o, part_ml, nsplit, split_len, nq, \
                  nkv, page_size, window, scale, waves, s
#define TLIE_CASE(DT)                                        \
  case DT:                                                   \
    status = launch_attention<DT, 1>(TLIE_ARGS);             \
    break;
#define TLIE_CASE4(DT)                                       \
  case DT:                                                   \
    status = launch_attention<DT, 4>(TLIE_ARGS);             \
    break;
#define TLIE_CASE2(DT)                                       \
  case DT:                                                   \
    status = launch_attention<DT, 2>(TLIE_ARGS);             \
    break;
#define TLIE_SHARED(DT)                                                              \
  case DT:                                                                           \
    status = col_tiles == 2 ? launch_attention<DT, 2, true>(TLIE_ARGS)               \
                            : launch_attention<DT, 1, true>(TLIE_ARGS);              \
    break;
  if (shared) {
    switch (d / 16) {
      TLIE_SHARED(1) TLIE_SHARED(2) TLIE_SHARED(3) TLIE_SHARED(4) TLIE_SHARED(5) TLIE_SHARED(6) TLIE_SHARED(7) TLIE_SHARED(8)
    }
  } else if (col_tiles == 1) {
    switch (d / 16) {
      TLIE_CASE(1) TLIE_CASE(2) TLIE_CASE(3) TLIE_CASE(4) TLIE_CASE(5) TLIE_CASE(6) TLIE_CASE(7) TLIE_CASE(8)
      TLIE_CASE(9) TLIE_CASE(10) TLIE_CASE(11) TLIE_CASE(12) TLIE_CASE(13) TLIE_CASE(14) TLIE_CASE(15) TLIE_CASE(16)
    }
  } else if (col_tiles == 4) {
    switch (d / 16) { TLIE_CASE4(1) TLIE_CASE4(2) TLIE_CASE4(3) TLIE_CASE4(4) }
  } else {
    switch (d / 16) {
      TLIE_CASE2(1) TLIE_CASE2(2) TLIE_CASE2(3) TLIE_CASE2(4) TLIE_CASE2(5) TLIE_CASE2(6) TLIE_CASE2(7) TLIE_CASE2(8)
    }
  }
#undef TLIE_CASE
#undef TLIE_SHARED
#undef TLIE_CASE2
#undef TLIE_CASE4
#undef TLIE_ARGS
  if (status != kOk || nsplit == 1) return status;
  hipLaunchKernelGGL(attention_merge_kernel, dim3(tokens * nq), dim3(64), nsplit * sizeof(float), s, part_o, part_ml,
                     (uint16_t*)out, nsplit, d);
  return launch_status();
}

extern "C" int tlie_attention_mfma(const void* q, const void* cache, const int* block_table, int max_blocks,
                                   const void* tiles, int num_tiles, int col_tiles, const int* positions, void* out,
                                   float* part_o, float* part_ml, int nsplit, int split_len, int tokens, int nq, int nkv,
                                   int d, int page_size, int window, float scale, int waves, int shared, void* stream) {
  return attention_entry(q, cache, block_table, max_blocks, tiles, num_tiles, col_tiles, positions, out, part_o, part_ml, nsplit,
                         split_len, tokens, nq, nkv, d, page_size, window, scale, waves, shared, stream);
}

// ---- the same attention for callers that cannot allocate (declared and described in no_alloc.h) ----------
// The partial results of the key parts (what `part_o` and `part_ml` bring in above) live in this array, of
// which every GPU the library runs on holds its own copy until the process ends.
static __device__ __align__(256) unsigned char scratch[TLIE_NO_ALLOC_SCRATCH_BYTES];

// In host code the array's name is only a stand-in for the symbol: its device address is asked for once
// per device, with that device current, and kept; kernels are handed that address, never the name.
static void* scratch_address() {
  static std::mutex guard;
  static void* address[64] = {};
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return nullptr;
  std::lock_guard<std::mutex> lock(guard);
  if (address[device] == nullptr) {
    void* found = nullptr;
    if (hipGetSymbolAddress(&found, HIP_SYMBOL(scratch)) != hipSuccess || found == nullptr) {
      (void)hipGetLastError();
      return nullptr;
    }
    address[device] = found;
  }
  return address[device];
}

extern "C" int tlie_attention_mfma_no_alloc(const void* q, const void* cache, const int* block_table, int max_blocks,
                                            const void* tiles, int num_tiles, int col_tiles, const int* positions, void* out,
                                            int nsplit, int split_len, int tokens, int nq, int nkv, int d, int page_size,
                                            int window, float scale, int waves, int shared, void* stream) {
  if (tokens <= 0 || nq <= 0 || d <= 0 || nsplit < 1) return kBadArgument;
  float *part_o = nullptr, *part_ml = nullptr;
  if (nsplit > 1) {
    // [tokens * nq * nsplit] rows of d floats, then as many pairs (maximum, sum), the pairs at a multiple of 256 bytes
    const size_t rows = static_cast<size_t>(tokens) * nq * nsplit;
    const size_t o_bytes = (rows * d * sizeof(float) + 255) / 256 * 256;
    if (o_bytes + rows * 2 * sizeof(float) > TLIE_NO_ALLOC_SCRATCH_BYTES) return kScratchTooSmall;
    unsigned char* base = static_cast<unsigned char*>(scratch_address());
    if (base == nullptr) return kLaunchFailed;
    part_o = reinterpret_cast<float*>(base);
    part_ml = reinterpret_cast<float*>(base + o_bytes);
  }
  return attention_entry(q, cache, block_table, max_blocks, tiles, num_tiles, col_tiles, positions, out, part_o, part_ml, nsplit,
                         split_len, tokens, nq, nkv, d, page_size, window, scale, waves, shared, stream);
}
