// y = x . W^T for at most 16 rows of x (decoding at small batch), bfloat16 on the matrix cores, with
// what stands before and after the product in the layer folded into it, so that a decode step
// needs fewer kernels: the scale of the RMSNorm before it, the bias, and then either the SiLU gate,
// or the add into the residual together with the next norm's inputs.
//
// reference: one token's layer in the reference is 15 launches (2 norms, 7 products, rotation,
// cache write, attention, SiLU, 2 adds; src/cuda/model.cu:406-475).  On this machine a dependent
// launch costs 2 to 3 us even inside a replayed graph, as much as streaming a whole projection
// matrix, so the count of launches decides the speed of decoding.  Finishing a split-K sum across
// workgroups costs about as much (the L2 caches of the chip's eight dies do not see each other's
// lines, so the parts have to travel through memory); here the sum stays inside a workgroup.
//
// A workgroup owns one MFMA strip of W's rows (16, or 8 when W has too few rows to give every CU
// a workgroup) and all of K: its 4, 8 or 16 waves take a part of K each, read W and x straight
// into the MFMA operands (no LDS staging: a wave's part of x is as small as its part of W), and
// add their results up through LDS in a fixed order.  Because the workgroup then holds complete
// sums, the epilogue can finish the layer's arithmetic:
//
//   * row scale: y[m, :] *= rsqrt(ssq[m] / width + eps).  RMSNorm(h) * g . W^T equals
//     r * ((h * g) . W^T) with r the row's scalar, so the product runs on bfloat16(h * g) (stored
//     by the previous epilogue, see below) and r is applied here; ssq[m] is the sum of the partial
//     sums of squares that the previous epilogue left per 16 columns.
//   * store: float32 [M, N] (qkv for the rotation kernel; logits).
//   * SiLU gate: W's rows alternate gate and up (g0, u0, g1, u1, ...); out[m, i] = silu(g) * u,
//     bfloat16 [M, N / 2].
//   * residual: residual[m, n] += y (float32, in place: every element has one owner), and for the
//     norm that reads the residual next: xg[m, n] = bfloat16(residual * g_next[n]) and the partial
//     sums of squares per row and 16 columns.
//   * rotation and cache write, for the fused q/k/v projection: the rows of W are stored so that
//     the two elements of a rotation pair, (i, i + rot_dim / 2) of a head, are neighbours
//     (positions 2i and 2i + 1); a pair then sits in two adjacent lanes, is turned by the token's
//     angle, and goes to q or to the cache row of the token's slot (what rope_cache.hip does as a
//     kernel of its own for longer steps).
#include "common.h"

namespace tlie {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

union RowPack {
  uint4 u;
  bf16x8 v;
};

constexpr int kEpilogueStore = 0, kEpilogueSilu = 1, kEpilogueResidual = 2, kEpilogueRope = 3;

struct RowsArgs {
  const uint16_t* x;          // [M, K] bfloat16
  const uint16_t* w;          // [N, K] bfloat16
  const uint16_t* bias;       // [N] or null
  int M, N, K, k_per_wave;    // k_per_wave: multiple of 64
  int rows_per_block;         // even, up to 16; or 32
  // row scale (null: none)
  const float* ssq_in;        // [strips_in, 16] partial sums of squares of the normed input's rows, over any split of its columns
  int strips_in;
  float inv_width, eps;       // 1 / width of the normed input
  // outputs
  float* y;                   // store: [M, N]
  uint16_t* act;              // SiLU: [M, N / 2]
  float* residual;            // residual: [M, N], updated in place
  const uint16_t* next_weight;  // residual: [N] bfloat16 weight of the next norm, or null
  const float* next_weight_f32; // the same when that weight is kept in float32
  uint16_t* xg;               // residual: [M, N] bfloat16(residual * next weight), or null
  float* ssq_out;             // residual: [ceil(N / rows_per_block), 16], or null
  // rotation and cache write: N = (nq + 2 nkv) * d, heads in the order q | k | v
  const int* positions;       // [M]
  const int* slot_map;        // [M] cache row of each token (page * page_size + row), or -1
  const float* inv_freq;      // [rot_dim / 2], or null: no rotation
  int rot_dim, nq, nkv, d, page_size;
  uint16_t* q_out;            // [M, nq * d]
  uint16_t* cache;            // [pages, 2, nkv, page_size * d]: keys [row][dim], values [dim][row]
};

// S whole steps of 64 k for every strip: all of W's pieces are asked for first (16 bytes a lane and piece;
// with 8 steps 16 loads per lane and strip in flight: the weights come from HBM and a wave has nothing
// else to do meanwhile), then x, which comes from the caches, in halves of up to 4 steps.
// k: the lane's first k of the chunk (lanes of group g take k + 16 g .. + 16 of every step).
// w_lane, x_lane: whether this lane's row of the strip, and its token, exist: the others load nothing (one
// condition around all loads of a kind), multiply what their registers happen to hold, and their results,
// rows and columns of their own, are never stored.
template <int STRIPS, int S>
__device__ __forceinline__ void rows_chunk(const uint16_t* (&w_row)[STRIPS], const uint16_t* x_row, int k,
                                           bool w_lane, bool x_lane, floatx4 (&acc)[STRIPS]) {
  RowPack wa[STRIPS][S][2];
  if (w_lane) {
#pragma unroll
    for (int st = 0; st < STRIPS; ++st)
#pragma unroll
      for (int s = 0; s < S; ++s)
#pragma unroll
        for (int h = 0; h < 2; ++h) wa[st][s][h].u = *reinterpret_cast<const uint4*>(w_row[st] + k + s * 64 + h * 8);
  }
  // (the compiler would rather ask for a few pieces, multiply, and ask for the next: it is told not to move
  // anything across these lines, so that all of the chunk's weights are on their way before the first wait)
  __builtin_amdgcn_sched_barrier(0);
  constexpr int kHalf = S > 4 ? 4 : S;
#pragma unroll
  for (int first = 0; first < S; first += kHalf) {
    RowPack xb[kHalf][2];
    if (x_lane) {
#pragma unroll
      for (int s = 0; s < kHalf; ++s)
#pragma unroll
        for (int h = 0; h < 2; ++h)
          if (first + s < S) xb[s][h].u = *reinterpret_cast<const uint4*>(x_row + k + (first + s) * 64 + h * 8);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int st = 0; st < STRIPS; ++st)
#pragma unroll
      for (int s = 0; s < kHalf; ++s)
        if (first + s < S) {
          acc[st] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[st][first + s][0].v, xb[s][0].v, acc[st], 0, 0, 0);
          acc[st] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[st][first + s][1].v, xb[s][1].v, acc[st], 0, 0, 0);
        }
  }
}

// The last step of a K that is no multiple of 64 (K is one of 8): a lane whose k lies beyond K reads the
// row's last 8 values instead and gets zeros for x.
template <int STRIPS>
__device__ __forceinline__ void rows_last_step(const uint16_t* (&w_row)[STRIPS], const uint16_t* x_row, int k, int k_end,
                                               floatx4 (&acc)[STRIPS]) {
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int kk = k + h * 8, from = min(kk, k_end - 8);
    RowPack xb;
    xb.u = *reinterpret_cast<const uint4*>(x_row + from);
    if (kk >= k_end) xb.u = make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int st = 0; st < STRIPS; ++st) {
      RowPack wa;
      wa.u = *reinterpret_cast<const uint4*>(w_row[st] + from);
      acc[st] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa.v, xb.v, acc[st], 0, 0, 0);
    }
  }
}

// WAVES: 2, 4, 8 or 16 waves share K (more waves for a long K or few strips, fewer when the strips
// alone fill the chip: every wave costs a dispatch).  STRIPS: MFMA strips of 16 rows of W a
// workgroup (2 when W has rows in plenty: each wave's part of x then serves twice the weights).
// With one strip a workgroup the kernel is held to the registers of 4 waves a SIMD (128): a few more, and a
// compute unit holds 3 workgroups of 4 waves where it held 4, which the products with many strips pay for
// (Llama-3-8B's gate/up at batch 1: 57 us against 54).
template <int EPILOGUE, int WAVES, int STRIPS>
__global__ void __launch_bounds__(WAVES * 64, STRIPS == 1 ? 4 : 2)
gemm_rows_kernel(const RowsArgs a) {
  __shared__ float partial[STRIPS][WAVES][64][4];   // each wave's 16 x 16 sums per strip
  __shared__ float scale_part[WAVES * 4][16];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);     // (the same for the wave's lanes: what depends on it alone is scalar)
  const int col = lane & 15, grp = lane >> 4;
  const int block_row = blockIdx.x * a.rows_per_block;
  const int strip_rows = STRIPS == 1 ? a.rows_per_block : 16;                 // with 8 rows a block, half the strip is idle
  const int k_begin = wave * a.k_per_wave, k_end = min(a.K, k_begin + a.k_per_wave);
  // (a row beyond the matrix, in its last strip, becomes the last row: read again, never stored)
  const uint16_t* w_row[STRIPS];
#pragma unroll
  for (int st = 0; st < STRIPS; ++st)
    w_row[st] = a.w + static_cast<size_t>(min(block_row + st * 16 + col, a.N - 1)) * a.K;
  const uint16_t* x_row = a.x + static_cast<size_t>(min(col, a.M - 1)) * a.K;
  const bool w_lane = col < strip_rows, x_lane = col < a.M;

  // the norm's partial sums of squares are asked for before the weights, and added up after the
  // products: their way from the L2 is hidden behind the weights' way from memory
  // (the (wave, group) pairs share the strips of the previous product; token = col)
  constexpr int kScaleLoads = 4;
  float scale_value[kScaleLoads];
  const int part = wave * 4 + grp;
  if (a.ssq_in != nullptr) {
#pragma unroll
    for (int i = 0; i < kScaleLoads; ++i) {
      const int s = part + i * WAVES * 4;
      scale_value[i] = s < a.strips_in ? a.ssq_in[s * 16 + col] : 0.f;
    }
  }

  // What the epilogue needs besides the sums is asked for now as well, for the same reason: each
  // thread knows its outputs (token = t / 16, row = t % 16 of a strip; see below) from the start.
  constexpr int kTurns = (256 + WAVES * 64 - 1) / (WAVES * 64);     // outputs of a strip per thread
  float pre_bias[STRIPS][kTurns], pre_old[STRIPS][kTurns], pre_g[STRIPS][kTurns];
  float pre_sine[STRIPS][kTurns], pre_cosine[STRIPS][kTurns];
  int pre_slot[STRIPS][kTurns];
#pragma unroll
  for (int st = 0; st < STRIPS; ++st)
#pragma unroll
    for (int turn = 0; turn < kTurns; ++turn) {
      const int t = threadIdx.x + turn * WAVES * 64;
      const int token = t >> 4, nn = t & 15, n = block_row + st * 16 + nn;
      const bool live = t < 256 && token < a.M && nn < strip_rows && n < a.N;
      pre_bias[st][turn] = live && a.bias != nullptr ? bf16_bits_to_float(a.bias[n]) : 0.f;
      pre_old[st][turn] = pre_g[st][turn] = pre_sine[st][turn] = 0.f;
      pre_cosine[st][turn] = 1.f;
      pre_slot[st][turn] = -1;
      if (EPILOGUE == kEpilogueResidual && live) {
        pre_old[st][turn] = a.residual[static_cast<size_t>(token) * a.N + n];
        if (a.xg != nullptr) pre_g[st][turn] = a.next_weight != nullptr ? bf16_bits_to_float(a.next_weight[n]) : a.next_weight_f32[n];
      }
      if (EPILOGUE == kEpilogueRope && live) {
        const int head = n / a.d, p = n % a.d;
        if (a.inv_freq != nullptr && head < a.nq + a.nkv && p < a.rot_dim)
          sincosf(static_cast<float>(a.positions[token]) * a.inv_freq[p >> 1], &pre_sine[st][turn], &pre_cosine[st][turn]);
        if (head >= a.nq) pre_slot[st][turn] = a.slot_map[token];
      }
    }

  floatx4 acc[STRIPS];
#pragma unroll
  for (int st = 0; st < STRIPS; ++st) acc[st] = floatx4{0.f, 0.f, 0.f, 0.f};
  // No load stands under a lane's condition (such a load costs a dozen instructions around it, and a wave
  // issues 24 in a row here): the wave's part of K is taken in chunks of up to 8 whole steps of 64, each
  // chunk straight-line code for its number of steps, which is the same for all lanes; a K that is no
  // multiple of 64 ends in a step of its own.
  for (int k0 = k_begin; k0 < k_end; k0 += 512) {
    const int steps = min(8, (k_end - k0) >> 6);
    const int k = k0 + grp * 16;
    switch (steps) {
      case 8: rows_chunk<STRIPS, 8>(w_row, x_row, k, w_lane, x_lane, acc); break;
      case 7: rows_chunk<STRIPS, 7>(w_row, x_row, k, w_lane, x_lane, acc); break;
      case 6: rows_chunk<STRIPS, 6>(w_row, x_row, k, w_lane, x_lane, acc); break;
      case 5: rows_chunk<STRIPS, 5>(w_row, x_row, k, w_lane, x_lane, acc); break;
      case 4: rows_chunk<STRIPS, 4>(w_row, x_row, k, w_lane, x_lane, acc); break;
      case 3: rows_chunk<STRIPS, 3>(w_row, x_row, k, w_lane, x_lane, acc); break;
      case 2: rows_chunk<STRIPS, 2>(w_row, x_row, k, w_lane, x_lane, acc); break;
      case 1: rows_chunk<STRIPS, 1>(w_row, x_row, k, w_lane, x_lane, acc); break;
      default: break;
    }
    if (steps < 8 && k0 + steps * 64 < k_end) rows_last_step<STRIPS>(w_row, x_row, k + steps * 64, k_end, acc);
  }
  // acc[st][j] = sum over this wave's k of W[block_row + st*16 + grp*4 + j][k] * x[col][k]
#pragma unroll
  for (int st = 0; st < STRIPS; ++st)
#pragma unroll
    for (int j = 0; j < 4; ++j) partial[st][wave][lane][j] = acc[st][j];
  if (a.ssq_in != nullptr) {
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < kScaleLoads; ++i) sum += scale_value[i];
    for (int s = part + kScaleLoads * WAVES * 4; s < a.strips_in; s += WAVES * 4) sum += a.ssq_in[s * 16 + col];
    scale_part[part][col] = sum;
  }
  __syncthreads();

  // one thread per output of a strip: token = t / 16, row = t % 16, so a token's outputs sit in
  // 16 consecutive lanes; the 256 outputs of each strip go round the workgroup's threads (whole
  // waves at a time: 256 is a multiple of 64)
#pragma unroll
  for (int st = 0; st < STRIPS; ++st)
#pragma unroll
    for (int turn = 0; turn < kTurns; ++turn) {
      const int t = threadIdx.x + turn * WAVES * 64;
      if (t >= 256) break;                                   // the same for a whole wave
      const int token = t >> 4, nn = t & 15, n = block_row + st * 16 + nn;
      const int from_lane = (nn >> 2) * 16 + token, from_j = nn & 3;    // where the MFMA left this output
      float value = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) value += partial[st][w][from_lane][from_j];
      if (a.ssq_in != nullptr) {
        float ssq = 0.f;
#pragma unroll
        for (int p = 0; p < WAVES * 4; ++p) ssq += scale_part[p][token];
        value *= rsqrtf(ssq * a.inv_width + a.eps);
      }
      const bool live = token < a.M && nn < strip_rows && n < a.N;
      value += pre_bias[st][turn];

      if (EPILOGUE == kEpilogueStore) {
        if (live) a.y[static_cast<size_t>(token) * a.N + n] = value;
      } else if (EPILOGUE == kEpilogueSilu) {
        const float up = __shfl_down(value, 1, 64);          // the odd row next to this even one
        if (live && (nn & 1) == 0) {
          const float gated = (value / (1.f + expf(-value))) * up;
          a.act[static_cast<size_t>(token) * (a.N / 2) + (n >> 1)] = __bfloat16_as_ushort(__float2bfloat16(gated));
        }
      } else if (EPILOGUE == kEpilogueRope) {
        const float other = __shfl_xor(value, 1, 64);        // the pair's other element, when this one is rotated
        if (live) {
          const int head = n / a.d, p = n % a.d;
          float result = value;
          int e = p;
          if (a.inv_freq != nullptr && head < a.nq + a.nkv && p < a.rot_dim) {
            const int i = p >> 1, half = a.rot_dim >> 1;
            const float sine = pre_sine[st][turn], cosine = pre_cosine[st][turn];
            if (p & 1) {
              e = i + half;
              result = value * cosine + other * sine;        // second' = second cos + first sin
            } else {
              e = i;
              result = value * cosine - other * sine;        // first' = first cos - second sin
            }
          }
          const uint16_t bits = __bfloat16_as_ushort(__float2bfloat16(result));
          if (head < a.nq) {
            a.q_out[(static_cast<size_t>(token) * a.nq + head) * a.d + e] = bits;
          } else {
            const int slot = pre_slot[st][turn];
            if (slot >= 0) {
              const size_t head_stride = static_cast<size_t>(a.page_size) * a.d;
              uint16_t* page = a.cache + static_cast<size_t>(slot / a.page_size) * 2 * a.nkv * head_stride;
              const int row = slot % a.page_size;
              if (head < a.nq + a.nkv)
                page[(head - a.nq) * head_stride + static_cast<size_t>(row) * a.d + e] = bits;
              else
                page[(head - a.nq) * head_stride + static_cast<size_t>(e) * a.page_size + row] = bits;
            }
          }
        }
      } else {
        float updated = 0.f;
        if (live) {
          updated = pre_old[st][turn] + value;
          a.residual[static_cast<size_t>(token) * a.N + n] = updated;
          if (a.xg != nullptr)
            a.xg[static_cast<size_t>(token) * a.N + n] = __bfloat16_as_ushort(__float2bfloat16(updated * pre_g[st][turn]));
        }
        if (a.ssq_out != nullptr) {
          float square = updated * updated;
          square += __shfl_xor(square, 1, 64);
          square += __shfl_xor(square, 2, 64);
          square += __shfl_xor(square, 4, 64);
          square += __shfl_xor(square, 8, 64);
          // one row of partial sums per strip of each block of W's rows
          if (nn == 0) a.ssq_out[(blockIdx.x * STRIPS + st) * 16 + token] = square;
        }
      }
    }
}

// residual[t, :] = table[token[t], :] as float; and for the first norm, as the residual epilogue
// above leaves them: xg = bfloat16(residual * g), partial sums of squares per 16 columns.
template <typename W, typename G>
__global__ void embed_rows_kernel(const int* __restrict__ tokens, const W* __restrict__ table,
                                  float* __restrict__ residual, const G* __restrict__ next_weight,
                                  uint16_t* __restrict__ xg, float* __restrict__ ssq_out, int hidden) {
  const int t = blockIdx.x;
  const W* row = table + static_cast<size_t>(tokens[t]) * hidden;
  for (int base = 0; base < hidden; base += blockDim.x) {
    const int i = base + threadIdx.x;
    float value = 0.f;
    if (i < hidden) {
      value = to_float(row[i]);
      residual[static_cast<size_t>(t) * hidden + i] = value;
      xg[static_cast<size_t>(t) * hidden + i] = __bfloat16_as_ushort(__float2bfloat16(value * to_float(next_weight[i])));
    }
    float square = value * value;
    square += __shfl_xor(square, 1, 64);
    square += __shfl_xor(square, 2, 64);
    square += __shfl_xor(square, 4, 64);
    square += __shfl_xor(square, 8, 64);
    if ((threadIdx.x & 15) == 0 && i < hidden) ssq_out[(i >> 4) * 16 + t] = square;
  }
}

// The same with four elements a thread and blocks side by side over the row (hidden % 4 == 0):
// grid (tokens, ceil(hidden / (4 * blockDim.x))).
template <typename W, typename G>
__global__ void embed_rows_wide_kernel(const int* __restrict__ tokens, const W* __restrict__ table,
                                       float* __restrict__ residual, const G* __restrict__ next_weight,
                                       uint16_t* __restrict__ xg, float* __restrict__ ssq_out, int hidden) {
  const int t = blockIdx.x;
  const int i = (blockIdx.y * blockDim.x + threadIdx.x) * 4;
  const bool live = i < hidden;
  float v[4] = {0.f, 0.f, 0.f, 0.f}, g[4] = {0.f, 0.f, 0.f, 0.f};
  if (live) {
    const W* row = table + static_cast<size_t>(tokens[t]) * hidden + i;
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = to_float(row[j]), g[j] = to_float(next_weight[i + j]);   // adjacent: the compiler joins the loads
    store4(residual + static_cast<size_t>(t) * hidden + i, v[0], v[1], v[2], v[3]);
    store4(reinterpret_cast<bf16*>(xg) + static_cast<size_t>(t) * hidden + i, v[0] * g[0], v[1] * g[1], v[2] * g[2], v[3] * g[3]);
  }
  float square = (v[0] * v[0] + v[1] * v[1]) + (v[2] * v[2] + v[3] * v[3]);
  square += __shfl_xor(square, 1, 64);
  square += __shfl_xor(square, 2, 64);
  if ((threadIdx.x & 3) == 0 && live) ssq_out[(i >> 4) * 16 + t] = square;
}

}  // namespace tlie

using namespace tlie;

// x [M, K], w [N, K], bias [N] or null: bfloat16; M <= 16, K % 8 == 0.
// ssq_in [strips_in, 16] or null (then no row scale); width: the normed input's width.
// epilogue 0: y float [M, N].  1: act bfloat16 [M, N / 2], N even, W's rows alternating gate, up.
// 2: residual float [M, N] += y; if xg is given, next_weight [N] (bfloat16 if next_weight_dtype is 1,
// else float) and xg bfloat16 [M, N]; if ssq_out is given, float [ceil(N / rows_per_block) * max(1, rows_per_block / 16), 16]
// (all of it is written).
// waves: 2, 4, 8 or 16, how many waves of a workgroup share K.  rows_per_block: an even number up to 16 (the rest of the
// strip of 16 is idle), or 32 (two strips, with at most 8 waves).
// 3: the rotation and cache write of rope_cache.hip on W's rows in paired order (see above): positions, slot_map [M],
// inv_freq [rot_dim / 2] or null, q_out bfloat16 [M, nq * d], cache bfloat16 [pages, 2, nkv, page_size * d];
// N = (nq + 2 nkv) * d.
extern "C" int tlie_gemm_rows(const void* x, const void* w, const void* bias, int M, int N, int K, const float* ssq_in,
                              int strips_in, int width, float eps, int epilogue, float* y, void* act, float* residual,
                              const void* next_weight, int next_weight_dtype, void* xg, float* ssq_out,
                              const int* positions, const int* slot_map, const float* inv_freq, int rot_dim, int nq,
                              int nkv, int d, int page_size, void* q_out, void* cache, int waves, int rows_per_block,
                              void* stream) {
  if (M <= 0 || M > 16 || N <= 0 || K <= 0 || (K & 7) != 0 || (waves != 2 && waves != 4 && waves != 8 && waves != 16)) return kBadArgument;
  if (!(rows_per_block >= 2 && rows_per_block <= 16 && rows_per_block % 2 == 0) && !(rows_per_block == 32 && waves <= 8)) return kBadArgument;
  if (ssq_in != nullptr && (strips_in <= 0 || width <= 0)) return kBadArgument;
  if (epilogue == kEpilogueStore && y == nullptr) return kBadArgument;
  if (epilogue == kEpilogueSilu && (act == nullptr || (N & 1) != 0)) return kBadArgument;
  if (epilogue == kEpilogueResidual && (residual == nullptr || (xg != nullptr && next_weight == nullptr))) return kBadArgument;
  if (epilogue == kEpilogueRope &&
      (positions == nullptr || slot_map == nullptr || q_out == nullptr || cache == nullptr || nq <= 0 || nkv <= 0 || d <= 0 ||
       page_size <= 0 || N != (nq + 2 * nkv) * d || rot_dim < 0 || rot_dim > d || (rot_dim & 1) != 0 || (d & 1) != 0))
    return kBadArgument;
  RowsArgs a;
  a.x = (const uint16_t*)x, a.w = (const uint16_t*)w, a.bias = (const uint16_t*)bias;
  a.M = M, a.N = N, a.K = K, a.rows_per_block = rows_per_block;
  a.k_per_wave = ((K + waves - 1) / waves + 63) / 64 * 64;
  a.ssq_in = ssq_in, a.strips_in = strips_in, a.inv_width = width > 0 ? 1.f / static_cast<float>(width) : 0.f, a.eps = eps;
  a.y = y, a.act = (uint16_t*)act, a.residual = residual;
  a.next_weight = next_weight_dtype == kBF16 ? (const uint16_t*)next_weight : nullptr;
  a.next_weight_f32 = next_weight_dtype == kBF16 ? nullptr : (const float*)next_weight;
  a.xg = (uint16_t*)xg, a.ssq_out = ssq_out;
  a.positions = positions, a.slot_map = slot_map, a.inv_freq = inv_freq, a.rot_dim = rot_dim;
  a.nq = nq, a.nkv = nkv, a.d = d, a.page_size = page_size, a.q_out = (uint16_t*)q_out, a.cache = (uint16_t*)cache;
  const dim3 grid((N + rows_per_block - 1) / rows_per_block);
  hipStream_t s = (hipStream_t)stream;
#define TLIE_CASE(E)                                                                                  \
  if (epilogue == E) {                                                                                \
    if (rows_per_block == 32 && waves == 8)                                                           \
      hipLaunchKernelGGL((gemm_rows_kernel<E, 8, 2>), grid, dim3(512), 0, s, a);                       \
    else if (rows_per_block == 32 && waves == 4)                                                      \
      hipLaunchKernelGGL((gemm_rows_kernel<E, 4, 2>), grid, dim3(256), 0, s, a);                       \
    else if (rows_per_block == 32)                                                                    \
      hipLaunchKernelGGL((gemm_rows_kernel<E, 2, 2>), grid, dim3(128), 0, s, a);                       \
    else if (waves == 16)                                                                             \
      hipLaunchKernelGGL((gemm_rows_kernel<E, 16, 1>), grid, dim3(1024), 0, s, a);                     \
    else if (waves == 8)                                                                              \
      hipLaunchKernelGGL((gemm_rows_kernel<E, 8, 1>), grid, dim3(512), 0, s, a);                       \
    else if (waves == 4)                                                                              \
      hipLaunchKernelGGL((gemm_rows_kernel<E, 4, 1>), grid, dim3(256), 0, s, a);                       \
    else                                                                                              \
      hipLaunchKernelGGL((gemm_rows_kernel<E, 2, 1>), grid, dim3(128), 0, s, a);                       \
    return launch_status();                                                                           \
  }
  TLIE_CASE(kEpilogueStore)
  TLIE_CASE(kEpilogueSilu)
  TLIE_CASE(kEpilogueResidual)
  TLIE_CASE(kEpilogueRope)
#undef TLIE_CASE
  return kBadArgument;
}

// tokens [T] (T <= 16), table [vocab, hidden]; residual float [T, hidden]; next_weight [hidden];
// xg bfloat16 [T, hidden]; ssq_out float [ceil(hidden / 16), 16].
extern "C" int tlie_embed_rows(const int* tokens, const void* table, int table_dtype, float* residual,
                               const void* next_weight, int next_weight_dtype, void* xg, float* ssq_out, int num_tokens,
                               int hidden, void* stream) {
  if (num_tokens <= 0 || num_tokens > 16 || hidden <= 0) return kBadArgument;
  hipStream_t s = (hipStream_t)stream;
  const bool wide = (hidden & 3) == 0 &&
                    ((reinterpret_cast<uintptr_t>(table) | reinterpret_cast<uintptr_t>(residual) |
                      reinterpret_cast<uintptr_t>(next_weight) | reinterpret_cast<uintptr_t>(xg)) & 15) == 0;
  const dim3 grid(num_tokens, wide ? (hidden + 1023) / 1024 : 1), block(256);
#define TLIE_CASE(WC, W, GC, G)                                                                                      \
  if (table_dtype == WC && next_weight_dtype == GC) {                                                                \
    if (wide)                                                                                                        \
      hipLaunchKernelGGL((embed_rows_wide_kernel<W, G>), grid, block, 0, s, tokens, (const W*)table, residual,        \
                         (const G*)next_weight, (uint16_t*)xg, ssq_out, hidden);                                     \
    else                                                                                                             \
      hipLaunchKernelGGL((embed_rows_kernel<W, G>), grid, block, 0, s, tokens, (const W*)table, residual,             \
                         (const G*)next_weight, (uint16_t*)xg, ssq_out, hidden);                                     \
    return launch_status();                                                                                          \
  }
  TLIE_CASE(kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kF32, float)
  TLIE_CASE(kF32, float, kBF16, bf16)
  TLIE_CASE(kF32, float, kF32, float)
#undef TLIE_CASE
  return kBadArgument;
}
