// y[M, N] = x[M, K] . W[N, K]^T (+ bias[N]) with every product and sum in true 32-bit: plain
// v_fma_f32 on values widened to float, no matrix instruction, no reduced-precision mode.
//
// reference: the only product of the reference's device path is a library call with 16-bit
// inputs and 32-bit accumulation (GemmFp16RowMajor, src/cuda/kernels.cu:342-368); its 32-bit
// model multiplies row by vector in a plain loop (src/model.cpp:65-72).  This kernel is that
// plain loop, tiled through LDS: a 64x64 tile of y per 256-thread block, 16 columns of K per
// step, each thread a 4x4 patch.
//
// The order of the sum of one output is fixed by K alone: K is cut into blocks of 512 from index 0;
// within a block the products are added one by one in index order (a chain of fused multiply-adds
// that starts at zero), and the blocks' sums are added to a total, which starts at zero, in index
// order.  Whatever M and N are, and whichever of the kernels below runs, an output gets the same
// bits: a token's result does not depend on what else is in the batch.  (Blocks, and not one chain
// over all of K, so that a product of few rows can give the blocks to different waves: a chain of
// 5632 dependent multiply-adds alone takes longer than reading the whole matrix.)
#include "common.h"

#include <type_traits>

namespace tlie {

constexpr int kTileM = 64, kTileN = 64, kTileK = 16;
constexpr int kBlockK = 512;          // the blocks of K whose sums are formed apart (a multiple of every tile's width)

template <typename X, typename W, typename O>
__global__ void __launch_bounds__(256)
gemm_generic_kernel(const X* __restrict__ x, const W* __restrict__ w, const W* __restrict__ bias,
                    O* __restrict__ y, int M, int N, int K) {
  __shared__ float xs[kTileK][kTileM + 4];
  __shared__ float ws[kTileK][kTileN + 4];
  const int m0 = blockIdx.y * kTileM, n0 = blockIdx.x * kTileN;
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;   // patch: rows ty*4.., cols tx*4..
  float acc[4][4] = {}, total[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += kTileK) {
    // 64 rows x 16 k of each operand: 1024 values, 4 per thread
    for (int i = threadIdx.x; i < kTileM * kTileK; i += 256) {
      const int r = i / kTileK, c = i % kTileK;
      const int m = m0 + r, n = n0 + r, k = k0 + c;
      xs[c][r] = (m < M && k < K) ? to_float(x[static_cast<size_t>(m) * K + k]) : 0.f;
      ws[c][r] = (n < N && k < K) ? to_float(w[static_cast<size_t>(n) * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int c = 0; c < kTileK; ++c) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[c][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[c][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    if ((k0 + kTileK) % kBlockK == 0 || k0 + kTileK >= K) {     // a block of K ends: its sums join the totals
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) total[i][j] += acc[i][j], acc[i][j] = 0.f;
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = total[i][j];
      if (bias) v += to_float(bias[n]);
      y[static_cast<size_t>(m) * N + n] = from_float<O>(v);
    }
  }
}

// The same sums for few rows of x (decoding, short portions): with M below 64 the tiles above leave
// most of their threads idle and give the chip N / 64 workgroups, each walking K in steps of 16
// between barriers.  Here a workgroup owns 16 columns of y and all M <= 16 * MT rows: a team of 256
// threads, thread (n, m) adding up y[m + 16 i][n] for i < MT with the chain of the kernel above
// (same blocks, same order: the same bits, so a step may take either).  TEAMS teams of a workgroup
// take the blocks of K in turn (team t the blocks t, t + TEAMS, ...), leave their blocks' sums in
// LDS, and the first team adds them up in index order.  W and x come through LDS in tiles of KT k,
// kAhead tiles of W asked for ahead (the weights come from memory and nothing else occupies the
// workgroup meanwhile), x, which comes from the caches, one tile ahead.
constexpr int kFewN = 16;
constexpr int kFewMaxBlocks = 16;      // blocks of K whose sums the teams can park in LDS (K up to 8192)

template <typename X, typename W, typename O, int MT, int TEAMS, int KT>
__global__ void __launch_bounds__(256 * TEAMS)
gemm_generic_few_kernel(const X* __restrict__ x, const W* __restrict__ w, const W* __restrict__ bias,
                        O* __restrict__ y, int M, int N, int K) {
  constexpr int kPer = KT / 16;                          // values of a tile's row a thread brings (8 or 4)
  constexpr int kAhead = 4;
  __shared__ __attribute__((aligned(16))) float ws[TEAMS][kFewN][KT + 4];
  __shared__ __attribute__((aligned(16))) float xs[TEAMS][16 * MT][KT + 4];
  __shared__ float sums[TEAMS > 1 ? kFewMaxBlocks : 1][256];
  const int n0 = blockIdx.x * kFewN;
  const int team = threadIdx.x >> 8, t = threadIdx.x & 255;
  const int tn = t % 16, tm = t / 16;
  const int load_row = t / 16, load_col = (t % 16) * kPer;
  const int blocks = (K + kBlockK - 1) / kBlockK;
  constexpr int kTilesPerBlock = kBlockK / KT;
  const int rounds = (blocks + TEAMS - 1) / TEAMS;       // every team walks so many blocks (the last may be beyond K: zeros)
  const int tiles = rounds * kTilesPerBlock;
  // tile q of this team: block (q / tiles per block) * TEAMS + team, k from block * 512 + (q % tiles per block) * KT
  auto tile_k = [&](int q) { return ((q / kTilesPerBlock) * TEAMS + team) * kBlockK + (q % kTilesPerBlock) * KT; };
  float w_ring[kAhead][kPer], x_next[MT][kPer];
  // (whole 16-byte loads where the rows allow them: both operands float, K a multiple of 4, bases aligned)
  const bool wide = std::is_same<X, float>::value && std::is_same<W, float>::value && (K & 3) == 0 &&
                    ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) & 15) == 0;
  auto fetch_row = [&](float (&out)[kPer], const auto* base, bool live, int k) {
    using Source = std::remove_cv_t<std::remove_pointer_t<decltype(base)>>;
    if (std::is_same<Source, float>::value && wide && k + kPer <= K) {
#pragma unroll
      for (int j = 0; j < kPer; j += 4) {
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (live) v = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(base) + k + j);
        out[j] = v.x, out[j + 1] = v.y, out[j + 2] = v.z, out[j + 3] = v.w;
      }
      return;
    }
#pragma unroll
    for (int j = 0; j < kPer; ++j) out[j] = (live && k + j < K) ? to_float(base[k + j]) : 0.f;
  };
  auto fetch_w = [&](float (&out)[kPer], int q) {
    const int n = n0 + load_row;
    fetch_row(out, w + static_cast<size_t>(min(n, N - 1)) * K, n < N, tile_k(q) + load_col);
  };
  auto fetch_x = [&](int q) {
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const int m = load_row + 16 * i;
      fetch_row(x_next[i], x + static_cast<size_t>(min(m, M - 1)) * K, m < M, tile_k(q) + load_col);
    }
  };
  float acc[MT], total[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) acc[i] = 0.f, total[i] = 0.f;
#pragma unroll
  for (int j = 0; j < kAhead; ++j)
    if (j < tiles) fetch_w(w_ring[j], j);
  fetch_x(0);
  for (int base = 0; base < tiles; base += kAhead) {
#pragma unroll
    for (int j = 0; j < kAhead; ++j) {
      const int q = base + j;
      if (q >= tiles) break;                               // (the same for the whole workgroup)
      __syncthreads();                                     // the last tile has been used
#pragma unroll
      for (int e = 0; e < kPer; e += 4)
        *reinterpret_cast<float4*>(&ws[team][load_row][load_col + e]) = make_float4(w_ring[j][e], w_ring[j][e + 1], w_ring[j][e + 2], w_ring[j][e + 3]);
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int e = 0; e < kPer; e += 4)
          *reinterpret_cast<float4*>(&xs[team][load_row + 16 * i][load_col + e]) = make_float4(x_next[i][e], x_next[i][e + 1], x_next[i][e + 2], x_next[i][e + 3]);
      __syncthreads();
      if (q + kAhead < tiles) fetch_w(w_ring[j], q + kAhead);
      if (q + 1 < tiles) fetch_x(q + 1);
      // (beyond K a tile holds zeros, as the tiles of the kernel above do: adding them changes nothing;
      // eight steps unrolled: the reads from LDS of several steps are asked for together, ahead of the
      // chain of multiply-adds that waits for them)
#pragma unroll 8
      for (int c = 0; c < KT; c += 4) {
        const float4 b = *reinterpret_cast<const float4*>(&ws[team][tn][c]);
#pragma unroll
        for (int i = 0; i < MT; ++i) {
          const float4 a = *reinterpret_cast<const float4*>(&xs[team][tm + 16 * i][c]);
          acc[i] = fmaf(a.x, b.x, acc[i]);
          acc[i] = fmaf(a.y, b.y, acc[i]);
          acc[i] = fmaf(a.z, b.z, acc[i]);
          acc[i] = fmaf(a.w, b.w, acc[i]);
        }
      }
      if (q % kTilesPerBlock == kTilesPerBlock - 1) {     // the team's block ends
        const int block = (q / kTilesPerBlock) * TEAMS + team;
        if (TEAMS == 1) {
#pragma unroll
          for (int i = 0; i < MT; ++i) total[i] += acc[i];
        } else if (block < blocks) {
          sums[block][t] = acc[0];
        }
#pragma unroll
        for (int i = 0; i < MT; ++i) acc[i] = 0.f;
      }
    }
  }
  if (TEAMS > 1) {
    __syncthreads();
    if (team != 0) return;
    for (int b = 0; b < blocks; ++b) total[0] += sums[b][t];   // in index order
  }
  const int n = n0 + tn;
  if (n >= N) return;
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    const int m = tm + 16 * i;
    if (m >= M) continue;
    float v = total[i];
    if (bias) v += to_float(bias[n]);
    y[static_cast<size_t>(m) * N + n] = from_float<O>(v);
  }
}

}  // namespace tlie

using namespace tlie;

extern "C" int tlie_gemm_generic(const void* x, int x_dtype, const void* w, int w_dtype, const void* bias,
                                 void* y, int y_dtype, int M, int N, int K, void* stream) {
  if (M <= 0 || N <= 0 || K <= 0) return kBadArgument;
  const dim3 grid((N + kTileN - 1) / kTileN, (M + kTileM - 1) / kTileM);
  if (grid.y > 65535) return kBadArgument;
  hipStream_t s = (hipStream_t)stream;
  const dim3 few((N + kFewN - 1) / kFewN);
#define TLIE_CASE(XC, X, WC, W, OC, O)                                                                       \
  if (x_dtype == XC && w_dtype == WC && y_dtype == OC) {                                                     \
    if (M <= 16 && K >= 2 * kBlockK && K <= kFewMaxBlocks * kBlockK)                                         \
      hipLaunchKernelGGL((gemm_generic_few_kernel<X, W, O, 1, 4, 64>), few, dim3(1024), 0, s, (const X*)x,    \
                         (const W*)w, (const W*)bias, (O*)y, M, N, K);                                       \
    else if (M <= 16)                                                                                        \
      hipLaunchKernelGGL((gemm_generic_few_kernel<X, W, O, 1, 1, 128>), few, dim3(256), 0, s, (const X*)x,    \
                         (const W*)w, (const W*)bias, (O*)y, M, N, K);                                       \
    else if (M <= 64)                                                                                        \
      hipLaunchKernelGGL((gemm_generic_few_kernel<X, W, O, 4, 1, 128>), few, dim3(256), 0, s, (const X*)x,    \
                         (const W*)w, (const W*)bias, (O*)y, M, N, K);                                       \
    else                                                                                                     \
      hipLaunchKernelGGL((gemm_generic_kernel<X, W, O>), grid, dim3(256), 0, s, (const X*)x, (const W*)w,     \
                         (const W*)bias, (O*)y, M, N, K);                                                    \
    return launch_status();                                                                                  \
  }
  TLIE_CASE(kF32, float, kF32, float, kF32, float)
  TLIE_CASE(kBF16, bf16, kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kBF16, bf16, kF32, float)
  TLIE_CASE(kBF16, bf16, kF32, float, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kF32, float, kF32, float)
#undef TLIE_CASE
  return kBadArgument;
}
