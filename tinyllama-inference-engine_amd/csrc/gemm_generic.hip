// y[M, N] = x[M, K] . W[N, K]^T (+ bias[N]) with every product and sum in true 32-bit: plain
// v_fma_f32 on values widened to float, no matrix instruction, no reduced-precision mode.
//
// reference: the only product of the reference's device path is a library call with 16-bit
// inputs and 32-bit accumulation (GemmFp16RowMajor, src/cuda/kernels.cu:342-368); its 32-bit
// model multiplies row by vector in a plain loop (src/model.cpp:65-72).  This kernel is that
// plain loop, tiled through LDS: a 64x64 tile of y per 256-thread block, 16 columns of K per
// step, each thread a 4x4 patch.  The sum over K of one output runs in index order whatever M
// and N are, so a token's result does not depend on what else is in the batch.
#include "common.h"

#include <type_traits>

namespace tlie {

constexpr int kTileM = 64, kTileN = 64, kTileK = 16;

template <typename X, typename W, typename O>
__global__ void __launch_bounds__(256)
gemm_generic_kernel(const X* __restrict__ x, const W* __restrict__ w, const W* __restrict__ bias,
                    O* __restrict__ y, int M, int N, int K) {
  __shared__ float xs[kTileK][kTileM + 4];
  __shared__ float ws[kTileK][kTileN + 4];
  const int m0 = blockIdx.y * kTileM, n0 = blockIdx.x * kTileN;
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;   // patch: rows ty*4.., cols tx*4..
  float acc[4][4] = {};
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
      float v = acc[i][j];
      if (bias) v += to_float(bias[n]);
      y[static_cast<size_t>(m) * N + n] = from_float<O>(v);
    }
  }
}

// The same sums for few rows of x (decoding, short portions): with M below 64 the tiles above leave
// most of their threads idle and give the chip N / 64 workgroups, each walking K in steps of 16
// between barriers.  Here a workgroup owns 16 columns of y and all M <= 16 * MT rows: thread
// (n, m) adds up y[m + 16 i][n] for i < MT, one multiply-add per k in index order, exactly the
// chain of the kernel above, so the two give the same bits and a step may take either.  W and x
// come through LDS in tiles of 128 k, the next tile asked for while the current one is used.
constexpr int kFewN = 16, kFewK = 128;

template <typename X, typename W, typename O, int MT>
__global__ void __launch_bounds__(256)
gemm_generic_few_kernel(const X* __restrict__ x, const W* __restrict__ w, const W* __restrict__ bias,
                        O* __restrict__ y, int M, int N, int K) {
  __shared__ __attribute__((aligned(16))) float ws[kFewN][kFewK + 4];
  __shared__ __attribute__((aligned(16))) float xs[16 * MT][kFewK + 4];
  const int n0 = blockIdx.x * kFewN;
  const int tn = threadIdx.x % 16, tm = threadIdx.x / 16;
  // what a thread brings of each tile: W: 16 rows x 128 k = 2048 values, 8 a thread (row r, k c..c+7);
  // x: 16 MT rows x 128 k, 8 MT a thread
  const int load_row = threadIdx.x / 16, load_col = (threadIdx.x % 16) * 8;
  float w_next[8], x_next[MT][8];
  // (whole 16-byte loads where the rows allow them: both operands float, K a multiple of 4, bases aligned)
  const bool wide = std::is_same<X, float>::value && std::is_same<W, float>::value && (K & 3) == 0 &&
                    ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) & 15) == 0;
  auto fetch = [&](int k0) {
    const int k = k0 + load_col, n = n0 + load_row;
    if (wide && k + 8 <= K) {
      float4 lo = make_float4(0.f, 0.f, 0.f, 0.f), hi = lo;
      if (n < N) {
        const float4* source = reinterpret_cast<const float4*>(reinterpret_cast<const float*>(w) + static_cast<size_t>(n) * K + k);
        lo = source[0], hi = source[1];
      }
      w_next[0] = lo.x, w_next[1] = lo.y, w_next[2] = lo.z, w_next[3] = lo.w;
      w_next[4] = hi.x, w_next[5] = hi.y, w_next[6] = hi.z, w_next[7] = hi.w;
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const int m = load_row + 16 * i;
        lo = make_float4(0.f, 0.f, 0.f, 0.f), hi = lo;
        if (m < M) {
          const float4* source = reinterpret_cast<const float4*>(reinterpret_cast<const float*>(x) + static_cast<size_t>(m) * K + k);
          lo = source[0], hi = source[1];
        }
        x_next[i][0] = lo.x, x_next[i][1] = lo.y, x_next[i][2] = lo.z, x_next[i][3] = lo.w;
        x_next[i][4] = hi.x, x_next[i][5] = hi.y, x_next[i][6] = hi.z, x_next[i][7] = hi.w;
      }
      return;
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      w_next[j] = (n < N && k + j < K) ? to_float(w[static_cast<size_t>(n) * K + k + j]) : 0.f;
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const int m = load_row + 16 * i;
        x_next[i][j] = (m < M && k + j < K) ? to_float(x[static_cast<size_t>(m) * K + k + j]) : 0.f;
      }
    }
  };
  float acc[MT];
#pragma unroll
  for (int i = 0; i < MT; ++i) acc[i] = 0.f;
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += kFewK) {
    __syncthreads();                                     // the last tile has been used
    *reinterpret_cast<float4*>(&ws[load_row][load_col]) = make_float4(w_next[0], w_next[1], w_next[2], w_next[3]);
    *reinterpret_cast<float4*>(&ws[load_row][load_col + 4]) = make_float4(w_next[4], w_next[5], w_next[6], w_next[7]);
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      *reinterpret_cast<float4*>(&xs[load_row + 16 * i][load_col]) = make_float4(x_next[i][0], x_next[i][1], x_next[i][2], x_next[i][3]);
      *reinterpret_cast<float4*>(&xs[load_row + 16 * i][load_col + 4]) = make_float4(x_next[i][4], x_next[i][5], x_next[i][6], x_next[i][7]);
    }
    __syncthreads();
    if (k0 + kFewK < K) fetch(k0 + kFewK);
    // (beyond K the tile holds zeros, as the tiles of the kernel above do: adding them changes nothing)
    const int width = min(kFewK, (K - k0 + 3) & ~3);
    for (int c = 0; c < width; c += 4) {
      const float4 b = *reinterpret_cast<const float4*>(&ws[tn][c]);
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        const float4 a = *reinterpret_cast<const float4*>(&xs[tm + 16 * i][c]);
        acc[i] = fmaf(a.x, b.x, acc[i]);
        acc[i] = fmaf(a.y, b.y, acc[i]);
        acc[i] = fmaf(a.z, b.z, acc[i]);
        acc[i] = fmaf(a.w, b.w, acc[i]);
      }
    }
  }
  const int n = n0 + tn;
  if (n >= N) return;
#pragma unroll
  for (int i = 0; i < MT; ++i) {
    const int m = tm + 16 * i;
    if (m >= M) continue;
    float v = acc[i];
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
    if (M <= 16)                                                                                             \
      hipLaunchKernelGGL((gemm_generic_few_kernel<X, W, O, 1>), few, dim3(256), 0, s, (const X*)x,            \
                         (const W*)w, (const W*)bias, (O*)y, M, N, K);                                       \
    else if (M <= 64)                                                                                        \
      hipLaunchKernelGGL((gemm_generic_few_kernel<X, W, O, 4>), few, dim3(256), 0, s, (const X*)x,            \
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
