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

}  // namespace tlie

using namespace tlie;

extern "C" int tlie_gemm_generic(const void* x, int x_dtype, const void* w, int w_dtype, const void* bias,
                                 void* y, int y_dtype, int M, int N, int K, void* stream) {
  if (M <= 0 || N <= 0 || K <= 0) return kBadArgument;
  const dim3 grid((N + kTileN - 1) / kTileN, (M + kTileM - 1) / kTileM);
  if (grid.y > 65535) return kBadArgument;
  hipStream_t s = (hipStream_t)stream;
#define TLIE_CASE(XC, X, WC, W, OC, O)                                                                       \
  if (x_dtype == XC && w_dtype == WC && y_dtype == OC) {                                                     \
    hipLaunchKernelGGL((gemm_generic_kernel<X, W, O>), grid, dim3(256), 0, s, (const X*)x, (const W*)w,       \
                       (const W*)bias, (O*)y, M, N, K);                                                      \
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
