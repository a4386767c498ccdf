// Shared device helpers for the gfx950 kernels: storage types, wave64 and block reductions.
//
// Storage is float or bfloat16; arithmetic that the engine promises in 32-bit (softmax, norms,
// rotation angles, the residual sum) is done on floats obtained with to_float().
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

namespace tlie {

constexpr int kWave = 64;

// dtype codes of the C interface
constexpr int kF32 = 0;
constexpr int kBF16 = 1;

typedef __hip_bfloat16 bf16;

__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16 v) { return __bfloat162float(v); }

template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_float<bf16>(float v) { return __float2bfloat16(v); }

// bfloat16 bits <-> float without going through the class type (for packed 16-byte loads)
__device__ __forceinline__ float bf16_bits_to_float(uint16_t bits) {
  return __uint_as_float(static_cast<uint32_t>(bits) << 16);
}
__device__ __forceinline__ float bf16_lo(uint32_t pair) { return __uint_as_float(pair << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t pair) { return __uint_as_float(pair & 0xffff0000u); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int offset = kWave / 2; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int offset = kWave / 2; offset > 0; offset >>= 1) v = fmaxf(v, __shfl_xor(v, offset, kWave));
  return v;
}

// Block-wide reductions over up to 16 waves; `scratch` holds at least 16 floats of LDS.
// Every thread of the block must call them; every thread gets the result.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int waves = (blockDim.x + kWave - 1) / kWave;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < waves; ++w) total += scratch[w];
  return total;
}
__device__ __forceinline__ float block_max(float v, float* scratch) {
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  const int waves = (blockDim.x + kWave - 1) / kWave;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = -INFINITY;
  for (int w = 0; w < waves; ++w) total = fmaxf(total, scratch[w]);
  return total;
}

// The sum over `nsplit` partial results that lie `stride` elements apart, four loads in flight at a
// time.  The order of the additions is fixed (four interleaved chains, then their sum), so the
// result does not vary from run to run.
template <typename D>
__device__ __forceinline__ float sum_splits(const D* __restrict__ first, int nsplit, size_t stride) {
  if (nsplit == 1) return to_float(first[0]);
  float a = 0.f, b = 0.f, c = 0.f, d = 0.f;
  int s = 0;
  for (; s + 3 < nsplit; s += 4) {
    a += to_float(first[(s + 0) * stride]);
    b += to_float(first[(s + 1) * stride]);
    c += to_float(first[(s + 2) * stride]);
    d += to_float(first[(s + 3) * stride]);
  }
  for (; s < nsplit; ++s) a += to_float(first[s * stride]);
  return (a + b) + (c + d);
}

// Error codes returned by the C entry points (0 = launched).
constexpr int kOk = 0;
constexpr int kBadArgument = -1;   // a size or dtype the kernel does not take
constexpr int kLaunchFailed = -2;  // hipGetLastError() reported an error after the launch

inline int launch_status() { return hipGetLastError() == hipSuccess ? kOk : kLaunchFailed; }

}  // namespace tlie
