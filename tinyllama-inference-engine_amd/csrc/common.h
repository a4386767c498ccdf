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

// two floats to two bfloat16 (round to nearest even) in one instruction, v_cvt_pk_bf16_f32
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float floatx2;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  const bf16x2 r = __builtin_convertvector((floatx2{lo, hi}), bf16x2);
  return *reinterpret_cast<const uint32_t*>(&r);
}

// Eight consecutive elements (the address a multiple of 16 bytes for bfloat16, of 32 for float) as floats.
__device__ __forceinline__ void load8(const float* p, float (&v)[8]) {
  const float4 a = reinterpret_cast<const float4*>(p)[0], b = reinterpret_cast<const float4*>(p)[1];
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void load8(const bf16* p, float (&v)[8]) {
  const uint4 u = *reinterpret_cast<const uint4*>(p);
  v[0] = bf16_lo(u.x); v[1] = bf16_hi(u.x); v[2] = bf16_lo(u.y); v[3] = bf16_hi(u.y);
  v[4] = bf16_lo(u.z); v[5] = bf16_hi(u.z); v[6] = bf16_lo(u.w); v[7] = bf16_hi(u.w);
}
__device__ __forceinline__ void store8(float* p, const float (&v)[8]) {
  reinterpret_cast<float4*>(p)[0] = make_float4(v[0], v[1], v[2], v[3]);
  reinterpret_cast<float4*>(p)[1] = make_float4(v[4], v[5], v[6], v[7]);
}
__device__ __forceinline__ void store8(bf16* p, const float (&v)[8]) {
  *reinterpret_cast<uint4*>(p) = make_uint4(pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4], v[5]), pack_bf16(v[6], v[7]));
}
__device__ __forceinline__ void store4(float* p, float a, float b, float c, float d) {
  *reinterpret_cast<float4*>(p) = make_float4(a, b, c, d);
}
__device__ __forceinline__ void store4(bf16* p, float a, float b, float c, float d) {
  *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16(a, b), pack_bf16(c, d));
}

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
constexpr int kScratchTooSmall = -4;  // the sizes need more scratch memory than the library's own array holds

inline int launch_status() { return hipGetLastError() == hipSuccess ? kOk : kLaunchFailed; }

}  // namespace tlie
