// Two microbenchmarks that give the roofline's ceilings as this machine delivers them, beside the
// published ones: how fast a kernel that does nothing else reads memory, and how fast the matrix
// cores multiply bfloat16 when nothing else is asked of them.  The measurement program reports both
// with its records, so that a fraction of the published peak can be read against what is reachable.
// reference: none (its benchmarks time its kernels, benchmarks/kernel_benchmarks.cu:127-163, and
// quote no ceiling).
#include "common.h"

namespace tlie {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;

// every workgroup reads its own contiguous share with 16-byte loads, eight in flight per thread
__global__ void __launch_bounds__(512) stream_read_kernel(const uint4* __restrict__ data, size_t per_block, unsigned* __restrict__ sink) {
  const uint4* p = data + blockIdx.x * per_block + threadIdx.x;
  const size_t steps = per_block / blockDim.x;
  constexpr int kDepth = 8;
  uint4 ring[kDepth];
  unsigned acc = 0;
#pragma unroll
  for (int j = 0; j < kDepth; ++j) ring[j] = j < steps ? p[static_cast<size_t>(j) * blockDim.x] : make_uint4(0, 0, 0, 0);
  for (size_t i = 0; i < steps; i += kDepth) {
#pragma unroll
    for (int j = 0; j < kDepth; ++j) {
      acc ^= ring[j].x ^ ring[j].y ^ ring[j].z ^ ring[j].w;
      const size_t next = i + j + kDepth;
      if (next < steps) ring[j] = p[next * blockDim.x];
    }
  }
  if (acc == 0x9e3779b9u) sink[0] = acc;                 // (keeps the loads alive; practically never true)
}

// eight independent chains of v_mfma_f32_32x32x16_bf16 per wave
__global__ void __launch_bounds__(256) mfma_bf16_kernel(int iterations, float* __restrict__ sink) {
  bf16x8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) a[i] = static_cast<__bf16>(0.001f * (threadIdx.x + i)), b[i] = static_cast<__bf16>(0.002f * (i + 1));
  floatx16 acc[8];
#pragma unroll
  for (int c = 0; c < 8; ++c)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[c][i] = 0.f;
  for (int it = 0; it < iterations; ++it) {
#pragma unroll
    for (int c = 0; c < 8; ++c) acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[c], 0, 0, 0);
  }
  float total = 0.f;
#pragma unroll
  for (int c = 0; c < 8; ++c) total += acc[c][0] + acc[c][15];
  if (total == 12345.678f) sink[0] = total;
}

}  // namespace tlie

using namespace tlie;

// Reads `bytes` (a multiple of 16) once.  blocks: workgroups of 512 threads (the caller gives a few per CU).
extern "C" int tlie_probe_stream_read(const void* data, unsigned long long bytes, int blocks, unsigned* sink, void* stream) {
  if (data == nullptr || sink == nullptr || blocks <= 0 || bytes < 16ull * 512 * blocks) return kBadArgument;
  const size_t per_block = bytes / 16 / blocks / 512 * 512;
  hipLaunchKernelGGL(stream_read_kernel, dim3(blocks), dim3(512), 0, (hipStream_t)stream, (const uint4*)data, per_block, sink);
  return launch_status();
}

// The bytes the call above reads for the same arguments.
extern "C" unsigned long long tlie_probe_stream_read_bytes(unsigned long long bytes, int blocks) {
  if (blocks <= 0) return 0;
  return bytes / 16 / blocks / 512 * 512 * 16 * blocks;
}

// blocks workgroups of 4 waves, each wave 8 * iterations products of 32 x 32 x 16 (32768 flops each).
extern "C" int tlie_probe_mfma_bf16(int iterations, int blocks, float* sink, void* stream) {
  if (iterations <= 0 || blocks <= 0 || sink == nullptr) return kBadArgument;
  hipLaunchKernelGGL(mfma_bf16_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, iterations, sink);
  return launch_status();
}
