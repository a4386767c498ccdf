// y = x . W^T for many rows of x (prompt steps), bfloat16 on the matrix cores: this library's own
// product of many rows, which runs where the vendor's library cannot be called (its file is not beside
// torch, or it has no algorithm for a shape within its workspace).
//
// reference: every product of the reference's device path is a library call (cublasGemmEx,
// src/cuda/kernels.cu:342-368); so are this engine's products of more than 64 rows.  Measured against
// that library on the MI355X (2048 tokens, TinyLlama's four matrices): this kernel reaches 0.5 to 0.7
// PFLOP/s where the library reaches 0.7 to 1.05, so the library stays the first choice; the plain
// 32-bit kernel, the only stand-in before, reaches 0.06.
//
// A workgroup of four waves owns a tile of 128 rows of W by 128 tokens and all of K.  K is walked
// in steps of 64: the step's 128 x 64 pieces of W and of x go from global memory straight into LDS
// (global_load_lds_dwordx4: no registers in between), two buffers in turn, so that a step's loads fly
// while the step before it is multiplied; two workgroups fit a compute unit and fill each other's
// waits.  LDS rows are 128 bytes; the 16-byte piece c of row r lies at piece c ^ (r % 8), so that the
// 8 lanes that read one piece of 8 neighbouring rows hit all banks once.  Each wave multiplies 64 rows
// of W by 64 tokens with v_mfma_f32_32x32x16_bf16, W as the first operand: a lane then holds, for one
// token, groups of four neighbouring outputs, which it stores as 8 or 16 bytes.
#include "common.h"

namespace tlie {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
typedef __attribute__((address_space(3))) uint32_t lds_word;

constexpr int kTileRows = 128;              // rows of W, and tokens, a workgroup
constexpr int kTileK = 64;                  // k values a step
constexpr int kTilePieces = kTileRows * kTileK / 8;   // 16-byte pieces of one operand's part of a step

// One 16-byte piece per lane from global memory into LDS at `base` + lane * 16 (base: the same for the wave).
__device__ __forceinline__ void load_piece(const uint16_t* from, uint4* base) {
  // (C-style casts: the address spaces are what the builtin's signature asks for)
  __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)from,
                                   (lds_word*)static_cast<uintptr_t>(static_cast<uint32_t>(reinterpret_cast<uintptr_t>(base))), 16, 0, 0);
}

// x [M, K], w [N, K] bfloat16; out bfloat16 [M, N] or out_f32 float [M, N].  K % 64 == 0, N % 4 == 0.
__global__ void __launch_bounds__(256, 2)
gemm_tiles_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w, uint16_t* __restrict__ out,
                  float* __restrict__ out_f32, int M, int N, int K, int tiles_n, int tiles_m) {
  // two buffers, each W's part [128 rows][8 pieces] and then x's part; two arrays, named apart in the code
  // below, so that the compiler knows that a step's reads do not touch what the next step's loads write
  __shared__ __attribute__((aligned(16))) uint4 buffer0[2][kTilePieces];
  __shared__ __attribute__((aligned(16))) uint4 buffer1[2][kTilePieces];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // Workgroups are dealt to the chip's eight dies in turn; a die's workgroups take neighbouring
  // tiles (the same rows of W, all tokens), so that a die's L2 reads those rows of W once.
  const int total = tiles_n * tiles_m;
  const int per_die = (total + 7) / 8;
  const int id = (blockIdx.x & 7) * per_die + (blockIdx.x >> 3);
  if (id >= total) return;                                           // (the same for the whole workgroup)
  const int n0 = (id / tiles_m) * kTileRows, m0 = (id % tiles_m) * kTileRows;

  // ---- what this lane brings into LDS each step: 4 pieces of W and 4 of x ----
  const uint16_t* from_w[4];
  const uint16_t* from_x[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int piece = wave * 256 + i * 64 + lane;                    // its place in LDS
    const int row = piece >> 3, c = (piece & 7) ^ (row & 7);         // what lies there: piece c of row `row`
    from_w[i] = w + static_cast<size_t>(min(n0 + row, N - 1)) * K + c * 8;      // (rows beyond the matrix: its last row, never stored)
    from_x[i] = x + static_cast<size_t>(min(m0 + row, M - 1)) * K + c * 8;
  }
  auto issue = [&](int step, uint4 (&buffer)[2][kTilePieces]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      load_piece(from_w[i] + step * kTileK, &buffer[0][wave * 256 + i * 64]);
      load_piece(from_x[i] + step * kTileK, &buffer[1][wave * 256 + i * 64]);
    }
  };

  floatx16 acc[2][2];
#pragma unroll
  for (int fn = 0; fn < 2; ++fn)
#pragma unroll
    for (int fm = 0; fm < 2; ++fm)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[fn][fm][r] = 0.f;

  // where this lane's operands lie in a buffer: row (lane % 32) of a group of 32, piece 2 kk + lane / 32
  const int wave_n = (wave & 1) * 64, wave_m = (wave >> 1) * 64;
  const int swizzle = lane & 7, high = lane >> 5;
  const int steps = K / kTileK;
  auto multiply = [&](const uint4 (&buffer)[2][kTilePieces]) {
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      const int piece = (kk * 2 + high) ^ swizzle;
      uint4 wv[2], xv[2];
#pragma unroll
      for (int f = 0; f < 2; ++f) {
        wv[f] = buffer[0][(wave_n + f * 32 + (lane & 31)) * 8 + piece];
        xv[f] = buffer[1][(wave_m + f * 32 + (lane & 31)) * 8 + piece];
      }
#pragma unroll
      for (int fn = 0; fn < 2; ++fn)
#pragma unroll
        for (int fm = 0; fm < 2; ++fm)
          acc[fn][fm] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const bf16x8*>(&wv[fn]),
                                                                *reinterpret_cast<const bf16x8*>(&xv[fm]), acc[fn][fm], 0, 0, 0);
    }
  };
  issue(0, buffer0);
  for (int step = 0; step < steps; step += 2) {
    __builtin_amdgcn_s_waitcnt(0x0f70);            // vmcnt(0): this wave's pieces of the step have landed
    __syncthreads();                               // everyone's have; and the other buffer has been read by all
    if (step + 1 < steps) issue(step + 1, buffer1);
    multiply(buffer0);
    if (step + 1 >= steps) break;
    __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();
    if (step + 2 < steps) issue(step + 2, buffer0);
    multiply(buffer1);
  }

  // acc[fn][fm][4 g + j] = y[token m0 + wave_m + 32 fm + lane % 32][output n0 + wave_n + 32 fn + 8 g + 4 (lane / 32) + j]
#pragma unroll
  for (int fm = 0; fm < 2; ++fm) {
    const int m = m0 + wave_m + fm * 32 + (lane & 31);
    if (m >= M) continue;
#pragma unroll
    for (int fn = 0; fn < 2; ++fn)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = n0 + wave_n + fn * 32 + g * 8 + high * 4;       // the first of four neighbouring outputs
        if (n >= N) continue;                                         // (N is a multiple of 4)
        const float v0 = acc[fn][fm][g * 4], v1 = acc[fn][fm][g * 4 + 1], v2 = acc[fn][fm][g * 4 + 2], v3 = acc[fn][fm][g * 4 + 3];
        if (out_f32 != nullptr)
          *reinterpret_cast<float4*>(out_f32 + static_cast<size_t>(m) * N + n) = make_float4(v0, v1, v2, v3);
        else
          *reinterpret_cast<uint2*>(out + static_cast<size_t>(m) * N + n) = make_uint2(pack_bf16(v0, v1), pack_bf16(v2, v3));
      }
  }
}

}  // namespace tlie

using namespace tlie;

// x [M, K], w [N, K]: bfloat16; K a multiple of 64, N a multiple of 4.  out: bfloat16 [M, N], or float [M, N] when
// out_is_f32 is not 0.
extern "C" int tlie_gemm_tiles(const void* x, const void* w, void* out, int out_is_f32, int M, int N, int K, void* stream) {
  if (M <= 0 || N <= 0 || K <= 0 || (K % kTileK) != 0 || (N & 3) != 0 || out == nullptr) return kBadArgument;
  const int tiles_n = (N + kTileRows - 1) / kTileRows, tiles_m = (M + kTileRows - 1) / kTileRows;
  const long long total = static_cast<long long>(tiles_n) * tiles_m;
  if (total > (1 << 28)) return kBadArgument;
  const dim3 grid(static_cast<unsigned>((total + 7) / 8 * 8));
  hipLaunchKernelGGL(gemm_tiles_kernel, grid, dim3(256), 0, (hipStream_t)stream, (const uint16_t*)x, (const uint16_t*)w,
                     out_is_f32 ? nullptr : (uint16_t*)out, out_is_f32 ? (float*)out : nullptr, M, N, K, tiles_n, tiles_m);
  return launch_status();
}
