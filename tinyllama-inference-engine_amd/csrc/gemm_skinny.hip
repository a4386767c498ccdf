// y = x . W^T for few rows of x (a decode batch, or a short step): bfloat16 in, float partial
// sums out, on the matrix cores.  The kernel is bound by reading W once from HBM, so W goes
// straight from global memory into the MFMA operand registers (every element of W is used by one
// wave only); x, which every wave needs, is staged through LDS.
//
// reference: every product of the reference's device path is one library call per projection
// (GemmFp16RowMajor, src/cuda/kernels.cu:342-368), also for one token.  A matrix of 2048 rows
// gives a 256-CU part too few waves when each wave takes whole rows, so K is split over
// `nsplit` workgroups in y and the partial sums [nsplit, M, N] are left to the consumer (the
// norm, rotation or activation kernel that reads them next) to add up.
//
// v_mfma_f32_16x16x32_bf16: operand A = 16 rows of W x 32 k, operand B = 16 rows of x x 32 k,
// C[w row][x row].  Lane l supplies row (l & 15) and the 8 k values of group (l >> 4).  Which k
// values a slot stands for is free as long as A and B agree, so a lane takes 16 consecutive k of
// its row per 64-wide step (two MFMAs): its loads are 32 contiguous bytes and a row's four lanes
// read 128 contiguous bytes.
#include "common.h"

namespace tlie {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

union Pack16 {
  uint4 u;
  bf16x8 v;
};

constexpr int kSkinnyPad = 8;                // bf16 elements of padding per LDS row (16 bytes): rows fall on different banks

// NT: tiles of 16 rows of x (M <= 16 * NT).  RS: strips of 16 rows of W per wave: with more rows
// of x, more strips share each read of x from LDS.  A workgroup has blockDim.x / 64 waves, at most
// MAXWAVES and at least MINWAVES, and takes 16 * RS rows of W per wave: the caller picks the number of waves and the
// split's length so that the workgroups are as many as the compute units, or a multiple (a compute
// unit draws some 20 GB/s from memory whatever its waves ask for, so the product takes as long as
// the unit with the most bytes; 176 workgroups on 256 units measured 3.1 TB/s, 256 of them 4.3).
// CHUNK: k values staged in LDS at a time.
// split_len: k values per split (multiple of 64).  K % 8 == 0.
// GATED: K is not split (one split holds all of it), W's rows alternate gate and up (g0, u0, g1, u1, ...),
// and the workgroup, which then holds complete sums, stores silu(gate) * up as bfloat16 [M, N / 2] in `act`
// instead of partial sums: the activation kernel's launch, and the partial sums' way to memory and back, go.
template <int NT, int RS, int CHUNK, int MINWAVES, int MAXWAVES, bool GATED = false>
__global__ void __launch_bounds__(64 * MAXWAVES)
gemm_skinny_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w, const uint16_t* __restrict__ bias,
                   float* __restrict__ y, uint16_t* __restrict__ act, int M, int N, int K, int split_len) {
  constexpr int kStride = CHUNK + kSkinnyPad;
  constexpr int kSteps = CHUNK / 64;
  __shared__ __attribute__((aligned(16))) uint16_t xs[NT * 16 * kStride];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int split = blockIdx.y;
  const int k_begin = split * split_len, k_end = min(K, k_begin + split_len);
  const int wave_row = (blockIdx.x * (blockDim.x >> 6) + wave) * 16 * RS;
  const int group = lane >> 4;
  const uint16_t* w_row[RS];
  bool active[RS];
#pragma unroll
  for (int r = 0; r < RS; ++r) {
    active[r] = wave_row + r * 16 < N;
    w_row[r] = w + static_cast<size_t>(min(wave_row + r * 16 + (lane & 15), N - 1)) * K;
  }

  floatx4 acc[RS][NT];
#pragma unroll
  for (int r = 0; r < RS; ++r)
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[r][t] = floatx4{0.f, 0.f, 0.f, 0.f};

  // Two sets of operand registers in turn: the next chunk's part of W, and its part of x, are asked
  // for before the current chunk is multiplied, so that memory and the matrix cores work at once.
  constexpr int kVectors = CHUNK / 8;                                  // 16-byte pieces of a staged row of x
  constexpr int kStage = (NT * 16 * kVectors + 64 * MINWAVES - 1) / (64 * MINWAVES);   // pieces a thread stages
  Pack16 a[2][RS][kSteps][2];
  uint4 staged[kStage];
  auto load_w = [&](int c0, Pack16 (&buf)[RS][kSteps][2]) {
    const int c1 = min(k_end, c0 + CHUNK);
#pragma unroll
    for (int r = 0; r < RS; ++r)
#pragma unroll
      for (int s = 0; s < kSteps; ++s) {
        const int k = c0 + s * 64 + group * 16;
        buf[r][s][0].u = (active[r] && k < c1) ? *reinterpret_cast<const uint4*>(w_row[r] + k) : make_uint4(0, 0, 0, 0);
        buf[r][s][1].u = (active[r] && k + 8 < c1) ? *reinterpret_cast<const uint4*>(w_row[r] + k + 8) : make_uint4(0, 0, 0, 0);
      }
  };
  auto load_x = [&](int c0) {
    const int c1 = min(k_end, c0 + CHUNK);
#pragma unroll
    for (int j = 0; j < kStage; ++j) {
      const int i = threadIdx.x + j * blockDim.x;
      const int token = i / kVectors, k = c0 + (i % kVectors) * 8;
      staged[j] = (token < M && k < c1) ? *reinterpret_cast<const uint4*>(x + static_cast<size_t>(token) * K + k)
                                        : make_uint4(0, 0, 0, 0);
    }
  };
  auto store_x = [&]() {
#pragma unroll
    for (int j = 0; j < kStage; ++j) {
      const int i = threadIdx.x + j * blockDim.x;
      if (i < NT * 16 * kVectors) *reinterpret_cast<uint4*>(xs + (i / kVectors) * kStride + (i % kVectors) * 8) = staged[j];
    }
  };
  auto multiply = [&](int c0, Pack16 (&buf)[RS][kSteps][2]) {
    const int c1 = min(k_end, c0 + CHUNK);
#pragma unroll
    for (int s = 0; s < kSteps; ++s) {
      if (c0 + s * 64 >= c1) break;          // the same for every lane
      const int offset = s * 64 + group * 16;
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const uint16_t* x_row = xs + (t * 16 + (lane & 15)) * kStride + offset;
        Pack16 b0, b1;
        b0.u = *reinterpret_cast<const uint4*>(x_row);
        b1.u = *reinterpret_cast<const uint4*>(x_row + 8);
#pragma unroll
        for (int r = 0; r < RS; ++r) {
          acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(buf[r][s][0].v, b0.v, acc[r][t], 0, 0, 0);
          acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(buf[r][s][1].v, b1.v, acc[r][t], 0, 0, 0);
        }
      }
    }
  };
  load_w(k_begin, a[0]);
  load_x(k_begin);
  for (int c0 = k_begin; c0 < k_end; c0 += 2 * CHUNK) {
#pragma unroll
    for (int turn = 0; turn < 2; ++turn) {
      const int mine = c0 + turn * CHUNK;
      if (mine >= k_end) break;
      __syncthreads();                       // the previous chunk's reads of xs are done
      store_x();
      __syncthreads();
      if (mine + CHUNK < k_end) {
        load_w(mine + CHUNK, a[turn ^ 1]);
        load_x(mine + CHUNK);
      }
      multiply(mine, a[turn]);
    }
  }
  // acc[r][t][j] = y[token t*16 + (lane & 15)][wave_row + r*16 + group*4 + j]
#pragma unroll
  for (int r = 0; r < RS; ++r) {
    if (!active[r]) continue;
    const int n0 = wave_row + r * 16 + group * 4;
    float add[4] = {0.f, 0.f, 0.f, 0.f};
    if (bias != nullptr && split == 0) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (n0 + j < N) add[j] = bf16_bits_to_float(bias[n0 + j]);
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      const int token = t * 16 + (lane & 15);
      if (token >= M) continue;
      if (GATED) {
        // (N is even and n0 a multiple of 4: a gate and its up are neighbours in this lane)
        const float g0 = acc[r][t][0] + add[0], u0 = acc[r][t][1] + add[1], g1 = acc[r][t][2] + add[2], u1 = acc[r][t][3] + add[3];
        uint16_t* gated = act + static_cast<size_t>(token) * (N / 2) + (n0 >> 1);
        if (n0 + 3 < N)
          *reinterpret_cast<uint32_t*>(gated) = pack_bf16((g0 / (1.f + expf(-g0))) * u0, (g1 / (1.f + expf(-g1))) * u1);
        else if (n0 + 1 < N)
          gated[0] = __bfloat16_as_ushort(__float2bfloat16((g0 / (1.f + expf(-g0))) * u0));
        continue;
      }
      float* out = y + (static_cast<size_t>(split) * M + token) * N + n0;
      if ((N & 3) == 0 && n0 + 3 < N) {
        *reinterpret_cast<float4*>(out) =
            make_float4(acc[r][t][0] + add[0], acc[r][t][1] + add[1], acc[r][t][2] + add[2], acc[r][t][3] + add[3]);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (n0 + j < N) out[j] = acc[r][t][j] + add[j];
      }
    }
  }
}

}  // namespace tlie

using namespace tlie;

namespace {

template <int NT, int RS, bool GATED>
int launch_skinny(dim3 grid, int waves, hipStream_t s, const uint16_t* x, const uint16_t* w, const uint16_t* bias, float* y,
                  uint16_t* act, int M, int N, int K, int split_len) {
  // (the staged chunk is as long as the registers allow for the workgroup's size)
  const dim3 block(64 * waves);
  if (waves == 3) {
    constexpr int kChunk = NT <= 2 ? 512 : 256;
    hipLaunchKernelGGL((gemm_skinny_kernel<NT, RS, kChunk, 3, 3, GATED>), grid, block, 0, s, x, w, bias, y, act, M, N, K, split_len);
  } else if (waves <= 4) {
    constexpr int kChunk = NT <= 2 ? 512 : 256;
    hipLaunchKernelGGL((gemm_skinny_kernel<NT, RS, kChunk, 4, 4, GATED>), grid, block, 0, s, x, w, bias, y, act, M, N, K, split_len);
  } else if (waves <= 8) {
    constexpr int kChunk = RS == 1 ? 256 : 128;
    hipLaunchKernelGGL((gemm_skinny_kernel<NT, RS, kChunk, 5, 8, GATED>), grid, block, 0, s, x, w, bias, y, act, M, N, K, split_len);
  } else {
    if constexpr (RS == 1)
      hipLaunchKernelGGL((gemm_skinny_kernel<NT, 1, (NT <= 2 ? 256 : 128), 9, 16, GATED>), grid, block, 0, s, x, w, bias, y, act, M, N, K, split_len);
    else
      return kBadArgument;
  }
  return launch_status();
}

template <bool GATED>
int dispatch_skinny(dim3 grid, int waves, int strips, int tiles, hipStream_t s, const uint16_t* x, const uint16_t* w,
                    const uint16_t* bias, float* y, uint16_t* act, int M, int N, int K, int split_len) {
  if (tiles <= 1) return launch_skinny<1, 1, GATED>(grid, waves, s, x, w, bias, y, act, M, N, K, split_len);
  if (tiles == 2) return launch_skinny<2, 1, GATED>(grid, waves, s, x, w, bias, y, act, M, N, K, split_len);
  if (strips == 1) return launch_skinny<4, 1, GATED>(grid, waves, s, x, w, bias, y, act, M, N, K, split_len);
  return launch_skinny<4, 2, GATED>(grid, waves, s, x, w, bias, y, act, M, N, K, split_len);
}

}  // namespace

// x [M, K], w [N, K], bias [N] or null: bfloat16.  y: float [nsplit, M, N] with
// nsplit = ceil(K / split_len).  M <= 64, K % 8 == 0, split_len % 64 == 0.
// waves: 3 to 16 waves a workgroup; strips: 1 or 2 strips of 16 rows of W per wave (2 only for more
// than 32 rows of x and up to 8 waves); a workgroup takes 16 * strips * waves rows of W.
// act (or null): with it, split_len must cover K (one split), N must be even, W's rows alternate gate and up, and
// bfloat16 silu(gate) * up [M, N / 2] is stored there instead of y (which may then be null).
extern "C" int tlie_gemm_skinny(const void* x, const void* w, const void* bias, float* y, void* act, int M, int N, int K,
                                int split_len, int waves, int strips, void* stream) {
  if (M <= 0 || M > 64 || N <= 0 || K <= 0 || (K & 7) != 0 || split_len <= 0 || (split_len & 63) != 0) return kBadArgument;
  if (waves < 3 || waves > 16 || strips < 1 || strips > 2 || (strips == 2 && (M <= 32 || waves > 8))) return kBadArgument;
  const int nsplit = (K + split_len - 1) / split_len;
  if (act != nullptr ? (nsplit != 1 || (N & 1) != 0) : y == nullptr) return kBadArgument;
  const int tiles = (M + 15) / 16;
  const int rows_per_block = 16 * strips * waves;
  const dim3 grid((N + rows_per_block - 1) / rows_per_block, nsplit);
  if (grid.y > 65535) return kBadArgument;
  hipStream_t s = (hipStream_t)stream;
  const uint16_t* xp = (const uint16_t*)x;
  const uint16_t* wp = (const uint16_t*)w;
  const uint16_t* bp = (const uint16_t*)bias;
  if (act != nullptr) return dispatch_skinny<true>(grid, waves, strips, tiles, s, xp, wp, bp, y, (uint16_t*)act, M, N, K, split_len);
  return dispatch_skinny<false>(grid, waves, strips, tiles, s, xp, wp, bp, y, nullptr, M, N, K, split_len);
}
