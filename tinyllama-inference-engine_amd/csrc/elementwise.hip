// Token-parallel kernels: embedding gather, residual-add + RMSNorm, SiLU*mul.
//
// A matrix product's result reaches these kernels either as one [rows, cols] array in the
// activation type, or as `nsplit` float partial sums [nsplit, rows, cols] that a split-K product
// left unsummed; the consumer adds them up, in a fixed order, so no separate reduction runs.
#include "common.h"

namespace tlie {

// ---- embedding: residual[t, :] = table[token[t], :] as float -------------------------------
// reference: a row copy per token (src/model.cpp:94-97, src/cuda/model.cu:388-391)
template <typename W>
__global__ void embed_gather_kernel(const int* __restrict__ tokens, const W* __restrict__ table,
                                    float* __restrict__ residual, int hidden) {
  const int t = blockIdx.x;
  const W* row = table + static_cast<size_t>(tokens[t]) * hidden;
  float* out = residual + static_cast<size_t>(t) * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) out[i] = to_float(row[i]);
}

// ---- residual += delta (+ bias); out = RMSNorm(residual) * weight ----------------------------
// reference: y = x * rsqrt(mean(x^2) + eps) * w, sum in float (src/cuda/kernels.cu:67-84);
// the add before it is AddInPlace (kernels.cu:208-215).  Here the residual stays in float.
// rows != nullptr: row r of the output comes from residual row rows[r] (and delta row rows[r]);
// the residual is then left untouched (used for the final norm at the wanted positions).
template <typename D, typename W, typename O>
__global__ void add_rmsnorm_kernel(float* __restrict__ residual, const D* __restrict__ delta, int nsplit,
                                   size_t split_stride, const W* __restrict__ weight, float eps, O* __restrict__ out,
                                   const int* __restrict__ rows, int hidden) {
  extern __shared__ float row_cache[];           // hidden floats, then 16 for the reduction
  float* scratch = row_cache + hidden;
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  float* res = residual + static_cast<size_t>(src) * hidden;
  float square = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float v = res[i];
    if (delta) {
      v += sum_splits(delta + static_cast<size_t>(src) * hidden + i, nsplit, split_stride);
      if (!rows) res[i] = v;
    }
    row_cache[i] = v;
    square += v * v;
  }
  const float total = block_sum(square, scratch);
  const float scale = rsqrtf(total / static_cast<float>(hidden) + eps);
  if (out) {
    O* o = out + static_cast<size_t>(r) * hidden;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) o[i] = from_float<O>(row_cache[i] * scale * to_float(weight[i]));
  }
}

// The same with eight elements a thread (16-byte loads and stores): hidden % 8 == 0; the summands
// of a split product are added in the order of their index.
template <typename D, typename W, typename O>
__global__ void add_rmsnorm_wide_kernel(float* __restrict__ residual, const D* __restrict__ delta, int nsplit,
                                        size_t split_stride, const W* __restrict__ weight, float eps,
                                        O* __restrict__ out, const int* __restrict__ rows, int hidden) {
  extern __shared__ float row_cache[];           // hidden floats, then 16 for the reduction
  float* scratch = row_cache + hidden;
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  float* res = residual + static_cast<size_t>(src) * hidden;
  float square = 0.f;
  for (int i = threadIdx.x * 8; i < hidden; i += blockDim.x * 8) {
    float v[8];
    load8(res + i, v);
    if (delta) {
      const D* part = delta + static_cast<size_t>(src) * hidden + i;
      float d[8];
      load8(part, d);
      for (int s = 1; s < nsplit; ++s) {
        float more[8];
        load8(part + s * split_stride, more);
#pragma unroll
        for (int j = 0; j < 8; ++j) d[j] += more[j];
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] += d[j];
      if (!rows) store8(res + i, v);
    }
    store8(row_cache + i, v);
#pragma unroll
    for (int j = 0; j < 8; ++j) square += v[j] * v[j];
  }
  const float total = block_sum(square, scratch);
  const float scale = rsqrtf(total / static_cast<float>(hidden) + eps);
  if (out) {
    O* o = out + static_cast<size_t>(r) * hidden;
    for (int i = threadIdx.x * 8; i < hidden; i += blockDim.x * 8) {
      float v[8], w[8];
      load8(row_cache + i, v);                   // the thread's own entries
      load8(weight + i, w);
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = v[j] * scale * w[j];
      store8(o + i, v);
    }
  }
}

// ---- act[t, i] = silu(gate[t, i]) * up[t, i]; gate_up is [rows, 2 * inter], either [gate | up] or,
// interleaved, g0 u0 g1 u1 ... (the layout the gated product of few rows wants of its weight) -------
// reference: (g / (1 + exp(-g))) * u in float (src/cuda/kernels.cu:198-206)
template <typename D, typename O>
__global__ void silu_mul_kernel(const D* __restrict__ gate_up, int nsplit, size_t split_stride,
                                O* __restrict__ out, int rows, int inter, int interleaved) {
  const size_t total = static_cast<size_t>(rows) * inter;
  for (size_t index = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; index < total;
       index += static_cast<size_t>(gridDim.x) * blockDim.x) {
    const size_t t = index / inter, i = index % inter;
    const D* base = gate_up + t * 2 * inter;
    const float g = sum_splits(base + (interleaved ? 2 * i : i), nsplit, split_stride);
    const float u = sum_splits(base + (interleaved ? 2 * i + 1 : inter + i), nsplit, split_stride);
    out[index] = from_float<O>((g / (1.f + expf(-g))) * u);
  }
}

// Eight results a thread from sixteen inputs: inter % 8 == 0; the summands of a split product are
// added in the order of their index.
template <typename D, typename O>
__global__ void silu_mul_wide_kernel(const D* __restrict__ gate_up, int nsplit, size_t split_stride, O* __restrict__ out,
                                     int rows, int inter, int interleaved) {
  const int per_row = inter / 8;
  const size_t total = static_cast<size_t>(rows) * per_row;
  for (size_t index = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; index < total;
       index += static_cast<size_t>(gridDim.x) * blockDim.x) {
    const size_t t = index / per_row;
    const int i = static_cast<int>(index % per_row) * 8;
    const D* base = gate_up + t * 2 * inter;
    float a[8], b[8], g[8], u[8];
    const int first = interleaved ? 2 * i : i, second = interleaved ? 2 * i + 8 : inter + i;
    load8(base + first, a);
    load8(base + second, b);
    for (int s = 1; s < nsplit; ++s) {
      float more[8];
      load8(base + s * split_stride + first, more);
#pragma unroll
      for (int j = 0; j < 8; ++j) a[j] += more[j];
      load8(base + s * split_stride + second, more);
#pragma unroll
      for (int j = 0; j < 8; ++j) b[j] += more[j];
    }
    if (interleaved) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        g[j] = a[2 * j]; u[j] = a[2 * j + 1];
        g[4 + j] = b[2 * j]; u[4 + j] = b[2 * j + 1];
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) g[j] = a[j], u[j] = b[j];
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) g[j] = (g[j] / (1.f + expf(-g[j]))) * u[j];
    store8(out + t * inter + i, g);
  }
}

// ---- out[r, c] = product[r, c] + bias[c] ------------------------------------------------------
// For a product that a library made without its bias (steps of many rows): the bias joins the
// float sums, as in the kernels that add it themselves, and the result is rounded once.
// reference: AddBiasKernel after the library's product (src/cuda/kernels.cu:198-206).
template <typename B, typename O>
__global__ void add_bias_kernel(const float* __restrict__ product, const B* __restrict__ bias, O* __restrict__ out,
                                size_t total, int cols) {
  for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < total; i += static_cast<size_t>(gridDim.x) * blockDim.x)
    out[i] = from_float<O>(product[i] + to_float(bias[i % cols]));
}

}  // namespace tlie

using namespace tlie;

extern "C" int tlie_embed_gather(const int* tokens, const void* table, int table_dtype, float* residual,
                                 int num_tokens, int hidden, void* stream) {
  if (num_tokens <= 0 || hidden <= 0) return kBadArgument;
  const int threads = hidden >= 1024 ? 256 : 64;
  if (table_dtype == kF32)
    hipLaunchKernelGGL(embed_gather_kernel<float>, dim3(num_tokens), dim3(threads), 0, (hipStream_t)stream,
                       tokens, (const float*)table, residual, hidden);
  else if (table_dtype == kBF16)
    hipLaunchKernelGGL(embed_gather_kernel<bf16>, dim3(num_tokens), dim3(threads), 0, (hipStream_t)stream,
                       tokens, (const bf16*)table, residual, hidden);
  else
    return kBadArgument;
  return launch_status();
}

template <typename D, typename W, typename O>
static int launch_add_rmsnorm(float* residual, const void* delta, int nsplit, size_t split_stride,
                              const void* weight, float eps, void* out,
                              const int* rows, int num_rows, int hidden, hipStream_t stream) {
  const size_t lds = (static_cast<size_t>(hidden) + 16) * sizeof(float);
  if (lds > 160 * 1024) return kBadArgument;
  const bool aligned = ((reinterpret_cast<uintptr_t>(residual) | reinterpret_cast<uintptr_t>(delta) |
                         reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(out)) & 31) == 0;
  if ((hidden & 7) == 0 && aligned && (nsplit == 1 || (split_stride * sizeof(D)) % 32 == 0)) {
    const int chunks = hidden / 8;
    const int wide = chunks >= 1024 ? 1024 : (chunks + 63) / 64 * 64;
    hipLaunchKernelGGL((add_rmsnorm_wide_kernel<D, W, O>), dim3(num_rows), dim3(wide), lds, stream, residual,
                       (const D*)delta, nsplit, split_stride, (const W*)weight, eps, (O*)out, rows, hidden);
    return launch_status();
  }
  const int threads = hidden >= 2048 ? 1024 : (hidden >= 1024 ? 512 : (hidden >= 256 ? 256 : 64));
  hipLaunchKernelGGL((add_rmsnorm_kernel<D, W, O>), dim3(num_rows), dim3(threads), lds, stream, residual,
                     (const D*)delta, nsplit, split_stride, (const W*)weight, eps, (O*)out, rows, hidden);
  return launch_status();
}

// delta may be null (no add); rows may be null (all rows, residual updated in place);
// out may be null (residual update only).
extern "C" int tlie_add_rmsnorm(float* residual, const void* delta, int delta_dtype, int nsplit,
                                long long split_stride, const void* weight, int weight_dtype,
                                float eps, void* out, int out_dtype, const int* rows, int num_rows, int hidden,
                                void* stream) {
  if (num_rows <= 0 || hidden <= 0 || nsplit < 1) return kBadArgument;
  hipStream_t s = (hipStream_t)stream;
#define TLIE_CASE(DC, D, WC, W, OC, O)                                                                     \
  if (delta_dtype == DC && weight_dtype == WC && out_dtype == OC)                                          \
    return launch_add_rmsnorm<D, W, O>(residual, delta, nsplit, (size_t)split_stride, weight, eps, out, \
                                       rows, num_rows, hidden, s);
  TLIE_CASE(kF32, float, kF32, float, kF32, float)
  TLIE_CASE(kF32, float, kF32, float, kBF16, bf16)
  TLIE_CASE(kF32, float, kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kF32, float, kBF16, bf16)
  TLIE_CASE(kF32, float, kBF16, bf16, kF32, float)
#undef TLIE_CASE
  return kBadArgument;
}

extern "C" int tlie_silu_mul(const void* gate_up, int in_dtype, int nsplit, long long split_stride, void* out,
                             int out_dtype, int rows, int inter, int interleaved, void* stream) {
  if (rows <= 0 || inter <= 0 || nsplit < 1) return kBadArgument;
  const size_t total = static_cast<size_t>(rows) * inter;
  const int threads = 256;
  const int blocks = static_cast<int>(total / threads + 1 < 65536 ? total / threads + 1 : 65536);
  hipStream_t s = (hipStream_t)stream;
  const bool aligned = ((reinterpret_cast<uintptr_t>(gate_up) | reinterpret_cast<uintptr_t>(out)) & 31) == 0;
  if ((inter & 7) == 0 && aligned && (nsplit == 1 || (in_dtype == kF32 && (split_stride & 7) == 0))) {
    const size_t groups = total / 8;
    const int wide = static_cast<int>(groups / threads + 1 < 65536 ? groups / threads + 1 : 65536);
    if (in_dtype == kF32 && out_dtype == kF32)
      hipLaunchKernelGGL((silu_mul_wide_kernel<float, float>), dim3(wide), dim3(threads), 0, s, (const float*)gate_up,
                         nsplit, (size_t)split_stride, (float*)out, rows, inter, interleaved);
    else if (in_dtype == kF32 && out_dtype == kBF16)
      hipLaunchKernelGGL((silu_mul_wide_kernel<float, bf16>), dim3(wide), dim3(threads), 0, s, (const float*)gate_up,
                         nsplit, (size_t)split_stride, (bf16*)out, rows, inter, interleaved);
    else if (in_dtype == kBF16 && out_dtype == kBF16)
      hipLaunchKernelGGL((silu_mul_wide_kernel<bf16, bf16>), dim3(wide), dim3(threads), 0, s, (const bf16*)gate_up,
                         nsplit, (size_t)split_stride, (bf16*)out, rows, inter, interleaved);
    else
      return kBadArgument;
    return launch_status();
  }
  if (in_dtype == kF32 && out_dtype == kF32)
    hipLaunchKernelGGL((silu_mul_kernel<float, float>), dim3(blocks), dim3(threads), 0, s, (const float*)gate_up, nsplit,
                       (size_t)split_stride, (float*)out, rows, inter, interleaved);
  else if (in_dtype == kF32 && out_dtype == kBF16)
    hipLaunchKernelGGL((silu_mul_kernel<float, bf16>), dim3(blocks), dim3(threads), 0, s, (const float*)gate_up, nsplit,
                       (size_t)split_stride, (bf16*)out, rows, inter, interleaved);
  else if (in_dtype == kBF16 && out_dtype == kBF16)
    hipLaunchKernelGGL((silu_mul_kernel<bf16, bf16>), dim3(blocks), dim3(threads), 0, s, (const bf16*)gate_up, nsplit,
                       (size_t)split_stride, (bf16*)out, rows, inter, interleaved);
  else
    return kBadArgument;
  return launch_status();
}

// product float [rows, cols], bias [cols] (float or bfloat16), out [rows, cols] (float: may be `product` itself; or bfloat16).
extern "C" int tlie_add_bias(const float* product, const void* bias, int bias_dtype, void* out, int out_dtype, int rows,
                             int cols, void* stream) {
  if (rows <= 0 || cols <= 0) return kBadArgument;
  const size_t total = static_cast<size_t>(rows) * cols;
  const int threads = 256;
  const int blocks = static_cast<int>((total + threads - 1) / threads < 16384 ? (total + threads - 1) / threads : 16384);
  hipStream_t s = (hipStream_t)stream;
#define TLIE_CASE(BC, B, OC, O)                                                                                  \
  if (bias_dtype == BC && out_dtype == OC) {                                                                     \
    hipLaunchKernelGGL((add_bias_kernel<B, O>), dim3(blocks), dim3(threads), 0, s, product, (const B*)bias, (O*)out, \
                       total, cols);                                                                             \
    return launch_status();                                                                                      \
  }
  TLIE_CASE(kF32, float, kF32, float)
  TLIE_CASE(kF32, float, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kF32, float)
  TLIE_CASE(kBF16, bf16, kBF16, bf16)
#undef TLIE_CASE
  return kBadArgument;
}
