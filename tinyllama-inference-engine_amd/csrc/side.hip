// What a layer that runs its sublayers side by side does to the residual, and pieces of a per-layer token input.
//
//   residual_update   x[t, :] += mult * (a[t, :] + b[t, :])            a, b: products (b optional); optionally a copy of
//                                                                      the new x in the activation type (for a product)
//   side_gate         g[t, j] = gelu_tanh(pre[t, j]) * table[token[t], offset + j]
//   residual_inject   x[t, :] = or += table[token[t], :] + vector      (table or vector optional)
//
// The residual is float, and so are all sums here.
#include "common.h"

namespace tlie {

__device__ __forceinline__ float gelu_tanh(float z) {
  return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <typename D, typename A>
__global__ void __launch_bounds__(256)
residual_update_kernel(float* __restrict__ residual, const D* __restrict__ a, int a_nsplit, size_t a_stride,
                       const D* __restrict__ b, int b_nsplit, size_t b_stride, float mult, size_t count,
                       A* __restrict__ copy, bool wide) {
  if (wide) {
    // eight elements a thread and load (no partial sums, a count that is a multiple of 8, addresses at multiples of 32 bytes)
    for (size_t i = (static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x) * 8; i < count; i += static_cast<size_t>(gridDim.x) * 2048) {
      float x[8], av[8], bv[8];
      load8(residual + i, x);
      load8(a + i, av);
      if (b != nullptr) load8(b + i, bv);
#pragma unroll
      for (int j = 0; j < 8; ++j) x[j] += mult * (b != nullptr ? av[j] + bv[j] : av[j]);
      store8(residual + i, x);
      if (copy != nullptr) store8(copy + i, x);
    }
    return;
  }
  for (size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x; i < count; i += static_cast<size_t>(gridDim.x) * 256) {
    float delta = sum_splits(a + i, a_nsplit, a_stride);
    if (b != nullptr) delta += sum_splits(b + i, b_nsplit, b_stride);
    const float v = residual[i] + mult * delta;
    residual[i] = v;
    if (copy != nullptr) copy[i] = from_float<A>(v);
  }
}

template <typename D, typename W, typename A>
__global__ void __launch_bounds__(256)
side_gate_kernel(const D* __restrict__ pre, int nsplit, size_t split_stride, const int* __restrict__ tokens,
                 const W* __restrict__ table, int table_row, int table_offset, int sd, A* __restrict__ out) {
  const int t = blockIdx.x;
  const W* e = table + static_cast<size_t>(tokens[t]) * table_row + table_offset;
  for (int j = threadIdx.x; j < sd; j += 256) {
    const float z = sum_splits(pre + static_cast<size_t>(t) * sd + j, nsplit, split_stride);
    out[static_cast<size_t>(t) * sd + j] = from_float<A>(gelu_tanh(z) * to_float(e[j]));
  }
}

template <typename W>
__global__ void __launch_bounds__(256)
residual_inject_kernel(float* __restrict__ residual, const int* __restrict__ tokens, const W* __restrict__ table,
                       const W* __restrict__ vector, int width, int accumulate) {
  const int t = blockIdx.x;
  float* x = residual + static_cast<size_t>(t) * width;
  const W* row = table != nullptr ? table + static_cast<size_t>(tokens[t]) * width : nullptr;
  for (int c = threadIdx.x; c < width; c += 256) {
    float v = accumulate ? x[c] : 0.f;
    if (row != nullptr) v += to_float(row[c]);
    if (vector != nullptr) v += to_float(vector[c]);
    x[c] = v;
  }
}

}  // namespace tlie

using namespace tlie;

// residual: float [count]; a, b (b may be null): products [nsplit][count] of in_dtype; copy (or null): [count] of copy_dtype.
extern "C" int tlie_residual_update(float* residual, const void* a, int a_nsplit, long long a_stride, const void* b,
                                    int b_nsplit, long long b_stride, int in_dtype, float mult, long long count, void* copy,
                                    int copy_dtype, void* stream) {
  if (count <= 0 || a == nullptr || a_nsplit < 1 || (b != nullptr && b_nsplit < 1)) return kBadArgument;
  const bool wide = a_nsplit == 1 && (b == nullptr || b_nsplit == 1) && (count & 7) == 0 &&
                    ((reinterpret_cast<uintptr_t>(residual) | reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) |
                      reinterpret_cast<uintptr_t>(copy)) & 31) == 0;
  long long blocks = wide ? (count / 8 + 255) / 256 : (count + 255) / 256;
  if (blocks > 65535LL * 16) blocks = 65535LL * 16;
  hipStream_t s = (hipStream_t)stream;
#define TLIE_CASE(DC, D, AC, A)                                                                                       \
  if (in_dtype == DC && copy_dtype == AC) {                                                                           \
    hipLaunchKernelGGL((residual_update_kernel<D, A>), dim3((unsigned)blocks), dim3(256), 0, s, residual, (const D*)a,  \
                       a_nsplit, (size_t)a_stride, (const D*)b, b_nsplit, (size_t)b_stride, mult, (size_t)count,       \
                       (A*)copy, wide);                                                                                     \
    return launch_status();                                                                                           \
  }
  TLIE_CASE(kF32, float, kF32, float)
  TLIE_CASE(kF32, float, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kF32, float)
#undef TLIE_CASE
  return kBadArgument;
}

// pre: a product [nsplit][tokens][sd] of in_dtype; tokens int32 [tokens]; table [vocab, table_row] of w_dtype, of which
// columns table_offset .. + sd are read; out [tokens, sd] of out_dtype.
extern "C" int tlie_side_gate(const void* pre, int in_dtype, int nsplit, long long split_stride, const int* tokens,
                              const void* table, int w_dtype, int table_row, int table_offset, int sd, void* out,
                              int out_dtype, int tokens_count, void* stream) {
  if (tokens_count <= 0 || sd <= 0 || nsplit < 1 || table_offset < 0 || table_offset + sd > table_row || tokens == nullptr ||
      table == nullptr)
    return kBadArgument;
  hipStream_t s = (hipStream_t)stream;
#define TLIE_CASE(DC, D, WC, W, AC, A)                                                                                \
  if (in_dtype == DC && w_dtype == WC && out_dtype == AC) {                                                           \
    hipLaunchKernelGGL((side_gate_kernel<D, W, A>), dim3(tokens_count), dim3(256), 0, s, (const D*)pre, nsplit,        \
                       (size_t)split_stride, tokens, (const W*)table, table_row, table_offset, sd, (A*)out);          \
    return launch_status();                                                                                           \
  }
  TLIE_CASE(kF32, float, kF32, float, kF32, float)
  TLIE_CASE(kF32, float, kBF16, bf16, kF32, float)
  TLIE_CASE(kF32, float, kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kF32, float, kF32, float, kBF16, bf16)
#undef TLIE_CASE
  return kBadArgument;
}

// residual[t, :] = (accumulate ? residual[t, :] : 0) + table[tokens[t], :] + vector; table [vocab, width] and
// vector [width] of w_dtype, either may be null.
extern "C" int tlie_residual_inject(float* residual, const int* tokens, const void* table, const void* vector, int w_dtype,
                                    int tokens_count, int width, int accumulate, void* stream) {
  if (tokens_count <= 0 || width <= 0 || (table != nullptr && tokens == nullptr)) return kBadArgument;
  hipStream_t s = (hipStream_t)stream;
  if (w_dtype == kF32)
    hipLaunchKernelGGL((residual_inject_kernel<float>), dim3(tokens_count), dim3(256), 0, s, residual, tokens,
                       (const float*)table, (const float*)vector, width, accumulate);
  else if (w_dtype == kBF16)
    hipLaunchKernelGGL((residual_inject_kernel<bf16>), dim3(tokens_count), dim3(256), 0, s, residual, tokens,
                       (const bf16*)table, (const bf16*)vector, width, accumulate);
  else
    return kBadArgument;
  return launch_status();
}
