// What a layer that runs its sublayers side by side does to the residual, and a per-layer token input after it.
//
//   residual_update   x[t, :] += mult * (a[t, :] + b[t, :])            a, b: products (b optional)
//   ... with a side input, then, with e = table[token[t], offset .. offset + sd):
//                     g = gelu_tanh(gate x) * e           gate: [sd, width], on the x just brought up to date
//                     y = proj g                          proj: [width, sd]
//                     x += mult * y / sqrt(mean(y^2) + eps) * norm
//   residual_inject   x[t, :] = or += table[token[t], :] + vector      (table or vector optional)
//
// The residual is float, and so are all sums here; a token is a workgroup's.
#include "common.h"

namespace tlie {

__device__ __forceinline__ float gelu_tanh(float z) {
  return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <typename D, typename W>
__global__ void __launch_bounds__(256)
residual_update_kernel(float* __restrict__ residual, const D* __restrict__ a, int a_nsplit, size_t a_stride,
                       const D* __restrict__ b, int b_nsplit, size_t b_stride, float mult, int width,
                       const int* __restrict__ tokens, const W* __restrict__ table, int table_row, int table_offset, int sd,
                       const W* __restrict__ gate, const W* __restrict__ proj, const W* __restrict__ norm, float eps) {
  extern __shared__ float lds[];
  float* xs = lds;                                     // width: the residual after the sublayers
  float* ys = xs + width;                              // width: the side input before its norm
  float* gs = ys + width;                              // sd
  float* scratch = gs + sd;                            // 16
  const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float* x = residual + static_cast<size_t>(t) * width;
  for (int c = threadIdx.x; c < width; c += 256) {
    float delta = sum_splits(a + static_cast<size_t>(t) * width + c, a_nsplit, a_stride);
    if (b != nullptr) delta += sum_splits(b + static_cast<size_t>(t) * width + c, b_nsplit, b_stride);
    const float v = x[c] + mult * delta;
    if (table == nullptr) x[c] = v;
    else xs[c] = v;
  }
  if (table == nullptr) return;                        // (the same for every thread)
  __syncthreads();
  const W* e = table + static_cast<size_t>(tokens[t]) * table_row + table_offset;
  for (int j = wave; j < sd; j += 4) {
    const W* weights = gate + static_cast<size_t>(j) * width;
    float sum = 0.f;
    for (int c = lane; c < width; c += 64) sum += to_float(weights[c]) * xs[c];
    sum = wave_sum(sum);
    if (lane == 0) gs[j] = gelu_tanh(sum) * to_float(e[j]);
  }
  __syncthreads();
  float squares = 0.f;
  for (int c = threadIdx.x; c < width; c += 256) {
    const W* weights = proj + static_cast<size_t>(c) * sd;
    float y = 0.f;
    for (int j = 0; j < sd; ++j) y += to_float(weights[j]) * gs[j];
    ys[c] = y;
    squares += y * y;
  }
  const float r = 1.f / sqrtf(block_sum(squares, scratch) / static_cast<float>(width) + eps);
  for (int c = threadIdx.x; c < width; c += 256) x[c] = xs[c] + mult * ys[c] * r * to_float(norm[c]);
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

// residual: float [tokens, width]; a, b (b may be null): products [nsplit][tokens][width] of in_dtype.  With a side input
// (table not null): tokens int32 [tokens]; table [vocab, table_row] of which columns table_offset .. + sd are this layer's;
// gate [sd, width], proj [width, sd], norm [width], all of w_dtype.
extern "C" int tlie_residual_update(float* residual, const void* a, int a_nsplit, long long a_stride, const void* b,
                                    int b_nsplit, long long b_stride, int in_dtype, float mult, int tokens_count, int width,
                                    const int* tokens, const void* table, int table_row, int table_offset, int sd,
                                    const void* gate, const void* proj, const void* norm, int w_dtype, float eps,
                                    void* stream) {
  if (tokens_count <= 0 || width <= 0 || a == nullptr || a_nsplit < 1 || (b != nullptr && b_nsplit < 1)) return kBadArgument;
  size_t lds = 0;
  if (table != nullptr) {
    if (tokens == nullptr || gate == nullptr || proj == nullptr || norm == nullptr || sd <= 0 || table_offset < 0 ||
        table_offset + sd > table_row || !(eps > 0.f))
      return kBadArgument;
    lds = (2 * static_cast<size_t>(width) + sd + 16) * sizeof(float);
    if (lds > 64 * 1024) return kBadArgument;
  }
  hipStream_t s = (hipStream_t)stream;
#define TLIE_CASE(DC, D, WC, W)                                                                                       \
  if (in_dtype == DC && w_dtype == WC) {                                                                              \
    hipLaunchKernelGGL((residual_update_kernel<D, W>), dim3(tokens_count), dim3(256), lds, s, residual, (const D*)a,   \
                       a_nsplit, (size_t)a_stride, (const D*)b, b_nsplit, (size_t)b_stride, mult, width, tokens,       \
                       (const W*)table, table_row, table_offset, sd, (const W*)gate, (const W*)proj, (const W*)norm,   \
                       eps);                                                                                          \
    return launch_status();                                                                                           \
  }
  TLIE_CASE(kF32, float, kF32, float)
  TLIE_CASE(kF32, float, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kF32, float)
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
