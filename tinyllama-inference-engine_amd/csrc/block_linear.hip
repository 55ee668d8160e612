// Block-diagonal products: the columns of x fall into `blocks` parts and part b is multiplied by a
// matrix of its own,
//     y[t, b, o] = sum_i x[t, b, i] * w[b][i][o] (+ bias[b][o]),
// with float sums.  The gates of a gated linear recurrence are such products (the recurrence's channels
// in blocks), and so are the per-head products of latent attention (a head's queries onto the latent
// space, its attended latent vector onto the head's values).  The weights are kept transposed, [in][out]
// per block, so that neighbouring threads read neighbouring outputs.
//
// x and y are addressed by strides (a row's, a block's), so that a part of a wider array can be read
// (the unrotated dims of every head's query) or written (the first dims of every head's key-side query)
// where it lies.  A workgroup takes 16 rows of x and 64 outputs of one block; x passes through LDS in
// pieces of 128 inner values, and a sum is one chain of additions in the order of the inner index,
// whatever the step's rows are: a row's result does not depend on how the step was cut.
#include "common.h"

namespace tlie {

constexpr int kBlockRows = 16, kBlockCols = 64, kBlockInner = 128;

template <typename X, typename W, typename Y>
__global__ void __launch_bounds__(256)
block_linear_kernel(const X* __restrict__ x, long long x_row, long long x_block, const W* __restrict__ wt,
                    const W* __restrict__ bias, Y* __restrict__ y, long long y_row, long long y_block, int rows,
                    int inner, int outer) {
  __shared__ float tile[kBlockRows][kBlockInner];
  const int b = blockIdx.y, row0 = blockIdx.x * kBlockRows;
  const int o = blockIdx.z * kBlockCols + (threadIdx.x & 63), quarter = threadIdx.x >> 6;   // rows quarter * 4 .. + 3 of the tile
  const W* w = wt + static_cast<size_t>(b) * inner * outer;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < inner; k0 += kBlockInner) {
    __syncthreads();                               // the piece before has been read
    for (int e = threadIdx.x; e < kBlockRows * kBlockInner; e += 256) {
      const int r = e / kBlockInner, i = e % kBlockInner;
      tile[r][i] = (row0 + r < rows && k0 + i < inner)
                       ? to_float(x[static_cast<size_t>(row0 + r) * x_row + static_cast<size_t>(b) * x_block + k0 + i]) : 0.f;
    }
    __syncthreads();
    if (o < outer) {
      const int count = min(kBlockInner, inner - k0);
      for (int i = 0; i < count; ++i) {
        const float weight = to_float(w[static_cast<size_t>(k0 + i) * outer + o]);
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] += tile[quarter * 4 + j][i] * weight;
      }
    }
  }
  if (o >= outer) return;
  const float shift = bias != nullptr ? to_float(bias[static_cast<size_t>(b) * outer + o]) : 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int r = row0 + quarter * 4 + j;
    if (r < rows) y[static_cast<size_t>(r) * y_row + static_cast<size_t>(b) * y_block + o] = from_float<Y>(acc[j] + shift);
  }
}

}  // namespace tlie

using namespace tlie;

// x: rows of x_row elements, block b's `inner` values from b * x_block on; wt: [blocks][inner][outer];
// bias: [blocks][outer] or null; y: rows of y_row elements, block b's `outer` results from b * y_block on.
// The caller has checked that the strides keep every access inside its array.
extern "C" int tlie_block_linear(const void* x, int x_dtype, long long x_row, long long x_block, const void* wt, int w_dtype,
                                 const void* bias, void* y, int y_dtype, long long y_row, long long y_block, int rows,
                                 int blocks, int inner, int outer, void* stream) {
  if (rows <= 0 || blocks <= 0 || blocks > 65535 || inner <= 0 || outer <= 0) return kBadArgument;
  const dim3 grid((rows + kBlockRows - 1) / kBlockRows, blocks, (outer + kBlockCols - 1) / kBlockCols);
  if (grid.z > 65535) return kBadArgument;
  hipStream_t s = (hipStream_t)stream;
#define TLIE_CASE(XC, X, WC, W, YC, Y)                                                                            \
  if (x_dtype == XC && w_dtype == WC && y_dtype == YC) {                                                           \
    hipLaunchKernelGGL((block_linear_kernel<X, W, Y>), grid, dim3(256), 0, s, (const X*)x, x_row, x_block,          \
                       (const W*)wt, (const W*)bias, (Y*)y, y_row, y_block, rows, inner, outer);                   \
    return launch_status();                                                                                        \
  }
  TLIE_CASE(kF32, float, kF32, float, kF32, float)
  TLIE_CASE(kBF16, bf16, kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kBF16, bf16, kF32, float)
  TLIE_CASE(kF32, float, kBF16, bf16, kF32, float)
  TLIE_CASE(kF32, float, kBF16, bf16, kBF16, bf16)
#undef TLIE_CASE
  return kBadArgument;
}
