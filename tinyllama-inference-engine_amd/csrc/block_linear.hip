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

// The same product on the matrix cores, for steps of many rows: bfloat16 weights kept as they are stored,
// [blocks][outer][inner]; x bfloat16, or float that is rounded to bfloat16 as it becomes an operand; float
// sums.  A wave takes 32 rows of x and 64 outputs of one block, a workgroup of four waves 128 rows: every
// operand goes from memory (the weights of a block are small: from the caches) straight into the registers
// of v_mfma_f32_16x16x32_bf16, whose A operand is 16 rows of the weight (a lane: row lane % 16, 8 inner values
// from (lane / 16) * 8 on) and whose B operand is 16 rows of x laid out alike; a lane then holds 4 consecutive
// outputs of one row of x.  inner % 32 == 0, and all offsets and strides of x multiples of 8 elements.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4_t;

__device__ __forceinline__ bf16x8_t operand_of(const bf16* p) { return *reinterpret_cast<const bf16x8_t*>(p); }
__device__ __forceinline__ bf16x8_t operand_of(const float* p) {
  const float4 lo = *reinterpret_cast<const float4*>(p), hi = *reinterpret_cast<const float4*>(p + 4);
  union { uint32_t w[4]; bf16x8_t v; } packed;
  packed.w[0] = pack_bf16(lo.x, lo.y), packed.w[1] = pack_bf16(lo.z, lo.w);
  packed.w[2] = pack_bf16(hi.x, hi.y), packed.w[3] = pack_bf16(hi.z, hi.w);
  return packed.v;
}

template <typename X, typename Y>
__global__ void __launch_bounds__(256)
block_linear_mfma_kernel(const X* __restrict__ x, long long x_row, long long x_block, const bf16* __restrict__ w,
                         const bf16* __restrict__ bias, Y* __restrict__ y, long long y_row, long long y_block, int rows,
                         int inner, int outer) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, col = lane & 15, grp = lane >> 4;
  const int b = blockIdx.y, row0 = blockIdx.x * 128 + wave * 32, out0 = blockIdx.z * 64;
  if (row0 >= rows) return;                        // (the whole wave)
  // rows and outputs past the end are read from the last one and not stored
  const X* x_at[2];
  const bf16* w_at[4];
#pragma unroll
  for (int r = 0; r < 2; ++r)
    x_at[r] = x + static_cast<size_t>(min(row0 + r * 16 + col, rows - 1)) * x_row + static_cast<size_t>(b) * x_block + grp * 8;
#pragma unroll
  for (int o = 0; o < 4; ++o)
    w_at[o] = w + (static_cast<size_t>(b) * outer + min(out0 + o * 16 + col, outer - 1)) * inner + grp * 8;
  floatx4_t acc[2][4];
#pragma unroll
  for (int r = 0; r < 2; ++r)
#pragma unroll
    for (int o = 0; o < 4; ++o) acc[r][o] = floatx4_t{0.f, 0.f, 0.f, 0.f};
  for (int k = 0; k < inner; k += 32) {
    bf16x8_t from_x[2], from_w[4];
#pragma unroll
    for (int r = 0; r < 2; ++r) from_x[r] = operand_of(x_at[r] + k);
#pragma unroll
    for (int o = 0; o < 4; ++o) from_w[o] = operand_of(w_at[o] + k);
#pragma unroll
    for (int r = 0; r < 2; ++r)
#pragma unroll
      for (int o = 0; o < 4; ++o) acc[r][o] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(from_w[o], from_x[r], acc[r][o], 0, 0, 0);
  }
  // acc[r][o][j] is output out0 + o * 16 + grp * 4 + j of row row0 + r * 16 + col
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    const int row = row0 + r * 16 + col;
    if (row >= rows) continue;
#pragma unroll
    for (int o = 0; o < 4; ++o)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int out = out0 + o * 16 + grp * 4 + j;
        if (out < outer) {
          const float shift = bias != nullptr ? to_float(bias[static_cast<size_t>(b) * outer + out]) : 0.f;
          y[static_cast<size_t>(row) * y_row + static_cast<size_t>(b) * y_block + out] = from_float<Y>(acc[r][o][j] + shift);
        }
      }
  }
}

}  // namespace tlie

using namespace tlie;

// w: bfloat16 [blocks][outer][inner] (as stored: [out, in] per block); otherwise as tlie_block_linear.
extern "C" int tlie_block_linear_mfma(const void* x, int x_dtype, long long x_row, long long x_block, const void* w,
                                      const void* bias, void* y, int y_dtype, long long y_row, long long y_block, int rows,
                                      int blocks, int inner, int outer, void* stream) {
  if (rows <= 0 || blocks <= 0 || blocks > 65535 || inner <= 0 || inner % 32 != 0 || outer <= 0) return kBadArgument;
  if (x_row % 8 != 0 || x_block % 8 != 0 || (reinterpret_cast<uintptr_t>(x) & (x_dtype == kF32 ? 31 : 15)) != 0 ||
      (reinterpret_cast<uintptr_t>(w) & 15) != 0)
    return kBadArgument;
  const dim3 grid((rows + 127) / 128, blocks, (outer + 63) / 64);
  if (grid.z > 65535) return kBadArgument;
  hipStream_t s = (hipStream_t)stream;
#define TLIE_CASE(XC, X, YC, Y)                                                                                   \
  if (x_dtype == XC && y_dtype == YC) {                                                                           \
    hipLaunchKernelGGL((block_linear_mfma_kernel<X, Y>), grid, dim3(256), 0, s, (const X*)x, x_row, x_block,        \
                       (const bf16*)w, (const bf16*)bias, (Y*)y, y_row, y_block, rows, inner, outer);             \
    return launch_status();                                                                                       \
  }
  TLIE_CASE(kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kF32, float)
  TLIE_CASE(kF32, float, kF32, float)
  TLIE_CASE(kF32, float, kBF16, bf16)
#undef TLIE_CASE
  return kBadArgument;
}

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
