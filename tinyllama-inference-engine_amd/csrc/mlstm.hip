// The matrix memory of an mLSTM layer, token by token.  Per head, with a query q (scaled by the caller's
// factor), a key k (dim values each) and a value v (vdim values), and two numbers a token, the log input gate
// i and the log forget gate f:
//   i = cap * tanh(pre_i / cap)          f = logsigmoid(cap * tanh(pre_f / cap))
//   m' = max(f + m, i)
//   S' = exp(f + m - m') S + exp(i - m') k v^T         (S: dim x vdim)
//   n' = exp(f + m - m') n + exp(i - m') k
//   o  = S'^T q / (max(|n' . q|, exp(-m')) + 1e-6)
// S, n and m are the request's state (zero when it is admitted) and are carried from step to step; all of
// this is float whatever type q, k and v come in.
//
// The gates do not depend on the memory: a first kernel walks each sequence's gates alone and leaves, per token and
// head, keep = exp(f + m - m'), take = exp(i - m') and exp(-m'), and the head's m after the step in the state.
//
// The memory itself: a workgroup is one wave and owns 64 columns of one head's S for one sequence of the step: lane l
// keeps column l of its tile, S[0 .. dim)[l], in registers, and walks tokens in order.  n is spread over the lanes
// (lane l keeps n[l], n[l + 64], ...), every tile keeps a copy of its own of n (so that no workgroup reads what
// another one writes), and the state row of a head is laid out tile by tile:
// [tiles][dim * 64 (S, [d][lane]) + dim (n) + 1 (m, the first tile's only)].  Queries and keys of four tokens at a time
// go through LDS (every lane needs all of them).
//
// A sequence that brings many tokens is taken in slices of 32 tokens that run side by side: every slice is walked
// from a memory of zero and leaves where it ends and the product of its keeps (S' = keep S + take k v^T is linear
// in S); a second kernel gives every slice its start, start(c + 1) = keeps(c) * start(c) + end(c), and the state its
// new value; a third walks every slice again from its start and writes the results.
#include "common.h"

namespace tlie {

constexpr int kMlstmBatch = 4, kMlstmSlice = 32;

// gates: float [tokens, 2 * heads] (input gates' pre-activations, then forget gates'); values: float [tokens, heads, 4]
// (keep, take, exp(-m), unused).  One wave per (sequence, head); m is the state's, read and written here only.
__global__ void __launch_bounds__(64)
mlstm_gates_kernel(const float* __restrict__ gates, float* __restrict__ values, float* __restrict__ state,
                   const int* __restrict__ seq_start, const int* __restrict__ seq_slot, int heads, size_t head_floats,
                   size_t m_offset, float cap) {
  const int seq = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int slot = seq_slot[seq];
  if (slot < 0) return;
  const int first = seq_start[seq], last = seq_start[seq + 1];
  if (first >= last) return;
  float* m_place = state + (static_cast<size_t>(slot) * heads + h) * head_floats + m_offset;
  float m = *m_place;
  // (a chunk's two pre-activations are asked for while the chunk before it is worked on)
  float pre_i = first + lane < last ? gates[static_cast<size_t>(first + lane) * 2 * heads + h] : 0.f;
  float pre_f = first + lane < last ? gates[static_cast<size_t>(first + lane) * 2 * heads + heads + h] : 0.f;
  for (int t0 = first; t0 < last; t0 += 64) {
    const int t = t0 + lane, count = min(64, last - t0);
    const float now_i = pre_i, now_f = pre_f;
    if (t + 64 < last) {
      pre_i = gates[static_cast<size_t>(t + 64) * 2 * heads + h];
      pre_f = gates[static_cast<size_t>(t + 64) * 2 * heads + heads + h];
    }
    float ig = 0.f, fg = 0.f;
    if (lane < count) {
      ig = cap * tanhf(now_i / cap);
      const float x = cap * tanhf(now_f / cap);
      fg = fminf(x, 0.f) - log1pf(expf(-fabsf(x)));
    }
    // m' = max(m + f, i) token by token is a chain of the maps m -> max(m + F, I); two in a row are one of the same
    // kind, (F1 + F2, max(I1 + F2, I2)), so the wave forms every token's map of all tokens up to it in six steps
    float F = lane < count ? fg : 0.f, I = lane < count ? ig : -INFINITY;
#pragma unroll
    for (int offset = 1; offset < 64; offset <<= 1) {
      const float Fb = __shfl_up(F, offset, 64), Ib = __shfl_up(I, offset, 64);
      if (lane >= offset) {
        I = fmaxf(Ib + F, I);
        F = Fb + F;
      }
    }
    const float after = fmaxf(m + F, I);               // m after this lane's token
    float before = __shfl_up(after, 1, 64);
    if (lane == 0) before = m;
    if (lane < count) {
      float4 out;
      out.x = expf(fg + before - after), out.y = expf(ig - after), out.z = expf(-after), out.w = 0.f;
      *reinterpret_cast<float4*>(values + (static_cast<size_t>(t) * heads + h) * 4) = out;
    }
    m = __shfl(after, count - 1, 64);
  }
  if (lane == 0) *m_place = m;
}

// MODE 0: the sequence's tokens of the step from the state, results and the new state written.
// MODE 1: a slice from zero; no results; where it ends and the product of its keeps go to `parts`.
// MODE 2: a slice from the start that `parts` now holds for it; results written.
// parts: float [sequences, slices, heads, tiles, dim * 64 + dim + 1] (S, n, the product of the slice's keeps).
// A workgroup has WAVES waves; wave w keeps dims w * DW .. (w + 1) * DW of its lanes' columns of S (and of n), so that
// a column of up to 256 dims stays in registers; the waves' parts of a token's sums meet in LDS, once a batch.
// (Measured at 8 heads, a prompt of 2048 tokens and a decode step of 8 requests: 128 x 256 as 1 x 128, 2 x 64, 4 x 32
// dims: 324, 239, 311 us and 30, 18, 13 us; 256 x 512 as 1 x 256, 2 x 128, 4 x 64: 2171, 1390, 990 us and 39, 34, 22 us:
// a step of single tokens takes four waves, a sliced walk two up to 128 dims and four beyond.)
template <typename D, int DW, int WAVES, int MODE>
__global__ void __launch_bounds__(64 * WAVES)
mlstm_scan_kernel(const D* __restrict__ fused, int nsplit, size_t split_stride, int row_width, int q_col, int k_col,
                  int v_col, const float* __restrict__ values, float* __restrict__ state, float* __restrict__ parts,
                  const int* __restrict__ seq_start, const int* __restrict__ seq_slot, float* __restrict__ out, int heads,
                  int dim, int vdim, int tiles, int slices, float q_scale) {
  constexpr int NJ = DW >= 64 ? DW / 64 : 1, DMAX = DW * WAVES;
  __shared__ __attribute__((aligned(16))) float qs[kMlstmBatch][DMAX];
  __shared__ __attribute__((aligned(16))) float ks[kMlstmBatch][DMAX];
  __shared__ float met[WAVES][kMlstmBatch][65];        // a wave's part of a token's S^T q (64 lanes) and of n . q
  const int seq = MODE == 0 ? blockIdx.x : blockIdx.x / slices, slice = MODE == 0 ? 0 : blockIdx.x % slices;
  const int h = blockIdx.y, tile = blockIdx.z, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int base = wave * DW;                          // this wave's first dim
  const int slot = seq_slot[seq];
  if (slot < 0) return;                                // a sequence that pads a recorded step: no state is its own
  int first = seq_start[seq], last = seq_start[seq + 1];
  if (MODE != 0) {
    first += slice * kMlstmSlice;
    last = min(last, first + kMlstmSlice);
  }
  if (first >= last) return;
  const int col = tile * 64 + lane;
  const bool live = col < vdim;
  const size_t tile_floats = static_cast<size_t>(dim) * 64 + dim + 1;
  float* st = MODE == 0 ? state + ((static_cast<size_t>(slot) * heads + h) * tiles + tile) * tile_floats
                        : parts + (((static_cast<size_t>(seq) * slices + slice) * heads + h) * tiles + tile) * tile_floats;
  float S[DW];
  float n[NJ];
#pragma unroll
  for (int d = 0; d < DW; ++d) S[d] = MODE != 1 && base + d < dim ? st[(base + d) * 64 + lane] : 0.f;
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const int d = base + lane + 64 * j;
    n[j] = MODE != 1 && lane + 64 * j < DW && d < dim ? st[static_cast<size_t>(dim) * 64 + d] : 0.f;
  }
  float keeps = 1.f;

  // a batch of tokens is asked for while the batch before it is worked on: its queries, keys, values and gates wait
  // in registers (a wave is alone on its SIMD where slices are few, and nothing else would hide the loads' way)
  float rq[kMlstmBatch][NJ], rk[kMlstmBatch][NJ], rv[kMlstmBatch];
  float4 rg[kMlstmBatch];
  auto fetch = [&](int t0) {
    const int nb = min(kMlstmBatch, last - t0);
#pragma unroll
    for (int b = 0; b < kMlstmBatch; ++b) {
      const D* row = fused + static_cast<size_t>(t0 + b) * row_width;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int d = base + lane + 64 * j;
        const bool there = b < nb && lane + 64 * j < DW && d < dim;
        rq[b][j] = MODE != 1 && there ? sum_splits(row + q_col + h * dim + d, nsplit, split_stride) * q_scale : 0.f;
        rk[b][j] = there ? sum_splits(row + k_col + h * dim + d, nsplit, split_stride) : 0.f;
      }
      rv[b] = b < nb && live ? sum_splits(row + v_col + h * vdim + col, nsplit, split_stride) : 0.f;
      rg[b] = b < nb ? *reinterpret_cast<const float4*>(values + (static_cast<size_t>(t0 + b) * heads + h) * 4)
                     : make_float4(1.f, 0.f, 1.f, 0.f);
    }
  };
  fetch(first);
  for (int t0 = first; t0 < last; t0 += kMlstmBatch) {
    const int nb = min(kMlstmBatch, last - t0);
    __syncthreads();                                   // the batch before has been read
    float vv[kMlstmBatch], keep[kMlstmBatch], take[kMlstmBatch], floor_[kMlstmBatch];
#pragma unroll
    for (int b = 0; b < kMlstmBatch; ++b) {
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        if (lane + 64 * j < DW) {
          if (MODE != 1) qs[b][base + lane + 64 * j] = rq[b][j];
          ks[b][base + lane + 64 * j] = rk[b][j];
        }
      }
      vv[b] = rv[b], keep[b] = rg[b].x, take[b] = rg[b].y, floor_[b] = rg[b].z;
    }
    __syncthreads();
    if (t0 + kMlstmBatch < last) fetch(t0 + kMlstmBatch);
    float top[kMlstmBatch], under[kMlstmBatch];         // this wave's part of S^T q and of n . q, a token each
#pragma unroll
    for (int b = 0; b < kMlstmBatch; ++b) {
      top[b] = under[b] = 0.f;
      if (b >= nb) continue;                           // (the same for the whole wave)
      const float tv = take[b] * vv[b];
      float acc = 0.f;
#pragma unroll
      for (int d0 = 0; d0 < DW; d0 += 4) {
        if (base + d0 < dim) {                         // (entries from dim on are zeros in LDS and stay zeros in S)
          const float4 k4 = *reinterpret_cast<const float4*>(&ks[b][base + d0]);
          S[d0 + 0] = keep[b] * S[d0 + 0] + k4.x * tv;
          S[d0 + 1] = keep[b] * S[d0 + 1] + k4.y * tv;
          S[d0 + 2] = keep[b] * S[d0 + 2] + k4.z * tv;
          S[d0 + 3] = keep[b] * S[d0 + 3] + k4.w * tv;
          if (MODE != 1) {
            const float4 q4 = *reinterpret_cast<const float4*>(&qs[b][base + d0]);
            acc += S[d0 + 0] * q4.x;
            acc += S[d0 + 1] * q4.y;
            acc += S[d0 + 2] * q4.z;
            acc += S[d0 + 3] * q4.w;
          }
        }
      }
      float partial = 0.f;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        if (lane + 64 * j < DW) {
          n[j] = keep[b] * n[j] + take[b] * ks[b][base + lane + 64 * j];
          if (MODE != 1) partial += n[j] * qs[b][base + lane + 64 * j];
        }
      }
      if (MODE == 1) keeps *= keep[b];
      else top[b] = acc, under[b] = wave_sum(partial);
    }
    if (MODE == 1) continue;
    if (WAVES > 1) {
#pragma unroll
      for (int b = 0; b < kMlstmBatch; ++b) {
        met[wave][b][lane] = top[b];
        if (lane == 0) met[wave][b][64] = under[b];
      }
      __syncthreads();
      if (wave != 0) continue;
#pragma unroll
      for (int b = 0; b < kMlstmBatch; ++b) {
#pragma unroll
        for (int w = 1; w < WAVES; ++w) top[b] += met[w][b][lane], under[b] += met[w][b][64];
      }
    }
#pragma unroll
    for (int b = 0; b < kMlstmBatch; ++b) {
      if (b >= nb) continue;
      const float bottom = fmaxf(fabsf(under[b]), floor_[b]) + 1e-6f;
      if (live) out[(static_cast<size_t>(t0 + b) * heads + h) * vdim + col] = top[b] / bottom;
    }
  }
  if (MODE == 2) return;
#pragma unroll
  for (int d = 0; d < DW; ++d)
    if (base + d < dim) st[(base + d) * 64 + lane] = S[d];
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const int d = base + lane + 64 * j;
    if (lane + 64 * j < DW && d < dim) st[static_cast<size_t>(dim) * 64 + d] = n[j];
  }
  if (MODE == 1 && threadIdx.x == 0) st[static_cast<size_t>(dim) * 64 + dim] = keeps;
}

// Every slice's start from the state and the slices before it, in place: where a slice's end stood its start stands
// afterwards; the state gets what the last slice leaves.  A thread an element of (S, n) of a (sequence, head, tile).
__global__ void __launch_bounds__(256)
mlstm_carry_kernel(float* __restrict__ parts, float* __restrict__ state, const int* __restrict__ seq_start,
                   const int* __restrict__ seq_slot, int heads, int tiles, int slices, int dim) {
  const int seq = blockIdx.x, unit = blockIdx.y;       // unit: head * tiles + tile
  const int slot = seq_slot[seq];
  if (slot < 0) return;
  const int count = seq_start[seq + 1] - seq_start[seq];
  const int used = (count + kMlstmSlice - 1) / kMlstmSlice;
  const size_t tile_floats = static_cast<size_t>(dim) * 64 + dim + 1;
  const int elements = dim * 64 + dim;
  float* st = state + (static_cast<size_t>(slot) * heads * tiles + unit) * tile_floats;
  for (int e = blockIdx.z * 256 + threadIdx.x; e < elements; e += gridDim.z * 256) {
    float value = st[e];
    const size_t stride = static_cast<size_t>(heads) * tiles * tile_floats;
    float* part = parts + (static_cast<size_t>(seq) * slices * heads * tiles + unit) * tile_floats;
    int c = 0;
    for (; c + 4 <= used; c += 4) {                    // (four slices' ends asked for together; the chain is the sums' only)
      float end[4], keeps[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) end[u] = part[(c + u) * stride + e], keeps[u] = part[(c + u) * stride + elements];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        part[(c + u) * stride + e] = value;
        value = keeps[u] * value + end[u];
      }
    }
    for (; c < used; ++c) {
      const float end = part[c * stride + e], keeps = part[c * stride + elements];
      part[c * stride + e] = value;
      value = keeps * value + end;
    }
    if (used > 0) st[e] = value;
  }
}

}  // namespace tlie

using namespace tlie;

// fused: a product [nsplit][tokens][row_width] whose columns q_col .. hold the heads' queries (dim each), k_col ..
// their keys, v_col .. their values (vdim each); gates: float [tokens, 2 * heads], the input gates' and then the
// forget gates' pre-activations; values: float [tokens, heads, 4], scratch for what the gates become; state: float
// [slots, heads, tiles, dim * 64 + dim + 1], tiles = ceil(vdim / 64); seq_start [sequences + 1], seq_slot [sequences]
// (negative: skipped); out: float [tokens, heads * vdim].  slices 0: every sequence's tokens are walked in order;
// slices > 0 (at least ceil(most tokens of a sequence / 32)): in slices of 32 tokens side by side, with parts: float
// [sequences, slices, heads, tiles, dim * 64 + dim + 1] as scratch.
extern "C" int tlie_mlstm_scan(const void* fused, int dtype, int nsplit, long long split_stride, int row_width, int q_col,
                               int k_col, int v_col, const float* gates, float* values, float* state, const int* seq_start,
                               const int* seq_slot, float* out, int sequences, int heads, int dim, int vdim, float cap,
                               float q_scale, int slices, float* parts, void* stream) {
  if (sequences <= 0 || heads <= 0 || dim <= 0 || dim > 256 || vdim <= 0 || nsplit < 1 || !(cap > 0.f)) return kBadArgument;
  const int tiles = (vdim + 63) / 64;
  if (heads > 65535 || tiles > 65535 || slices < 0 || (slices > 0 && parts == nullptr) || values == nullptr) return kBadArgument;
  if (q_col < 0 || k_col < 0 || v_col < 0 || q_col + heads * dim > row_width || k_col + heads * dim > row_width ||
      v_col + heads * vdim > row_width)
    return kBadArgument;
  hipStream_t s = (hipStream_t)stream;
  const size_t tile_floats = static_cast<size_t>(dim) * 64 + dim + 1;
  hipLaunchKernelGGL(mlstm_gates_kernel, dim3(sequences, heads), dim3(64), 0, s, gates, values, state, seq_start, seq_slot,
                     heads, tiles * tile_floats, tile_floats - 1, cap);
  if (launch_status() != kOk) return kLaunchFailed;
#define TLIE_LAUNCH(D, DW, WAVES, MODE, GRID)                                                                         \
  hipLaunchKernelGGL((mlstm_scan_kernel<D, DW, WAVES, MODE>), GRID, dim3(64 * WAVES), 0, s, (const D*)fused, nsplit,   \
                     (size_t)split_stride, row_width, q_col, k_col, v_col, values, state, parts, seq_start, seq_slot,  \
                     out, heads, dim, vdim, tiles, slices, q_scale)
#define TLIE_SIZES(D, MODE, GRID)                                                                                     \
  if (dim <= 32) TLIE_LAUNCH(D, 32, 1, MODE, GRID);                                                                   \
  else if (dim <= 64) { if (MODE == 0) TLIE_LAUNCH(D, 32, 2, MODE, GRID); else TLIE_LAUNCH(D, 64, 1, MODE, GRID); }   \
  else if (dim <= 128) { if (MODE == 0) TLIE_LAUNCH(D, 32, 4, MODE, GRID); else TLIE_LAUNCH(D, 64, 2, MODE, GRID); }  \
  else TLIE_LAUNCH(D, 64, 4, MODE, GRID)
#define TLIE_TYPES(MODE, GRID)                                                                                        \
  if (dtype == kF32) { TLIE_SIZES(float, MODE, GRID); }                                                               \
  else if (dtype == kBF16) { TLIE_SIZES(bf16, MODE, GRID); }                                                          \
  else return kBadArgument
  if (slices == 0) {
    const dim3 grid(sequences, heads, tiles);
    TLIE_TYPES(0, grid);
    return launch_status();
  }
  if (static_cast<long long>(sequences) * slices > 2147483647LL) return kBadArgument;
  const dim3 sliced(sequences * slices, heads, tiles);
  TLIE_TYPES(1, sliced);
  if (launch_status() != kOk) return kLaunchFailed;
  const int elements = dim * 64 + dim;
  int across = (elements + 255) / 256;
  if (across > 16) across = 16;
  if (heads * tiles > 65535) return kBadArgument;
  hipLaunchKernelGGL(mlstm_carry_kernel, dim3(sequences, heads * tiles, across), dim3(256), 0, s, parts, state, seq_start,
                     seq_slot, heads, tiles, slices, dim);
  if (launch_status() != kOk) return kLaunchFailed;
  TLIE_TYPES(2, sliced);
#undef TLIE_TYPES
#undef TLIE_SIZES
#undef TLIE_LAUNCH
  return launch_status();
}
