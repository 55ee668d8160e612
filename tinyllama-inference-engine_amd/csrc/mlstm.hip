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
// A workgroup is one wave and owns 64 columns of one head's S for one sequence of the step: lane l keeps
// column l of its tile, S[0 .. dim)[l], in registers, and walks the sequence's tokens of the step in order.
// n is spread over the lanes (lane l keeps n[l], n[l + 64], ...), every tile keeps a copy of its own of n
// and m (so that no workgroup reads what another one writes), and the state row of a head is laid out tile
// by tile: [tiles][dim * 64 (S, [d][lane]) + dim (n) + 1 (m)].  Queries and keys of four tokens at a time go
// through LDS (every lane needs all of them); the order of a token's sums never depends on how the step
// was cut or on what else is in it.
#include "common.h"

namespace tlie {

constexpr int kMlstmBatch = 4;

template <typename D, int DMAX>
__global__ void __launch_bounds__(64)
mlstm_scan_kernel(const D* __restrict__ fused, int nsplit, size_t split_stride, int row_width, int q_col, int k_col,
                  int v_col, const float* __restrict__ gates, float* __restrict__ state,
                  const int* __restrict__ seq_start, const int* __restrict__ seq_slot, float* __restrict__ out, int heads,
                  int dim, int vdim, int tiles, float cap, float q_scale) {
  constexpr int NJ = DMAX >= 64 ? DMAX / 64 : 1;
  __shared__ __attribute__((aligned(16))) float qs[kMlstmBatch][DMAX];
  __shared__ __attribute__((aligned(16))) float ks[kMlstmBatch][DMAX];
  const int seq = blockIdx.x, h = blockIdx.y, tile = blockIdx.z, lane = threadIdx.x;
  const int slot = seq_slot[seq];
  if (slot < 0) return;                                // a sequence that pads a recorded step: no state is its own
  const int first = seq_start[seq], last = seq_start[seq + 1];
  if (first >= last) return;
  const int col = tile * 64 + lane;
  const bool live = col < vdim;
  const size_t tile_floats = static_cast<size_t>(dim) * 64 + dim + 1;
  float* st = state + ((static_cast<size_t>(slot) * heads + h) * tiles + tile) * tile_floats;
  float S[DMAX];
#pragma unroll
  for (int d = 0; d < DMAX; ++d) S[d] = d < dim ? st[d * 64 + lane] : 0.f;
  float n[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const int d = lane + 64 * j;
    n[j] = d < dim ? st[static_cast<size_t>(dim) * 64 + d] : 0.f;
  }
  float m = st[static_cast<size_t>(dim) * 64 + dim];
  const int gate_row = 2 * heads;

  for (int t0 = first; t0 < last; t0 += kMlstmBatch) {
    const int nb = min(kMlstmBatch, last - t0);
    __syncthreads();                                   // the batch before has been read
    float vv[kMlstmBatch], gi[kMlstmBatch], gf[kMlstmBatch];
#pragma unroll
    for (int b = 0; b < kMlstmBatch; ++b) {
      const D* row = fused + static_cast<size_t>(t0 + b) * row_width;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int d = lane + 64 * j;
        if (d < DMAX) {
          const bool there = b < nb && d < dim;
          qs[b][d] = there ? sum_splits(row + q_col + h * dim + d, nsplit, split_stride) * q_scale : 0.f;
          ks[b][d] = there ? sum_splits(row + k_col + h * dim + d, nsplit, split_stride) : 0.f;
        }
      }
      vv[b] = b < nb && live ? sum_splits(row + v_col + h * vdim + col, nsplit, split_stride) : 0.f;
      gi[b] = b < nb ? gates[static_cast<size_t>(t0 + b) * gate_row + h] : 0.f;
      gf[b] = b < nb ? gates[static_cast<size_t>(t0 + b) * gate_row + heads + h] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int b = 0; b < kMlstmBatch; ++b) {
      if (b >= nb) break;                              // (the same for the whole wave)
      const float ig = cap * tanhf(gi[b] / cap);
      const float x = cap * tanhf(gf[b] / cap);
      const float fg = fminf(x, 0.f) - log1pf(expf(-fabsf(x)));
      const float m_new = fmaxf(fg + m, ig);
      const float keep = expf(fg + m - m_new), take = expf(ig - m_new);
      m = m_new;
      const float tv = take * vv[b];
      float acc = 0.f;
#pragma unroll
      for (int d0 = 0; d0 < DMAX; d0 += 4) {
        if (d0 < dim) {                                // (entries from dim on are zeros in LDS and stay zeros in S)
          const float4 k4 = *reinterpret_cast<const float4*>(&ks[b][d0]);
          const float4 q4 = *reinterpret_cast<const float4*>(&qs[b][d0]);
          S[d0 + 0] = keep * S[d0 + 0] + k4.x * tv;
          acc += S[d0 + 0] * q4.x;
          S[d0 + 1] = keep * S[d0 + 1] + k4.y * tv;
          acc += S[d0 + 1] * q4.y;
          S[d0 + 2] = keep * S[d0 + 2] + k4.z * tv;
          acc += S[d0 + 2] * q4.z;
          S[d0 + 3] = keep * S[d0 + 3] + k4.w * tv;
          acc += S[d0 + 3] * q4.w;
        }
      }
      float partial = 0.f;
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int d = lane + 64 * j;
        if (d < DMAX) {
          n[j] = keep * n[j] + take * ks[b][d];
          partial += n[j] * qs[b][d];
        }
      }
      const float nq = wave_sum(partial);
      const float bottom = fmaxf(fabsf(nq), expf(-m)) + 1e-6f;
      if (live) out[(static_cast<size_t>(t0 + b) * heads + h) * vdim + col] = acc / bottom;
    }
  }
#pragma unroll
  for (int d = 0; d < DMAX; ++d)
    if (d < dim) st[d * 64 + lane] = S[d];
#pragma unroll
  for (int j = 0; j < NJ; ++j) {
    const int d = lane + 64 * j;
    if (d < dim) st[static_cast<size_t>(dim) * 64 + d] = n[j];
  }
  if (lane == 0) st[static_cast<size_t>(dim) * 64 + dim] = m;
}

}  // namespace tlie

using namespace tlie;

// fused: a product [nsplit][tokens][row_width] whose columns q_col .. hold the heads' queries (dim each), k_col ..
// their keys, v_col .. their values (vdim each); gates: float [tokens, 2 * heads], the input gates' and then the
// forget gates' pre-activations; state: float [slots, heads, tiles, dim * 64 + dim + 1], tiles = ceil(vdim / 64);
// seq_start [sequences + 1], seq_slot [sequences] (negative: skipped); out: float [tokens, heads * vdim].
extern "C" int tlie_mlstm_scan(const void* fused, int dtype, int nsplit, long long split_stride, int row_width, int q_col,
                               int k_col, int v_col, const float* gates, float* state, const int* seq_start,
                               const int* seq_slot, float* out, int sequences, int heads, int dim, int vdim, float cap,
                               float q_scale, void* stream) {
  if (sequences <= 0 || heads <= 0 || dim <= 0 || dim > 256 || vdim <= 0 || nsplit < 1 || !(cap > 0.f)) return kBadArgument;
  const int tiles = (vdim + 63) / 64;
  if (heads > 65535 || tiles > 65535) return kBadArgument;
  if (q_col < 0 || k_col < 0 || v_col < 0 || q_col + heads * dim > row_width || k_col + heads * dim > row_width ||
      v_col + heads * vdim > row_width)
    return kBadArgument;
  const dim3 grid(sequences, heads, tiles);
  hipStream_t s = (hipStream_t)stream;
#define TLIE_LAUNCH(D, DMAX)                                                                                          \
  hipLaunchKernelGGL((mlstm_scan_kernel<D, DMAX>), grid, dim3(64), 0, s, (const D*)fused, nsplit, (size_t)split_stride, \
                     row_width, q_col, k_col, v_col, gates, state, seq_start, seq_slot, out, heads, dim, vdim, tiles,  \
                     cap, q_scale)
#define TLIE_SIZES(D)                                                                                                 \
  if (dim <= 32) TLIE_LAUNCH(D, 32); else if (dim <= 64) TLIE_LAUNCH(D, 64); else if (dim <= 128) TLIE_LAUNCH(D, 128); \
  else TLIE_LAUNCH(D, 256)
  if (dtype == kF32) { TLIE_SIZES(float); }
  else if (dtype == kBF16) { TLIE_SIZES(bf16); }
  else return kBadArgument;
#undef TLIE_SIZES
#undef TLIE_LAUNCH
  return launch_status();
}
