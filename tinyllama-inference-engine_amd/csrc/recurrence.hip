// A gated linear recurrence behind a short causal convolution, with state per request.
//
//   u_t = bias + sum_j taps[n-1-j] * x_(t-j)         per channel, zeros before the sequence's start
//   r_t = sigmoid(gate_r(u_t)), i_t = sigmoid(gate_i(u_t))      (the gates' products are the block-diagonal kernel's)
//   a_t = exp(-c * r_t * softplus(lambda)),   S_t = a_t * S_(t-1) + sqrt(1 - a_t^2) * i_t * u_t,   S = 0 before the start
//   out_t = S_t * gelu_tanh(y_t)
//
// A request's state is one row of the state area, [taps][channels] floats: rows 0 .. taps-2 hold the last
// taps - 1 inputs x of the convolution, oldest first, row taps - 1 holds S.  A step brings any number of
// tokens of a sequence (consecutive in the step); what comes before them is read from the state, and
// the state is brought up to the step's last token.  Everything here is float: the convolution's sums,
// the gates, the decay and its logarithm, the state.  sqrt(1 - a^2) is formed as sqrt(-expm1(2 log a)),
// which keeps its digits where a is close to 1.
//
// Tokens and sequences whose request slot is negative pad a recorded step: nothing is read or written
// for them.
//
// A step that brings many tokens of a sequence takes the recurrence in slices of kSlice tokens: one
// kernel leaves every slice's product of decays P and its end state E from a start of zero (and the
// state the sequence came with), a second one gives every slice its carry, carry_z = P_(z-1) carry_(z-1) +
// E_(z-1) from the sequence's state on, and walks the slice from there as the one-kernel form walks the
// whole sequence.  The slices of a sequence then run side by side; the decays are computed twice.
#include "common.h"

namespace tlie {

__device__ __forceinline__ float sigmoid_f(float v) { return 1.f / (1.f + expf(-v)); }
__device__ __forceinline__ float softplus_f(float v) { return v > 20.f ? v : log1pf(expf(v)); }
__device__ __forceinline__ float gelu_tanh_f(float z) {
  return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// what token t does to channel c's state: S <- a * S + b
__device__ __forceinline__ void decay_and_drive(const float* __restrict__ gates, const float* __restrict__ u, size_t t,
                                                size_t gate_row, size_t gate_at, int block_width, int channels, int c,
                                                float rate, float& a, float& b) {
  const float r = sigmoid_f(gates[t * gate_row + gate_at]);
  const float i = sigmoid_f(gates[t * gate_row + gate_at + block_width]);
  const float log_a = rate * r;
  a = expf(log_a);
  b = sqrtf(-expm1f(2.f * log_a)) * (i * u[t * channels + c]);
}

constexpr int kSlice = 32;             // tokens of a slice in the sliced form

// in: [nsplit][tokens][in_width], the convolution's inputs in columns x_col .. x_col + channels - 1.
// u: [tokens][channels] float.  One thread a (token, channel).
template <typename D, typename W>
__global__ void causal_conv_kernel(const D* __restrict__ in, int nsplit, size_t split_stride, int in_width, int x_col,
                                   const W* __restrict__ taps, const W* __restrict__ bias, const float* __restrict__ state,
                                   const int* __restrict__ token_seq, const int* __restrict__ token_slot,
                                   const int* __restrict__ seq_start, float* __restrict__ u, int channels, int ntaps) {
  const int t = blockIdx.x;
  const int slot = token_slot[t];
  if (slot < 0) return;
  const int k = t - seq_start[token_seq[t]];       // the token's index among its sequence's tokens of this step
  const float* held = state + static_cast<size_t>(slot) * ntaps * channels;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < channels; c += gridDim.y * blockDim.x) {
    float acc = bias != nullptr ? to_float(bias[c]) : 0.f;
    for (int j = 0; j < ntaps; ++j) {              // the input j tokens back meets tap n - 1 - j
      float x;
      if (k - j >= 0) x = sum_splits(in + static_cast<size_t>(t - j) * in_width + x_col + c, nsplit, split_stride);
      else x = held[static_cast<size_t>(ntaps - 1 + k - j) * channels + c];
      acc += to_float(taps[static_cast<size_t>(c) * ntaps + ntaps - 1 - j]) * x;
    }
    u[static_cast<size_t>(t) * channels + c] = acc;
  }
}

// gates: [tokens][blocks][2 * block_width] float, a block's r gates before its i gates, before the sigmoid.
// One thread a (sequence, channel): it walks the sequence's tokens of this step in order, then
// leaves S and the convolution's last inputs in the state.
template <typename D, typename W, typename O>
__global__ void gated_recurrence_kernel(const D* __restrict__ in, int nsplit, size_t split_stride, int in_width, int x_col,
                                        int y_col, const float* __restrict__ u, const float* __restrict__ gates,
                                        const W* __restrict__ lambda, float decay, float* __restrict__ state,
                                        const int* __restrict__ seq_start, const int* __restrict__ seq_slot,
                                        O* __restrict__ out, int channels, int block_width, int ntaps,
                                        const float* __restrict__ parts) {
  const int seq = blockIdx.x;
  const int slot = seq_slot[seq];
  if (slot < 0) return;
  const int first = seq_start[seq], count = seq_start[seq + 1] - first;
  if (count <= 0) return;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  float* held = state + static_cast<size_t>(slot) * ntaps * channels;
  const int block = c / block_width, inside = c % block_width;
  const size_t gate_row = static_cast<size_t>(channels) * 2, gate_at = static_cast<size_t>(block) * 2 * block_width + inside;
  const float rate = -decay * softplus_f(to_float(lambda[c]));
  // slices == 0: the whole sequence in this thread, from and to the state.  Otherwise this thread takes slice
  // blockIdx.z of its sequence, from the carry that the slices before it leave (`parts`, see below).
  const int slices = parts != nullptr ? static_cast<int>(gridDim.z) : 0;
  int begin = 0, end = count;
  float s;
  if (slices == 0) {
    s = held[static_cast<size_t>(ntaps - 1) * channels + c];
  } else {
    begin = blockIdx.z * kSlice, end = min(count, begin + kSlice);
    if (begin >= count) return;
    const float* mine = parts + static_cast<size_t>(seq) * (2 * slices + 1) * channels;
    s = mine[static_cast<size_t>(2 * slices) * channels + c];                    // the state the sequence came with
    for (int z = 0; z < static_cast<int>(blockIdx.z); ++z)
      s = mine[static_cast<size_t>(2 * z) * channels + c] * s + mine[static_cast<size_t>(2 * z + 1) * channels + c];
  }
  for (int k = begin; k < end; ++k) {
    const size_t t = static_cast<size_t>(first + k);
    float a, b;
    decay_and_drive(gates, u, t, gate_row, gate_at, block_width, channels, c, rate, a, b);
    s = a * s + b;
    const float y = sum_splits(in + t * in_width + y_col + c, nsplit, split_stride);
    out[t * channels + c] = from_float<O>(s * gelu_tanh_f(y));
  }
  if (end < count) return;                         // (only the sequence's last slice leaves the state)
  held[static_cast<size_t>(ntaps - 1) * channels + c] = s;
  // the last taps - 1 inputs of (what was held, then this step's): entry e of the new rows is entry
  // count + e of that sequence; rows are written in rising order and read at higher indices only
  for (int e = 0; e < ntaps - 1; ++e) {
    const int from = count + e;
    float x;
    if (from < ntaps - 1) x = held[static_cast<size_t>(from) * channels + c];
    else x = sum_splits(in + static_cast<size_t>(first + from - (ntaps - 1)) * in_width + x_col + c, nsplit, split_stride);
    held[static_cast<size_t>(e) * channels + c] = x;
  }
}

// parts: [sequences][2 * slices + 1][channels]: for slice z the product of its decays at 2z and its end state
// from a start of zero at 2z + 1 (the last slice of a sequence leaves none: nobody reads it); at 2 * slices the
// state the sequence came with (the kernel above reads it from here, since its last slice writes the state
// while other slices may still want the old one).
__global__ void recurrence_slices_kernel(const float* __restrict__ u, const float* __restrict__ gates, const void* __restrict__ lambda,
                                         int lambda_is_bf16, float decay, const float* __restrict__ state,
                                         const int* __restrict__ seq_start, const int* __restrict__ seq_slot,
                                         float* __restrict__ parts, int channels, int block_width, int ntaps) {
  const int seq = blockIdx.x, slices = gridDim.z;
  const int slot = seq_slot[seq];
  if (slot < 0) return;
  const int first = seq_start[seq], count = seq_start[seq + 1] - first;
  const int begin = blockIdx.z * kSlice, end = min(count, begin + kSlice);
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels || count <= 0) return;
  float* mine = parts + static_cast<size_t>(seq) * (2 * slices + 1) * channels;
  if (blockIdx.z == 0)
    mine[static_cast<size_t>(2 * slices) * channels + c] = state[(static_cast<size_t>(slot) * ntaps + ntaps - 1) * channels + c];
  if (end >= count) return;                        // past the sequence, or its last slice
  const int block = c / block_width, inside = c % block_width;
  const size_t gate_row = static_cast<size_t>(channels) * 2, gate_at = static_cast<size_t>(block) * 2 * block_width + inside;
  const float lam = lambda_is_bf16 ? to_float(static_cast<const bf16*>(lambda)[c]) : static_cast<const float*>(lambda)[c];
  const float rate = -decay * softplus_f(lam);
  float product = 1.f, s = 0.f;
  for (int k = begin; k < end; ++k) {
    float a, b;
    decay_and_drive(gates, u, static_cast<size_t>(first + k), gate_row, gate_at, block_width, channels, c, rate, a, b);
    s = a * s + b;
    product *= a;
  }
  mine[static_cast<size_t>(2 * blockIdx.z) * channels + c] = product;
  mine[static_cast<size_t>(2 * blockIdx.z + 1) * channels + c] = s;
}

}  // namespace tlie

using namespace tlie;

extern "C" int tlie_causal_conv(const void* in, int in_dtype, int nsplit, long long split_stride, int in_width, int x_col,
                                const void* taps, const void* bias, int weight_dtype, const float* state,
                                const int* token_seq, const int* token_slot, const int* seq_start, float* u, int tokens,
                                int channels, int ntaps, void* stream) {
  if (tokens <= 0 || channels <= 0 || ntaps <= 0 || nsplit < 1 || x_col < 0 || x_col + channels > in_width) return kBadArgument;
  const int threads = channels >= 256 ? 256 : 64;
  int across = (channels + threads - 1) / threads;
  if (across > 64) across = 64;
  const dim3 grid(tokens, across);
  hipStream_t s = (hipStream_t)stream;
#define TLIE_CASE(DC, D, WC, W)                                                                                   \
  if (in_dtype == DC && weight_dtype == WC) {                                                                     \
    hipLaunchKernelGGL((causal_conv_kernel<D, W>), grid, dim3(threads), 0, s, (const D*)in, nsplit,                 \
                       (size_t)split_stride, in_width, x_col, (const W*)taps, (const W*)bias, state, token_seq,    \
                       token_slot, seq_start, u, channels, ntaps);                                                 \
    return launch_status();                                                                                       \
  }
  TLIE_CASE(kF32, float, kF32, float)
  TLIE_CASE(kF32, float, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kBF16, bf16)
#undef TLIE_CASE
  return kBadArgument;
}

extern "C" int tlie_gated_recurrence(const void* in, int in_dtype, int nsplit, long long split_stride, int in_width,
                                     int x_col, int y_col, const float* u, const float* gates, const void* lambda,
                                     int weight_dtype, float decay, float* state, const int* seq_start, const int* seq_slot,
                                     void* out, int out_dtype, int seqs, int channels, int block_width, int ntaps,
                                     int slices, float* parts, void* stream) {
  // slices 0: a thread walks all of a sequence's tokens of the step.  slices > 0 (then no sequence brings more than
  // slices * 32 tokens, and parts holds seqs * (2 * slices + 1) * channels floats): the sliced form.
  if (slices < 0 || slices > 65535 || (slices > 0 && parts == nullptr)) return kBadArgument;
  if (seqs <= 0 || channels <= 0 || ntaps <= 0 || nsplit < 1 || block_width <= 0 || channels % block_width != 0) return kBadArgument;
  if (x_col < 0 || x_col + channels > in_width || y_col < 0 || y_col + channels > in_width) return kBadArgument;
  const dim3 grid(seqs, (channels + 63) / 64, slices > 0 ? slices : 1);
  if (grid.y > 65535) return kBadArgument;
  hipStream_t s = (hipStream_t)stream;
  if (slices > 0) {
    if (weight_dtype != kF32 && weight_dtype != kBF16) return kBadArgument;
    hipLaunchKernelGGL(recurrence_slices_kernel, grid, dim3(64), 0, s, u, gates, lambda, weight_dtype == kBF16 ? 1 : 0, decay,
                       state, seq_start, seq_slot, parts, channels, block_width, ntaps);
    if (launch_status() != kOk) return kLaunchFailed;
  }
  const float* carried = slices > 0 ? parts : nullptr;
#define TLIE_CASE(DC, D, WC, W, OC, O)                                                                            \
  if (in_dtype == DC && weight_dtype == WC && out_dtype == OC) {                                                   \
    hipLaunchKernelGGL((gated_recurrence_kernel<D, W, O>), grid, dim3(64), 0, s, (const D*)in, nsplit,              \
                       (size_t)split_stride, in_width, x_col, y_col, u, gates, (const W*)lambda, decay, state,     \
                       seq_start, seq_slot, (O*)out, channels, block_width, ntaps, carried);                       \
    return launch_status();                                                                                        \
  }
  TLIE_CASE(kF32, float, kF32, float, kF32, float)
  TLIE_CASE(kF32, float, kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kBF16, bf16, kBF16, bf16)
#undef TLIE_CASE
  return kBadArgument;
}
