// Kernels around a sublayer's input that the framework's RMS-norm kernels do not cover:
//
//   layer_norm      residual += s1 * delta1 + s2 * delta2 (both optional), optionally a weighted sum over the
//                   residuals of earlier layers in its place, then (x - mean) / sqrt(var + eps) * w + b
//   input_conv      h + conv(h): a short causal convolution per channel over each sequence's tokens, whose last
//                   inputs are a request's state
//   token_shift     several blends of a token's input with the input of the token before it (a request's state)
//   xielu           an activation with two learned numbers
//
// Sums, means, variances and the convolution's sums are float.  Tokens and sequences whose request slot is negative
// pad a recorded step: no state is read or written for them.
#include "common.h"

namespace tlie {

// One workgroup a row.  rows == nullptr: row t of the residual gets the deltas added in place.  With a history
// (count > 0): the residual is the history's last entry, history[count - 1], and what is normed (and written to
// `mixed`, the residual of the layer to come) is sum_j hw[j] * history[j][t].  rows != nullptr: only the rows named
// there, nothing but `out` written.  out == nullptr: no norm, only the sums.
template <typename D1, typename D2, typename W, typename O>
__global__ void __launch_bounds__(256)
layer_norm_kernel(float* __restrict__ residual, const D1* __restrict__ d1, int n1, size_t stride1, float s1,
                  const D2* __restrict__ d2, int n2, size_t stride2, float s2, const float* __restrict__ history,
                  size_t history_stride, int history_count, const W* __restrict__ history_weight, float* __restrict__ mixed,
                  const W* __restrict__ weight, const W* __restrict__ bias, float eps, O* __restrict__ out,
                  const int* __restrict__ rows, int hidden) {
  extern __shared__ float row_values[];
  __shared__ float scratch[16];
  const int t = rows != nullptr ? rows[blockIdx.x] : blockIdx.x;
  const size_t at = static_cast<size_t>(t) * hidden;
  float sum = 0.f;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    float x = residual[at + c];
    if (d1 != nullptr) x += s1 * sum_splits(d1 + at + c, n1, stride1);
    if (d2 != nullptr) x += s2 * sum_splits(d2 + at + c, n2, stride2);
    if (rows == nullptr && (d1 != nullptr || d2 != nullptr)) residual[at + c] = x;
    if (history_count > 0) {
      float y = 0.f;
      for (int j = 0; j + 1 < history_count; ++j) y += to_float(history_weight[j]) * history[j * history_stride + at + c];
      x = y + to_float(history_weight[history_count - 1]) * x;
      if (rows == nullptr) mixed[at + c] = x;
    }
    row_values[c] = x;
    sum += x;
  }
  if (out == nullptr) return;
  const float mean = block_sum(sum, scratch) / static_cast<float>(hidden);
  float squares = 0.f;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    const float d = row_values[c] - mean;
    squares += d * d;
  }
  const float r = 1.f / sqrtf(block_sum(squares, scratch) / static_cast<float>(hidden) + eps);
  O* dst = out + static_cast<size_t>(blockIdx.x) * hidden;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    float v = (row_values[c] - mean) * r * to_float(weight[c]);
    if (bias != nullptr) v += to_float(bias[c]);
    dst[c] = from_float<O>(v);
  }
}

constexpr int kMaxTaps = 8;

// h: float [tokens, channels]; taps: [channels, ntaps], tap j weighs the input ntaps - 1 - j tokens back; state: float
// [slots, ntaps - 1, channels] (a slot's rows `slot_stride` floats after the slot's before it), the last inputs, oldest first.  Workgroups 0 .. tokens - 1 take a token each that
// needs nothing of the state (its index among its sequence's tokens of the step is at least ntaps - 1); workgroups
// tokens .. tokens + sequences - 1 take a sequence each: its first tokens, which read the state, and then the state's
// new rows, so that no workgroup reads state that another one writes.
template <typename W, typename O>
__global__ void __launch_bounds__(256)
input_conv_kernel(const float* __restrict__ h, const W* __restrict__ taps, float* __restrict__ state,
                  const int* __restrict__ token_seq, const int* __restrict__ token_slot, const int* __restrict__ seq_start,
                  const int* __restrict__ seq_slot, O* __restrict__ out, int tokens, int channels, int ntaps, size_t slot_stride) {
  const int back = ntaps - 1;
  if (static_cast<int>(blockIdx.x) < tokens) {
    const int t = blockIdx.x;
    if (token_slot[t] < 0) {                           // a token that pads a recorded step: zeros, so that what follows stays finite
      for (int c = threadIdx.x; c < channels; c += blockDim.x) out[static_cast<size_t>(t) * channels + c] = from_float<O>(0.f);
      return;
    }
    if (t - seq_start[token_seq[t]] < back) return;
    for (int c = threadIdx.x; c < channels; c += blockDim.x) {
      float acc = h[static_cast<size_t>(t) * channels + c];
      for (int j = 0; j < ntaps; ++j)
        acc += to_float(taps[static_cast<size_t>(c) * ntaps + j]) * h[static_cast<size_t>(t - back + j) * channels + c];
      out[static_cast<size_t>(t) * channels + c] = from_float<O>(acc);
    }
    return;
  }
  const int seq = blockIdx.x - tokens;
  const int slot = seq_slot[seq];
  if (slot < 0) return;
  const int first = seq_start[seq], count = seq_start[seq + 1] - first;
  if (count <= 0) return;
  float* held = state + static_cast<size_t>(slot) * slot_stride;
  for (int c = threadIdx.x; c < channels; c += blockDim.x) {
    float old[kMaxTaps], w[kMaxTaps];
#pragma unroll
    for (int j = 0; j < kMaxTaps; ++j) {
      old[j] = j < back ? held[static_cast<size_t>(j) * channels + c] : 0.f;      // the input back - j tokens before the step
      w[j] = j < ntaps ? to_float(taps[static_cast<size_t>(c) * ntaps + j]) : 0.f;
    }
    // input at index i among the step's tokens of this sequence; negative: before the step
    auto input = [&](int i) {
      if (i >= 0) return h[static_cast<size_t>(first + i) * channels + c];
      float v = 0.f;
#pragma unroll
      for (int j = 0; j < kMaxTaps; ++j) v = (j == back + i) ? old[j] : v;
      return v;
    };
    const int early = count < back ? count : back;
    for (int k = 0; k < early; ++k) {
      float acc = h[static_cast<size_t>(first + k) * channels + c];
#pragma unroll
      for (int j = 0; j < kMaxTaps; ++j)
        if (j < ntaps) acc += w[j] * input(k - back + j);
      out[static_cast<size_t>(first + k) * channels + c] = from_float<O>(acc);
    }
    float fresh[kMaxTaps];
#pragma unroll
    for (int j = 0; j < kMaxTaps; ++j) fresh[j] = j < back ? input(count - back + j) : 0.f;
#pragma unroll
    for (int j = 0; j < kMaxTaps; ++j)
      if (j < back) held[static_cast<size_t>(j) * channels + c] = fresh[j];
  }
}

// x: [tokens, width] in the activation type; mu: [mixes, width]; state: float [slots, width], the input of the token
// before the step; out: [mixes][tokens][width], out[m][t] = x_t + (x_(t-1) - x_t) * mu[m].  Workgroups 0 .. tokens - 1:
// tokens that have their predecessor in the step; workgroups from `tokens` on: a sequence's first token, then the state.
template <typename A, typename W>
__global__ void __launch_bounds__(256)
token_shift_kernel(const A* __restrict__ x, const W* __restrict__ mu, float* __restrict__ state,
                   const int* __restrict__ token_seq, const int* __restrict__ token_slot, const int* __restrict__ seq_start,
                   const int* __restrict__ seq_slot, A* __restrict__ out, int tokens, int width, int mixes, size_t slot_stride) {
  int t;
  float* held = nullptr;
  int last = 0;
  if (static_cast<int>(blockIdx.x) < tokens) {
    t = blockIdx.x;
    if (token_slot[t] < 0) {                           // a token that pads a recorded step: zeros
      for (int m = 0; m < mixes; ++m)
        for (int c = threadIdx.x; c < width; c += blockDim.x) out[(static_cast<size_t>(m) * tokens + t) * width + c] = from_float<A>(0.f);
      return;
    }
    if (t == seq_start[token_seq[t]]) return;
  } else {
    const int seq = blockIdx.x - tokens, slot = seq_slot[seq];
    if (slot < 0 || seq_start[seq + 1] <= seq_start[seq]) return;
    t = seq_start[seq], last = seq_start[seq + 1] - 1;
    held = state + static_cast<size_t>(slot) * slot_stride;
  }
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float now = to_float(x[static_cast<size_t>(t) * width + c]);
    const float before = held != nullptr ? held[c] : to_float(x[static_cast<size_t>(t - 1) * width + c]);
    for (int m = 0; m < mixes; ++m)
      out[(static_cast<size_t>(m) * tokens + t) * width + c] = from_float<A>(now + (before - now) * to_float(mu[static_cast<size_t>(m) * width + c]));
    if (held != nullptr) held[c] = to_float(x[static_cast<size_t>(last) * width + c]);
  }
}

__device__ __forceinline__ float softplus_of(float v) { return v > 20.f ? v : log1pf(expf(v)); }

// out = softplus(p) z^2 + z / 2 for z > 0, (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2 otherwise; (p, q) = numbers[0], [1].
template <typename D, typename W, typename O>
__global__ void __launch_bounds__(256)
xielu_kernel(const D* __restrict__ in, int nsplit, size_t split_stride, const W* __restrict__ numbers, O* __restrict__ out,
             size_t count) {
  const float up = softplus_of(to_float(numbers[0])), down = 0.5f + softplus_of(to_float(numbers[1]));
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < count; i += static_cast<size_t>(gridDim.x) * blockDim.x) {
    const float z = sum_splits(in + i, nsplit, split_stride);
    const float v = z > 0.f ? up * z * z + 0.5f * z : down * (expm1f(z) - z) + 0.5f * z;
    out[i] = from_float<O>(v);
  }
}

}  // namespace tlie

using namespace tlie;

// residual: float [tokens, hidden] (changed in place when there are deltas and no rows); d1, d2 (or null): products of
// d1_dtype, d2_dtype; history (or null, with history_count 0): float, entry j at history + j * history_stride, the last
// entry being the residual itself; history_weight: [history_count] of w_dtype; mixed: float [tokens, hidden]; weight,
// bias (bias may be null) [hidden] of w_dtype; out (or null) [count, hidden] of out_dtype; rows (or null): int [count].
extern "C" int tlie_layer_norm(float* residual, const void* d1, int d1_dtype, int n1, long long stride1, float s1,
                               const void* d2, int d2_dtype, int n2, long long stride2, float s2, const float* history,
                               long long history_stride, int history_count, const void* history_weight, float* mixed,
                               const void* weight, const void* bias, int w_dtype, float eps, void* out, int out_dtype,
                               const int* rows, int count, int hidden, void* stream) {
  if (count <= 0 || hidden <= 0 || hidden > 16000 || history_count < 0 || n1 < 1 || n2 < 1) return kBadArgument;
  if (history_count > 0 && (history == nullptr || history_weight == nullptr || (rows == nullptr && mixed == nullptr))) return kBadArgument;
  if (out != nullptr && (weight == nullptr || !(eps > 0.f))) return kBadArgument;
  hipStream_t s = (hipStream_t)stream;
  const size_t lds = static_cast<size_t>(hidden) * sizeof(float);
#define TLIE_CASE(C1, D1, C2, D2, WC, W, OC, O)                                                                          \
  if (d1_dtype == C1 && d2_dtype == C2 && w_dtype == WC && out_dtype == OC) {                                            \
    hipLaunchKernelGGL((layer_norm_kernel<D1, D2, W, O>), dim3(count), dim3(256), lds, s, residual, (const D1*)d1, n1,    \
                       (size_t)stride1, s1, (const D2*)d2, n2, (size_t)stride2, s2, history, (size_t)history_stride,      \
                       history_count, (const W*)history_weight, mixed, (const W*)weight, (const W*)bias, eps, (O*)out,    \
                       rows, hidden);                                                                                    \
    return launch_status();                                                                                              \
  }
  TLIE_CASE(kF32, float, kF32, float, kF32, float, kF32, float)
  TLIE_CASE(kF32, float, kF32, float, kBF16, bf16, kF32, float)
  TLIE_CASE(kF32, float, kF32, float, kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kF32, float, kBF16, bf16, kF32, float)
  TLIE_CASE(kF32, float, kBF16, bf16, kBF16, bf16, kF32, float)
  TLIE_CASE(kBF16, bf16, kBF16, bf16, kBF16, bf16, kF32, float)
  TLIE_CASE(kBF16, bf16, kF32, float, kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kF32, float, kBF16, bf16, kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kBF16, bf16, kBF16, bf16, kBF16, bf16)
#undef TLIE_CASE
  return kBadArgument;
}

extern "C" int tlie_input_conv(const float* h, const void* taps, int taps_dtype, float* state, const int* token_seq,
                               const int* token_slot, const int* seq_start, const int* seq_slot, void* out, int out_dtype,
                               int tokens, int sequences, int channels, int ntaps, long long slot_stride, void* stream) {
  if (tokens <= 0 || sequences <= 0 || channels <= 0 || ntaps < 1 || ntaps > kMaxTaps) return kBadArgument;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(tokens + sequences);
#define TLIE_CASE(WC, W, OC, O)                                                                                          \
  if (taps_dtype == WC && out_dtype == OC) {                                                                             \
    hipLaunchKernelGGL((input_conv_kernel<W, O>), grid, dim3(256), 0, s, h, (const W*)taps, state, token_seq, token_slot, \
                       seq_start, seq_slot, (O*)out, tokens, channels, ntaps, (size_t)slot_stride);                                           \
    return launch_status();                                                                                              \
  }
  TLIE_CASE(kF32, float, kF32, float)
  TLIE_CASE(kBF16, bf16, kF32, float)
  TLIE_CASE(kBF16, bf16, kBF16, bf16)
#undef TLIE_CASE
  return kBadArgument;
}

extern "C" int tlie_token_shift(const void* x, int dtype, const void* mu, int mu_dtype, float* state, const int* token_seq,
                                const int* token_slot, const int* seq_start, const int* seq_slot, void* out, int tokens,
                                int sequences, int width, int mixes, long long slot_stride, void* stream) {
  if (tokens <= 0 || sequences <= 0 || width <= 0 || mixes <= 0) return kBadArgument;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid(tokens + sequences);
#define TLIE_CASE(AC, A, WC, W)                                                                                          \
  if (dtype == AC && mu_dtype == WC) {                                                                                   \
    hipLaunchKernelGGL((token_shift_kernel<A, W>), grid, dim3(256), 0, s, (const A*)x, (const W*)mu, state, token_seq,    \
                       token_slot, seq_start, seq_slot, (A*)out, tokens, width, mixes, (size_t)slot_stride);                                  \
    return launch_status();                                                                                              \
  }
  TLIE_CASE(kF32, float, kF32, float)
  TLIE_CASE(kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kF32, float)
#undef TLIE_CASE
  return kBadArgument;
}

// in: a product [nsplit][count] of in_dtype; numbers: [2] of n_dtype; out: [count] of out_dtype.
extern "C" int tlie_xielu(const void* in, int in_dtype, int nsplit, long long split_stride, const void* numbers, int n_dtype,
                          void* out, int out_dtype, long long count, void* stream) {
  if (count <= 0 || nsplit < 1) return kBadArgument;
  hipStream_t s = (hipStream_t)stream;
  long long blocks = (count + 255) / 256;
  if (blocks > 8192) blocks = 8192;
#define TLIE_CASE(IC, D, NC, W, OC, O)                                                                                   \
  if (in_dtype == IC && n_dtype == NC && out_dtype == OC) {                                                              \
    hipLaunchKernelGGL((xielu_kernel<D, W, O>), dim3((unsigned)blocks), dim3(256), 0, s, (const D*)in, nsplit,            \
                       (size_t)split_stride, (const W*)numbers, (O*)out, (size_t)count);                                 \
    return launch_status();                                                                                              \
  }
  TLIE_CASE(kF32, float, kF32, float, kF32, float)
  TLIE_CASE(kF32, float, kBF16, bf16, kF32, float)
  TLIE_CASE(kF32, float, kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kBF16, bf16, kBF16, bf16)
#undef TLIE_CASE
  return kBadArgument;
}
