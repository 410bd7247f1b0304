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

// The same with eight elements a thread (16- and 32-byte loads and stores): hidden % 8 == 0, and the parts of a split
// product lie a multiple of eight elements apart; the summands of a split product are added in the order of their index.
template <typename D>
__device__ __forceinline__ void load8_splits(const D* __restrict__ part, int nsplit, size_t stride, float (&d)[8]) {
  load8(part, d);
  for (int s = 1; s < nsplit; ++s) {
    float more[8];
    load8(part + s * stride, more);
#pragma unroll
    for (int j = 0; j < 8; ++j) d[j] += more[j];
  }
}

template <typename D1, typename D2, typename W, typename O>
__global__ void __launch_bounds__(256)
layer_norm_wide_kernel(float* __restrict__ residual, const D1* __restrict__ d1, int n1, size_t stride1, float s1,
                       const D2* __restrict__ d2, int n2, size_t stride2, float s2, const float* __restrict__ history,
                       size_t history_stride, int history_count, const W* __restrict__ history_weight, float* __restrict__ mixed,
                       const W* __restrict__ weight, const W* __restrict__ bias, float eps, O* __restrict__ out,
                       const int* __restrict__ rows, int hidden) {
  extern __shared__ float row_values[];
  __shared__ float scratch[16];
  const int t = rows != nullptr ? rows[blockIdx.x] : blockIdx.x;
  const size_t at = static_cast<size_t>(t) * hidden;
  float sum = 0.f;
  for (int c = threadIdx.x * 8; c < hidden; c += blockDim.x * 8) {
    float x[8];
    load8(residual + at + c, x);
    if (d1 != nullptr) {
      float d[8];
      load8_splits(d1 + at + c, n1, stride1, d);
#pragma unroll
      for (int j = 0; j < 8; ++j) x[j] += s1 * d[j];
    }
    if (d2 != nullptr) {
      float d[8];
      load8_splits(d2 + at + c, n2, stride2, d);
#pragma unroll
      for (int j = 0; j < 8; ++j) x[j] += s2 * d[j];
    }
    if (rows == nullptr && (d1 != nullptr || d2 != nullptr)) store8(residual + at + c, x);
    if (history_count > 0) {
      float y[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      for (int j = 0; j + 1 < history_count; ++j) {
        float earlier[8];
        load8(history + j * history_stride + at + c, earlier);
        const float w = to_float(history_weight[j]);
#pragma unroll
        for (int e = 0; e < 8; ++e) y[e] += w * earlier[e];
      }
      const float w = to_float(history_weight[history_count - 1]);
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] = y[e] + w * x[e];
      if (rows == nullptr) store8(mixed + at + c, x);
    }
    store8(row_values + c, x);                        // (a thread reads back only what it wrote itself)
#pragma unroll
    for (int j = 0; j < 8; ++j) sum += x[j];
  }
  if (out == nullptr) return;
  const float mean = block_sum(sum, scratch) / static_cast<float>(hidden);
  float squares = 0.f;
  for (int c = threadIdx.x * 8; c < hidden; c += blockDim.x * 8) {
    float x[8];
    load8(row_values + c, x);
#pragma unroll
    for (int j = 0; j < 8; ++j) squares += (x[j] - mean) * (x[j] - mean);
  }
  const float r = 1.f / sqrtf(block_sum(squares, scratch) / static_cast<float>(hidden) + eps);
  O* dst = out + static_cast<size_t>(blockIdx.x) * hidden;
  for (int c = threadIdx.x * 8; c < hidden; c += blockDim.x * 8) {
    float x[8], w[8];
    load8(row_values + c, x);
    load8(weight + c, w);
#pragma unroll
    for (int j = 0; j < 8; ++j) x[j] = (x[j] - mean) * r * w[j];
    if (bias != nullptr) {
      load8(bias + c, w);
#pragma unroll
      for (int j = 0; j < 8; ++j) x[j] += w[j];
    }
    store8(dst + c, x);
  }
}

constexpr int kMaxTaps = 8, kConvTokens = 8;

__device__ __forceinline__ void store1(float* p, float v) { *p = v; }
__device__ __forceinline__ void store1(bf16* p, float v) { *p = __float2bfloat16(v); }

// Four consecutive elements as floats (the address a multiple of 16 bytes for float, of 8 for bfloat16).
__device__ __forceinline__ float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load4(const bf16* p) {
  const uint2 u = *reinterpret_cast<const uint2*>(p);
  return make_float4(bf16_lo(u.x), bf16_hi(u.x), bf16_lo(u.y), bf16_hi(u.y));
}

// h: float [tokens, channels]; taps: [channels, ntaps], tap j weighs the input ntaps - 1 - j tokens back; state: float
// [slots, ntaps - 1, channels] (a slot's rows `slot_stride` floats after the slot's before it), the last inputs, oldest
// first.  Every thread owns V consecutive channels (V = 4 where the channels are a multiple of 4), blockIdx.y a stretch
// of 256 * V channels.  The first ceil(tokens / kConvTokens) workgroups (in x) take kConvTokens tokens each, those of
// them that need nothing of the state (a token's index among its sequence's tokens of the step is at least ntaps - 1);
// the `sequences` workgroups after them take a sequence each: its first tokens, which read the state, and then the state's new rows, so that no workgroup reads
// state that another one writes.
template <typename W, typename O, int V>
__global__ void __launch_bounds__(256)
input_conv_kernel(const float* __restrict__ h, const W* __restrict__ taps, float* __restrict__ state,
                  const int* __restrict__ token_seq, const int* __restrict__ token_slot, const int* __restrict__ seq_start,
                  const int* __restrict__ seq_slot, O* __restrict__ out, int tokens, int channels, int ntaps, size_t slot_stride) {
  const int back = ntaps - 1;
  const int c = (blockIdx.y * 256 + threadIdx.x) * V;
  if (c >= channels) return;
  auto read = [&](const float* p, float (&v)[V]) {
    if (V == 4) {
      const float4 x = load4(p);
      v[0] = x.x, v[V > 1 ? 1 : 0] = x.y, v[V > 2 ? 2 : 0] = x.z, v[V > 3 ? 3 : 0] = x.w;
    } else {
      v[0] = p[0];
    }
  };
  auto write = [&](O* p, const float (&v)[V]) {
    if (V == 4) store4(p, v[0], v[V > 1 ? 1 : 0], v[V > 2 ? 2 : 0], v[V > 3 ? 3 : 0]);
    else p[0] = from_float<O>(v[0]);
  };
  float w[kMaxTaps][V];                                // this thread's channels' taps
#pragma unroll
  for (int j = 0; j < kMaxTaps; ++j)
#pragma unroll
    for (int e = 0; e < V; ++e) w[j][e] = j < ntaps ? to_float(taps[static_cast<size_t>(c + e) * ntaps + j]) : 0.f;
  const int token_blocks = (tokens + kConvTokens - 1) / kConvTokens;
  if (static_cast<int>(blockIdx.x) < token_blocks) {
    const int t0 = blockIdx.x * kConvTokens, t1 = min(tokens, t0 + kConvTokens);
    for (int t = t0; t < t1; ++t) {                    // (the taps are read once for these tokens; the rows come from the cache)
      if (token_slot[t] < 0) {                         // a token that pads a recorded step: zeros, so that what follows stays finite
        float zero[V];
#pragma unroll
        for (int e = 0; e < V; ++e) zero[e] = 0.f;
        write(out + static_cast<size_t>(t) * channels + c, zero);
        continue;
      }
      if (t - seq_start[token_seq[t]] < back) continue;
      float acc[V];
      read(h + static_cast<size_t>(t) * channels + c, acc);
#pragma unroll
      for (int j = 0; j < kMaxTaps; ++j) {
        if (j < ntaps) {
          float x[V];
          read(h + static_cast<size_t>(t - back + j) * channels + c, x);
#pragma unroll
          for (int e = 0; e < V; ++e) acc[e] += w[j][e] * x[e];
        }
      }
      write(out + static_cast<size_t>(t) * channels + c, acc);
    }
    return;
  }
  const int seq = blockIdx.x - token_blocks;
  const int slot = seq_slot[seq];
  if (slot < 0) return;
  const int first = seq_start[seq], count = seq_start[seq + 1] - first;
  if (count <= 0) return;
  float* held = state + static_cast<size_t>(slot) * slot_stride;
  // the input at index i among the step's tokens of this sequence; negative: before the step, from the state
  auto input = [&](int i, float (&v)[V]) {
    if (i >= 0) read(h + static_cast<size_t>(first + i) * channels + c, v);
    else read(held + static_cast<size_t>(back + i) * channels + c, v);
  };
  const int early = count < back ? count : back;
  for (int k = 0; k < early; ++k) {
    float acc[V];
    read(h + static_cast<size_t>(first + k) * channels + c, acc);
#pragma unroll
    for (int j = 0; j < kMaxTaps; ++j) {
      if (j < ntaps) {
        float x[V];
        input(k - back + j, x);
#pragma unroll
        for (int e = 0; e < V; ++e) acc[e] += w[j][e] * x[e];
      }
    }
    write(out + static_cast<size_t>(first + k) * channels + c, acc);
  }
  float fresh[kMaxTaps][V];                            // (all read before any is written: a short step keeps old rows)
#pragma unroll
  for (int j = 0; j < kMaxTaps; ++j)
    if (j < back) input(count - back + j, fresh[j]);
#pragma unroll
  for (int j = 0; j < kMaxTaps; ++j) {
    if (j < back) {
      if (V == 4) store4(held + static_cast<size_t>(j) * channels + c, fresh[j][0], fresh[j][V > 1 ? 1 : 0], fresh[j][V > 2 ? 2 : 0], fresh[j][V > 3 ? 3 : 0]);
      else held[static_cast<size_t>(j) * channels + c] = fresh[j][0];
    }
  }
}

// x: [tokens, width] in the activation type; mu: [mixes, width]; state: float [slots, width], the input of the token
// before the step; out: [mixes][tokens][width], out[m][t] = x_t + (x_(t-1) - x_t) * mu[m].  A thread owns V consecutive
// columns (V = 4 where the width is a multiple of 4), blockIdx.y a stretch of 256 * V columns.  Workgroups 0 ..
// tokens - 1 (in x): tokens that have their predecessor in the step; workgroups from `tokens` on: a sequence's first
// token, then the state.
template <typename A, typename W, int V>
__global__ void __launch_bounds__(256)
token_shift_kernel(const A* __restrict__ x, const W* __restrict__ mu, float* __restrict__ state,
                   const int* __restrict__ token_seq, const int* __restrict__ token_slot, const int* __restrict__ seq_start,
                   const int* __restrict__ seq_slot, A* __restrict__ out, int tokens, int width, int mixes, size_t slot_stride) {
  const int c = (blockIdx.y * 256 + threadIdx.x) * V;
  if (c >= width) return;
  auto read = [&](auto* p, float (&v)[V]) {
    if (V == 4) {
      const float4 q = load4(p);
      v[0] = q.x, v[V > 1 ? 1 : 0] = q.y, v[V > 2 ? 2 : 0] = q.z, v[V > 3 ? 3 : 0] = q.w;
    } else {
      v[0] = to_float(p[0]);
    }
  };
  auto write = [&](auto* p, const float (&v)[V]) {
    if (V == 4) store4(p, v[0], v[V > 1 ? 1 : 0], v[V > 2 ? 2 : 0], v[V > 3 ? 3 : 0]);
    else store1(p, v[0]);
  };
  int t;
  float* held = nullptr;
  int last = 0;
  if (static_cast<int>(blockIdx.x) < tokens) {
    t = blockIdx.x;
    if (token_slot[t] < 0) {                           // a token that pads a recorded step: zeros
      float zero[V];
#pragma unroll
      for (int e = 0; e < V; ++e) zero[e] = 0.f;
      for (int m = 0; m < mixes; ++m) write(out + (static_cast<size_t>(m) * tokens + t) * width + c, zero);
      return;
    }
    if (t == seq_start[token_seq[t]]) return;
  } else {
    const int seq = blockIdx.x - tokens, slot = seq_slot[seq];
    if (slot < 0 || seq_start[seq + 1] <= seq_start[seq]) return;
    t = seq_start[seq], last = seq_start[seq + 1] - 1;
    held = state + static_cast<size_t>(slot) * slot_stride;
  }
  float now[V], before[V];
  read(x + static_cast<size_t>(t) * width + c, now);
  if (held != nullptr) read(held + c, before);
  else read(x + static_cast<size_t>(t - 1) * width + c, before);
  for (int m = 0; m < mixes; ++m) {
    float blend[V], result[V];
    read(mu + static_cast<size_t>(m) * width + c, blend);
#pragma unroll
    for (int e = 0; e < V; ++e) result[e] = now[e] + (before[e] - now[e]) * blend[e];
    write(out + (static_cast<size_t>(m) * tokens + t) * width + c, result);
  }
  if (held != nullptr) {
    float kept[V];
    read(x + static_cast<size_t>(last) * width + c, kept);
    write(held + c, kept);
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

// The same with eight elements a thread: count % 8 == 0 and the parts of a split product a multiple of eight apart.
template <typename D, typename W, typename O>
__global__ void __launch_bounds__(256)
xielu_wide_kernel(const D* __restrict__ in, int nsplit, size_t split_stride, const W* __restrict__ numbers, O* __restrict__ out,
                  size_t count) {
  const float up = softplus_of(to_float(numbers[0])), down = 0.5f + softplus_of(to_float(numbers[1]));
  for (size_t i = (static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x) * 8; i < count; i += static_cast<size_t>(gridDim.x) * blockDim.x * 8) {
    float z[8];
    load8_splits(in + i, nsplit, split_stride, z);
#pragma unroll
    for (int j = 0; j < 8; ++j) z[j] = z[j] > 0.f ? up * z[j] * z[j] + 0.5f * z[j] : down * (expm1f(z[j]) - z[j]) + 0.5f * z[j];
    store8(out + i, z);
  }
}

}  // namespace tlie

using namespace tlie;

static inline bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

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
  // eight elements a thread where rows, parts of split products and earlier results all begin at multiples of eight
  const bool wide = hidden % 8 == 0 && (d1 == nullptr || n1 == 1 || stride1 % 8 == 0) && (d2 == nullptr || n2 == 1 || stride2 % 8 == 0) &&
                    (history_count == 0 || history_stride % 8 == 0) && aligned16(residual) && aligned16(d1) && aligned16(d2) &&
                    aligned16(history) && aligned16(mixed) && aligned16(weight) && aligned16(bias) && aligned16(out);
  int threads = 64;                                    // as many waves as the row has work for (at most four)
  while (threads < 256 && threads * 8 < hidden) threads *= 2;
#define TLIE_CASE(C1, D1, C2, D2, WC, W, OC, O)                                                                          \
  if (d1_dtype == C1 && d2_dtype == C2 && w_dtype == WC && out_dtype == OC) {                                            \
    if (wide)                                                                                                            \
      hipLaunchKernelGGL((layer_norm_wide_kernel<D1, D2, W, O>), dim3(count), dim3(threads), lds, s, residual,            \
                         (const D1*)d1, n1, (size_t)stride1, s1, (const D2*)d2, n2, (size_t)stride2, s2, history,         \
                         (size_t)history_stride, history_count, (const W*)history_weight, mixed, (const W*)weight,        \
                         (const W*)bias, eps, (O*)out, rows, hidden);                                                     \
    else                                                                                                                 \
      hipLaunchKernelGGL((layer_norm_kernel<D1, D2, W, O>), dim3(count), dim3(256), lds, s, residual, (const D1*)d1, n1,  \
                         (size_t)stride1, s1, (const D2*)d2, n2, (size_t)stride2, s2, history, (size_t)history_stride,    \
                         history_count, (const W*)history_weight, mixed, (const W*)weight, (const W*)bias, eps, (O*)out,  \
                         rows, hidden);                                                                                  \
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
  const bool four = channels % 4 == 0 && slot_stride % 4 == 0 && aligned16(h) && aligned16(state) && aligned16(out);
  const int per_block = four ? 1024 : 256;
  const dim3 grid((tokens + kConvTokens - 1) / kConvTokens + sequences, (channels + per_block - 1) / per_block);
  if (grid.y > 65535) return kBadArgument;
#define TLIE_CASE(WC, W, OC, O)                                                                                          \
  if (taps_dtype == WC && out_dtype == OC) {                                                                             \
    if (four)                                                                                                            \
      hipLaunchKernelGGL((input_conv_kernel<W, O, 4>), grid, dim3(256), 0, s, h, (const W*)taps, state, token_seq,        \
                         token_slot, seq_start, seq_slot, (O*)out, tokens, channels, ntaps, (size_t)slot_stride);         \
    else                                                                                                                 \
      hipLaunchKernelGGL((input_conv_kernel<W, O, 1>), grid, dim3(256), 0, s, h, (const W*)taps, state, token_seq,        \
                         token_slot, seq_start, seq_slot, (O*)out, tokens, channels, ntaps, (size_t)slot_stride);         \
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
  const bool four = width % 4 == 0 && slot_stride % 4 == 0 && aligned16(x) && aligned16(mu) && aligned16(state) && aligned16(out);
  const int per_block = four ? 1024 : 256;
  const dim3 grid(tokens + sequences, (width + per_block - 1) / per_block);
  if (grid.y > 65535) return kBadArgument;
#define TLIE_CASE(AC, A, WC, W)                                                                                          \
  if (dtype == AC && mu_dtype == WC) {                                                                                   \
    if (four)                                                                                                            \
      hipLaunchKernelGGL((token_shift_kernel<A, W, 4>), grid, dim3(256), 0, s, (const A*)x, (const W*)mu, state,          \
                         token_seq, token_slot, seq_start, seq_slot, (A*)out, tokens, width, mixes, (size_t)slot_stride); \
    else                                                                                                                 \
      hipLaunchKernelGGL((token_shift_kernel<A, W, 1>), grid, dim3(256), 0, s, (const A*)x, (const W*)mu, state,          \
                         token_seq, token_slot, seq_start, seq_slot, (A*)out, tokens, width, mixes, (size_t)slot_stride); \
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
  if (blocks > 65536) blocks = 65536;
  const bool wide = count % 8 == 0 && (nsplit == 1 || split_stride % 8 == 0) && aligned16(in) && aligned16(out);
#define TLIE_CASE(IC, D, NC, W, OC, O)                                                                                   \
  if (in_dtype == IC && n_dtype == NC && out_dtype == OC) {                                                              \
    if (wide)                                                                                                            \
      hipLaunchKernelGGL((xielu_wide_kernel<D, W, O>), dim3((unsigned)((blocks + 7) / 8)), dim3(256), 0, s, (const D*)in,  \
                         nsplit, (size_t)split_stride, (const W*)numbers, (O*)out, (size_t)count);                        \
    else                                                                                                                 \
      hipLaunchKernelGGL((xielu_kernel<D, W, O>), dim3((unsigned)blocks), dim3(256), 0, s, (const D*)in, nsplit,          \
                         (size_t)split_stride, (const W*)numbers, (O*)out, (size_t)count);                                \
    return launch_status();                                                                                              \
  }
  TLIE_CASE(kF32, float, kF32, float, kF32, float)
  TLIE_CASE(kF32, float, kBF16, bf16, kF32, float)
  TLIE_CASE(kF32, float, kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kBF16, bf16, kBF16, bf16)
#undef TLIE_CASE
  return kBadArgument;
}
