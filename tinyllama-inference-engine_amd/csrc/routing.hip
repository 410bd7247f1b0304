// Products with a handful of outputs whose sums are float whatever the types (a router's logits, the gates of a
// recurrence), and what a routed feed-forward does with a router's scores.
//
//   few_outputs      out[t, n] = bias[n] + sum_k x[t, k] w[n, k]                          float out
//   ... as a router  s = sigmoid(out[t, :]); the `top` largest s (the lower index wins a tie) keep their s,
//                    all others become 0: scale[t, n]                                      float out
//   ... mode 1       the `top` largest sums themselves are picked, and keep their softmax over the picked ones only
//   ... extra        the last `extra` outputs stand outside the choice: each becomes its own sigmoid (a gate
//                    of something that every token uses)
//   routed_gate      hidden[t, c] = act(s g) * (s u), s = scale[t, c / block] for the first experts * block
//                    columns and 1 for the rest (a shared expert's), g and u side by side in gate_up[t, 2c], [2c + 1]
//   ... weigh 1      hidden[t, c] = s * act(g, u): the score weighs the expert's result (the second product is
//                    linear, so its input is weighed in the result's place); shared_scaled: the shared expert's
//                    columns take scale[t, experts] instead of 1; the experts' and the shared expert's gates have
//                    their own limits
//
// A token is a workgroup's: wave w of its four takes outputs w, w + 4, ..., lane l the inner indices l, l + 64,
// ...: the order of a sum depends on the sizes alone.
#include "common.h"

namespace tlie {

template <typename X, typename W>
__global__ void __launch_bounds__(256)
few_outputs_kernel(const X* __restrict__ x, const W* __restrict__ w, const W* __restrict__ bias, float* __restrict__ out,
                   int inner, int outputs, int top, int mode, int extra) {
  extern __shared__ float sums[];                      // outputs
  const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const X* row = x + static_cast<size_t>(t) * inner;
  // (eight inner indices a lane and load where the rows allow it: a wave then asks for a kilobyte or two at once, and a
  // sum of 2048 terms waits for memory four times, not sixteen)
  const bool wide = (inner & 7) == 0 && ((reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(w)) & 31) == 0;
  for (int n = wave; n < outputs; n += 4) {
    const W* weights = w + static_cast<size_t>(n) * inner;
    float a = 0.f, b = 0.f;
    if (wide) {
#pragma unroll 2
      for (int k = lane * 8; k < inner; k += 512) {
        float xv[8], wv[8];
        load8(row + k, xv);
        load8(weights + k, wv);
        a += xv[0] * wv[0];
        b += xv[1] * wv[1];
        a += xv[2] * wv[2];
        b += xv[3] * wv[3];
        a += xv[4] * wv[4];
        b += xv[5] * wv[5];
        a += xv[6] * wv[6];
        b += xv[7] * wv[7];
      }
    } else {
      int k = lane;
      for (; k + 64 < inner; k += 128) {
        a += to_float(row[k]) * to_float(weights[k]);
        b += to_float(row[k + 64]) * to_float(weights[k + 64]);
      }
      if (k < inner) a += to_float(row[k]) * to_float(weights[k]);
    }
    float total = wave_sum(a + b);
    if (bias != nullptr) total += to_float(bias[n]);
    if (top <= 0) {
      if (lane == 0) out[static_cast<size_t>(t) * outputs + n] = total;
    } else if (lane == 0) {
      sums[n] = (mode == 0 || n >= outputs - extra) ? 1.f / (1.f + expf(-total)) : total;
    }
  }
  if (top <= 0) return;
  __syncthreads();
  if (wave != 0) return;
  // the first wave picks: `top` times the largest score that is left, the lower index on a tie
  float* picked_out = out + static_cast<size_t>(t) * outputs;
  const int choices = outputs - extra;
  for (int n = lane; n < outputs; n += 64) picked_out[n] = n < choices ? 0.f : sums[n];
  const float gone = mode == 0 ? -2.f : -INFINITY;      // (below every score that is left)
  float first = 0.f, denominator = 0.f;                // mode 1: the largest picked sum, and the sum of the picked ones' exponentials
  int my_where = -1;
  float my_weight = 0.f;
  for (int round = 0; round < top; ++round) {
    float best = mode == 0 ? -1.f : -INFINITY;
    int where = 1 << 30;
    for (int n = lane; n < choices; n += 64) {
      const float s = sums[n];
      if (s > best) best = s, where = n;               // (ascending n: the first of equals stays)
    }
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
      const float other = __shfl_xor(best, offset, 64);
      const int other_where = __shfl_xor(where, offset, 64);
      if (other > best || (other == best && other_where < where)) best = other, where = other_where;
    }
    if (where >= choices) break;                       // fewer outputs than `top` (or sums that are not finite)
    if (round == 0) first = best;
    const float weight = mode == 0 ? best : expf(best - first);
    denominator += weight;
    if (mode == 1 && lane == round) my_where = where, my_weight = weight;      // (every lane holds the round's pick; lane `round` keeps it)
    if (lane == 0) {
      if (mode == 0) picked_out[where] = weight;
      sums[where] = gone;
    }
    // lane 0's writes are ordered before the other lanes' next reads of sums[] (one wave: LDS operations complete in order)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
  if (mode == 1 && my_where >= 0) picked_out[my_where] = my_weight / denominator;   // (at most 64 picks: one a lane)
}

// weigh 0: the score weighs the expert's input (act(s g) * (s u)); 1: its result (s * act(g, u)).  scale_cols: columns of a
// row of the scale matrix; shared_scaled: the columns after the experts' take scale[t, experts], not 1.  kind, alpha:
// the gate (see gated_value); limit, shared_limit: its limit for the experts' and for the shared expert's columns.
struct GateOptions {
  int weigh;
  int scale_cols;
  int shared_scaled;
  int kind;
  float alpha;
  float limit;
  float shared_limit;
};

template <typename D, typename A>
__global__ void __launch_bounds__(256)
routed_gate_kernel(const D* __restrict__ gate_up, int nsplit, size_t split_stride, const float* __restrict__ scale,
                   int experts, int block, A* __restrict__ out, int inter, bool wide, GateOptions options) {
  const int t = blockIdx.x;
  const D* row = gate_up + static_cast<size_t>(t) * 2 * inter;
  if (wide) {
    // four columns a thread: eight values in one load, four out in one store (no partial sums, four columns in one
    // expert's block, rows that start at multiples of 32 bytes)
    for (int c = (blockIdx.y * 256 + threadIdx.x) * 4; c < inter; c += gridDim.y * 1024) {
      const int e = c / block;
      const bool own = e < experts;
      const float s = own ? scale[static_cast<size_t>(t) * options.scale_cols + e]
                          : (options.shared_scaled ? scale[static_cast<size_t>(t) * options.scale_cols + experts] : 1.f);
      float v[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      if (s != 0.f) load8(row + 2 * c, v);
      A* to = out + static_cast<size_t>(t) * inter + c;
      const float limit = own ? options.limit : options.shared_limit;
      if (s == 0.f) store4(to, 0.f, 0.f, 0.f, 0.f);
      else if (options.weigh == 1)
        store4(to, s * gated_value(v[0], v[1], options.kind, options.alpha, limit), s * gated_value(v[2], v[3], options.kind, options.alpha, limit),
               s * gated_value(v[4], v[5], options.kind, options.alpha, limit), s * gated_value(v[6], v[7], options.kind, options.alpha, limit));
      else store4(to, gated_value(s * v[0], s * v[1], kGateSilu, 1.f, 0.f), gated_value(s * v[2], s * v[3], kGateSilu, 1.f, 0.f),
                  gated_value(s * v[4], s * v[5], kGateSilu, 1.f, 0.f), gated_value(s * v[6], s * v[7], kGateSilu, 1.f, 0.f));
    }
    return;
  }
  for (int c = blockIdx.y * 256 + threadIdx.x; c < inter; c += gridDim.y * 256) {
    const int e = c / block;
    const bool own = e < experts;
    const float s = own ? scale[static_cast<size_t>(t) * options.scale_cols + e]
                        : (options.shared_scaled ? scale[static_cast<size_t>(t) * options.scale_cols + experts] : 1.f);
    float v = 0.f;
    if (s != 0.f) {                                    // an expert the token does not use: silu(0) * 0
      const float g = sum_splits(row + 2 * c, nsplit, split_stride);
      const float u = sum_splits(row + 2 * c + 1, nsplit, split_stride);
      if (options.weigh == 1) v = s * gated_value(g, u, options.kind, options.alpha, own ? options.limit : options.shared_limit);
      else v = gated_value(s * g, s * u, kGateSilu, 1.f, 0.f);
    }
    out[static_cast<size_t>(t) * inter + c] = from_float<A>(v);
  }
}

}  // namespace tlie

using namespace tlie;

// x: [tokens, inner] of x_dtype; w: [outputs, inner] and bias (or null) [outputs] of w_dtype; out: float [tokens, outputs].
// top 0: the sums; top > 0: the router's scale matrix (see above).
// mode 0: sigmoid scores, the picked ones keep theirs; mode 1: the largest sums are picked and keep their softmax over the
// picked ones.  extra: trailing outputs outside the choice, which become their sigmoids (top > 0 only).
extern "C" int tlie_few_outputs(const void* x, int x_dtype, const void* w, const void* bias, int w_dtype, float* out,
                                int tokens, int inner, int outputs, int top, int mode, int extra, void* stream) {
  if (tokens <= 0 || inner <= 0 || outputs <= 0 || outputs > 4096 || top < 0) return kBadArgument;
  if (mode < 0 || mode > 1 || extra < 0 || (top == 0 && (mode != 0 || extra != 0)) || (top > 0 && top > outputs - extra) || (mode == 1 && top > 64)) return kBadArgument;
  hipStream_t s = (hipStream_t)stream;
  const size_t lds = static_cast<size_t>(outputs) * sizeof(float);
#define TLIE_CASE(XC, X, WC, W)                                                                                       \
  if (x_dtype == XC && w_dtype == WC) {                                                                               \
    hipLaunchKernelGGL((few_outputs_kernel<X, W>), dim3(tokens), dim3(256), lds, s, (const X*)x, (const W*)w,          \
                       (const W*)bias, out, inner, outputs, top, mode, extra);                                                     \
    return launch_status();                                                                                           \
  }
  TLIE_CASE(kF32, float, kF32, float)
  TLIE_CASE(kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kF32, float)
  TLIE_CASE(kF32, float, kBF16, bf16)
#undef TLIE_CASE
  return kBadArgument;
}

// gate_up: a product [nsplit][tokens][2 * inter], gate and up of a column side by side; scale: float [tokens, experts];
// the first experts * block columns are the experts', the rest a shared expert's; out: [tokens, inter] of out_dtype.
// weigh, scale_cols, shared_scaled, kind, alpha, limit, shared_limit: see GateOptions (weigh 0 takes the SiLU gate).
extern "C" int tlie_routed_gate(const void* gate_up, int in_dtype, int nsplit, long long split_stride, const float* scale,
                                int experts, int block, void* out, int out_dtype, int tokens, int inter, int weigh,
                                int scale_cols, int shared_scaled, int kind, float alpha, float limit, float shared_limit,
                                void* stream) {
  if (tokens <= 0 || inter <= 0 || experts < 0 || block <= 0 || nsplit < 1) return kBadArgument;
  if (weigh < 0 || weigh > 1 || scale_cols < experts + (shared_scaled ? 1 : 0) || (weigh == 0 && kind != kGateSilu)) return kBadArgument;
  if (kind != kGateSilu && kind != kGateClampedSwish) return kBadArgument;
  const GateOptions options{weigh, scale_cols, shared_scaled, kind, alpha, limit, shared_limit};
  if (static_cast<long long>(experts) * block > inter) return kBadArgument;
  const bool wide = nsplit == 1 && (inter & 3) == 0 && (block & 3) == 0 &&
                    ((reinterpret_cast<uintptr_t>(gate_up) | reinterpret_cast<uintptr_t>(out)) & 31) == 0;
  int across = (inter + (wide ? 1023 : 255)) / (wide ? 1024 : 256);
  if (across > 64) across = 64;
  const dim3 grid(tokens, across);
  hipStream_t s = (hipStream_t)stream;
#define TLIE_CASE(DC, D, AC, A)                                                                                       \
  if (in_dtype == DC && out_dtype == AC) {                                                                            \
    hipLaunchKernelGGL((routed_gate_kernel<D, A>), grid, dim3(256), 0, s, (const D*)gate_up, nsplit,                   \
                       (size_t)split_stride, scale, experts, block, (A*)out, inter, wide, options);                                  \
    return launch_status();                                                                                           \
  }
  TLIE_CASE(kF32, float, kF32, float)
  TLIE_CASE(kF32, float, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kBF16, bf16)
#undef TLIE_CASE
  return kBadArgument;
}
