// What stands between a mixer's per-head results and its output product when each head is normed by itself:
//   o[t, h, :]   = a[t, h, :]                                            one result a head, or
//                = a[t, first(h), :] - lambda * a[t, second(h), :]      two maps of attention a head, combined
//   out[t, h, e] = o[e] / sqrt(mean(o^2) + eps) * weight[h * dv + e] * mult * f(gate[t, h * dv + e])
// f is the sigmoid (gate_kind 0) or z * sigmoid(z) (gate_kind 1); weight and gate are optional (null: 1).  Everything is float; `a` holds floats, the gate is read from a
// product's columns (any type, possibly partial sums), out is in the activation type.
//
// Two maps: `a` then holds 2 * heads results a token in the order in which the attention kernel wants its
// query heads, those of one key head side by side: with r = heads / (key/value groups), head h = g * r + i has
// its first map at (2 g) * r + i and its second at (2 g + 1) * r + i.  A map's result may also come in `parts`
// pieces of dv / parts dims each (the attention kernel on the matrix cores takes value heads wider than the keys as
// several heads of the keys' size): piece p of the map of key head k = 2 g + m lies at ((k * parts + p) * r + i).
#include "common.h"

namespace tlie {

template <typename D, typename W, typename A>
__global__ void __launch_bounds__(256)
head_combine_kernel(const float* __restrict__ a, int heads, int dv, int pair_group, int parts, float lambda, float eps,
                    const W* __restrict__ weight, float mult, const D* __restrict__ gate, int gate_nsplit,
                    size_t gate_split_stride, int gate_row, int gate_col, int gate_kind, A* __restrict__ out) {
  const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int h = blockIdx.y * 4 + wave;
  if (h >= heads) return;                              // (a whole wave; no barrier follows)
  // where dim e of the head's first (and second) result lies: with two maps, a map's result may come in `parts`
  // pieces of dv / parts dims, the pieces of one key head's query heads piece by piece
  const int piece = dv / parts;
  const int g = pair_group > 0 ? h / pair_group : 0, i = pair_group > 0 ? h - g * pair_group : 0;
  const float* row = a + static_cast<size_t>(t) * (pair_group > 0 ? 2 : 1) * heads * dv;
  auto value = [&](int e) {
    if (pair_group <= 0) return row[static_cast<size_t>(h) * dv + e];
    const int p = e / piece, inside = e - p * piece;
    const float first = row[((static_cast<size_t>(2 * g) * parts + p) * pair_group + i) * piece + inside];
    const float second = row[((static_cast<size_t>(2 * g + 1) * parts + p) * pair_group + i) * piece + inside];
    return first - lambda * second;
  };
  auto emit = [&](int e, float normed) {
    const int c = h * dv + e;
    float v = normed * mult;
    if (weight != nullptr) v *= to_float(weight[c]);
    if (gate != nullptr) {
      const float z = sum_splits(gate + static_cast<size_t>(t) * gate_row + gate_col + c, gate_nsplit, gate_split_stride);
      v *= (gate_kind == 1 ? z : 1.f) / (1.f + expf(-z));
    }
    out[static_cast<size_t>(t) * heads * dv + c] = from_float<A>(v);
  };
  // a lane's dims (lane, lane + 64, ...) are read once and kept, up to 512 dims a head; beyond, read again
  constexpr int kKept = 8;
  const bool fits = dv <= 64 * kKept;
  float kept[kKept];
  float squares = 0.f;
#pragma unroll
  for (int i = 0; i < kKept; ++i) {
    const int e = lane + 64 * i;
    kept[i] = fits && e < dv ? value(e) : 0.f;
    squares += kept[i] * kept[i];
  }
  if (!fits) {
    for (int e = lane; e < dv; e += 64) {
      const float o = value(e);
      squares += o * o;
    }
  }
  const float r = 1.f / sqrtf(wave_sum(squares) / static_cast<float>(dv) + eps);
#pragma unroll
  for (int i = 0; i < kKept; ++i) {
    const int e = lane + 64 * i;
    if (fits && e < dv) emit(e, kept[i] * r);
  }
  if (fits) return;
  for (int e = lane; e < dv; e += 64) emit(e, value(e) * r);
}

}  // namespace tlie

using namespace tlie;

// a: float [tokens, (pair_group > 0 ? 2 : 1) * heads, dv]; weight (or null): [heads * dv] of weight_dtype; gate (or null):
// a product [nsplit][tokens][gate_row] of gate_dtype whose columns gate_col .. gate_col + heads * dv - 1 are read.
extern "C" int tlie_head_combine(const float* a, int tokens, int heads, int dv, int pair_group, int parts, float lambda, float eps,
                                 const void* weight, int weight_dtype, float mult, const void* gate, int gate_dtype,
                                 int gate_nsplit, long long gate_split_stride, int gate_row, int gate_col, int gate_kind,
                                 void* out, int out_dtype, void* stream) {
  if (tokens <= 0 || heads <= 0 || dv <= 0 || pair_group < 0 || (pair_group > 0 && heads % pair_group != 0)) return kBadArgument;
  if (parts < 1 || dv % parts != 0 || (parts > 1 && pair_group <= 0) || gate_kind < 0 || gate_kind > 1) return kBadArgument;
  if (gate != nullptr && (gate_nsplit < 1 || gate_col < 0 || gate_row < gate_col + heads * dv)) return kBadArgument;
  if (heads > 4 * 65535) return kBadArgument;
  const dim3 grid(tokens, (heads + 3) / 4);
  hipStream_t s = (hipStream_t)stream;
#define TLIE_CASE(GC, D, WC, W, AC, A)                                                                                   \
  if (gate_dtype == GC && weight_dtype == WC && out_dtype == AC) {                                                       \
    hipLaunchKernelGGL((head_combine_kernel<D, W, A>), grid, dim3(256), 0, s, a, heads, dv, pair_group, parts, lambda, eps,     \
                       (const W*)weight, mult, (const D*)gate, gate_nsplit, (size_t)gate_split_stride, gate_row, gate_col, \
                       gate_kind, (A*)out);                                                                                          \
    return launch_status();                                                                                              \
  }
  TLIE_CASE(kF32, float, kF32, float, kF32, float)
  TLIE_CASE(kF32, float, kF32, float, kBF16, bf16)
  TLIE_CASE(kF32, float, kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kF32, float, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kBF16, bf16, kBF16, bf16)
#undef TLIE_CASE
  return kBadArgument;
}
