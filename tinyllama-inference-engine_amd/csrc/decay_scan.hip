// Linear attention with a decaying matrix state, token by token.  Per head, with a query q and a key k (dim values
// each), a value v (vdim values) and a decay w per key channel:
//   KIND 0, 1:   S' = diag(w) S + k v^T,   o = S'^T q                       (S: dim x vdim)
//   KIND 2:      o = (S + diag(u) k v^T)^T q,   then S' = diag(w) S + k v^T   (u: a bonus per key channel that
//                only the current token gets)
// KIND 0 takes one decay a head (the same for every channel and token), KIND 1 and 2 one a token and channel.
// S is the request's state (zero when it is admitted) and is carried from step to step; the state, the decays and
// all sums are float whatever type q, k and v come in.  There is no softmax and no denominator.
//
// A workgroup owns 64 columns of one head's S for one sequence of the step: lane l keeps column l of its tile,
// S[0 .. dim)[l], in registers, split over the workgroup's waves by dims, and walks tokens in order.  The state row
// of a head is laid out tile by tile, [tiles][dim][64].  Queries, keys and decays of four tokens at a time go
// through LDS (every lane needs all of them); the waves' parts of a token's sums meet in LDS, once a batch.
//
// A sequence that brings many tokens is taken in slices of 32 tokens that run side by side: every slice is walked
// from a state of zero and leaves where it ends and, per channel, the product of its decays (the update is linear
// in S); a second kernel gives every slice its start, start(c + 1) = decays(c) * start(c) + end(c), and the state
// its new value; a third walks every slice again from its start and writes the results.
//
// Sequences whose request slot is negative pad a recorded step: nothing is read or written for them.
#include "common.h"

namespace tlie {

constexpr int kScanBatch = 4, kScanSlice = 32;

// Columns col .. of a product [nsplit][tokens][row] (possibly partial sums that lie `stride` elements apart).
struct ScanColumns {
  const void* data;
  int nsplit;
  long long stride;
  int row;
  int col;
};

// MODE 0: the sequence's tokens of the step from the state, results and the new state written.
// MODE 1: a slice from zero; no results; where it ends and the products of its decays go to `parts`.
// MODE 2: a slice from the start that `parts` now holds for it; results written.
// parts: float [sequences, slices, heads, tiles, dim * 64 + dim] (S, then a channel's product of decays).
template <typename D, int DW, int WAVES, int MODE, int KIND>
__global__ void __launch_bounds__(64 * WAVES)
decay_scan_kernel(ScanColumns qc, ScanColumns kc, ScanColumns vc, const float* __restrict__ decay,
                  const float* __restrict__ head_decay, const float* __restrict__ bonus, float q_scale, float k_scale,
                  float* __restrict__ state, float* __restrict__ parts, const int* __restrict__ seq_start,
                  const int* __restrict__ seq_slot, float* __restrict__ out, int heads, int dim, int vdim, int tiles,
                  int slices, size_t slot_stride) {
  constexpr int NJ = DW >= 64 ? DW / 64 : 1, DMAX = DW * WAVES;
  __shared__ __attribute__((aligned(16))) float qs[kScanBatch][DMAX];
  __shared__ __attribute__((aligned(16))) float ks[kScanBatch][DMAX];
  __shared__ __attribute__((aligned(16))) float ws[KIND >= 1 ? kScanBatch : 1][KIND >= 1 ? DMAX : 4];
  __shared__ __attribute__((aligned(16))) float us[KIND == 2 ? DMAX : 4];
  __shared__ float met[WAVES][kScanBatch][65];         // a wave's part of a token's S^T q (64 lanes) and of the bonus' sum
  const int seq = MODE == 0 ? blockIdx.x : blockIdx.x / slices, slice = MODE == 0 ? 0 : blockIdx.x % slices;
  const int h = blockIdx.y, tile = blockIdx.z, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int base = wave * DW;                          // this wave's first dim
  const int slot = seq_slot[seq];
  if (slot < 0) return;
  int first = seq_start[seq], last = seq_start[seq + 1];
  if (MODE != 0) {
    first += slice * kScanSlice;
    last = min(last, first + kScanSlice);
  }
  if (first >= last) return;
  const int col = tile * 64 + lane;
  const bool live = col < vdim;
  const size_t state_floats = static_cast<size_t>(dim) * 64, part_floats = state_floats + dim;
  float* st = MODE == 0 ? state + static_cast<size_t>(slot) * slot_stride + (static_cast<size_t>(h) * tiles + tile) * state_floats
                        : parts + (((static_cast<size_t>(seq) * slices + slice) * heads + h) * tiles + tile) * part_floats;
  const float head_w = KIND == 0 ? head_decay[h] : 1.f;
  float S[DW];
  float product[NJ];                                   // MODE 1: the product of the decays of this lane's channels
#pragma unroll
  for (int d = 0; d < DW; ++d) S[d] = MODE != 1 && base + d < dim ? st[(base + d) * 64 + lane] : 0.f;
#pragma unroll
  for (int j = 0; j < NJ; ++j) product[j] = 1.f;
  if (KIND == 2) {
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int d = base + lane + 64 * j;
      if (lane + 64 * j < DW) us[d] = d < dim ? bonus[h * dim + d] : 0.f;
    }
  }

  const D* qd = static_cast<const D*>(qc.data);
  const D* kd = static_cast<const D*>(kc.data);
  const D* vd = static_cast<const D*>(vc.data);
  // a batch of tokens is asked for while the batch before it is worked on
  float rq[kScanBatch][NJ], rk[kScanBatch][NJ], rw[kScanBatch][NJ], rv[kScanBatch];
  auto fetch = [&](int t0) {
    const int nb = min(kScanBatch, last - t0);
#pragma unroll
    for (int b = 0; b < kScanBatch; ++b) {
      const size_t t = static_cast<size_t>(t0 + b);
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        const int d = base + lane + 64 * j;
        const bool there = b < nb && lane + 64 * j < DW && d < dim;
        rq[b][j] = MODE != 1 && there ? sum_splits(qd + t * qc.row + qc.col + h * dim + d, qc.nsplit, static_cast<size_t>(qc.stride)) * q_scale : 0.f;
        rk[b][j] = there ? sum_splits(kd + t * kc.row + kc.col + h * dim + d, kc.nsplit, static_cast<size_t>(kc.stride)) * k_scale : 0.f;
        rw[b][j] = KIND >= 1 && there ? decay[t * heads * dim + h * dim + d] : 1.f;
      }
      rv[b] = b < nb && live ? sum_splits(vd + t * vc.row + vc.col + h * vdim + col, vc.nsplit, static_cast<size_t>(vc.stride)) : 0.f;
    }
  };
  fetch(first);
  for (int t0 = first; t0 < last; t0 += kScanBatch) {
    const int nb = min(kScanBatch, last - t0);
    __syncthreads();                                   // the batch before has been read
    float vv[kScanBatch];
#pragma unroll
    for (int b = 0; b < kScanBatch; ++b) {
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        if (lane + 64 * j < DW) {
          if (MODE != 1) qs[b][base + lane + 64 * j] = rq[b][j];
          ks[b][base + lane + 64 * j] = rk[b][j];
          if (KIND >= 1) ws[b][base + lane + 64 * j] = rw[b][j];
          if (MODE == 1 && b < nb) product[j] *= KIND >= 1 ? rw[b][j] : head_w;
        }
      }
      vv[b] = rv[b];
    }
    __syncthreads();
    if (t0 + kScanBatch < last) fetch(t0 + kScanBatch);
    float top[kScanBatch], extra[kScanBatch];           // this wave's part of S^T q and of sum(q u k), a token each
#pragma unroll
    for (int b = 0; b < kScanBatch; ++b) {
      top[b] = extra[b] = 0.f;
      if (b >= nb) continue;                           // (the same for the whole wave)
      const float v = vv[b];
      float acc = 0.f, side = 0.f;
#pragma unroll
      for (int d0 = 0; d0 < DW; d0 += 4) {
        if (base + d0 < dim) {                         // (entries from dim on are zeros in LDS and stay zeros in S)
          const float4 k4 = *reinterpret_cast<const float4*>(&ks[b][base + d0]);
          float4 w4 = make_float4(head_w, head_w, head_w, head_w), q4 = make_float4(0.f, 0.f, 0.f, 0.f);
          if (KIND >= 1) w4 = *reinterpret_cast<const float4*>(&ws[b][base + d0]);
          if (MODE != 1) q4 = *reinterpret_cast<const float4*>(&qs[b][base + d0]);
          if (KIND == 2 && MODE != 1) {                // the result reads the state before this token joins it
            const float4 u4 = *reinterpret_cast<const float4*>(&us[base + d0]);
            acc += S[d0 + 0] * q4.x;
            acc += S[d0 + 1] * q4.y;
            acc += S[d0 + 2] * q4.z;
            acc += S[d0 + 3] * q4.w;
            side += q4.x * (u4.x * k4.x);
            side += q4.y * (u4.y * k4.y);
            side += q4.z * (u4.z * k4.z);
            side += q4.w * (u4.w * k4.w);
          }
          S[d0 + 0] = w4.x * S[d0 + 0] + k4.x * v;
          S[d0 + 1] = w4.y * S[d0 + 1] + k4.y * v;
          S[d0 + 2] = w4.z * S[d0 + 2] + k4.z * v;
          S[d0 + 3] = w4.w * S[d0 + 3] + k4.w * v;
          if (KIND != 2 && MODE != 1) {
            acc += S[d0 + 0] * q4.x;
            acc += S[d0 + 1] * q4.y;
            acc += S[d0 + 2] * q4.z;
            acc += S[d0 + 3] * q4.w;
          }
        }
      }
      top[b] = acc, extra[b] = side;
    }
    if (MODE == 1) continue;
    if (WAVES > 1) {
#pragma unroll
      for (int b = 0; b < kScanBatch; ++b) {
        met[wave][b][lane] = top[b];
        if (lane == 0) met[wave][b][64] = extra[b];
      }
      __syncthreads();
      if (wave != 0) continue;
#pragma unroll
      for (int b = 0; b < kScanBatch; ++b) {
#pragma unroll
        for (int w = 1; w < WAVES; ++w) top[b] += met[w][b][lane], extra[b] += met[w][b][64];
      }
    }
#pragma unroll
    for (int b = 0; b < kScanBatch; ++b) {
      if (b >= nb) continue;
      float result = top[b];
      if (KIND == 2) result += extra[b] * vv[b];
      if (live) out[(static_cast<size_t>(t0 + b) * heads + h) * vdim + col] = result;
    }
  }
  if (MODE == 2) return;
#pragma unroll
  for (int d = 0; d < DW; ++d)
    if (base + d < dim) st[(base + d) * 64 + lane] = S[d];
  if (MODE == 1) {
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int d = base + lane + 64 * j;
      if (lane + 64 * j < DW && d < dim) st[state_floats + d] = product[j];
    }
  }
}

// Every slice's start from the state and the slices before it, in place: where a slice's end stood its start stands
// afterwards; the state gets what the last slice leaves.  A thread an element of S of a (sequence, head, tile).
__global__ void __launch_bounds__(256)
decay_carry_kernel(float* __restrict__ parts, float* __restrict__ state, const int* __restrict__ seq_start,
                   const int* __restrict__ seq_slot, int heads, int tiles, int slices, int dim, size_t slot_stride) {
  const int seq = blockIdx.x, unit = blockIdx.y;       // unit: head * tiles + tile
  const int slot = seq_slot[seq];
  if (slot < 0) return;
  const int count = seq_start[seq + 1] - seq_start[seq];
  const int used = (count + kScanSlice - 1) / kScanSlice;
  const size_t state_floats = static_cast<size_t>(dim) * 64, part_floats = state_floats + dim;
  const int elements = dim * 64;
  float* st = state + static_cast<size_t>(slot) * slot_stride + static_cast<size_t>(unit) * state_floats;
  const size_t stride = static_cast<size_t>(heads) * tiles * part_floats;
  float* part = parts + (static_cast<size_t>(seq) * slices * heads * tiles + unit) * part_floats;
  for (int e = blockIdx.z * 256 + threadIdx.x; e < elements; e += gridDim.z * 256) {
    const int d = e >> 6;
    float value = st[e];
    int c = 0;
    for (; c + 4 <= used; c += 4) {                    // (four slices' ends asked for together; the chain is the sums' only)
      float end[4], keeps[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) end[u] = part[(c + u) * stride + e], keeps[u] = part[(c + u) * stride + elements + d];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        part[(c + u) * stride + e] = value;
        value = keeps[u] * value + end[u];
      }
    }
    for (; c < used; ++c) {
      const float end = part[c * stride + e], keeps = part[c * stride + elements + d];
      part[c * stride + e] = value;
      value = keeps * value + end;
    }
    if (used > 0) st[e] = value;
  }
}

// out[t, c] = decay(z), z = bias[c] + sum_r weight[c, r] * f(low[t, r]); f the identity or tanh.
// kind 0: sigmoid(z)^(1 / tau), formed as exp(logsigmoid(z) / tau); kind 1: exp(-exp(z)).  Float throughout.
// A workgroup takes TT tokens (their low rows lie in LDS) and a thread a channel for all of them, so that a channel's
// weights are read once for the tile; a step of few tokens takes tiles of one, for the workgroups' number.
constexpr int kDecayTokens = 8, kDecayTiledFrom = 64;

template <typename W, int TT>
__global__ void __launch_bounds__(256)
low_rank_decay_kernel(const float* __restrict__ low, int nsplit, size_t split_stride, int inner_tanh, const W* __restrict__ weight,
                      const W* __restrict__ bias, int kind, float tau, float* __restrict__ out, int tokens, int channels, int rank) {
  extern __shared__ float shared_low[];                // [TT][rank]
  const int t0 = blockIdx.x * TT;
  const int count = min(TT, tokens - t0);
  for (int i = threadIdx.x; i < TT * rank; i += blockDim.x) {
    const int b = i / rank;
    const float v = b < count ? sum_splits(low + static_cast<size_t>(t0) * rank + i, nsplit, split_stride) : 0.f;
    shared_low[i] = inner_tanh ? tanhf(v) : v;
  }
  __syncthreads();
  const float inv_tau = 1.f / tau;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < channels; c += gridDim.y * blockDim.x) {
    float z[TT];
    const float start = bias != nullptr ? to_float(bias[c]) : 0.f;
#pragma unroll
    for (int b = 0; b < TT; ++b) z[b] = start;
    const W* row = weight + static_cast<size_t>(c) * rank;
    for (int r = 0; r < rank; ++r) {
      const float w = to_float(row[r]);
#pragma unroll
      for (int b = 0; b < TT; ++b) z[b] += w * shared_low[b * rank + r];
    }
#pragma unroll
    for (int b = 0; b < TT; ++b) {
      if (b >= count) break;
      float w;
      if (kind == 0) w = expf((fminf(z[b], 0.f) - log1pf(expf(-fabsf(z[b])))) * inv_tau);
      else w = expf(-expf(z[b]));
      out[static_cast<size_t>(t0 + b) * channels + c] = w;
    }
  }
}

// Heads of a product turned by their positions on their way into a scan: the first `rot_dim` dims of each head,
// dim i with dim i + rot_dim / 2, by the angle position * inv_freq[i]; the rest pass; the first `heads_a` heads are
// multiplied by scale_a afterwards, the others by scale_b; `tail` more columns follow unchanged.  Floats out.
template <typename D>
__global__ void __launch_bounds__(256)
rotate_heads_kernel(const D* __restrict__ in, int nsplit, size_t split_stride, int row, int col, const int* __restrict__ positions,
                    const float* __restrict__ inv_freq, int rot_dim, int heads, int heads_a, int dim, float scale_a,
                    float scale_b, int tail, float* __restrict__ out) {
  const int t = blockIdx.x;
  const int width = heads * dim + tail, half = rot_dim / 2;
  const D* src = in + static_cast<size_t>(t) * row + col;
  const float position = static_cast<float>(positions[t]);
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < width; c += gridDim.y * blockDim.x) {
    float value = sum_splits(src + c, nsplit, split_stride);
    if (c < heads * dim) {
      const int head = c / dim, d = c - head * dim;
      if (d < rot_dim) {
        const int i = d < half ? d : d - half;
        float sine, cosine;
        sincosf(position * inv_freq[i], &sine, &cosine);
        const float other = sum_splits(src + (d < half ? c + half : c - half), nsplit, split_stride);
        value = d < half ? value * cosine - other * sine : value * cosine + other * sine;
      }
      value *= head < heads_a ? scale_a : scale_b;
    }
    out[static_cast<size_t>(t) * width + c] = value;
  }
}

}  // namespace tlie

using namespace tlie;

// q, k, v: columns of products of one type (see ScanColumns), q and k `heads * dim` wide, v `heads * vdim`; decay:
// float [tokens, heads * dim] (kind 1, 2) or null; head_decay: float [heads] (kind 0) or null; bonus: float
// [heads * dim] (kind 2) or null; state: float [slots, heads, tiles, dim * 64], tiles = ceil(vdim / 64), a slot's row
// slot_stride floats after the one before it (a row may hold more than the scan's part); seq_start
// [sequences + 1], seq_slot [sequences] (negative: skipped); out: float [tokens, heads * vdim].  slices 0: every
// sequence's tokens are walked in order; slices > 0 (at least ceil(most tokens of a sequence / 32)): in slices of
// 32 tokens side by side, with parts: float [sequences, slices, heads, tiles, dim * 64 + dim] as scratch.
extern "C" int tlie_decay_scan(const void* q, int q_nsplit, long long q_stride, int q_row, int q_col, const void* k,
                               int k_nsplit, long long k_stride, int k_row, int k_col, const void* v, int v_nsplit,
                               long long v_stride, int v_row, int v_col, int dtype, int kind, const float* decay,
                               const float* head_decay, const float* bonus, float q_scale, float k_scale, float* state,
                               const int* seq_start, const int* seq_slot, float* out, int sequences, int heads, int dim,
                               int vdim, int slices, float* parts, long long slot_stride, void* stream) {
  if (sequences <= 0 || heads <= 0 || dim <= 0 || dim > 256 || vdim <= 0 || kind < 0 || kind > 2) return kBadArgument;
  if (q_nsplit < 1 || k_nsplit < 1 || v_nsplit < 1) return kBadArgument;
  if ((kind == 0 && head_decay == nullptr) || (kind >= 1 && decay == nullptr) || (kind == 2 && bonus == nullptr)) return kBadArgument;
  const int tiles = (vdim + 63) / 64;
  if (heads > 65535 || tiles > 65535 || slices < 0 || (slices > 0 && parts == nullptr)) return kBadArgument;
  if (slot_stride < static_cast<long long>(heads) * tiles * dim * 64) return kBadArgument;
  if (q_col < 0 || k_col < 0 || v_col < 0 || q_col + heads * dim > q_row || k_col + heads * dim > k_row ||
      v_col + heads * vdim > v_row)
    return kBadArgument;
  hipStream_t s = (hipStream_t)stream;
  const ScanColumns qc{q, q_nsplit, q_stride, q_row, q_col}, kc{k, k_nsplit, k_stride, k_row, k_col},
      vc{v, v_nsplit, v_stride, v_row, v_col};
#define TLIE_LAUNCH(D, DW, WAVES, MODE, KIND, GRID)                                                                   \
  hipLaunchKernelGGL((decay_scan_kernel<D, DW, WAVES, MODE, KIND>), GRID, dim3(64 * WAVES), 0, s, qc, kc, vc, decay,   \
                     head_decay, bonus, q_scale, k_scale, state, parts, seq_start, seq_slot, out, heads, dim, vdim,    \
                     tiles, slices, (size_t)slot_stride)
#define TLIE_SIZES(D, MODE, KIND, GRID)                                                                               \
  if (dim <= 32) TLIE_LAUNCH(D, 32, 1, MODE, KIND, GRID);                                                             \
  else if (dim <= 64) TLIE_LAUNCH(D, 32, 2, MODE, KIND, GRID);                                                        \
  else if (dim <= 128) TLIE_LAUNCH(D, 32, 4, MODE, KIND, GRID);                                                       \
  else TLIE_LAUNCH(D, 64, 4, MODE, KIND, GRID)
#define TLIE_KINDS(D, MODE, GRID)                                                                                     \
  if (kind == 0) { TLIE_SIZES(D, MODE, 0, GRID); }                                                                    \
  else if (kind == 1) { TLIE_SIZES(D, MODE, 1, GRID); }                                                               \
  else { TLIE_SIZES(D, MODE, 2, GRID); }
#define TLIE_TYPES(MODE, GRID)                                                                                        \
  if (dtype == kF32) { TLIE_KINDS(float, MODE, GRID) }                                                                \
  else if (dtype == kBF16) { TLIE_KINDS(bf16, MODE, GRID) }                                                           \
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
  int across = (dim * 64 + 255) / 256;
  if (across > 16) across = 16;
  if (heads * tiles > 65535) return kBadArgument;
  hipLaunchKernelGGL(decay_carry_kernel, dim3(sequences, heads * tiles, across), dim3(256), 0, s, parts, state, seq_start,
                     seq_slot, heads, tiles, slices, dim, (size_t)slot_stride);
  if (launch_status() != kOk) return kLaunchFailed;
  TLIE_TYPES(2, sliced);
#undef TLIE_TYPES
#undef TLIE_KINDS
#undef TLIE_SIZES
#undef TLIE_LAUNCH
  return launch_status();
}

// low: a float product [nsplit][tokens][rank]; weight [channels, rank] and bias [channels] (or null) of w_dtype; out: float [tokens, channels].
extern "C" int tlie_low_rank_decay(const float* low, int nsplit, long long split_stride, int inner_tanh, const void* weight, const void* bias, int w_dtype, int kind,
                                   float tau, float* out, int tokens, int channels, int rank, void* stream) {
  if (tokens <= 0 || channels <= 0 || rank <= 0 || rank > 1024 || nsplit < 1 || kind < 0 || kind > 1 || (kind == 0 && !(tau > 0.f))) return kBadArgument;
  int across = (channels + 255) / 256;
  if (across > 64) across = 64;
  const int tile = tokens >= kDecayTiledFrom ? kDecayTokens : 1;
  const dim3 grid((tokens + tile - 1) / tile, across);
  const size_t lds = static_cast<size_t>(tile) * rank * sizeof(float);
  hipStream_t s = (hipStream_t)stream;
#define TLIE_LAUNCH(W, TT)                                                                                             \
  hipLaunchKernelGGL((low_rank_decay_kernel<W, TT>), grid, dim3(256), lds, s, low, nsplit, (size_t)split_stride, inner_tanh, (const W*)weight, \
                     (const W*)bias, kind, tau, out, tokens, channels, rank)
  if (w_dtype == kF32) {
    if (tile == 1) TLIE_LAUNCH(float, 1);
    else TLIE_LAUNCH(float, kDecayTokens);
  } else if (w_dtype == kBF16) {
    if (tile == 1) TLIE_LAUNCH(bf16, 1);
    else TLIE_LAUNCH(bf16, kDecayTokens);
  } else return kBadArgument;
#undef TLIE_LAUNCH
  return launch_status();
}

// in: a product [nsplit][tokens][row]; columns col .. col + heads * dim + tail are read; out: float [tokens, heads * dim + tail].
extern "C" int tlie_rotate_heads(const void* in, int dtype, int nsplit, long long split_stride, int row, int col,
                                 const int* positions, const float* inv_freq, int rot_dim, int heads, int heads_a, int dim,
                                 float scale_a, float scale_b, int tail, float* out, int tokens, void* stream) {
  if (tokens <= 0 || heads <= 0 || dim <= 0 || rot_dim < 0 || rot_dim > dim || rot_dim % 2 != 0 || tail < 0 || nsplit < 1) return kBadArgument;
  if (col < 0 || col + heads * dim + tail > row || (rot_dim > 0 && inv_freq == nullptr)) return kBadArgument;
  hipStream_t s = (hipStream_t)stream;
  int across = (heads * dim + tail + 1023) / 1024;       // (about four columns a thread)
  if (across > 64) across = 64;
  const dim3 grid(tokens, across);
  if (dtype == kF32)
    hipLaunchKernelGGL((rotate_heads_kernel<float>), grid, dim3(256), 0, s, (const float*)in, nsplit, (size_t)split_stride,
                       row, col, positions, inv_freq, rot_dim, heads, heads_a, dim, scale_a, scale_b, tail, out);
  else if (dtype == kBF16)
    hipLaunchKernelGGL((rotate_heads_kernel<bf16>), grid, dim3(256), 0, s, (const bf16*)in, nsplit, (size_t)split_stride,
                       row, col, positions, inv_freq, rot_dim, heads, heads_a, dim, scale_a, scale_b, tail, out);
  else return kBadArgument;
  return launch_status();
}
