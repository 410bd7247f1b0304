// Latent attention's step between its first product and the attention kernel: the low-rank vector of
// every token is normed and cached, the one rotated key part that all heads share is rotated and
// cached beside it, and the queries are taken apart.
//
// The product's columns: for each of H heads `plain` unrotated query dims and `rot` rotated ones, then
// `rank` dims of the latent vector, then `rot` dims of the shared key part.  What the cache keeps per
// position is the normed latent vector c and the rotated key part, nothing per head: a page holds the
// rows [c | rotated part] of its positions, which the attention kernel reads as keys of size rank + rot of
// a single key head, and after them c once more, transposed ([rank][row]), which it reads as that head's
// values.  The heads' own key and value matrices are applied to the queries before and to the attended
// latent vectors after the attention (the block-diagonal products), which gives the same scores and
// results as expanding every cached position's keys and values.
// The value side of a page has `value_rows` rows of a page's positions: rank of them, or rank + rot when
// the attention kernel that reads the page wants values as wide as keys; rows from rank on are never
// written, and hold the zeros the pool was made with.
//
// Rotation: of a rotated part's first `turn` dims (turn <= rot, even; the rest pass unchanged) the pair
// (i, i + turn/2) by angle = float(position) * inv_freq[i], sines and cosines float.
// Norm: c = x * rsqrt(mean(x^2) + eps) * weight over the rank dims, in float.
#include "common.h"

namespace tlie {

// q_plain: [tokens][H * plain] (what the per-head product onto the latent space reads);
// q_wide:  [tokens][H][rank + rot]: only the last rot dims of every head are written here.
template <typename D, typename W, typename A>
__global__ void latent_place_kernel(const D* __restrict__ fused, int nsplit, size_t split_stride,
                                    const int* __restrict__ positions, const int* __restrict__ slot_map,
                                    const float* __restrict__ inv_freq, const W* __restrict__ norm_weight, float eps,
                                    A* __restrict__ q_plain, A* __restrict__ q_wide, A* __restrict__ cache, int heads,
                                    int plain, int rot, int turn, int rank, int value_rows, int page_size, int row_width) {
  extern __shared__ float lds[];
  const int half = turn / 2;
  float* cosines = lds;                  // half
  float* sines = cosines + half;         // half
  float* scratch = sines + half;         // 16
  const int t = blockIdx.x;
  const int per_head = plain + rot, q_width = heads * per_head, key = rank + rot;
  const D* in = fused + static_cast<size_t>(t) * row_width;        // (a row may hold more columns after these: someone else's)
  const float pos = static_cast<float>(positions[t]);
  for (int i = threadIdx.x; i < half; i += blockDim.x) sincosf(pos * inv_freq[i], &sines[i], &cosines[i]);
  float square = 0.f;
  for (int i = threadIdx.x; i < rank; i += blockDim.x) {
    const float v = sum_splits(in + q_width + i, nsplit, split_stride);
    square += v * v;
  }
  const float scale = rsqrtf(block_sum(square, scratch) / static_cast<float>(rank) + eps);   // (its barriers also order the angles)

  auto turned = [&](const D* part, int e) {        // element e of a rotated part that starts at `part`
    const float own = sum_splits(part + e, nsplit, split_stride);
    if (e >= turn) return own;
    if (e < half) return own * cosines[e] - sum_splits(part + e + half, nsplit, split_stride) * sines[e];
    return own * cosines[e - half] + sum_splits(part + e - half, nsplit, split_stride) * sines[e - half];
  };
  const int slot = slot_map[t];
  if (slot >= 0) {
    A* page = cache + static_cast<size_t>(slot / page_size) * page_size * (key + value_rows);
    const int row = slot % page_size;
    for (int i = threadIdx.x; i < key; i += blockDim.x) {
      if (i < rank) {
        const A c = from_float<A>(sum_splits(in + q_width + i, nsplit, split_stride) * scale * to_float(norm_weight[i]));
        page[static_cast<size_t>(row) * key + i] = c;
        page[static_cast<size_t>(page_size) * key + static_cast<size_t>(i) * page_size + row] = c;
      } else {
        page[static_cast<size_t>(row) * key + i] = from_float<A>(turned(in + q_width + rank, i - rank));
      }
    }
  }
  for (int c = threadIdx.x; c < q_width; c += blockDim.x) {
    const int head = c / per_head, e = c % per_head;
    if (e < plain)
      q_plain[(static_cast<size_t>(t) * heads + head) * plain + e] = from_float<A>(sum_splits(in + c, nsplit, split_stride));
    else
      q_wide[(static_cast<size_t>(t) * heads + head) * key + rank + (e - plain)] = from_float<A>(turned(in + head * per_head + plain, e - plain));
  }
}

}  // namespace tlie

using namespace tlie;

extern "C" int tlie_latent_place(const void* fused, int in_dtype, int nsplit, long long split_stride, const int* positions,
                                 const int* slot_map, const float* inv_freq, const void* norm_weight, int weight_dtype,
                                 float eps, void* q_plain, void* q_wide, void* cache, int act_dtype, int tokens, int heads,
                                 int plain, int rot, int turn, int rank, int value_rows, int page_size, int row_width, void* stream) {
  if (tokens <= 0 || heads <= 0 || plain <= 0 || rot < 0 || turn < 0 || turn > rot || turn % 2 != 0 || rank <= 0 || page_size <= 0 ||
      nsplit < 1)
    return kBadArgument;
  if (value_rows != rank && value_rows != rank + rot) return kBadArgument;
  if (turn > 0 && inv_freq == nullptr) return kBadArgument;
  if (row_width < heads * (plain + rot) + rank + rot) return kBadArgument;
  const int widest = heads * (plain + rot);
  const int threads = widest >= 1024 ? 1024 : (widest >= 256 ? 256 : 64);
  const size_t lds = (static_cast<size_t>(rot) + 16) * sizeof(float);
  hipStream_t s = (hipStream_t)stream;
#define TLIE_CASE(DC, D, WC, W, AC, A)                                                                              \
  if (in_dtype == DC && weight_dtype == WC && act_dtype == AC) {                                                     \
    hipLaunchKernelGGL((latent_place_kernel<D, W, A>), dim3(tokens), dim3(threads), lds, s, (const D*)fused, nsplit,   \
                       (size_t)split_stride, positions, slot_map, inv_freq, (const W*)norm_weight, eps, (A*)q_plain,  \
                       (A*)q_wide, (A*)cache, heads, plain, rot, turn, rank, value_rows, page_size, row_width);                                   \
    return launch_status();                                                                                          \
  }
  TLIE_CASE(kF32, float, kF32, float, kF32, float)
  TLIE_CASE(kF32, float, kF32, float, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kF32, float, kBF16, bf16)
  TLIE_CASE(kF32, float, kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kBF16, bf16, kBF16, bf16)
#undef TLIE_CASE
  return kBadArgument;
}
