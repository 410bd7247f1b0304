// Token-parallel kernels: embedding gather, residual-add + RMSNorm, SiLU*mul.
//
// A matrix product's result reaches these kernels either as one [rows, cols] array in the
// activation type, or as `nsplit` float partial sums [nsplit, rows, cols] that a split-K product
// left unsummed; the consumer adds them up, in a fixed order, so no separate reduction runs.
#include "common.h"

namespace tlie {

// ---- embedding: residual[t, :] = table[token[t], :] as float -------------------------------
// reference: a row copy per token (src/model.cpp:94-97, src/cuda/model.cu:388-391)
template <typename W>
__global__ void embed_gather_kernel(const int* __restrict__ tokens, const W* __restrict__ table,
                                    float* __restrict__ residual, int hidden) {
  const int t = blockIdx.x;
  const W* row = table + static_cast<size_t>(tokens[t]) * hidden;
  float* out = residual + static_cast<size_t>(t) * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) out[i] = to_float(row[i]);
}

// ---- residual += delta (+ bias); out = RMSNorm(residual) * weight ----------------------------
// reference: y = x * rsqrt(mean(x^2) + eps) * w, sum in float (src/cuda/kernels.cu:67-84);
// the add before it is AddInPlace (kernels.cu:208-215).  Here the residual stays in float.
// rows != nullptr: row r of the output comes from residual row rows[r] (and delta row rows[r]);
// the residual is then left untouched (used for the final norm at the wanted positions).
template <typename D, typename W, typename O>
__global__ void add_rmsnorm_kernel(float* __restrict__ residual, const D* __restrict__ delta, int nsplit,
                                   size_t split_stride, const W* __restrict__ weight, float eps, O* __restrict__ out,
                                   const int* __restrict__ rows, int hidden) {
  extern __shared__ float row_cache[];           // hidden floats, then 16 for the reduction
  float* scratch = row_cache + hidden;
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  float* res = residual + static_cast<size_t>(src) * hidden;
  float square = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    float v = res[i];
    if (delta) {
      v += sum_splits(delta + static_cast<size_t>(src) * hidden + i, nsplit, split_stride);
      if (!rows) res[i] = v;
    }
    row_cache[i] = v;
    square += v * v;
  }
  const float total = block_sum(square, scratch);
  const float scale = rsqrtf(total / static_cast<float>(hidden) + eps);
  if (out) {
    O* o = out + static_cast<size_t>(r) * hidden;
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) o[i] = from_float<O>(row_cache[i] * scale * to_float(weight[i]));
  }
}

// The same with eight elements a thread (16-byte loads and stores): hidden % 8 == 0; the summands
// of a split product are added in the order of their index.
template <typename D, typename W, typename O>
__global__ void add_rmsnorm_wide_kernel(float* __restrict__ residual, const D* __restrict__ delta, int nsplit,
                                        size_t split_stride, const W* __restrict__ weight, float eps,
                                        O* __restrict__ out, const int* __restrict__ rows, int hidden) {
  extern __shared__ float row_cache[];           // hidden floats, then 16 for the reduction
  float* scratch = row_cache + hidden;
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  float* res = residual + static_cast<size_t>(src) * hidden;
  float square = 0.f;
  for (int i = threadIdx.x * 8; i < hidden; i += blockDim.x * 8) {
    float v[8];
    load8(res + i, v);
    if (delta) {
      const D* part = delta + static_cast<size_t>(src) * hidden + i;
      float d[8];
      load8(part, d);
      for (int s = 1; s < nsplit; ++s) {
        float more[8];
        load8(part + s * split_stride, more);
#pragma unroll
        for (int j = 0; j < 8; ++j) d[j] += more[j];
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] += d[j];
      if (!rows) store8(res + i, v);
    }
    store8(row_cache + i, v);
#pragma unroll
    for (int j = 0; j < 8; ++j) square += v[j] * v[j];
  }
  const float total = block_sum(square, scratch);
  const float scale = rsqrtf(total / static_cast<float>(hidden) + eps);
  if (out) {
    O* o = out + static_cast<size_t>(r) * hidden;
    for (int i = threadIdx.x * 8; i < hidden; i += blockDim.x * 8) {
      float v[8], w[8];
      load8(row_cache + i, v);                   // the thread's own entries
      load8(weight + i, w);
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = v[j] * scale * w[j];
      store8(o + i, v);
    }
  }
}

// ---- act[t, i] = silu(gate[t, i]) * up[t, i]; gate_up is [rows, 2 * inter], either [gate | up] or,
// interleaved, g0 u0 g1 u1 ... (the layout the gated product of few rows wants of its weight) -------
// reference: (g / (1 + exp(-g))) * u in float (src/cuda/kernels.cu:198-206)
template <typename D, typename O>
__global__ void silu_mul_kernel(const D* __restrict__ gate_up, int nsplit, size_t split_stride,
                                O* __restrict__ out, int rows, int inter, int interleaved, int kind, float alpha, float limit) {
  const size_t total = static_cast<size_t>(rows) * inter;
  for (size_t index = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; index < total;
       index += static_cast<size_t>(gridDim.x) * blockDim.x) {
    const size_t t = index / inter, i = index % inter;
    const D* base = gate_up + t * 2 * inter;
    const float g = sum_splits(base + (interleaved ? 2 * i : i), nsplit, split_stride);
    const float u = sum_splits(base + (interleaved ? 2 * i + 1 : inter + i), nsplit, split_stride);
    out[index] = from_float<O>(gated_value(g, u, kind, alpha, limit));
  }
}

// Eight results a thread from sixteen inputs: inter % 8 == 0; the summands of a split product are
// added in the order of their index.
template <typename D, typename O>
__global__ void silu_mul_wide_kernel(const D* __restrict__ gate_up, int nsplit, size_t split_stride, O* __restrict__ out,
                                     int rows, int inter, int interleaved, int kind, float alpha, float limit) {
  const int per_row = inter / 8;
  const size_t total = static_cast<size_t>(rows) * per_row;
  for (size_t index = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; index < total;
       index += static_cast<size_t>(gridDim.x) * blockDim.x) {
    const size_t t = index / per_row;
    const int i = static_cast<int>(index % per_row) * 8;
    const D* base = gate_up + t * 2 * inter;
    float a[8], b[8], g[8], u[8];
    const int first = interleaved ? 2 * i : i, second = interleaved ? 2 * i + 8 : inter + i;
    load8(base + first, a);
    load8(base + second, b);
    for (int s = 1; s < nsplit; ++s) {
      float more[8];
      load8(base + s * split_stride + first, more);
#pragma unroll
      for (int j = 0; j < 8; ++j) a[j] += more[j];
      load8(base + s * split_stride + second, more);
#pragma unroll
      for (int j = 0; j < 8; ++j) b[j] += more[j];
    }
    if (interleaved) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        g[j] = a[2 * j]; u[j] = a[2 * j + 1];
        g[4 + j] = b[2 * j]; u[4 + j] = b[2 * j + 1];
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) g[j] = a[j], u[j] = b[j];
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) g[j] = gated_value(g[j], u[j], kind, alpha, limit);
    store8(out + t * inter + i, g);
  }
}

// ---- residual += RMSNorm(delta) * post_weight; out = RMSNorm(residual) * weight ---------------------
// For blocks that norm a sublayer's result before it joins the residual, and norm the residual again
// before the next sublayer: both in one pass over the row.  Sums of squares, scales and the residual
// sum are float.  rows != nullptr: only those rows, and the residual is left as it was; out may be
// null (the residual is brought up to date and nothing else).
template <typename D, typename W, typename O>
__global__ void norm_add_rmsnorm_kernel(float* __restrict__ residual, const D* __restrict__ delta, int nsplit,
                                        size_t split_stride, const W* __restrict__ post_weight, float post_eps,
                                        const W* __restrict__ weight, float eps, O* __restrict__ out,
                                        const int* __restrict__ rows, int hidden) {
  extern __shared__ float row_cache[];           // hidden floats, then 16 for the reductions
  float* scratch = row_cache + hidden;
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  float* res = residual + static_cast<size_t>(src) * hidden;
  float square = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float v = sum_splits(delta + static_cast<size_t>(src) * hidden + i, nsplit, split_stride);
    row_cache[i] = v;                            // (a thread reads back only what it wrote itself)
    square += v * v;
  }
  const float post_scale = rsqrtf(block_sum(square, scratch) / static_cast<float>(hidden) + post_eps);
  square = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float v = res[i] + row_cache[i] * post_scale * to_float(post_weight[i]);
    if (!rows) res[i] = v;
    row_cache[i] = v;
    square += v * v;
  }
  if (out == nullptr) return;                    // (the same for the whole grid)
  const float scale = rsqrtf(block_sum(square, scratch) / static_cast<float>(hidden) + eps);
  O* o = out + static_cast<size_t>(r) * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) o[i] = from_float<O>(row_cache[i] * scale * to_float(weight[i]));
}

// The same with eight elements a thread (16-byte loads and stores): hidden % 8 == 0; the summands of a split
// product are added in the order of their index.
template <typename D, typename W, typename O>
__global__ void norm_add_rmsnorm_wide_kernel(float* __restrict__ residual, const D* __restrict__ delta, int nsplit,
                                             size_t split_stride, const W* __restrict__ post_weight, float post_eps,
                                             const W* __restrict__ weight, float eps, O* __restrict__ out,
                                             const int* __restrict__ rows, int hidden) {
  extern __shared__ float row_cache[];           // hidden floats, then 16 for the reductions
  float* scratch = row_cache + hidden;
  const int r = blockIdx.x;
  const int src = rows ? rows[r] : r;
  float* res = residual + static_cast<size_t>(src) * hidden;
  float square = 0.f;
  for (int i = threadIdx.x * 8; i < hidden; i += blockDim.x * 8) {
    const D* part = delta + static_cast<size_t>(src) * hidden + i;
    float d[8];
    load8(part, d);
    for (int s = 1; s < nsplit; ++s) {
      float more[8];
      load8(part + s * split_stride, more);
#pragma unroll
      for (int j = 0; j < 8; ++j) d[j] += more[j];
    }
    store8(row_cache + i, d);                    // (a thread reads back only what it wrote itself)
#pragma unroll
    for (int j = 0; j < 8; ++j) square += d[j] * d[j];
  }
  const float post_scale = rsqrtf(block_sum(square, scratch) / static_cast<float>(hidden) + post_eps);
  square = 0.f;
  for (int i = threadIdx.x * 8; i < hidden; i += blockDim.x * 8) {
    float v[8], d[8], w[8];
    load8(res + i, v);
    load8(row_cache + i, d);
    load8(post_weight + i, w);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = v[j] + d[j] * post_scale * w[j];
    if (!rows) store8(res + i, v);
    store8(row_cache + i, v);
#pragma unroll
    for (int j = 0; j < 8; ++j) square += v[j] * v[j];
  }
  if (out == nullptr) return;                    // (the same for the whole grid)
  const float scale = rsqrtf(block_sum(square, scratch) / static_cast<float>(hidden) + eps);
  O* o = out + static_cast<size_t>(r) * hidden;
  for (int i = threadIdx.x * 8; i < hidden; i += blockDim.x * 8) {
    float v[8], w[8];
    load8(row_cache + i, v);
    load8(weight + i, w);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = v[j] * scale * w[j];
    store8(o + i, v);
  }
}

// ---- out[r, c] = product[r, c] + bias[c] ------------------------------------------------------
// For a product that a library made without its bias (steps of many rows): the bias joins the
// float sums, as in the kernels that add it themselves, and the result is rounded once.
// reference: AddBiasKernel after the library's product (src/cuda/kernels.cu:198-206).
template <typename B, typename O>
__global__ void add_bias_kernel(const float* __restrict__ product, const B* __restrict__ bias, O* __restrict__ out,
                                size_t total, int cols) {
  for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < total; i += static_cast<size_t>(gridDim.x) * blockDim.x)
    out[i] = from_float<O>(product[i] + to_float(bias[i % cols]));
}

// ---- values[t, c] *= sigmoid(pre[t, col + c]): a gate on a mixer's heads, its pre-activations columns col .. col + cols - 1
// of a wider product (row_width columns a row); the sigmoid and the product float -------------------------------------
template <typename D, typename A>
__global__ void sigmoid_gate_kernel(A* __restrict__ values, const D* __restrict__ pre, int nsplit, size_t split_stride,
                                    int col, int row_width, size_t total, int cols) {
  for (size_t index = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; index < total;
       index += static_cast<size_t>(gridDim.x) * blockDim.x) {
    const size_t t = index / cols, c = index % cols;
    const float z = sum_splits(pre + t * row_width + col + c, nsplit, split_stride);
    values[index] = from_float<A>(to_float(values[index]) / (1.f + expf(-z)));
  }
}

// The same with eight columns a thread (no partial sums, cols, col and row_width multiples of 8, 16-byte aligned arrays).
template <typename D, typename A>
__global__ void sigmoid_gate_wide_kernel(A* __restrict__ values, const D* __restrict__ pre, int col, int row_width, size_t groups, int cols) {
  const int per_row = cols / 8;
  for (size_t index = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; index < groups;
       index += static_cast<size_t>(gridDim.x) * blockDim.x) {
    const size_t t = index / per_row;
    const int c = static_cast<int>(index % per_row) * 8;
    float v[8], z[8];
    load8(values + t * cols + c, v);
    load8(pre + t * row_width + col + c, z);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = v[j] / (1.f + expf(-z[j]));
    store8(values + t * cols + c, v);
  }
}

// ---- x <- cap * tanh(x / cap), in place (capped logits) --------------------------------------------------------------
__global__ void softcap_kernel(float* __restrict__ x, size_t total, float cap) {
  for (size_t index = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; index < total;
       index += static_cast<size_t>(gridDim.x) * blockDim.x)
    x[index] = cap * tanhf(x[index] / cap);
}

}  // namespace tlie

using namespace tlie;

extern "C" int tlie_embed_gather(const int* tokens, const void* table, int table_dtype, float* residual,
                                 int num_tokens, int hidden, void* stream) {
  if (num_tokens <= 0 || hidden <= 0) return kBadArgument;
  const int threads = hidden >= 1024 ? 256 : 64;
  if (table_dtype == kF32)
    hipLaunchKernelGGL(embed_gather_kernel<float>, dim3(num_tokens), dim3(threads), 0, (hipStream_t)stream,
                       tokens, (const float*)table, residual, hidden);
  else if (table_dtype == kBF16)
    hipLaunchKernelGGL(embed_gather_kernel<bf16>, dim3(num_tokens), dim3(threads), 0, (hipStream_t)stream,
                       tokens, (const bf16*)table, residual, hidden);
  else
    return kBadArgument;
  return launch_status();
}

template <typename D, typename W, typename O>
static int launch_add_rmsnorm(float* residual, const void* delta, int nsplit, size_t split_stride,
                              const void* weight, float eps, void* out,
                              const int* rows, int num_rows, int hidden, hipStream_t stream) {
  const size_t lds = (static_cast<size_t>(hidden) + 16) * sizeof(float);
  if (lds > 160 * 1024) return kBadArgument;
  const bool aligned = ((reinterpret_cast<uintptr_t>(residual) | reinterpret_cast<uintptr_t>(delta) |
                         reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(out)) & 31) == 0;
  if ((hidden & 7) == 0 && aligned && (nsplit == 1 || (split_stride * sizeof(D)) % 32 == 0)) {
    const int chunks = hidden / 8;
    const int wide = chunks >= 1024 ? 1024 : (chunks + 63) / 64 * 64;
    hipLaunchKernelGGL((add_rmsnorm_wide_kernel<D, W, O>), dim3(num_rows), dim3(wide), lds, stream, residual,
                       (const D*)delta, nsplit, split_stride, (const W*)weight, eps, (O*)out, rows, hidden);
    return launch_status();
  }
  const int threads = hidden >= 2048 ? 1024 : (hidden >= 1024 ? 512 : (hidden >= 256 ? 256 : 64));
  hipLaunchKernelGGL((add_rmsnorm_kernel<D, W, O>), dim3(num_rows), dim3(threads), lds, stream, residual,
                     (const D*)delta, nsplit, split_stride, (const W*)weight, eps, (O*)out, rows, hidden);
  return launch_status();
}

// delta may be null (no add); rows may be null (all rows, residual updated in place);
// out may be null (residual update only).
extern "C" int tlie_add_rmsnorm(float* residual, const void* delta, int delta_dtype, int nsplit,
                                long long split_stride, const void* weight, int weight_dtype,
                                float eps, void* out, int out_dtype, const int* rows, int num_rows, int hidden,
                                void* stream) {
  if (num_rows <= 0 || hidden <= 0 || nsplit < 1) return kBadArgument;
  hipStream_t s = (hipStream_t)stream;
#define TLIE_CASE(DC, D, WC, W, OC, O)                                                                     \
  if (delta_dtype == DC && weight_dtype == WC && out_dtype == OC)                                          \
    return launch_add_rmsnorm<D, W, O>(residual, delta, nsplit, (size_t)split_stride, weight, eps, out, \
                                       rows, num_rows, hidden, s);
  TLIE_CASE(kF32, float, kF32, float, kF32, float)
  TLIE_CASE(kF32, float, kF32, float, kBF16, bf16)
  TLIE_CASE(kF32, float, kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kF32, float, kBF16, bf16)
  TLIE_CASE(kF32, float, kBF16, bf16, kF32, float)
#undef TLIE_CASE
  return kBadArgument;
}

// delta [nsplit][rows][hidden]; post_weight and weight [hidden] of one type; weight and out may be null
// together (no norm after the add); rows may be null (all rows, residual updated in place).
extern "C" int tlie_norm_add_rmsnorm(float* residual, const void* delta, int delta_dtype, int nsplit, long long split_stride,
                                     const void* post_weight, float post_eps, const void* weight, int weight_dtype, float eps,
                                     void* out, int out_dtype, const int* rows, int num_rows, int hidden, void* stream) {
  if (num_rows <= 0 || hidden <= 0 || nsplit < 1 || delta == nullptr || post_weight == nullptr) return kBadArgument;
  if ((out == nullptr) != (weight == nullptr)) return kBadArgument;
  const size_t lds = (static_cast<size_t>(hidden) + 16) * sizeof(float);
  if (lds > 160 * 1024) return kBadArgument;
  const int threads = hidden >= 4096 ? 1024 : (hidden >= 1024 ? 512 : (hidden >= 256 ? 256 : 64));
  hipStream_t s = (hipStream_t)stream;
  const bool aligned = ((reinterpret_cast<uintptr_t>(residual) | reinterpret_cast<uintptr_t>(delta) | reinterpret_cast<uintptr_t>(post_weight) |
                         reinterpret_cast<uintptr_t>(weight) | reinterpret_cast<uintptr_t>(out)) & 31) == 0;
  const size_t delta_size = delta_dtype == kF32 ? 4 : 2;
  const bool wide = (hidden & 7) == 0 && aligned && (nsplit == 1 || (static_cast<size_t>(split_stride) * delta_size) % 32 == 0);
  const int chunks = hidden / 8;
  const int wide_threads = chunks >= 1024 ? 1024 : (chunks + 63) / 64 * 64;
#define TLIE_CASE(DC, D, WC, W, OC, O)                                                                              \
  if (delta_dtype == DC && weight_dtype == WC && out_dtype == OC) {                                                 \
    if (wide) {                                                                                                     \
      hipLaunchKernelGGL((norm_add_rmsnorm_wide_kernel<D, W, O>), dim3(num_rows), dim3(wide_threads), lds, s, residual, \
                         (const D*)delta, nsplit, (size_t)split_stride, (const W*)post_weight, post_eps,            \
                         (const W*)weight, eps, (O*)out, rows, hidden);                                              \
      return launch_status();                                                                                       \
    }                                                                                                               \
    hipLaunchKernelGGL((norm_add_rmsnorm_kernel<D, W, O>), dim3(num_rows), dim3(threads), lds, s, residual,          \
                       (const D*)delta, nsplit, (size_t)split_stride, (const W*)post_weight, post_eps,              \
                       (const W*)weight, eps, (O*)out, rows, hidden);                                                \
    return launch_status();                                                                                         \
  }
  TLIE_CASE(kF32, float, kF32, float, kF32, float)
  TLIE_CASE(kF32, float, kF32, float, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kF32, float, kBF16, bf16)
  TLIE_CASE(kF32, float, kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kF32, float, kBF16, bf16, kF32, float)
#undef TLIE_CASE
  return kBadArgument;
}

extern "C" int tlie_silu_mul(const void* gate_up, int in_dtype, int nsplit, long long split_stride, void* out,
                             int out_dtype, int rows, int inter, int interleaved, int kind, float alpha, float limit,
                             void* stream) {
  if (rows <= 0 || inter <= 0 || nsplit < 1 || kind < 0 || kind > 1) return kBadArgument;
  const size_t total = static_cast<size_t>(rows) * inter;
  const int threads = 256;
  const int blocks = static_cast<int>(total / threads + 1 < 65536 ? total / threads + 1 : 65536);
  hipStream_t s = (hipStream_t)stream;
  const bool aligned = ((reinterpret_cast<uintptr_t>(gate_up) | reinterpret_cast<uintptr_t>(out)) & 31) == 0;
  if ((inter & 7) == 0 && aligned && (nsplit == 1 || (in_dtype == kF32 && (split_stride & 7) == 0))) {
    const size_t groups = total / 8;
    const int wide = static_cast<int>(groups / threads + 1 < 65536 ? groups / threads + 1 : 65536);
    if (in_dtype == kF32 && out_dtype == kF32)
      hipLaunchKernelGGL((silu_mul_wide_kernel<float, float>), dim3(wide), dim3(threads), 0, s, (const float*)gate_up,
                         nsplit, (size_t)split_stride, (float*)out, rows, inter, interleaved, kind, alpha, limit);
    else if (in_dtype == kF32 && out_dtype == kBF16)
      hipLaunchKernelGGL((silu_mul_wide_kernel<float, bf16>), dim3(wide), dim3(threads), 0, s, (const float*)gate_up,
                         nsplit, (size_t)split_stride, (bf16*)out, rows, inter, interleaved, kind, alpha, limit);
    else if (in_dtype == kBF16 && out_dtype == kBF16)
      hipLaunchKernelGGL((silu_mul_wide_kernel<bf16, bf16>), dim3(wide), dim3(threads), 0, s, (const bf16*)gate_up,
                         nsplit, (size_t)split_stride, (bf16*)out, rows, inter, interleaved, kind, alpha, limit);
    else
      return kBadArgument;
    return launch_status();
  }
  if (in_dtype == kF32 && out_dtype == kF32)
    hipLaunchKernelGGL((silu_mul_kernel<float, float>), dim3(blocks), dim3(threads), 0, s, (const float*)gate_up, nsplit,
                       (size_t)split_stride, (float*)out, rows, inter, interleaved, kind, alpha, limit);
  else if (in_dtype == kF32 && out_dtype == kBF16)
    hipLaunchKernelGGL((silu_mul_kernel<float, bf16>), dim3(blocks), dim3(threads), 0, s, (const float*)gate_up, nsplit,
                       (size_t)split_stride, (bf16*)out, rows, inter, interleaved, kind, alpha, limit);
  else if (in_dtype == kBF16 && out_dtype == kBF16)
    hipLaunchKernelGGL((silu_mul_kernel<bf16, bf16>), dim3(blocks), dim3(threads), 0, s, (const bf16*)gate_up, nsplit,
                       (size_t)split_stride, (bf16*)out, rows, inter, interleaved, kind, alpha, limit);
  else
    return kBadArgument;
  return launch_status();
}

// product float [rows, cols], bias [cols] (float or bfloat16), out [rows, cols] (float: may be `product` itself; or bfloat16).
extern "C" int tlie_add_bias(const float* product, const void* bias, int bias_dtype, void* out, int out_dtype, int rows,
                             int cols, void* stream) {
  if (rows <= 0 || cols <= 0) return kBadArgument;
  const size_t total = static_cast<size_t>(rows) * cols;
  const int threads = 256;
  const int blocks = static_cast<int>((total + threads - 1) / threads < 16384 ? (total + threads - 1) / threads : 16384);
  hipStream_t s = (hipStream_t)stream;
#define TLIE_CASE(BC, B, OC, O)                                                                                  \
  if (bias_dtype == BC && out_dtype == OC) {                                                                     \
    hipLaunchKernelGGL((add_bias_kernel<B, O>), dim3(blocks), dim3(threads), 0, s, product, (const B*)bias, (O*)out, \
                       total, cols);                                                                             \
    return launch_status();                                                                                      \
  }
  TLIE_CASE(kF32, float, kF32, float)
  TLIE_CASE(kF32, float, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kF32, float)
  TLIE_CASE(kBF16, bf16, kBF16, bf16)
#undef TLIE_CASE
  return kBadArgument;
}

// values: [rows, cols] of act_dtype, changed in place; pre: a product [nsplit][rows][row_width] whose columns
// col .. col + cols - 1 are the gate's pre-activations.
extern "C" int tlie_sigmoid_gate(void* values, int act_dtype, const void* pre, int pre_dtype, int nsplit, long long split_stride,
                                 int col, int row_width, int rows, int cols, void* stream) {
  if (rows <= 0 || cols <= 0 || col < 0 || col + cols > row_width || nsplit < 1) return kBadArgument;
  const size_t total = static_cast<size_t>(rows) * cols;
  hipStream_t s = (hipStream_t)stream;
  if (nsplit == 1 && cols % 8 == 0 && col % 8 == 0 && row_width % 8 == 0 && pre_dtype == act_dtype &&
      ((reinterpret_cast<uintptr_t>(values) | reinterpret_cast<uintptr_t>(pre)) & 31) == 0) {
    const size_t groups = total / 8;
    const int wide_blocks = static_cast<int>((groups + 255) / 256 < 16384 ? (groups + 255) / 256 : 16384);
    if (act_dtype == kBF16)
      hipLaunchKernelGGL((sigmoid_gate_wide_kernel<bf16, bf16>), dim3(wide_blocks), dim3(256), 0, s, (bf16*)values, (const bf16*)pre, col,
                         row_width, groups, cols);
    else
      hipLaunchKernelGGL((sigmoid_gate_wide_kernel<float, float>), dim3(wide_blocks), dim3(256), 0, s, (float*)values, (const float*)pre,
                         col, row_width, groups, cols);
    return launch_status();
  }
  const int blocks = static_cast<int>((total + 255) / 256 < 16384 ? (total + 255) / 256 : 16384);
#define TLIE_CASE(DC, D, AC, A)                                                                                  \
  if (pre_dtype == DC && act_dtype == AC) {                                                                      \
    hipLaunchKernelGGL((sigmoid_gate_kernel<D, A>), dim3(blocks), dim3(256), 0, s, (A*)values, (const D*)pre, nsplit, \
                       (size_t)split_stride, col, row_width, total, cols);                                       \
    return launch_status();                                                                                      \
  }
  TLIE_CASE(kF32, float, kF32, float)
  TLIE_CASE(kF32, float, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kBF16, bf16)
#undef TLIE_CASE
  return kBadArgument;
}

extern "C" int tlie_softcap(float* x, long long total, float cap, void* stream) {
  if (total <= 0 || !(cap > 0.f)) return kBadArgument;
  const long long wanted = (total + 255) / 256;
  hipLaunchKernelGGL(softcap_kernel, dim3(static_cast<unsigned>(wanted < 16384 ? wanted : 16384)), dim3(256), 0, (hipStream_t)stream,
                     x, static_cast<size_t>(total), cap);
  return launch_status();
}
