// A residual of several streams (hyper-connections): instead of one row x per token there are S rows
// x_0 .. x_{S-1}, [S][tokens][hidden] floats.  A sublayer reads a weighted sum of them, and its result y
// joins them after they have been mixed among themselves:
//
//   u     = sum_s read[s] x_s                       what the sublayer's norm reads
//   x_t  <- sum_s mix[s][t] x_s + write[t] * y      all streams at once, from the old ones
//
// One kernel does what stands between two sublayers: it brings the streams up to date with the result y
// that still waits (mix, write: of the sublayer that made y), forms the next sublayer's u (read: of the next
// sublayer), and norms it: out = u * rsqrt(mean(u^2) + eps) * weight.  Each of the three steps is optional:
//   delta == null    nothing waits, the streams are read as they are
//   read == null     no sublayer follows: nothing is normed
//   total != null    the sum of the (updated) streams is written there, [tokens][hidden] floats: what the
//                    model's last norm reads
// A token is a workgroup's; a thread holds the S values of a column in registers, so the update in place
// reads every old value before it writes a new one.  Everything is float.  S <= kStreamsLimit.
#include "common.h"

namespace tlie {

constexpr int kStreamsLimit = 8;     // the kernel is built for up to 4 streams (up to 1024 threads a token) and for up to 8

template <typename D, typename W, typename O, int VEC, int kMaxStreams>
__global__ void __launch_bounds__(kMaxStreams <= 4 ? 1024 : 256)
stream_norm_kernel(float* __restrict__ streams, size_t stream_stride, int count, const D* __restrict__ delta, int nsplit,
                   size_t split_stride, const float* __restrict__ mix, const float* __restrict__ write,
                   const float* __restrict__ read, const W* __restrict__ weight, float eps, O* __restrict__ out,
                   float* __restrict__ total, int hidden) {
  extern __shared__ float row_cache[];           // hidden floats (only when something is normed), then 16
  float* scratch = row_cache + (read != nullptr ? hidden : 0);
  const int t = blockIdx.x;
  float m[kMaxStreams][kMaxStreams], wr[kMaxStreams], rd[kMaxStreams];
#pragma unroll
  for (int s = 0; s < kMaxStreams; ++s) {
    wr[s] = (delta != nullptr && s < count) ? write[s] : 0.f;
    rd[s] = (read != nullptr && s < count) ? read[s] : 0.f;
#pragma unroll
    for (int r = 0; r < kMaxStreams; ++r) m[s][r] = (delta != nullptr && s < count && r < count) ? mix[s * count + r] : 0.f;
  }
  float square = 0.f;
  for (int i = threadIdx.x * VEC; i < hidden; i += blockDim.x * VEC) {
    float x[kMaxStreams][VEC], y[VEC], u[VEC], all[VEC];
#pragma unroll
    for (int s = 0; s < kMaxStreams; ++s) {
      if (s < count) {
        const float* from = streams + s * stream_stride + static_cast<size_t>(t) * hidden + i;
        if constexpr (VEC == 4) {
          const float4 v = *reinterpret_cast<const float4*>(from);
          x[s][0] = v.x; x[s][1] = v.y; x[s][2] = v.z; x[s][3] = v.w;
        } else {
          x[s][0] = from[0];
        }
      }
    }
    if (delta != nullptr) {
      const D* part = delta + static_cast<size_t>(t) * hidden + i;
      if constexpr (VEC == 4 && sizeof(D) == 4) {
        // partial sums of a split product, four columns a load, added in the order of their index
        float4 sum = *reinterpret_cast<const float4*>(part);
        for (int split = 1; split < nsplit; ++split) {
          const float4 more = *reinterpret_cast<const float4*>(part + split * split_stride);
          sum.x += more.x; sum.y += more.y; sum.z += more.z; sum.w += more.w;
        }
        y[0] = sum.x; y[1] = sum.y; y[2] = sum.z; y[3] = sum.w;
      } else {
#pragma unroll
        for (int j = 0; j < VEC; ++j) y[j] = sum_splits(part + j, nsplit, split_stride);
      }
      float fresh[kMaxStreams][VEC];
#pragma unroll
      for (int r = 0; r < kMaxStreams; ++r) {
        if (r < count) {
#pragma unroll
          for (int j = 0; j < VEC; ++j) {
            float sum = 0.f;
#pragma unroll
            for (int s = 0; s < kMaxStreams; ++s)
              if (s < count) sum += m[s][r] * x[s][j];
            fresh[r][j] = sum + wr[r] * y[j];
          }
        }
      }
#pragma unroll
      for (int r = 0; r < kMaxStreams; ++r) {
        if (r < count) {
#pragma unroll
          for (int j = 0; j < VEC; ++j) x[r][j] = fresh[r][j];
          float* to = streams + r * stream_stride + static_cast<size_t>(t) * hidden + i;
          if constexpr (VEC == 4) *reinterpret_cast<float4*>(to) = make_float4(x[r][0], x[r][1], x[r][2], x[r][3]);
          else to[0] = x[r][0];
        }
      }
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j) {
      u[j] = 0.f;
      all[j] = 0.f;
#pragma unroll
      for (int s = 0; s < kMaxStreams; ++s) {
        if (s < count) {
          u[j] += rd[s] * x[s][j];
          all[j] += x[s][j];
        }
      }
      square += u[j] * u[j];
    }
    if (read != nullptr) {
      // (u times the norm's weight waits in LDS: the second pass then only applies the row's scale)
#pragma unroll
      for (int j = 0; j < VEC; ++j) row_cache[i + j] = u[j] * to_float(weight[i + j]);
    }
    if (total != nullptr) {
#pragma unroll
      for (int j = 0; j < VEC; ++j) total[static_cast<size_t>(t) * hidden + i + j] = all[j];
    }
  }
  if (read == nullptr) return;
  const float scale = rsqrtf(block_sum(square, scratch) / static_cast<float>(hidden) + eps);
  O* o = out + static_cast<size_t>(t) * hidden;
  for (int i = threadIdx.x * VEC; i < hidden; i += blockDim.x * VEC) {
#pragma unroll
    for (int j = 0; j < VEC; ++j) o[i + j] = from_float<O>(row_cache[i + j] * scale);   // (the thread's own entries)
  }
}

// streams[s][t][:] = first[t][:] for every s: the streams start as copies of the embedding's output.
__global__ void stream_spread_kernel(const float* __restrict__ first, float* __restrict__ streams, size_t elements, int count) {
  for (size_t index = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; index < elements;
       index += static_cast<size_t>(gridDim.x) * blockDim.x) {
    const float v = first[index];
    for (int s = 0; s < count; ++s) streams[s * elements + index] = v;
  }
}

}  // namespace tlie

using namespace tlie;

// streams: float [count][tokens][hidden], changed in place when delta is given; delta: a product [nsplit][tokens][hidden]
// or null; mix: float [count][count] ([from][to]), write: float [count] (both needed with delta); read: float [count] or
// null; weight [hidden] and out [tokens][hidden] (needed with read); total: float [tokens][hidden] or null.
extern "C" int tlie_stream_norm(float* streams, int count, const void* delta, int delta_dtype, int nsplit, long long split_stride,
                                const float* mix, const float* write, const float* read, const void* weight, int weight_dtype,
                                float eps, void* out, int out_dtype, float* total, int tokens, int hidden, void* stream) {
  if (tokens <= 0 || hidden <= 0 || count <= 0 || count > kStreamsLimit || nsplit < 1) return kBadArgument;
  if (delta != nullptr && (mix == nullptr || write == nullptr)) return kBadArgument;
  if (read != nullptr && (weight == nullptr || out == nullptr || !(eps > 0.f))) return kBadArgument;
  const size_t lds = (static_cast<size_t>(read != nullptr ? hidden : 0) + 16) * sizeof(float);
  if (lds > 64 * 1024) return kBadArgument;
  const size_t stride = static_cast<size_t>(tokens) * hidden;
  const bool wide = (hidden & 3) == 0 && (split_stride & 3) == 0 &&
                    ((reinterpret_cast<uintptr_t>(streams) | reinterpret_cast<uintptr_t>(total) | reinterpret_cast<uintptr_t>(delta)) & 15) == 0;
  const int per_thread = wide ? 4 : 1;
  const int wanted = (hidden / per_thread + 63) / 64 * 64;
  // a step of few tokens has few workgroups: each then takes as many threads as its row has pieces, so that every load
  // of the row is asked for at once (up to 4 streams; beyond, the registers of 256 threads)
  const int most = count <= 4 && tokens <= 64 ? 1024 : 256;
  const int threads = wanted > most ? most : wanted;
  hipStream_t s = (hipStream_t)stream;
  if (delta == nullptr) delta_dtype = kF32;
  if (read == nullptr) weight_dtype = kF32, out_dtype = kF32;
#define TLIE_CASE(DC, D, WC, W, OC, O)                                                                                  \
  if (delta_dtype == DC && weight_dtype == WC && out_dtype == OC) {                                                     \
    if (wide && count <= 4)                                                                                             \
      hipLaunchKernelGGL((stream_norm_kernel<D, W, O, 4, 4>), dim3(tokens), dim3(threads), lds, s, streams, stride, count, \
                         (const D*)delta, nsplit, (size_t)split_stride, mix, write, read, (const W*)weight, eps, (O*)out, \
                         total, hidden);                                                                                \
    else if (wide)                                                                                                      \
      hipLaunchKernelGGL((stream_norm_kernel<D, W, O, 4, 8>), dim3(tokens), dim3(threads), lds, s, streams, stride, count, \
                         (const D*)delta, nsplit, (size_t)split_stride, mix, write, read, (const W*)weight, eps, (O*)out, \
                         total, hidden);                                                                                \
    else if (count <= 4)                                                                                                \
      hipLaunchKernelGGL((stream_norm_kernel<D, W, O, 1, 4>), dim3(tokens), dim3(threads), lds, s, streams, stride, count, \
                         (const D*)delta, nsplit, (size_t)split_stride, mix, write, read, (const W*)weight, eps, (O*)out, \
                         total, hidden);                                                                                \
    else                                                                                                                \
      hipLaunchKernelGGL((stream_norm_kernel<D, W, O, 1, 8>), dim3(tokens), dim3(threads), lds, s, streams, stride, count, \
                         (const D*)delta, nsplit, (size_t)split_stride, mix, write, read, (const W*)weight, eps, (O*)out, \
                         total, hidden);                                                                                \
    return launch_status();                                                                                             \
  }
  TLIE_CASE(kF32, float, kF32, float, kF32, float)
  TLIE_CASE(kF32, float, kF32, float, kBF16, bf16)
  TLIE_CASE(kF32, float, kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kBF16, bf16, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kF32, float, kBF16, bf16)
  TLIE_CASE(kBF16, bf16, kF32, float, kF32, float)
#undef TLIE_CASE
  return kBadArgument;
}

extern "C" int tlie_stream_spread(const float* first, float* streams, int count, long long elements, void* stream) {
  if (count <= 0 || elements <= 0) return kBadArgument;
  long long blocks = (elements + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(stream_spread_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, (hipStream_t)stream, first, streams,
                     static_cast<size_t>(elements), count);
  return launch_status();
}
