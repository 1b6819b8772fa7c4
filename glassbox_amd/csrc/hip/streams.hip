// A residual kept as several streams (hyper-connections).  Instead of one residual x there are S copies
// X[0..S-1], each [tokens, width] float32, stacked in one buffer.  A sublayer reads a weighted sum of them,
//   u = sum_s w_in[s] X[s] ,
// through its norm, and its output y [tokens, width] (float32) goes back into all of them at once:
//   X'[t] = sum_s mix[s, t] X[s] + w_out[t] y     (mix is indexed [from, to]) .
// At the end the model's norm reads sum_s X[s].  All sums are 32-bit, streams added in ascending s.
#include <algorithm>

#include "common.h"

using namespace gb;

GB_DEFINE_LAST_ERROR

namespace {

constexpr int kMaxStreams = 8;

// V neighbouring floats as one word where V is 4 (the caller has checked that such words are whole)
template <int V> __device__ __forceinline__ void load_v(const float* p, float (&v)[V]) {
  if constexpr (V == 4) {
    const f32x4 t = *reinterpret_cast<const f32x4*>(p);
    v[0] = t[0]; v[1] = t[1]; v[2] = t[2]; v[3] = t[3];
  } else {
#pragma unroll
    for (int e = 0; e < V; ++e) v[e] = p[e];
  }
}
template <int V> __device__ __forceinline__ void store_v(float* p, const float (&v)[V]) {
  if constexpr (V == 4) {
    *reinterpret_cast<f32x4*>(p) = f32x4{v[0], v[1], v[2], v[3]};
  } else {
#pragma unroll
    for (int e = 0; e < V; ++e) p[e] = v[e];
  }
}

// out[r, :] = gamma * u / sqrt(mean(u^2) + eps) with u = sum_s w_in[s] X[s][row] (w_in == nullptr: every weight 1);
// `rows` (optional) picks the input row of each output row.  One block an output row, V columns a thread at a time
// (V = 4: rows of whole 16-byte words); `sum` (optional) receives u.  With `mix` the streams are first updated by the
// sublayer before, X'[t] = sum_s mix[s, t] X[s] + w_out[t] y, written back, and u is taken from the new ones: one pass
// over the streams where the update and the next norm would make two.
template <typename G, typename O, int V>
__global__ void streams_norm_kernel(float* __restrict__ X, long long stream_stride, int S, const float* __restrict__ w_in,
                                    const G* __restrict__ gamma, const int32_t* __restrict__ rows, O* __restrict__ out,
                                    float* __restrict__ sum, int d, float eps, const float* __restrict__ mix,
                                    const float* __restrict__ w_out, const float* __restrict__ y) {
  __shared__ float scratch[17];
  extern __shared__ float u[];   // [d]
  const int r = blockIdx.x, tid = threadIdx.x, nt = blockDim.x;
  const size_t row = (size_t)(rows ? rows[r] : r) * d;
  float w[kMaxStreams];
#pragma unroll
  for (int s = 0; s < kMaxStreams; ++s) w[s] = s < S ? (w_in ? w_in[s] : 1.f) : 0.f;
  float ss = 0.f;
  for (int c = tid * V; c < d; c += nt * V) {
    float x[kMaxStreams][V], acc[V];
#pragma unroll
    for (int s = 0; s < kMaxStreams; ++s)
      if (s < S) load_v<V>(X + (size_t)s * stream_stride + row + c, x[s]);
    if (mix) {
      float yv[V], xn[kMaxStreams][V];
      load_v<V>(y + row + c, yv);
#pragma unroll
      for (int t = 0; t < kMaxStreams; ++t)
        if (t < S) {
#pragma unroll
          for (int e = 0; e < V; ++e) {
            float v = 0.f;
#pragma unroll
            for (int s = 0; s < kMaxStreams; ++s)
              if (s < S) v = fmaf(mix[s * S + t], x[s][e], v);
            xn[t][e] = fmaf(w_out[t], yv[e], v);
          }
          store_v<V>(X + (size_t)t * stream_stride + row + c, xn[t]);
        }
#pragma unroll
      for (int s = 0; s < kMaxStreams; ++s)
        if (s < S) {
#pragma unroll
          for (int e = 0; e < V; ++e) x[s][e] = xn[s][e];
        }
    }
#pragma unroll
    for (int e = 0; e < V; ++e) {
      acc[e] = 0.f;
#pragma unroll
      for (int s = 0; s < kMaxStreams; ++s)
        if (s < S) acc[e] = w_in ? fmaf(w[s], x[s][e], acc[e]) : acc[e] + x[s][e];
      u[c + e] = acc[e];
      ss = fmaf(acc[e], acc[e], ss);
    }
  }
  const float total = block_sum(ss, scratch);
  const float scale = 1.0f / sqrtf(total / (float)d + eps);
  for (int c = tid * V; c < d; c += nt * V) {
#pragma unroll
    for (int e = 0; e < V; ++e) {
      out[(size_t)r * d + c + e] = from_f<O>(to_f(gamma[c + e]) * (u[c + e] * scale));
      if (sum) sum[(size_t)r * d + c + e] = u[c + e];
    }
  }
}

// X'[t] = sum_s mix[s, t] X[s] + w_out[t] y, in place: an element of all streams is read before any is written.
__global__ void streams_mix_kernel(float* __restrict__ X, long long stream_stride, int S, const float* __restrict__ mix,
                                   const float* __restrict__ w_out, const float* __restrict__ y, long long count) {
  __shared__ float m[kMaxStreams * kMaxStreams + kMaxStreams];
  if (threadIdx.x < S * S) m[threadIdx.x] = mix[threadIdx.x];
  if (threadIdx.x < S) m[kMaxStreams * kMaxStreams + threadIdx.x] = w_out[threadIdx.x];
  __syncthreads();
  const long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count) return;
  float x[kMaxStreams];
#pragma unroll
  for (int s = 0; s < kMaxStreams; ++s) x[s] = s < S ? X[(size_t)s * stream_stride + i] : 0.f;
  const float yv = y[i];
#pragma unroll
  for (int t = 0; t < kMaxStreams; ++t) {
    if (t >= S) break;
    float v = 0.f;
#pragma unroll
    for (int s = 0; s < kMaxStreams; ++s)
      if (s < S) v = fmaf(m[s * S + t], x[s], v);
    X[(size_t)t * stream_stride + i] = fmaf(m[kMaxStreams * kMaxStreams + t], yv, v);
  }
}

}  // namespace

extern "C" int gb_streams_max() { return kMaxStreams; }

// mix, w_out, y (all or none; not with `rows`): the update of the streams by the sublayer before, done on the way.
extern "C" int gb_streams_norm(float* X, long long stream_stride, int S, const float* w_in, const void* gamma,
                               int gamma_dtype, const int32_t* rows, void* out, int out_dtype, float* sum, int m, int d,
                               float eps, const float* mix, const float* w_out, const float* y, hipStream_t stream) {
  GB_REQUIRE(m >= 0 && d > 0 && S >= 1 && S <= kMaxStreams, "streams_norm: bad sizes m=%d d=%d streams=%d (at most %d)", m, d, S,
             kMaxStreams);
  GB_REQUIRE(d <= 16384, "streams_norm: rows of %d columns do not fit a workgroup's memory", d);
  GB_REQUIRE((mix == nullptr) == (w_out == nullptr) && (mix == nullptr) == (y == nullptr) && (mix == nullptr || rows == nullptr),
             "streams_norm: the update of the streams takes mix, w_out and y together, and every row in its place");
  if (m == 0) return 0;
  const size_t smem = sizeof(float) * d;
  const bool words = d % 4 == 0 && stream_stride % 4 == 0 && (uintptr_t)X % 16 == 0 && (y == nullptr || (uintptr_t)y % 16 == 0);
  // a thread for every word of the row, up to 1,024: all of a row's loads are asked for at once
  const int per = words ? 4 : 1;
  const int threads = std::min(1024, std::max(64, ((d + per - 1) / per + 63) / 64 * 64));
#define GB_SN(G, O)                                                                                                     \
  if (words)                                                                                                            \
    hipLaunchKernelGGL((streams_norm_kernel<G, O, 4>), dim3(m), dim3(threads), smem, stream, X, stream_stride, S, w_in, \
                       (const G*)gamma, rows, (O*)out, sum, d, eps, mix, w_out, y);                                     \
  else                                                                                                                  \
    hipLaunchKernelGGL((streams_norm_kernel<G, O, 1>), dim3(m), dim3(threads), smem, stream, X, stream_stride, S, w_in, \
                       (const G*)gamma, rows, (O*)out, sum, d, eps, mix, w_out, y)
  if (gamma_dtype == kF32 && out_dtype == kF32) { GB_SN(float, float); }
  else if (gamma_dtype == kF32 && out_dtype == kBF16) { GB_SN(float, bf16); }
  else if (gamma_dtype == kBF16 && out_dtype == kBF16) { GB_SN(bf16, bf16); }
  else if (gamma_dtype == kBF16 && out_dtype == kF32) { GB_SN(bf16, float); }
  else return fail("streams_norm: unknown dtypes %d, %d", gamma_dtype, out_dtype);
#undef GB_SN
  return launched("streams_norm");
}

extern "C" int gb_streams_mix(float* X, long long stream_stride, int S, const float* mix, const float* w_out, const float* y,
                              long long count, hipStream_t stream) {
  GB_REQUIRE(count >= 0 && S >= 1 && S <= kMaxStreams, "streams_mix: bad sizes count=%lld streams=%d (at most %d)", count, S,
             kMaxStreams);
  GB_REQUIRE(stream_stride >= count, "streams_mix: streams overlap");
  if (count == 0) return 0;
  const long long blocks = (count + 255) / 256;
  GB_REQUIRE(blocks < (1ll << 31), "streams_mix: too many elements");
  hipLaunchKernelGGL(streams_mix_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, X, stream_stride, S, mix, w_out, y, count);
  return launched("streams_mix");
}

GB_TAPED(gb_streams_norm)
GB_TAPED(gb_streams_mix)
