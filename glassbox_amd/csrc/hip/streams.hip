// A residual kept as several streams (hyper-connections).  Instead of one residual x there are S copies
// X[0..S-1], each [tokens, width] float32, stacked in one buffer.  A sublayer reads a weighted sum of them,
//   u = sum_s w_in[s] X[s] ,
// through its norm, and its output y [tokens, width] (float32) goes back into all of them at once:
//   X'[t] = sum_s mix[s, t] X[s] + w_out[t] y     (mix is indexed [from, to]) .
// At the end the model's norm reads sum_s X[s].  All sums are 32-bit, streams added in ascending s.
#include "common.h"

using namespace gb;

GB_DEFINE_LAST_ERROR

namespace {

constexpr int kMaxStreams = 8;

// out[r, :] = gamma * u / sqrt(mean(u^2) + eps) with u = sum_s w_in[s] X[s][row] (w_in == nullptr: every weight 1);
// `rows` (optional) picks the input row of each output row.  One block an output row; `sum` (optional) receives u.
template <typename G, typename O>
__global__ void streams_norm_kernel(const float* __restrict__ X, long long stream_stride, int S,
                                    const float* __restrict__ w_in, const G* __restrict__ gamma,
                                    const int32_t* __restrict__ rows, O* __restrict__ out, float* __restrict__ sum, int d,
                                    float eps) {
  __shared__ float scratch[17];
  extern __shared__ float u[];   // [d]
  const int r = blockIdx.x, tid = threadIdx.x, nt = blockDim.x;
  const float* x0 = X + (size_t)(rows ? rows[r] : r) * d;
  float w[kMaxStreams];
#pragma unroll
  for (int s = 0; s < kMaxStreams; ++s) w[s] = s < S ? (w_in ? w_in[s] : 1.f) : 0.f;
  float ss = 0.f;
  for (int c = tid; c < d; c += nt) {
    float v = 0.f;
#pragma unroll
    for (int s = 0; s < kMaxStreams; ++s)
      if (s < S) v = w_in ? fmaf(w[s], x0[(size_t)s * stream_stride + c], v) : v + x0[(size_t)s * stream_stride + c];
    u[c] = v;
    ss = fmaf(v, v, ss);
  }
  const float total = block_sum(ss, scratch);
  const float scale = 1.0f / sqrtf(total / (float)d + eps);
  for (int c = tid; c < d; c += nt) {
    out[(size_t)r * d + c] = from_f<O>(to_f(gamma[c]) * (u[c] * scale));
    if (sum) sum[(size_t)r * d + c] = u[c];
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

extern "C" int gb_streams_norm(const float* X, long long stream_stride, int S, const float* w_in, const void* gamma,
                               int gamma_dtype, const int32_t* rows, void* out, int out_dtype, float* sum, int m, int d,
                               float eps, hipStream_t stream) {
  GB_REQUIRE(m >= 0 && d > 0 && S >= 1 && S <= kMaxStreams, "streams_norm: bad sizes m=%d d=%d streams=%d (at most %d)", m, d, S,
             kMaxStreams);
  GB_REQUIRE(d <= 16384, "streams_norm: rows of %d columns do not fit a workgroup's memory", d);
  if (m == 0) return 0;
  const int threads = d >= 1024 ? 256 : d >= 256 ? 128 : 64;
  const size_t smem = sizeof(float) * d;
#define GB_SN(G, O)                                                                                                     \
  hipLaunchKernelGGL((streams_norm_kernel<G, O>), dim3(m), dim3(threads), smem, stream, X, stream_stride, S, w_in,      \
                     (const G*)gamma, rows, (O*)out, sum, d, eps)
  if (gamma_dtype == kF32 && out_dtype == kF32) GB_SN(float, float);
  else if (gamma_dtype == kF32 && out_dtype == kBF16) GB_SN(float, bf16);
  else if (gamma_dtype == kBF16 && out_dtype == kBF16) GB_SN(bf16, bf16);
  else if (gamma_dtype == kBF16 && out_dtype == kF32) GB_SN(bf16, float);
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
