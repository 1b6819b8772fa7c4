// Routing of tokens to experts, and the experts' gated units.
//
//   s = sigmoid(z)                          z [n, E] the router's logits, 32-bit
//   chosen: the `top` experts with the largest s + correction (of equal ones the lower index)
//   weight of a chosen expert: s / (sum of the chosen s + 1e-20) * scale
//
// `route` leaves the result in two forms: the chosen experts and their weights a token ([n, top]), and a row of E
// weights a token with zeros for the experts not chosen (with `shared`, one more column: sigmoid of z's column E, the
// gate of an expert that every token uses).  `gated_units` turns the stacked gate and up projections of all experts
// into act = silu(gate) * up * weight, so that one product with the experts' down matrices side by side gives the
// weighted sum of the chosen experts' outputs (an expert not chosen contributes exact zeros).
#include "common.h"

using namespace gb;

GB_DEFINE_LAST_ERROR

namespace {

constexpr int kPerLane = 8;   // experts a lane: up to 512 experts
constexpr int kMaxTop = 16;

__global__ __launch_bounds__(4 * kWave) void route_kernel(const float* __restrict__ z, int ldz, int E,
                                                        const float* __restrict__ correction, int top, float scale,
                                                        int shared, float* __restrict__ combine, int32_t* __restrict__ ids,
                                                        float* __restrict__ wts, int n) {
  const int t = blockIdx.x * 4 + threadIdx.x / kWave, lane = threadIdx.x % kWave;
  if (t >= n) return;
  const float* row = z + (size_t)t * ldz;
  float s[kPerLane], c[kPerLane];
#pragma unroll
  for (int j = 0; j < kPerLane; ++j) {
    const int e = lane + j * kWave;
    s[j] = 0.f;
    c[j] = -INFINITY;
    if (e < E) {
      s[j] = 1.0f / (1.0f + expf(-row[e]));
      c[j] = s[j] + (correction ? correction[e] : 0.f);
    }
  }
  int chosen[kMaxTop];
  float cs[kMaxTop];
  float sum = 0.f;
#pragma unroll
  for (int k = 0; k < kMaxTop; ++k) {
    chosen[k] = -1;
    cs[k] = 0.f;
    if (k >= top) continue;
    float best = -INFINITY;
    int be = 0x7fffffff;
    float bs = 0.f;
#pragma unroll
    for (int j = 0; j < kPerLane; ++j) {
      const int e = lane + j * kWave;
      if (e < E && (c[j] > best || (c[j] == best && e < be))) {
        best = c[j];
        be = e;
        bs = s[j];
      }
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
      const float ob = __shfl_xor(best, off, kWave), os = __shfl_xor(bs, off, kWave);
      const int oe = __shfl_xor(be, off, kWave);
      if (ob > best || (ob == best && oe < be)) {
        best = ob;
        be = oe;
        bs = os;
      }
    }
    chosen[k] = be;
    cs[k] = bs;
    sum += bs;
#pragma unroll
    for (int j = 0; j < kPerLane; ++j)
      if (lane + j * kWave == be) c[j] = -INFINITY;   // taken
  }
  const float inv = scale / (sum + 1e-20f);
  const int cols = E + (shared ? 1 : 0);
#pragma unroll
  for (int j = 0; j < kPerLane; ++j) {
    const int e = lane + j * kWave;
    if (e >= E) continue;
    float w = 0.f;
#pragma unroll
    for (int k = 0; k < kMaxTop; ++k)
      if (k < top && chosen[k] == e) w = cs[k] * inv;
    combine[(size_t)t * cols + e] = w;
  }
  if (shared && lane == 0) combine[(size_t)t * cols + E] = 1.0f / (1.0f + expf(-row[E]));
#pragma unroll
  for (int k = 0; k < kMaxTop; ++k)
    if (k < top && lane == k % kWave) {
      ids[(size_t)t * top + k] = chosen[k];
      wts[(size_t)t * top + k] = cs[k] * inv;
    }
}

// act[t, j] = silu(g) * u * combine[t, expert of column j]: columns e * ff .. (e + 1) * ff - 1 are expert e's, the
// columns from E * ff on the shared expert's (weight in column E of combine).  Rows of `gu`: all gate columns, then all
// up columns.
template <typename I, typename O>
__global__ void gated_units_kernel(const I* __restrict__ gu, int ld, const float* __restrict__ combine, int cols, O* __restrict__ act,
                                   long long count, int inter, int E, int ff) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= count) return;
  const long long t = idx / inter;
  const int j = (int)(idx % inter);
  const int e = j < E * ff ? j / ff : E;
  const float w = combine[(size_t)t * cols + e];
  float y = 0.f;
  if (w != 0.f) {
    const I* row = gu + (size_t)t * ld;
    const float g = to_f(row[j]), u = to_f(row[inter + j]);
    y = g / (1.0f + expf(-g)) * u * w;
  }
  act[idx] = from_f<O>(y);
}

}  // namespace

extern "C" int gb_moe_route(const float* z, int ldz, int n, int E, const float* correction, int top, float scale, int shared,
                            float* combine, int32_t* ids, float* wts, hipStream_t stream) {
  GB_REQUIRE(n >= 0 && E > 0 && E <= kPerLane * kWave, "moe_route: %d experts (at most %d)", E, kPerLane * kWave);
  GB_REQUIRE(top > 0 && top <= kMaxTop && top <= E, "moe_route: %d chosen experts of %d (at most %d)", top, E, kMaxTop);
  GB_REQUIRE(ldz >= E + (shared ? 1 : 0), "moe_route: rows of %d logits for %d experts", ldz, E);
  if (n == 0) return 0;
  hipLaunchKernelGGL(route_kernel, dim3((unsigned)((n + 3) / 4)), dim3(4 * kWave), 0, stream, z, ldz, E, correction, top, scale,
                     shared, combine, ids, wts, n);
  return launched("moe_route");
}

extern "C" int gb_moe_gated_units(const void* gu, int in_dtype, int ld, const float* combine, int cols, void* act, int out_dtype,
                                  int n, int inter, int E, int ff, hipStream_t stream) {
  GB_REQUIRE(n >= 0 && inter > 0 && ld >= 2 * inter && E >= 0 && ff > 0 && E * ff <= inter && cols >= E + (E * ff < inter ? 1 : 0),
             "moe_gated_units: bad sizes n=%d inter=%d experts=%d of %d cols=%d", n, inter, E, ff, cols);
  if (n == 0) return 0;
  const long long count = (long long)n * inter;
  GB_REQUIRE((count + 255) / 256 < (1ll << 31), "moe_gated_units: too many elements");
  const dim3 grid((unsigned)((count + 255) / 256));
  if (in_dtype == kF32 && out_dtype == kF32)
    hipLaunchKernelGGL((gated_units_kernel<float, float>), grid, dim3(256), 0, stream, (const float*)gu, ld, combine, cols, (float*)act, count, inter, E, ff);
  else if (in_dtype == kF32 && out_dtype == kBF16)
    hipLaunchKernelGGL((gated_units_kernel<float, bf16>), grid, dim3(256), 0, stream, (const float*)gu, ld, combine, cols, (bf16*)act, count, inter, E, ff);
  else if (in_dtype == kBF16 && out_dtype == kBF16)
    hipLaunchKernelGGL((gated_units_kernel<bf16, bf16>), grid, dim3(256), 0, stream, (const bf16*)gu, ld, combine, cols, (bf16*)act, count, inter, E, ff);
  else
    return fail("moe_gated_units: no kernel for operand type %d and result type %d", in_dtype, out_dtype);
  return launched("moe_gated_units");
}

GB_TAPED(gb_moe_route)
GB_TAPED(gb_moe_gated_units)
