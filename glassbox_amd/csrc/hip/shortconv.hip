// A short causal convolution over time on every channel of stacked projections, and what attention does to its
// heads right after it: rotation of a part of each query and key head in neighbouring pairs, an RMS norm of the
// query and key heads without a weight, and the cache write.
//
//   y[t, c] = sum_j w[c, j] u[t - taps + 1 + j, c]        u: the projections, zero before the request's first token
//
// The last taps - 1 projections of each request live in its state slot, [taps - 1, channels] float32 (index i is the
// position `first position of the step` - (taps - 1) + i), so that a step goes on where the one before ended whatever
// the cut.  A row of the projections holds nh query heads and nkv key heads of `dim` channels, then nkv value heads of
// `vdim`; a row of the result holds the same heads, each in `hd` >= max(dim, vdim) columns, the rest zeros (the cache
// and the attention kernels work on heads of one size; zeros change neither a score nor a sum).
//
//   pairs (2i, 2i + 1), i < rot / 2, of a query or key head:  (a, b) -> (a cos - b sin, b cos + a sin), angles from
//   the step's table [n, rot / 2]; then the head divided by sqrt(mean of its dim squares + eps).
//
// One wave a (token, head); a lane takes pairs of neighbouring channels.  Everything is computed in 32-bit and
// rounded once, when it is stored.
#include "common.h"

using namespace gb;

GB_DEFINE_LAST_ERROR

namespace {

constexpr int kMaxTaps = 8;
constexpr int kPairsLane = 2;   // heads of up to 256 channels

template <typename T>
__global__ __launch_bounds__(4 * kWave) void conv_heads_kernel(
    const T* __restrict__ proj, int stride, const float* __restrict__ wconv, int taps, float* __restrict__ state,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ q_start, const int32_t* __restrict__ pos0,
    const int32_t* __restrict__ state_slots, const float* __restrict__ cosv, const float* __restrict__ sinv, int rot,
    float eps, int norm, T* __restrict__ out, int out_stride, int hd, const int32_t* __restrict__ slots,
    T* __restrict__ k_pages, T* __restrict__ v_pages, int page_size, int nh, int nkv, int dim, int vdim, int channels,
    long long units, int update_state) {
  const long long unit = (long long)blockIdx.x * 4 + threadIdx.x / kWave;
  if (unit >= units) return;
  const int heads = nh + 2 * nkv;
  const int t = (int)(unit / heads), u = (int)(unit % heads), lane = threadIdx.x % kWave;
  const bool is_q = u < nh, is_k = !is_q && u < nh + nkv;
  const int D = (is_q || is_k) ? dim : vdim;
  const int ch0 = is_q ? u * dim : is_k ? nh * dim + (u - nh) * dim : (nh + nkv) * dim + (u - nh - nkv) * vdim;
  const int seq = tok_seq[t], start = q_start[seq], first_pos = pos0[seq];
  const int pos = first_pos + (t - start);
  const int K = taps - 1;
  float* st = (wconv && K > 0) ? state + (size_t)state_slots[seq] * K * channels : nullptr;

  float y[kPairsLane][2];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < kPairsLane; ++j) {
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int c = (lane + j * kWave) * 2 + e;
      float acc = 0.f;
      if (c < D) {
        const int ch = ch0 + c;
        if (!wconv) {
          acc = to_f(proj[(size_t)t * stride + ch]);
        } else {
          float old[kMaxTaps];   // the channel's slot, as far as this token needs it or has to move it
#pragma unroll
          for (int i = 0; i < kMaxTaps - 1; ++i) old[i] = 0.f;
          if (st) {
#pragma unroll
            for (int i = 0; i < kMaxTaps - 1; ++i)
              if (i < K && (update_state || i >= t - start)) old[i] = st[(size_t)i * channels + ch];
          }
#pragma unroll
          for (int jt = 0; jt < kMaxTaps; ++jt) {
            if (jt >= taps) break;
            const int back = K - jt;   // how many tokens before this one
            float v = 0.f;
            if (t - back >= start) v = to_f(proj[(size_t)(t - back) * stride + ch]);
            else if (pos - back >= 0) {
              const int idx = (t - start) + jt;   // = (pos - back) - first_pos + K
#pragma unroll
              for (int i = 0; i < kMaxTaps - 1; ++i)
                if (i == idx) v = old[i];
            }
            acc = fmaf(wconv[(size_t)ch * taps + jt], v, acc);
          }
          if (update_state && st) {   // a step of single tokens: the slot moves on by one
#pragma unroll
            for (int i = 0; i < kMaxTaps - 1; ++i)
              if (i < K) st[(size_t)i * channels + ch] = i + 1 < K ? old[i + 1] : to_f(proj[(size_t)t * stride + ch]);
          }
        }
      }
      y[j][e] = acc;
    }
    const int p = lane + j * kWave;
    if (!(!is_q && !is_k) && 2 * p + 1 < rot && 2 * p + 1 < D) {
      const float cs = cosv[(size_t)t * (rot / 2) + p], sn = sinv[(size_t)t * (rot / 2) + p];
      const float a = y[j][0], b = y[j][1];
      y[j][0] = a * cs - b * sn;
      y[j][1] = b * cs + a * sn;
    }
    ss = fmaf(y[j][0], y[j][0], ss);
    ss = fmaf(y[j][1], y[j][1], ss);
  }
  float s = 1.f;
  if (norm && (is_q || is_k)) {
    ss = wave_sum(ss);
    s = 1.0f / sqrtf(ss / (float)D + eps);
  }
  const int slot = (!is_q && slots) ? slots[t] : -1;
  const int piece = key_piece(hd);
  T* kb = nullptr;
  T* vb = nullptr;
  if (slot >= 0) {
    const int kvh = is_k ? u - nh : u - nh - nkv;
    const size_t block = ((size_t)(slot / page_size) * nkv + kvh) * (size_t)page_size * hd;
    kb = k_pages + block;
    vb = v_pages + block;
  }
  T* orow = out + (size_t)t * out_stride + (size_t)u * hd;
#pragma unroll
  for (int j = 0; j < kPairsLane; ++j) {
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int c = (lane + j * kWave) * 2 + e;
      if (c >= hd) continue;
      const float val = c < D ? y[j][e] * s : 0.f;
      const T r = from_f<T>(val);
      orow[c] = r;
      if (slot >= 0) {
        if (is_k) kb[key_offset(slot % page_size, c, page_size, piece)] = r;
        else vb[(size_t)c * page_size + slot % page_size] = r;
      }
    }
  }
}

// The state after a step with prompt portions: a thread a (request, channel) reads what it keeps of the old slot and
// of the step's rows, then writes.
template <typename T>
__global__ void conv_state_kernel(const T* __restrict__ proj, int stride, float* __restrict__ state,
                                  const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
                                  const int32_t* __restrict__ state_slots, int channels, int taps) {
  const int seq = blockIdx.y, ch = blockIdx.x * blockDim.x + threadIdx.x;
  if (ch >= channels) return;
  const int L = q_len[seq], start = q_start[seq], K = taps - 1;
  float* st = state + (size_t)state_slots[seq] * K * channels + ch;
  float nv[kMaxTaps - 1];
#pragma unroll
  for (int i = 0; i < kMaxTaps - 1; ++i) {
    nv[i] = 0.f;
    if (i < K) {
      const int r = L - K + i;   // the step's row that lands here, if there is one
      nv[i] = r >= 0 ? to_f(proj[(size_t)(start + r) * stride + ch]) : st[(size_t)(i + L) * channels];
    }
  }
#pragma unroll
  for (int i = 0; i < kMaxTaps - 1; ++i)
    if (i < K) st[(size_t)i * channels] = nv[i];
}

}  // namespace

// proj [n, stride] (query, key, value heads as projected), wconv [channels, taps] float32 or nullptr (no convolution),
// state [slots, taps - 1, channels] float32, cos/sin [n, rot / 2] float32 (rot 0: no rotation), out [n, out_stride]
// with (nh + 2 nkv) heads of hd columns; slots (or nullptr) the cache rows of the tokens in pages of heads of hd.
// update_state: every request of the step brings one token, and the kernel moves the slots on itself; otherwise
// gb_conv_state does, after it.
extern "C" int gb_conv_heads(const void* proj, int dtype, int stride, const float* wconv, int taps, float* state,
                             const int32_t* tok_seq, const int32_t* q_start, const int32_t* pos0, const int32_t* state_slots,
                             const float* cosv, const float* sinv, int rot, float eps, int norm, void* out, int out_stride,
                             int hd, const int32_t* slots, void* k_pages, void* v_pages, int page_size, int n, int nh, int nkv,
                             int dim, int vdim, int update_state, hipStream_t stream) {
  GB_REQUIRE(n >= 0 && nh > 0 && nkv >= 0 && dim > 0 && vdim > 0 && hd >= dim && hd >= vdim,
             "conv_heads: bad sizes n=%d heads=%d+%d dim=%d vdim=%d hd=%d", n, nh, nkv, dim, vdim, hd);
  GB_REQUIRE(hd <= 2 * kWave * kPairsLane, "conv_heads: heads of %d columns are above %d", hd, 2 * kWave * kPairsLane);
  const int channels = (nh + nkv) * dim + nkv * vdim;
  GB_REQUIRE(stride >= channels && out_stride >= (nh + 2 * nkv) * hd, "conv_heads: rows shorter than their heads");
  GB_REQUIRE(!wconv || (taps >= 1 && taps <= kMaxTaps && (taps == 1 || state)), "conv_heads: %d taps (at most %d), with the state", taps, kMaxTaps);
  GB_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= dim && (rot == 0 || (cosv && sinv)), "conv_heads: %d rotated channels of %d", rot, dim);
  GB_REQUIRE(!slots || (k_pages && v_pages && page_size > 0), "conv_heads: cache rows without pages");
  GB_REQUIRE(tok_seq && q_start && pos0 && state_slots, "conv_heads: the step's tables are needed");
  if (n == 0) return 0;
  const long long units = (long long)n * (nh + 2 * nkv);
  GB_REQUIRE((units + 3) / 4 < (1ll << 31), "conv_heads: too many heads for one launch");
  const dim3 grid((unsigned)((units + 3) / 4));
  if (dtype == kF32)
    hipLaunchKernelGGL(conv_heads_kernel<float>, grid, dim3(4 * kWave), 0, stream, (const float*)proj, stride, wconv, taps, state,
                       tok_seq, q_start, pos0, state_slots, cosv, sinv, rot, eps, norm, (float*)out, out_stride, hd, slots,
                       (float*)k_pages, (float*)v_pages, page_size, nh, nkv, dim, vdim, channels, units, update_state);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(conv_heads_kernel<bf16>, grid, dim3(4 * kWave), 0, stream, (const bf16*)proj, stride, wconv, taps, state,
                       tok_seq, q_start, pos0, state_slots, cosv, sinv, rot, eps, norm, (bf16*)out, out_stride, hd, slots,
                       (bf16*)k_pages, (bf16*)v_pages, page_size, nh, nkv, dim, vdim, channels, units, update_state);
  else
    return fail("conv_heads: unknown dtype %d", dtype);
  return launched("conv_heads");
}

extern "C" int gb_conv_state(const void* proj, int dtype, int stride, float* state, const int32_t* q_start,
                             const int32_t* q_len, const int32_t* state_slots, int n_seqs, int channels, int taps,
                             hipStream_t stream) {
  GB_REQUIRE(n_seqs >= 0 && channels > 0 && stride >= channels && taps >= 1 && taps <= kMaxTaps, "conv_state: bad sizes requests=%d channels=%d taps=%d",
             n_seqs, channels, taps);
  GB_REQUIRE(n_seqs <= 65535, "conv_state: too many requests for one launch");
  if (n_seqs == 0 || taps == 1) return 0;
  const dim3 grid((unsigned)((channels + 255) / 256), (unsigned)n_seqs);
  if (dtype == kF32)
    hipLaunchKernelGGL(conv_state_kernel<float>, grid, dim3(256), 0, stream, (const float*)proj, stride, state, q_start, q_len,
                       state_slots, channels, taps);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(conv_state_kernel<bf16>, grid, dim3(256), 0, stream, (const bf16*)proj, stride, state, q_start, q_len,
                       state_slots, channels, taps);
  else
    return fail("conv_state: unknown dtype %d", dtype);
  return launched("conv_state");
}

GB_TAPED(gb_conv_heads)
GB_TAPED(gb_conv_state)
