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
// A few lanes a (token, head), as many as the head has pairs of neighbouring channels, so that a wave takes several
// short heads; a lane takes a pair.  A token whose taps all lie among the step's rows reads no state.  Everything is
// computed in 32-bit and rounded once, when it is stored.
#include "common.h"

using namespace gb;

GB_DEFINE_LAST_ERROR

namespace {

constexpr int kMaxTaps = 8;

// TAPS: the convolution's length (0: none).  LPU lanes a (token, head), a lane PPL pairs of neighbouring channels: heads
// of up to 2 * LPU * PPL columns; a wave takes 64 / LPU heads.
template <typename T, int TAPS, int LPU, int PPL>
__global__ __launch_bounds__(4 * kWave) void conv_heads_kernel(
    const T* __restrict__ proj, int stride, const float* __restrict__ wconv, float* __restrict__ state,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ q_start, const int32_t* __restrict__ pos0,
    const int32_t* __restrict__ state_slots, const float* __restrict__ cosv, const float* __restrict__ sinv, int rot,
    float eps, int norm, T* __restrict__ out, int out_stride, int hd, const int32_t* __restrict__ slots,
    T* __restrict__ k_pages, T* __restrict__ v_pages, int page_size, int nh, int nkv, int dim, int vdim, int channels,
    long long units, int update_state) {
  constexpr int K = TAPS > 0 ? TAPS - 1 : 0;
  constexpr int UPW = kWave / LPU;   // heads a wave
  const int lane = threadIdx.x % kWave, li = lane % LPU;
  const long long unit = ((long long)blockIdx.x * 4 + threadIdx.x / kWave) * UPW + lane / LPU;
  const bool live = unit < units;
  const int heads = nh + 2 * nkv;
  const int t = live ? (int)(unit / heads) : 0, u = live ? (int)(unit % heads) : 0;
  const bool is_q = u < nh, is_k = !is_q && u < nh + nkv;
  const int D = (is_q || is_k) ? dim : vdim;
  const int ch0 = is_q ? u * dim : is_k ? nh * dim + (u - nh) * dim : (nh + nkv) * dim + (u - nh - nkv) * vdim;
  const int seq = tok_seq[t], start = q_start[seq], first_pos = pos0[seq];
  const int off = t - start;           // the token's place in its request's rows of this step
  float* st = K > 0 ? state + (size_t)state_slots[seq] * K * channels : nullptr;
  const T* row = proj + (size_t)t * stride;

  float y[PPL][2];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < PPL; ++j) {
    const int p = li + j * LPU;
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int c = 2 * p + e;
      float acc = 0.f;
      if (live && c < D) {
        const int ch = ch0 + c;
        if (TAPS == 0) {
          acc = to_f(row[ch]);
        } else if (off >= K && !update_state) {   // every tap lies among the step's rows
#pragma unroll
          for (int jt = 0; jt < TAPS; ++jt)
            acc = fmaf(wconv[(size_t)ch * TAPS + jt], to_f(proj[(size_t)(t - (K - jt)) * stride + ch]), acc);
        } else {
          float old[K > 0 ? K : 1];   // the channel's slot: index i is the position `first_pos` - K + i
#pragma unroll
          for (int i = 0; i < K; ++i) old[i] = (update_state || i >= off) ? st[(size_t)i * channels + ch] : 0.f;
#pragma unroll
          for (int jt = 0; jt < TAPS; ++jt) {
            const int back = K - jt;   // how many tokens before this one
            float v = 0.f;
            if (off >= back) {
              v = to_f(proj[(size_t)(t - back) * stride + ch]);
            } else if (first_pos + off - back >= 0) {
#pragma unroll
              for (int i = 0; i < K; ++i)
                if (i == off + jt) v = old[i];   // = (position - back) - first_pos + K
            }
            acc = fmaf(wconv[(size_t)ch * TAPS + jt], v, acc);
          }
          if (update_state) {   // a step of single tokens: the slot moves on by one
#pragma unroll
            for (int i = 0; i < K; ++i) st[(size_t)i * channels + ch] = i + 1 < K ? old[i + 1 < K ? i + 1 : 0] : to_f(row[ch]);
          }
        }
      }
      y[j][e] = acc;
    }
    if (live && (is_q || is_k) && 2 * p + 1 < rot && 2 * p + 1 < D) {
      const float cs = cosv[(size_t)t * (rot / 2) + p], sn = sinv[(size_t)t * (rot / 2) + p];
      const float a = y[j][0], b = y[j][1];
      y[j][0] = a * cs - b * sn;
      y[j][1] = b * cs + a * sn;
    }
    ss = fmaf(y[j][0], y[j][0], ss);
    ss = fmaf(y[j][1], y[j][1], ss);
  }
  float s = 1.f;
  if (norm) {   // (value heads take part in the moves and keep s = 1)
#pragma unroll
    for (int o = LPU / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, kWave);
    if (is_q || is_k) s = 1.0f / sqrtf(ss / (float)D + eps);
  }
  if (!live) return;
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
  for (int j = 0; j < PPL; ++j) {
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int c = (li + j * LPU) * 2 + e;
      if (c >= hd) continue;
      const T r = from_f<T>(c < D ? y[j][e] * s : 0.f);
      orow[c] = r;
      if (slot >= 0) {
        if (is_k) kb[key_offset(slot % page_size, c, page_size, piece)] = r;
        else vb[(size_t)c * page_size + slot % page_size] = r;
      }
    }
  }
}

// The same for steps of many rows in bfloat16 whose heads are made of whole groups of eight channels (and that leave the
// cache write to the page-store kernel): a lane takes eight neighbouring channels of a head, so that every access to the
// rows is a 16-byte word, and `lpu` lanes (a power of two, at least hd / 8) a head; and it takes them for TT rows one
// after the other, so that it reads its channels' taps once and each row of the projections once: the last taps - 1
// rows wait in registers, whichever request they belong to, and a row whose request began fewer rows ago takes those
// taps from the request's slot or as zeros instead.  The taps are added up in the order of the kernel above: the
// convolution's sums are the same to the bit.
template <int TAPS, int TT>
__global__ __launch_bounds__(4 * kWave) void conv_heads_wide_kernel(
    const bf16* __restrict__ proj, int stride, const float* __restrict__ wconv, const float* __restrict__ state,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ q_start, const int32_t* __restrict__ pos0,
    const int32_t* __restrict__ state_slots, const float* __restrict__ cosv, const float* __restrict__ sinv, int rot,
    float eps, int norm, bf16* __restrict__ out, int out_stride, int hd, int nh, int nkv, int dim, int vdim, int channels,
    long long units, int lpu, int n) {
  constexpr int K = TAPS > 0 ? TAPS - 1 : 0;
  constexpr int NW = TAPS > 0 ? TAPS : 1;
  const int lane = threadIdx.x % kWave, li = lane % lpu;
  const long long unit = ((long long)blockIdx.x * 4 + threadIdx.x / kWave) * (kWave / lpu) + lane / lpu;
  const int c0 = li * 8;   // the first of the lane's eight columns of its head
  const bool live = unit < units && c0 < hd;
  const int heads = nh + 2 * nkv;
  const int t0 = live ? (int)(unit / heads) * TT : 0, u = live ? (int)(unit % heads) : 0;
  const bool is_q = u < nh, is_k = !is_q && u < nh + nkv;
  const int D = (is_q || is_k) ? dim : vdim;
  const int ch = (is_q ? u * dim : is_k ? nh * dim + (u - nh) * dim : (nh + nkv) * dim + (u - nh - nkv) * vdim) + c0;
  const bool has = live && c0 < D;

  float w[8 * NW];      // [channel][tap], as they lie in memory
  float win[NW][8];     // win[j]: the projections of row t - K + j
#pragma unroll
  for (int i = 0; i < 8 * NW; ++i) w[i] = 0.f;
#pragma unroll
  for (int j = 0; j < NW; ++j)
#pragma unroll
    for (int c = 0; c < 8; ++c) win[j][c] = 0.f;
  if (has) {
    if (TAPS > 0) {
#pragma unroll
      for (int i = 0; i < 2 * TAPS; ++i) {
        const float4 q = *reinterpret_cast<const float4*>(wconv + (size_t)ch * TAPS + 4 * i);
        w[4 * i] = q.x, w[4 * i + 1] = q.y, w[4 * i + 2] = q.z, w[4 * i + 3] = q.w;
      }
    }
#pragma unroll
    for (int j = 0; j < K; ++j) {   // rows t0 - K .. t0 - 1 of the step, as far as it has them
      const int r = t0 - K + j;
      if (r >= 0) {
        const bf16x8 x = *reinterpret_cast<const bf16x8*>(proj + (size_t)r * stride + ch);
#pragma unroll
        for (int c = 0; c < 8; ++c) win[j + 1][c] = (float)x[c];
      }
    }
  }
#pragma unroll 1
  for (int it = 0; it < TT; ++it) {
    const int t = t0 + it;
    const bool row = live && t < n;
    float y[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) y[c] = 0.f;
    if (row && has) {
#pragma unroll
      for (int j = 0; j < K; ++j)
#pragma unroll
        for (int c = 0; c < 8; ++c) win[j][c] = win[j + 1][c];
      const bf16x8 x = *reinterpret_cast<const bf16x8*>(proj + (size_t)t * stride + ch);
#pragma unroll
      for (int c = 0; c < 8; ++c) win[K][c] = (float)x[c];
      if (TAPS == 0) {
#pragma unroll
        for (int c = 0; c < 8; ++c) y[c] = win[0][c];
      } else {
        const int seq = tok_seq[t], off = t - q_start[seq], first_pos = pos0[seq];
#pragma unroll
        for (int jt = 0; jt < TAPS; ++jt) {
          const int back = K - jt;   // how many tokens before this one
          float v[8];
#pragma unroll
          for (int c = 0; c < 8; ++c) v[c] = win[jt][c];
          if (off < back) {
#pragma unroll
            for (int c = 0; c < 8; ++c) v[c] = 0.f;
            if (first_pos + off - back >= 0) {   // in the request's slot, at index off + jt
              const float* st = state + ((size_t)state_slots[seq] * K + (off + jt)) * channels + ch;
              const float4 lo = *reinterpret_cast<const float4*>(st), hi = *reinterpret_cast<const float4*>(st + 4);
              v[0] = lo.x, v[1] = lo.y, v[2] = lo.z, v[3] = lo.w, v[4] = hi.x, v[5] = hi.y, v[6] = hi.z, v[7] = hi.w;
            }
          }
#pragma unroll
          for (int c = 0; c < 8; ++c) y[c] = fmaf(w[c * NW + jt], v[c], y[c]);
        }
      }
      if (is_q || is_k) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int p = c0 / 2 + i;
          if (2 * p + 1 < rot) {
            const float cs = cosv[(size_t)t * (rot / 2) + p], sn = sinv[(size_t)t * (rot / 2) + p];
            const float a = y[2 * i], b = y[2 * i + 1];
            y[2 * i] = a * cs - b * sn;
            y[2 * i + 1] = b * cs + a * sn;
          }
        }
      }
    }
    float s = 1.f;
    if (norm) {   // (value heads take part in the moves and keep s = 1)
      float ss = 0.f;
#pragma unroll
      for (int c = 0; c < 8; ++c) ss = fmaf(y[c], y[c], ss);
      for (int o = lpu / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, kWave);
      if (is_q || is_k) s = 1.0f / sqrtf(ss / (float)D + eps);
    }
    if (row) {
      bf16x8 r;
#pragma unroll
      for (int c = 0; c < 8; ++c) r[c] = (bf16)(y[c] * s);   // (columns from D on are zero already)
      *reinterpret_cast<bf16x8*>(out + (size_t)t * out_stride + (size_t)u * hd + c0) = r;
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
  GB_REQUIRE(hd <= 4 * kWave, "conv_heads: heads of %d columns are above %d", hd, 4 * kWave);
  const int channels = (nh + nkv) * dim + nkv * vdim;
  GB_REQUIRE(stride >= channels && out_stride >= (nh + 2 * nkv) * hd, "conv_heads: rows shorter than their heads");
  GB_REQUIRE(!wconv || (taps >= 1 && taps <= kMaxTaps && (taps == 1 || state)), "conv_heads: %d taps (at most %d), with the state", taps, kMaxTaps);
  GB_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= dim && (rot == 0 || (cosv && sinv)), "conv_heads: %d rotated channels of %d", rot, dim);
  GB_REQUIRE(!slots || (k_pages && v_pages && page_size > 0), "conv_heads: cache rows without pages");
  GB_REQUIRE(tok_seq && q_start && pos0 && state_slots, "conv_heads: the step's tables are needed");
  if (n == 0) return 0;
  const long long units = (long long)n * (nh + 2 * nkv);
  const int tp = wconv ? taps : 0;
  if (dtype == kBF16 && !slots && !update_state && n > 64 && dim % 8 == 0 && vdim % 8 == 0 && hd % 8 == 0 && hd <= 8 * kWave &&
      stride % 8 == 0 && out_stride % 8 == 0 && (uintptr_t)proj % 16 == 0 && (uintptr_t)out % 16 == 0 &&
      (uintptr_t)wconv % 16 == 0 && (uintptr_t)state % 16 == 0) {
    int lpu = 1;
    while (lpu * 8 < hd) lpu *= 2;
    // eight rows a lane where that still leaves the chip a few thousand waves, else two
    const long long units8 = (long long)((n + 7) / 8) * (nh + 2 * nkv);
    const int tt = (units8 + kWave / lpu - 1) / (kWave / lpu) >= 2048 ? 8 : 2;
    const long long wide_units = (long long)((n + tt - 1) / tt) * (nh + 2 * nkv);
    const long long waves = (wide_units + kWave / lpu - 1) / (kWave / lpu);
    GB_REQUIRE((waves + 3) / 4 < (1ll << 31), "conv_heads: too many heads for one launch");
    const dim3 grid((unsigned)((waves + 3) / 4));
#define GB_WIDE_T(TP, TT)                                                                                                    \
  hipLaunchKernelGGL((conv_heads_wide_kernel<TP, TT>), grid, dim3(4 * kWave), 0, stream, (const bf16*)proj, stride, wconv,     \
                     state, tok_seq, q_start, pos0, state_slots, cosv, sinv, rot, eps, norm, (bf16*)out, out_stride, hd, nh,   \
                     nkv, dim, vdim, channels, wide_units, lpu, n)
#define GB_WIDE(TP)                     \
  case TP:                              \
    if (tt == 8) GB_WIDE_T(TP, 8);      \
    else GB_WIDE_T(TP, 2);              \
    break;
    switch (tp) {
      GB_WIDE(0) GB_WIDE(1) GB_WIDE(2) GB_WIDE(3) GB_WIDE(4) GB_WIDE(5) GB_WIDE(6) GB_WIDE(7) GB_WIDE(8)
    }
#undef GB_WIDE
#undef GB_WIDE_T
    return launched("conv_heads (wide)");
  }
  const int pairs = (hd + 1) / 2;
  int lpu = 4;
  while (lpu < pairs && lpu < kWave) lpu *= 2;
  const int ppl = pairs > kWave ? 2 : 1;
  const long long waves = (units + kWave / lpu - 1) / (kWave / lpu);
  GB_REQUIRE((waves + 3) / 4 < (1ll << 31), "conv_heads: too many heads for one launch");
  const dim3 grid((unsigned)((waves + 3) / 4));
#define GB_CONV(TT, TP, LPU, PPL)                                                                                            \
  hipLaunchKernelGGL((conv_heads_kernel<TT, TP, LPU, PPL>), grid, dim3(4 * kWave), 0, stream, (const TT*)proj, stride, wconv,  \
                     state, tok_seq, q_start, pos0, state_slots, cosv, sinv, rot, eps, norm, (TT*)out, out_stride, hd, slots,  \
                     (TT*)k_pages, (TT*)v_pages, page_size, nh, nkv, dim, vdim, channels, units, update_state)
#define GB_CONV_L(TT, TP)                                                  \
  switch (ppl == 2 ? 128 : lpu) {                                          \
    case 4: GB_CONV(TT, TP, 4, 1); break;                                  \
    case 8: GB_CONV(TT, TP, 8, 1); break;                                  \
    case 16: GB_CONV(TT, TP, 16, 1); break;                                \
    case 32: GB_CONV(TT, TP, 32, 1); break;                                \
    case 64: GB_CONV(TT, TP, 64, 1); break;                                \
    default: GB_CONV(TT, TP, 64, 2); break;                                \
  }
#define GB_CONV_T(TT)                                                      \
  switch (tp) {                                                            \
    case 0: GB_CONV_L(TT, 0) break;                                        \
    case 1: GB_CONV_L(TT, 1) break;                                        \
    case 2: GB_CONV_L(TT, 2) break;                                        \
    case 3: GB_CONV_L(TT, 3) break;                                        \
    case 4: GB_CONV_L(TT, 4) break;                                        \
    case 5: GB_CONV_L(TT, 5) break;                                        \
    case 6: GB_CONV_L(TT, 6) break;                                        \
    case 7: GB_CONV_L(TT, 7) break;                                        \
    default: GB_CONV_L(TT, 8) break;                                       \
  }
  if (dtype == kF32) {
    GB_CONV_T(float)
  } else if (dtype == kBF16) {
    GB_CONV_T(bf16)
  } else {
    return fail("conv_heads: unknown dtype %d", dtype);
  }
#undef GB_CONV_T
#undef GB_CONV_L
#undef GB_CONV
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
