// Linear attention with a decayed matrix state per (request, head): retention (one fixed decay a head) and
// gated linear attention (a decay per key channel and token).
//
//   S_t = diag(a_t) S_(t-1) + k_t v_t^T      S: [dk, dv], a_t: one number a head, or a vector over the dk rows
//   o_t = S_t^T q_t
//
// The state is 32-bit and lives in a slot per live request, [heads, dv, dk]: a column of S (one value channel)
// lies in a row of memory.  Columns never meet: column j of S_t depends on column j of S_(t-1), k_t and v_t[j]
// alone.  So a wave owns eight columns, eight lanes a column, a lane R = ceil(dk / 8) of its rows in registers, and
// walks its request's tokens of the step in order: the same additions in the same order whether a prompt comes
// whole, in portions or token by token.  A workgroup (four waves, 32 columns of one head) stages the tokens'
// q, k and decays through LDS sixteen tokens at a time, the next sixteen on their way from memory meanwhile.
// q, k and the decays come in 32-bit (what the kernels below prepare), v in the activations' type.
//
// A long portion of a prompt would leave the chip to the few waves of its request, one token after the other.  It is
// cut into segments of `seg_len` tokens that run side by side: segment 0 goes on from the request's state, every other
// one starts from nothing and leaves its own end state E and the product D of its decays in a workspace.  A second
// kernel gives a segment the state S0 it should have started from (folded from the segments before it:
// S <- D S + E) and adds what that state contributes to each token's output, (q_t * P_t)^T S0 with P_t the product of
// the decays from the segment's first token to t; the last segment writes the request's state, D S0 + E.  Portions of
// up to `seg_len` tokens take none of this.
//
// Around it: `retention_prep` (rotation of the first `rot` dimensions of the q and k heads in rotate-half pairs,
// k scaled), `gla_prep` (q scaled, decays sigmoid(z)^(1/tau) from the low-rank projection z = A2 t + b), and
// `head_norm_gate` (each head's output divided by its root mean square, an optional weight over dv, times
// silu(gate), written in the activations' type for the output projection).
#include "common.h"

using namespace gb;

GB_DEFINE_LAST_ERROR

namespace {

constexpr int kTokens = 16;    // tokens staged at a time
constexpr int kLanesCol = 8;   // lanes a column of the state
constexpr int kColsWave = kWave / kLanesCol;
constexpr int kWaves = 4;
constexpr int kColsBlock = kColsWave * kWaves;
constexpr int kThreads = kWaves * kWave;
constexpr int kPiece = 1024;   // elements of a row a workgroup of the preparing kernels takes

// Sum over the eight lanes of a column (lanes 8c .. 8c+7), by data-parallel moves inside the wave's rows of 16 lanes:
// neighbours, pairs of neighbours, then the other half of the eight.  Every lane of the eight gets the sum.
__device__ __forceinline__ float sum8(float v) {
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xf, 0xf, false));   // quad_perm [1,0,3,2]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xf, 0xf, false));   // quad_perm [2,3,0,1]
  v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xf, 0xf, false));  // row_half_mirror
  return v;
}

// What a workgroup of either kernel works on: its request's segment.
struct Segment {
  int seq, seg, n_segs, first, count;
  __device__ __forceinline__ Segment(const int32_t* q_start, const int32_t* q_len, int z, int segs, int seg_len) {
    seq = z / segs;
    seg = z % segs;
    const int all = q_len[seq];
    n_segs = segs > 1 ? (all + seg_len - 1) / seg_len : 1;
    first = q_start[seq] + seg * seg_len;
    count = n_segs > 1 ? min(seg_len, all - seg * seg_len) : all;
  }
};

template <typename T, int R, bool GATED>
__global__ __launch_bounds__(kThreads) void scan_kernel(
    const float* __restrict__ q, const float* __restrict__ k, const float* __restrict__ a, const float* __restrict__ head_decay,
    const T* __restrict__ v, int v_stride, float* __restrict__ out, float* __restrict__ state,
    const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len, const int32_t* __restrict__ pos0,
    const int32_t* __restrict__ state_slots, int nh, int dk, int dv, int sc, int a_head, int segs, int seg_len, float* __restrict__ seg_state,
    float* __restrict__ seg_decay) {
  constexpr int DKP = R * kLanesCol;                       // rows, padded
  constexpr int PER = (kTokens * DKP) / kThreads;          // staged elements a thread and array (R >= 2)
  __shared__ float qs[kTokens][DKP], ks[kTokens][DKP], ds[GATED ? kTokens : 1][GATED ? DKP : 1];
  __shared__ float vs[kTokens][kColsBlock];
  const Segment sg(q_start, q_len, blockIdx.z, segs, seg_len);
  if (sg.seg >= sg.n_segs) return;
  const int seq = sg.seq, h = blockIdx.y, col0 = blockIdx.x * kColsBlock;
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int rg = lane % kLanesCol;                          // which R rows of the column
  const int cb = wave * kColsWave + lane / kLanesCol;       // column within the block
  const int col = col0 + cb;
  const int first = sg.first, count = sg.count;
  const int width = nh * dk;
  const bool live = col < dv;
  const bool cut = sg.n_segs > 1;                           // the request's portion runs as several segments

  float S[R], P[GATED ? R : 1];
  float* slot_row = state + (((size_t)state_slots[seq] * nh + h) * sc + (live ? col : 0)) * dk + rg * R;
  // where the end state goes: the request's slot, or, of a segment, the workspace
  float* srow = cut ? seg_state + (((size_t)blockIdx.z * nh + h) * dv + (live ? col : 0)) * dk + rg * R : slot_row;
  // a request's first tokens start from an empty state, whatever the slot held; so does every segment but the first
  const bool fresh = pos0[seq] == 0 || sg.seg > 0;
#pragma unroll
  for (int m = 0; m < R; ++m) S[m] = (!fresh && live && rg * R + m < dk) ? slot_row[m] : 0.f;
#pragma unroll
  for (int m = 0; m < (GATED ? R : 1); ++m) P[m] = 1.f;
  const float decay = GATED ? 1.f : head_decay[h];

  float nq[PER], nk[PER], na[GATED ? PER : 1], nv[2];
  auto fetch = [&](int t0) {   // tokens t0 .. t0 + kTokens - 1 of this request's rows into registers
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      const int idx = tid + e * kThreads, tok = idx / DKP, ch = idx % DKP;
      const bool ok = t0 + tok < count && ch < dk;
      const size_t at = (size_t)(first + t0 + tok) * width + (size_t)h * dk + ch;
      nq[e] = ok ? q[at] : 0.f;
      nk[e] = ok ? k[at] : 0.f;
      if (GATED) na[e] = ok ? a[a_head ? (size_t)(first + t0 + tok) * nh + h : at] : 0.f;
    }
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int idx = tid + e * kThreads, tok = idx / kColsBlock, c = idx % kColsBlock;
      const bool ok = t0 + tok < count && col0 + c < dv;
      nv[e] = ok ? to_f(v[(size_t)(first + t0 + tok) * v_stride + (size_t)h * dv + col0 + c]) : 0.f;
    }
  };
  static_assert(kTokens * kColsBlock == 2 * kThreads, "two staged values of v a thread");

  fetch(0);
  for (int t0 = 0; t0 < count; t0 += kTokens) {
    __syncthreads();   // the tokens before have been read
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      const int idx = tid + e * kThreads;
      (&qs[0][0])[idx] = nq[e];
      (&ks[0][0])[idx] = nk[e];
      if (GATED) (&ds[0][0])[idx] = na[e];
    }
#pragma unroll
    for (int e = 0; e < 2; ++e) (&vs[0][0])[tid + e * kThreads] = nv[e];
    __syncthreads();
    if (t0 + kTokens < count) fetch(t0 + kTokens);
    const int here = min(kTokens, count - t0);
    // U tokens at a time: their operands are read from LDS together, the state goes through them in order (one
    // multiply-add a token and row is all that waits for the token before), and their outputs' sums over the rows and
    // over the eight lanes of a column run side by side
    constexpr int U = R <= 8 ? 4 : R == 16 ? 2 : 1;
    float* orow = out + (size_t)(first + t0) * ((size_t)nh * dv) + (size_t)h * dv + col;
    int j = 0;
    for (; j + U <= here; j += U) {
      float kk[U][R], qq[U][R], aa[GATED ? U : 1][GATED ? R : 1], vv[U], part[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        vv[u] = vs[j + u][cb];
#pragma unroll
        for (int m = 0; m < R; ++m) {
          kk[u][m] = ks[j + u][rg * R + m];
          qq[u][m] = qs[j + u][rg * R + m];
          if (GATED) aa[u][m] = ds[j + u][rg * R + m];
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        part[u] = 0.f;
#pragma unroll
        for (int m = 0; m < R; ++m) {
          S[m] = fmaf(GATED ? aa[u][m] : decay, S[m], kk[u][m] * vv[u]);
          part[u] = fmaf(S[m], qq[u][m], part[u]);
        }
        if (GATED && cut) {
#pragma unroll
          for (int m = 0; m < R; ++m) P[m] *= aa[u][m];
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) part[u] = sum8(part[u]);
      if (rg == 0 && live) {
#pragma unroll
        for (int u = 0; u < U; ++u) orow[(size_t)(j + u) * ((size_t)nh * dv)] = part[u];
      }
    }
    for (; j < here; ++j) {   // the same sums, token by token
      const float vv = vs[j][cb];
      float part = 0.f;
#pragma unroll
      for (int m = 0; m < R; ++m) {
        S[m] = fmaf(GATED ? ds[j][rg * R + m] : decay, S[m], ks[j][rg * R + m] * vv);
        part = fmaf(S[m], qs[j][rg * R + m], part);
        if (GATED && cut) P[m] *= ds[j][rg * R + m];
      }
      part = sum8(part);
      if (rg == 0 && live) orow[(size_t)j * ((size_t)nh * dv)] = part;
    }
  }
  if (live) {
#pragma unroll
    for (int m = 0; m < R; ++m)
      if (rg * R + m < dk) srow[m] = S[m];
  }
  if (GATED && cut && blockIdx.x == 0 && cb == 0) {   // the segment's decays, once a head
    float* drow = seg_decay + ((size_t)blockIdx.z * nh + h) * dk + rg * R;
#pragma unroll
    for (int m = 0; m < R; ++m)
      if (rg * R + m < dk) drow[m] = P[m];
  }
}

// The second kernel of a portion that ran as segments (see the top of the file): same grid, same lanes.
template <int R, bool GATED>
__global__ __launch_bounds__(kThreads) void scan_join_kernel(
    const float* __restrict__ q, const float* __restrict__ a, const float* __restrict__ head_decay, float* __restrict__ out,
    float* __restrict__ state, const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
    const int32_t* __restrict__ state_slots, int nh, int dk, int dv, int sc, int a_head, int segs, int seg_len, const float* __restrict__ seg_state,
    const float* __restrict__ seg_decay) {
  constexpr int DKP = R * kLanesCol;
  constexpr int PER = (kTokens * DKP) / kThreads;
  __shared__ float qs[kTokens][DKP], ds[GATED ? kTokens : 1][GATED ? DKP : 1];
  const Segment sg(q_start, q_len, blockIdx.z, segs, seg_len);
  if (sg.n_segs <= 1 || sg.seg == 0 || sg.seg >= sg.n_segs) return;   // nothing was cut, or the segment started from the state
  const int h = blockIdx.y, col0 = blockIdx.x * kColsBlock;
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int rg = lane % kLanesCol, cb = wave * kColsWave + lane / kLanesCol, col = col0 + cb;
  const int first = sg.first, count = sg.count, width = nh * dk;
  const bool live = col < dv;
  const float decay = GATED ? 1.f : head_decay[h];
  float whole = 1.f;   // a full segment's decay, for a decay a head: the same products in the same order as token by token
  if (!GATED)
    for (int i = 0; i < seg_len; ++i) whole *= decay;

  // the state this segment should have started from: the end states of the segments before it, folded in order
  const size_t cell0 = (size_t)sg.seq * segs;
  auto e_row = [&](int sgm) { return seg_state + ((((cell0 + sgm) * nh + h) * dv + (live ? col : 0)) * dk) + rg * R; };
  float S0[R];
#pragma unroll
  for (int m = 0; m < R; ++m) S0[m] = (live && rg * R + m < dk) ? e_row(0)[m] : 0.f;
  constexpr int F = R <= 8 ? 4 : 1;   // segments whose end states are asked for together
  for (int s0 = 1; s0 < sg.seg; s0 += F) {
    float e[F][R], d[F][GATED ? R : 1];
#pragma unroll
    for (int f = 0; f < F; ++f) {
      const int sgm = min(s0 + f, sg.seg - 1);
      const float* ep = e_row(sgm);
      const float* dp = seg_decay + ((cell0 + sgm) * nh + h) * dk + rg * R;
#pragma unroll
      for (int m = 0; m < R; ++m) {
        const bool ok = live && rg * R + m < dk;
        e[f][m] = ok ? ep[m] : 0.f;
        if (GATED) d[f][m] = ok ? dp[m] : 0.f;
      }
    }
#pragma unroll
    for (int f = 0; f < F; ++f) {
      if (s0 + f >= sg.seg) break;
#pragma unroll
      for (int m = 0; m < R; ++m) S0[m] = fmaf(GATED ? d[f][m] : whole, S0[m], e[f][m]);
    }
  }

  float P[R];   // the decays from the segment's first token on
#pragma unroll
  for (int m = 0; m < R; ++m) P[m] = 1.f;
  float nq[PER], na[GATED ? PER : 1];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      const int idx = tid + e * kThreads, tok = idx / DKP, ch = idx % DKP;
      const bool ok = t0 + tok < count && ch < dk;
      const size_t at = (size_t)(first + t0 + tok) * width + (size_t)h * dk + ch;
      nq[e] = ok ? q[at] : 0.f;
      if (GATED) na[e] = ok ? a[a_head ? (size_t)(first + t0 + tok) * nh + h : at] : 0.f;
    }
  };
  fetch(0);
  for (int t0 = 0; t0 < count; t0 += kTokens) {
    __syncthreads();
#pragma unroll
    for (int e = 0; e < PER; ++e) {
      (&qs[0][0])[tid + e * kThreads] = nq[e];
      if (GATED) (&ds[0][0])[tid + e * kThreads] = na[e];
    }
    __syncthreads();
    if (t0 + kTokens < count) fetch(t0 + kTokens);
    const int here = min(kTokens, count - t0);
    float* orow = out + (size_t)(first + t0) * ((size_t)nh * dv) + (size_t)h * dv + col;
    constexpr int U = R <= 8 ? 4 : R == 16 ? 2 : 1;   // tokens at a time, as in the first kernel
    // what the first kernel left of these tokens' outputs, asked for before the arithmetic that is added to it
    float was[kTokens];
#pragma unroll
    for (int u = 0; u < kTokens; ++u) was[u] = (rg == 0 && live && u < here) ? orow[(size_t)u * ((size_t)nh * dv)] : 0.f;
    int j = 0;
#pragma unroll
    for (int jj = 0; jj < kTokens; jj += U) {
      if (jj + U > here) break;
      j = jj + U;
      float qq[U][R], aa[GATED ? U : 1][GATED ? R : 1], part[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int m = 0; m < R; ++m) {
          qq[u][m] = qs[jj + u][rg * R + m];
          if (GATED) aa[u][m] = ds[jj + u][rg * R + m];
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        part[u] = 0.f;
#pragma unroll
        for (int m = 0; m < R; ++m) {
          P[m] *= GATED ? aa[u][m] : decay;
          part[u] = fmaf(qq[u][m] * P[m], S0[m], part[u]);
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) part[u] = sum8(part[u]);
      if (rg == 0 && live) {
#pragma unroll
        for (int u = 0; u < U; ++u) orow[(size_t)(jj + u) * ((size_t)nh * dv)] = was[jj + u] + part[u];
      }
    }
    for (; j < here; ++j) {
      float part = 0.f;
#pragma unroll
      for (int m = 0; m < R; ++m) {
        P[m] *= GATED ? ds[j][rg * R + m] : decay;
        part = fmaf(qs[j][rg * R + m] * P[m], S0[m], part);
      }
      part = sum8(part);
      if (rg == 0 && live) orow[(size_t)j * ((size_t)nh * dv)] += part;
    }
  }
  if (sg.seg == sg.n_segs - 1 && live) {   // the request's state after the portion
    const float* e = e_row(sg.seg);
    float* srow = state + (((size_t)state_slots[sg.seq] * nh + h) * sc + col) * dk + rg * R;
#pragma unroll
    for (int m = 0; m < R; ++m)
      if (rg * R + m < dk) srow[m] = fmaf(P[m], S0[m], e[m]);
  }
}

// q32, k32 [n, nh * dk] from the q and k heads of the projection's rows: dimensions i < rot of a head in pairs
// (i, i + rot / 2), i < rot / 2, turned by the row's angles (cos, sin [n, rot / 2]); the rest as they are; k times k_scale.
template <typename T>
__global__ void retention_prep_kernel(const T* __restrict__ proj, int stride, int q_off, int k_off,
                                      const float* __restrict__ cosv, const float* __restrict__ sinv, float* __restrict__ q32,
                                      float* __restrict__ k32, int nh, int dk, int rot, float k_scale) {
  const int t = blockIdx.x, width = nh * dk, half = rot / 2;
  const T* row = proj + (size_t)t * stride;
  // (a workgroup a row and piece of kPiece elements: a step of few rows still spreads over the chip)
  for (int e = blockIdx.y * kPiece + threadIdx.x; e < min(2 * width, (int)(blockIdx.y + 1) * kPiece); e += blockDim.x) {
    const bool is_k = e >= width;
    const int c = is_k ? e - width : e, d = c % dk;
    const T* src = row + (is_k ? k_off : q_off);
    float x = to_f(src[c]);
    if (d < rot) {
      const bool lower = d < half;
      const int i = lower ? d : d - half;
      const float other = to_f(src[lower ? c + half : c - half]);
      const float cs = cosv[(size_t)t * half + i], sn = sinv[(size_t)t * half + i];
      // (u, w) -> (u cos - w sin, w cos + u sin)
      x = lower ? x * cs - other * sn : x * cs + other * sn;
    }
    if (is_k) k32[(size_t)t * width + c] = x * k_scale;
    else q32[(size_t)t * width + c] = x;
  }
}

__device__ __forceinline__ float log_sigmoid(float z) {
  // log(1 / (1 + exp(-z))) without overflow on either side
  return z >= 0.f ? -log1pf(expf(-z)) : z - log1pf(expf(z));
}

// q32 = q * q_scale, k32 = k, decay[t, c] = sigmoid(z)^(1/tau) with z = sum_r A2[c, r] low[t, r] + b[c]; with `zin`
// the sums come from there (a matrix product made them) and a2 is not read
template <typename T>
__global__ void gla_prep_kernel(const T* __restrict__ proj, int stride, int q_off, int k_off, int low_off,
                                const T* __restrict__ a2, const float* __restrict__ zin,
                                const float* __restrict__ a2_bias, float* __restrict__ q32,
                                float* __restrict__ k32, float* __restrict__ decay, int width, int rank, float q_scale,
                                float inv_tau) {
  extern __shared__ float low[];   // [rank]
  const int t = blockIdx.x;
  const T* row = proj + (size_t)t * stride;
  if (!zin) {
    for (int r = threadIdx.x; r < rank; r += blockDim.x) low[r] = to_f(row[low_off + r]);
    __syncthreads();
  }
  for (int c = blockIdx.y * kPiece + threadIdx.x; c < min(width, (int)(blockIdx.y + 1) * kPiece); c += blockDim.x) {
    q32[(size_t)t * width + c] = to_f(row[q_off + c]) * q_scale;
    k32[(size_t)t * width + c] = to_f(row[k_off + c]);
    float z = 0.f;
    if (zin) {
      z = zin[(size_t)t * width + c];
    } else {
      const T* w = a2 + (size_t)c * rank;
      for (int r = 0; r < rank; ++r) z = fmaf(to_f(w[r]), low[r], z);
    }
    z += a2_bias ? a2_bias[c] : 0.f;
    decay[(size_t)t * width + c] = expf(log_sigmoid(z) * inv_tau);
  }
}

// out[t, h, :] = w * o / sqrt(mean(o^2) + eps) * silu(gate[t, h, :])  (w == nullptr: no weight).  One wave a (token, head),
// four waves a workgroup.
template <typename T>
__global__ __launch_bounds__(4 * kWave) void head_norm_gate_kernel(const float* __restrict__ o, const T* __restrict__ gate,
                                                                 int gate_stride, const float* __restrict__ w,
                                                                 T* __restrict__ out, int nh, int dv, float eps, int pairs) {
  const int pair = blockIdx.x * 4 + threadIdx.x / kWave;
  if (pair >= pairs) return;
  const int t = pair / nh, h = pair % nh, lane = threadIdx.x % kWave;
  const float* orow = o + ((size_t)t * nh + h) * dv;
  float ss = 0.f;
  for (int d = lane; d < dv; d += kWave) ss = fmaf(orow[d], orow[d], ss);
  ss = wave_sum(ss);
  const float s = 1.0f / sqrtf(ss / (float)dv + eps);
  for (int d = lane; d < dv; d += kWave) {
    const float g = to_f(gate[(size_t)t * gate_stride + (size_t)h * dv + d]);
    const float act = g / (1.0f + expf(-g));
    const float y = (w ? w[d] : 1.0f) * (orow[d] * s);
    out[((size_t)t * nh + h) * dv + d] = from_f<T>(y * act);
  }
}

// The same with sixteen lanes a (token, head), a lane words of four values, sixteen heads a workgroup: for every dv that
// is a multiple of 4 up to 256, whatever the number of rows (a head's sum is then added up in one order always).
template <typename T>
__global__ __launch_bounds__(256) void head_norm_gate_words_kernel(const float* __restrict__ o, const T* __restrict__ gate,
                                                                 int gate_stride, const float* __restrict__ w,
                                                                 T* __restrict__ out, int nh, int dv, float eps, int pairs) {
  constexpr int IT = 4;
  typedef T quad __attribute__((ext_vector_type(4)));
  const int pair = blockIdx.x * 16 + threadIdx.x / 16, li = threadIdx.x % 16;
  const bool live = pair < pairs;
  const int t = live ? pair / nh : 0, h = live ? pair % nh : 0;
  const float* orow = o + ((size_t)t * nh + h) * dv;
  f32x4 x[IT];
  float ss = 0.f;
#pragma unroll
  for (int it = 0; it < IT; ++it) {
    const int d0 = (it * 16 + li) * 4;
    if (live && d0 < dv) {
      x[it] = *reinterpret_cast<const f32x4*>(orow + d0);
#pragma unroll
      for (int e = 0; e < 4; ++e) ss = fmaf(x[it][e], x[it][e], ss);
    }
  }
#pragma unroll
  for (int off = 1; off < 16; off <<= 1) ss += __shfl_xor(ss, off, kWave);
  const float s = 1.0f / sqrtf(ss / (float)dv + eps);
#pragma unroll
  for (int it = 0; it < IT; ++it) {
    const int d0 = (it * 16 + li) * 4;
    if (live && d0 < dv) {
      const quad g4 = *reinterpret_cast<const quad*>(gate + (size_t)t * gate_stride + (size_t)h * dv + d0);
      quad y;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float g = to_f(g4[e]);
        y[e] = from_f<T>(((w ? w[d0 + e] : 1.0f) * (x[it][e] * s)) * (g / (1.0f + expf(-g))));
      }
      *reinterpret_cast<quad*>(out + ((size_t)t * nh + h) * dv + d0) = y;
    }
  }
}

// ---------------------------------------------------------------- matrix memory with exponential gates (mLSTM)
// Per head, with a log input gate i_t, a log forget gate f_t and a running maximum m (m before the first token: 0):
//   m_t = max(f_t + m_(t-1), i_t)
//   S_t = exp(f_t + m_(t-1) - m_t) S_(t-1) + exp(i_t - m_t) k_t v_t^T,   n_t the same with k_t alone
//   o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6)
// which is the recurrence above with the decay a_t = exp(f_t + m_(t-1) - m_t) a token and head, the keys times
// b_t = exp(i_t - m_t), and n as one more value channel whose v is 1.  The gates are capped,
// i = cap tanh(z_i / cap), f = log sigmoid(cap tanh(z_f / cap)), z the projections plus their biases.

// The gates of every (token, head), side by side: coef[t, h] = (f, i, .) for the kernel below.
__global__ void mlstm_gate_values_kernel(const float* __restrict__ z, int ldz, const float* __restrict__ bias_i,
                                         const float* __restrict__ bias_f, float cap, float* __restrict__ coef, int n, int nh) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= n * nh) return;
  const int t = idx / nh, h = idx % nh;
  const float* row = z + (size_t)t * ldz;
  coef[(size_t)idx * 3 + 1] = cap * tanhf((row[h] + (bias_i ? bias_i[h] : 0.f)) / cap);
  coef[(size_t)idx * 3] = log_sigmoid(cap * tanhf((row[nh + h] + (bias_f ? bias_f[h] : 0.f)) / cap));
}

// One wave a (request, head): 256 tokens at a time, each lane four tokens in a row.  A token's gates are the pair (F, I)
// that stands for m -> max(F + m, I) (first (F1, I1), then (F2, I2): (F1 + F2, max(I1 + F2, I2))): a lane folds its
// four, the wave scans the 64 results, and each lane walks its four tokens again from the maximum that the lanes
// before it leave.  Writes coef[t, h] = (a_t, b_t, exp(-m_t)) and leaves the request's last m in its state slot at
// `m_at` of the head's block.
__global__ __launch_bounds__(kWave) void mlstm_gates_kernel(float* __restrict__ coef,
                                                          float* __restrict__ state, long long head_floats, long long m_at,
                                                          const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
                                                          const int32_t* __restrict__ pos0, const int32_t* __restrict__ state_slots,
                                                          int nh) {
  constexpr int TPL = 4;   // tokens a lane
  const int seq = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int start = q_start[seq], L = q_len[seq];
  float* mp = state + ((size_t)state_slots[seq] * nh + h) * head_floats + m_at;
  float carry = pos0[seq] == 0 ? 0.f : *mp;
  for (int base = 0; base < L; base += kWave * TPL) {
    const int t0 = base + lane * TPL;
    float fg[TPL], ig[TPL];
    float F = 0.f, I = -INFINITY;   // the lane's tokens folded (tokens beyond the last are the identity)
#pragma unroll
    for (int j = 0; j < TPL; ++j) {
      fg[j] = 0.f;
      ig[j] = -INFINITY;
      if (t0 + j < L) {
        const float* c = coef + ((size_t)(start + t0 + j) * nh + h) * 3;
        fg[j] = c[0];
        ig[j] = c[1];
      }
      I = fmaxf(I + fg[j], ig[j]);
      F += fg[j];
    }
#pragma unroll
    for (int off = 1; off < kWave; off <<= 1) {
      const float Fo = __shfl_up(F, off, kWave), Io = __shfl_up(I, off, kWave);
      if (lane >= off) {
        I = fmaxf(Io + F, I);
        F = Fo + F;
      }
    }
    // what the lanes before this one make of the maximum that the chunk began with
    const float Fb = __shfl_up(F, 1, kWave), Ib = __shfl_up(I, 1, kWave);
    float m = lane == 0 ? carry : fmaxf(Fb + carry, Ib);
#pragma unroll
    for (int j = 0; j < TPL; ++j) {
      const float before = m;
      m = fmaxf(fg[j] + before, ig[j]);
      if (t0 + j < L) {
        float* c = coef + ((size_t)(start + t0 + j) * nh + h) * 3;
        c[0] = expf(fg[j] + before - m);
        c[1] = expf(ig[j] - m);
        c[2] = expf(-m);
      }
    }
    carry = __shfl(m, kWave - 1, kWave);   // (lanes beyond the last token hold the identity: their m is the last token's)
  }
  if (lane == 0 && L > 0) *mp = carry;
}

// Both kernels above in one for a step in which every request brings one token: a thread a (request, head).
__global__ void mlstm_gates_single_kernel(const float* __restrict__ z, int ldz, const float* __restrict__ bias_i,
                                          const float* __restrict__ bias_f, float cap, float* __restrict__ coef,
                                          float* __restrict__ state, long long head_floats, long long m_at,
                                          const int32_t* __restrict__ q_start, const int32_t* __restrict__ pos0,
                                          const int32_t* __restrict__ state_slots, int n_seqs, int nh) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= n_seqs * nh) return;
  const int seq = idx / nh, h = idx % nh, t = q_start[seq];
  const float* row = z + (size_t)t * ldz;
  const float ig = cap * tanhf((row[h] + (bias_i ? bias_i[h] : 0.f)) / cap);
  const float fg = log_sigmoid(cap * tanhf((row[nh + h] + (bias_f ? bias_f[h] : 0.f)) / cap));
  float* mp = state + ((size_t)state_slots[seq] * nh + h) * head_floats + m_at;
  const float before = pos0[seq] == 0 ? 0.f : *mp;
  const float m = fmaxf(fg + before, ig);
  float* c = coef + ((size_t)t * nh + h) * 3;
  c[0] = expf(fg + before - m);
  c[1] = expf(ig - m);
  c[2] = expf(-m);
  *mp = m;
}

// q32 = q * q_scale, k32 = k * b_t, decay[t, h] = a_t, vext[t, h, :] = (v[t, h, :], 1): the scan's operands
template <typename T>
__global__ void mlstm_prep_kernel(const T* __restrict__ proj, int stride, int q_off, int k_off, int v_off,
                                  const float* __restrict__ coef, float* __restrict__ q32, float* __restrict__ k32,
                                  float* __restrict__ decay, T* __restrict__ vext, int nh, int dk, int dv, float q_scale) {
  const int t = blockIdx.x;
  const T* row = proj + (size_t)t * stride;
  const int width = nh * dk, vw = nh * (dv + 1);
  for (int c = blockIdx.y * kPiece + threadIdx.x; c < min(width, (int)(blockIdx.y + 1) * kPiece); c += blockDim.x) {
    const int h = c / dk;
    q32[(size_t)t * width + c] = to_f(row[q_off + c]) * q_scale;
    k32[(size_t)t * width + c] = to_f(row[k_off + c]) * coef[((size_t)t * nh + h) * 3 + 1];
  }
  for (int c = blockIdx.y * kPiece + threadIdx.x; c < min(vw, (int)(blockIdx.y + 1) * kPiece); c += blockDim.x) {
    const int h = c / (dv + 1), d = c % (dv + 1);
    vext[(size_t)t * vw + c] = d < dv ? row[v_off + h * dv + d] : from_f<T>(1.0f);
  }
  if (blockIdx.y == 0)
    for (int h = threadIdx.x; h < nh; h += blockDim.x) decay[(size_t)t * nh + h] = coef[((size_t)t * nh + h) * 3];
}

// out[t, h, :] = w[h, :] * y / sqrt(mean(y^2) + eps) * sigmoid(gate[t, h, :]),  y = o[t, h, :dv] / (max(|o[t, h, dv]|,
// exp(-m_t)) + 1e-6); o holds dv + 1 sums a head, the last the normaliser's.  Sixteen lanes a (token, head), sixteen
// heads a workgroup; a lane takes every sixteenth channel, so a head's sum is added up in one order whatever the step.
template <typename T>
__global__ __launch_bounds__(4 * kWave) void mlstm_out_kernel(const float* __restrict__ o, const float* __restrict__ coef,
                                                            const T* __restrict__ gate, int gate_stride,
                                                            const float* __restrict__ w, T* __restrict__ out, int nh, int dv,
                                                            float eps, int pairs) {
  constexpr int LPH = 16;   // lanes a head
  const int pair = blockIdx.x * (4 * kWave / LPH) + threadIdx.x / LPH, li = threadIdx.x % LPH;
  const bool live = pair < pairs;
  const int t = live ? pair / nh : 0, h = live ? pair % nh : 0;
  const float* orow = o + ((size_t)t * nh + h) * (dv + 1);
  const float inv = 1.0f / (fmaxf(fabsf(orow[dv]), coef[((size_t)t * nh + h) * 3 + 2]) + 1e-6f);
  float ss = 0.f;
  for (int d = li; d < dv; d += LPH) {
    const float y = orow[d] * inv;
    ss = fmaf(y, y, ss);
  }
#pragma unroll
  for (int off = LPH / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, kWave);
  if (!live) return;
  const float s = inv / sqrtf(ss / (float)dv + eps);
  for (int d = li; d < dv; d += LPH) {
    const float g = to_f(gate[(size_t)t * gate_stride + (size_t)h * dv + d]);
    const float y = (w ? w[(size_t)h * dv + d] : 1.0f) * (orow[d] * s);
    out[((size_t)t * nh + h) * dv + d] = from_f<T>(y / (1.0f + expf(-g)));
  }
}

template <typename T, bool GATED>
int launch_scan(int R, dim3 grid, hipStream_t stream, const float* q, const float* k, const float* a, const float* head_decay,
                const void* v, int v_stride, float* out, float* state, const int32_t* q_start, const int32_t* q_len,
                const int32_t* pos0, const int32_t* slots, int nh, int dk, int dv, int sc, int a_head, int segs, int seg_len, float* seg_state,
                float* seg_decay) {
#define GB_SCAN(RR)                                                                                                          \
  case RR:                                                                                                                   \
    hipLaunchKernelGGL((scan_kernel<T, RR, GATED>), grid, dim3(kThreads), 0, stream, q, k, a, head_decay, (const T*)v, v_stride, \
                       out, state, q_start, q_len, pos0, slots, nh, dk, dv, sc, a_head, segs, seg_len, seg_state, seg_decay); \
    if (segs > 1)                                                                                                            \
      hipLaunchKernelGGL((scan_join_kernel<RR, GATED>), grid, dim3(kThreads), 0, stream, q, a, head_decay, out, state, q_start, \
                         q_len, slots, nh, dk, dv, sc, a_head, segs, seg_len, (const float*)seg_state, (const float*)seg_decay); \
    break;
  switch (R) {
    GB_SCAN(2) GB_SCAN(4) GB_SCAN(8) GB_SCAN(16) GB_SCAN(32)
    default: return fail("linear_scan: no kernel for %d rows a lane", R);
  }
#undef GB_SCAN
  return launched("linear_scan");
}

}  // namespace

// The recurrence over the rows of a step.  q, k [n, nh * dk] float32; `a` [n, nh * dk] float32 decays a key channel
// (a_head: [n, nh], a decay a token and head, the same for all its key channels), or
// nullptr with head_decay [nh] float32; v rows of nh * dv in the activations' type (row stride v_stride); out [n, nh * dv]
// float32; state [slots, nh, state_cols, dk] float32 with state_cols >= dv (rows beyond dv are the caller's).  Request s of the step brings rows q_start[s] .. + q_len[s] - 1, starts at
// position pos0[s] (0: from an empty state) and keeps its state in slot state_slots[s].
// segs > 1: no request brings more than segs * seg_len rows, and those that bring more than seg_len run as segments of
// seg_len rows side by side; seg_ws holds gb_linear_scan_floats(n_seqs, nh, dk, dv, segs) floats.
extern "C" long long gb_linear_scan_floats(int n_seqs, int nh, int dk, int dv, int segs) {
  return segs > 1 ? (long long)n_seqs * segs * nh * ((long long)dv * dk + dk) : 0;
}

extern "C" int gb_linear_scan(const float* q, const float* k, const float* a, const float* head_decay, const void* v,
                              int v_dtype, int v_stride, float* out, float* state, const int32_t* q_start,
                              const int32_t* q_len, const int32_t* pos0, const int32_t* state_slots, int n_seqs, int nh,
                              int dk, int dv, int state_cols, int a_head, int segs, int seg_len, float* seg_ws, long long seg_ws_floats,
                              hipStream_t stream) {
  GB_REQUIRE(state_cols >= dv, "linear_scan: a state of %d columns a head holds fewer than the %d value channels", state_cols, dv);
  GB_REQUIRE(n_seqs >= 0 && nh > 0 && dk > 0 && dv > 0, "linear_scan: bad sizes requests=%d heads=%d dk=%d dv=%d", n_seqs, nh, dk, dv);
  GB_REQUIRE(dk <= 32 * kLanesCol, "linear_scan: a key size of %d is above the supported %d", dk, 32 * kLanesCol);
  GB_REQUIRE((a != nullptr) != (head_decay != nullptr), "linear_scan: a decay a head or a decay a key channel, one of the two");
  GB_REQUIRE(v_stride >= nh * dv, "linear_scan: value rows of %d hold fewer than %d heads of %d", v_stride, nh, dv);
  GB_REQUIRE(segs >= 1 && (segs == 1 || (seg_len >= kTokens && seg_ws != nullptr &&
                                          seg_ws_floats >= gb_linear_scan_floats(n_seqs, nh, dk, dv, segs))),
             "linear_scan: %d segments of %d rows need a workspace of %lld floats", segs, seg_len,
             gb_linear_scan_floats(n_seqs, nh, dk, dv, segs));
  GB_REQUIRE((long long)n_seqs * segs <= 65535 && nh <= 65535, "linear_scan: too many requests, segments or heads for one launch");
  if (n_seqs == 0) return 0;
  float* seg_state = seg_ws;
  float* seg_decay = segs > 1 ? seg_ws + (size_t)n_seqs * segs * nh * dv * dk : nullptr;
  int R = 2;
  while (R * kLanesCol < dk) R *= 2;
  const dim3 grid((unsigned)((dv + kColsBlock - 1) / kColsBlock), (unsigned)nh, (unsigned)(n_seqs * segs));
  const bool gated = a != nullptr;
  if (v_dtype == kF32)
    return gated ? launch_scan<float, true>(R, grid, stream, q, k, a, head_decay, v, v_stride, out, state, q_start, q_len, pos0, state_slots, nh, dk, dv, state_cols, a_head, segs, seg_len, seg_state, seg_decay)
                 : launch_scan<float, false>(R, grid, stream, q, k, a, head_decay, v, v_stride, out, state, q_start, q_len, pos0, state_slots, nh, dk, dv, state_cols, a_head, segs, seg_len, seg_state, seg_decay);
  if (v_dtype == kBF16)
    return gated ? launch_scan<bf16, true>(R, grid, stream, q, k, a, head_decay, v, v_stride, out, state, q_start, q_len, pos0, state_slots, nh, dk, dv, state_cols, a_head, segs, seg_len, seg_state, seg_decay)
                 : launch_scan<bf16, false>(R, grid, stream, q, k, a, head_decay, v, v_stride, out, state, q_start, q_len, pos0, state_slots, nh, dk, dv, state_cols, a_head, segs, seg_len, seg_state, seg_decay);
  return fail("linear_scan: unknown dtype %d", v_dtype);
}

extern "C" int gb_retention_prep(const void* proj, int dtype, int stride, int q_off, int k_off, const float* cosv,
                                 const float* sinv, float* q32, float* k32, int n, int nh, int dk, int rot, float k_scale,
                                 hipStream_t stream) {
  GB_REQUIRE(n >= 0 && nh > 0 && dk > 0 && rot >= 0 && rot <= dk && rot % 2 == 0, "retention_prep: bad sizes n=%d heads=%d dk=%d rot=%d",
             n, nh, dk, rot);
  GB_REQUIRE(q_off >= 0 && k_off >= 0 && q_off + nh * dk <= stride && k_off + nh * dk <= stride, "retention_prep: heads beyond the row");
  GB_REQUIRE(rot == 0 || (cosv && sinv), "retention_prep: rotation without tables");
  GB_REQUIRE(n <= 2147483647 && (2 * nh * dk + kPiece - 1) / kPiece <= 65535, "retention_prep: rows too long for one launch");
  if (n == 0) return 0;
  const int threads = nh * dk >= 512 ? 256 : 128;
  if (dtype == kF32)
    hipLaunchKernelGGL(retention_prep_kernel<float>, dim3(n, (2 * nh * dk + kPiece - 1) / kPiece), dim3(threads), 0, stream, (const float*)proj, stride, q_off, k_off,
                       cosv, sinv, q32, k32, nh, dk, rot, k_scale);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(retention_prep_kernel<bf16>, dim3(n, (2 * nh * dk + kPiece - 1) / kPiece), dim3(threads), 0, stream, (const bf16*)proj, stride, q_off, k_off,
                       cosv, sinv, q32, k32, nh, dk, rot, k_scale);
  else
    return fail("retention_prep: unknown dtype %d", dtype);
  return launched("retention_prep");
}

extern "C" int gb_gla_prep(const void* proj, int dtype, int stride, int q_off, int k_off, int low_off, const void* a2,
                           const float* zin, const float* a2_bias, float* q32, float* k32, float* decay, int n, int width, int rank,
                           float q_scale, float inv_tau, hipStream_t stream) {
  GB_REQUIRE(n >= 0 && width > 0 && rank > 0 && rank <= 4096, "gla_prep: bad sizes n=%d width=%d rank=%d", n, width, rank);
  GB_REQUIRE(a2 != nullptr || zin != nullptr, "gla_prep: neither the decay's second matrix nor its products");
  GB_REQUIRE(q_off >= 0 && k_off >= 0 && low_off >= 0 && q_off + width <= stride && k_off + width <= stride &&
                 low_off + rank <= stride, "gla_prep: heads beyond the row");
  if (n == 0) return 0;
  const int threads = width >= 512 ? 256 : 128;
  const size_t smem = sizeof(float) * rank;
  if (dtype == kF32)
    hipLaunchKernelGGL(gla_prep_kernel<float>, dim3(n, (width + kPiece - 1) / kPiece), dim3(threads), smem, stream, (const float*)proj, stride, q_off, k_off,
                       low_off, (const float*)a2, zin, a2_bias, q32, k32, decay, width, rank, q_scale, inv_tau);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(gla_prep_kernel<bf16>, dim3(n, (width + kPiece - 1) / kPiece), dim3(threads), smem, stream, (const bf16*)proj, stride, q_off, k_off,
                       low_off, (const bf16*)a2, zin, a2_bias, q32, k32, decay, width, rank, q_scale, inv_tau);
  else
    return fail("gla_prep: unknown dtype %d", dtype);
  return launched("gla_prep");
}

extern "C" int gb_head_norm_gate(const float* o, const void* gate, int dtype, int gate_stride, const float* w, void* out, int n,
                                 int nh, int dv, float eps, hipStream_t stream) {
  GB_REQUIRE(n >= 0 && nh > 0 && dv > 0 && gate_stride >= nh * dv, "head_norm_gate: bad sizes n=%d heads=%d dv=%d", n, nh, dv);
  GB_REQUIRE((long long)n * nh < (1ll << 31), "head_norm_gate: too many (token, head) pairs");
  if (n == 0) return 0;
  const int pairs = n * nh, gw = dtype == kF32 ? 16 : 8;   // (a gate word of four values: 16 or 8 bytes)
  if (dv % 4 == 0 && dv <= 256 && gate_stride % 4 == 0 && (uintptr_t)gate % gw == 0 && (uintptr_t)o % 16 == 0 &&
      (uintptr_t)out % gw == 0 && (dtype == kF32 || dtype == kBF16)) {
    const dim3 grid((unsigned)((pairs + 15) / 16));
    if (dtype == kF32)
      hipLaunchKernelGGL(head_norm_gate_words_kernel<float>, grid, dim3(256), 0, stream, o, (const float*)gate, gate_stride, w,
                         (float*)out, nh, dv, eps, pairs);
    else
      hipLaunchKernelGGL(head_norm_gate_words_kernel<bf16>, grid, dim3(256), 0, stream, o, (const bf16*)gate, gate_stride, w,
                         (bf16*)out, nh, dv, eps, pairs);
    return launched("head_norm_gate");
  }
  if (dtype == kF32)
    hipLaunchKernelGGL(head_norm_gate_kernel<float>, dim3((unsigned)((n * nh + 3) / 4)), dim3(4 * kWave), 0, stream, o,
                       (const float*)gate, gate_stride, w, (float*)out, nh, dv, eps, n * nh);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(head_norm_gate_kernel<bf16>, dim3((unsigned)((n * nh + 3) / 4)), dim3(4 * kWave), 0, stream, o,
                       (const bf16*)gate, gate_stride, w, (bf16*)out, nh, dv, eps, n * nh);
  else
    return fail("head_norm_gate: unknown dtype %d", dtype);
  return launched("head_norm_gate");
}

// z [n, ldz] float32: the input gates' projections of the nh heads, then the forget gates'; biases float32 [nh] or nullptr;
// coef [n, nh, 3] float32 (n: the step's rows) receives (a_t, b_t, exp(-m_t)); the running maximum of head h of a request lives at
// state[slot][h * head_floats + m_at].  single: every request of the step brings one row, and one kernel does it all.
extern "C" int gb_mlstm_gates(const float* z, int ldz, const float* bias_i, const float* bias_f, float cap, float* coef,
                              float* state, long long head_floats, long long m_at, const int32_t* q_start,
                              const int32_t* q_len, const int32_t* pos0, const int32_t* state_slots, int n_seqs, int nh,
                              int n, int single, hipStream_t stream) {
  GB_REQUIRE(n_seqs >= 0 && nh > 0 && ldz >= 2 * nh && cap > 0.f, "mlstm_gates: bad sizes requests=%d heads=%d ldz=%d cap=%g", n_seqs, nh, ldz, cap);
  GB_REQUIRE(head_floats > 0 && m_at >= 0 && m_at < head_floats, "mlstm_gates: the maximum lies outside its head's state");
  GB_REQUIRE(n_seqs <= 2147483647 && nh <= 65535, "mlstm_gates: too many heads for one launch");
  GB_REQUIRE(n >= 0 && (long long)n * nh < (1ll << 31), "mlstm_gates: too many (token, head) pairs");
  if (n_seqs == 0 || n == 0) return 0;
  if (single) {
    GB_REQUIRE(n == n_seqs, "mlstm_gates: a step of single tokens brings %d rows for %d requests", n, n_seqs);
    hipLaunchKernelGGL(mlstm_gates_single_kernel, dim3((unsigned)((n_seqs * nh + 255) / 256)), dim3(256), 0, stream, z, ldz, bias_i,
                       bias_f, cap, coef, state, head_floats, m_at, q_start, pos0, state_slots, n_seqs, nh);
    return launched("mlstm_gates (single tokens)");
  }
  hipLaunchKernelGGL(mlstm_gate_values_kernel, dim3((unsigned)((n * nh + 255) / 256)), dim3(256), 0, stream, z, ldz, bias_i, bias_f,
                     cap, coef, n, nh);
  hipLaunchKernelGGL(mlstm_gates_kernel, dim3(n_seqs, nh), dim3(kWave), 0, stream, coef, state, head_floats, m_at, q_start, q_len,
                     pos0, state_slots, nh);
  return launched("mlstm_gates");
}

extern "C" int gb_mlstm_prep(const void* proj, int dtype, int stride, int q_off, int k_off, int v_off, const float* coef,
                             float* q32, float* k32, float* decay, void* vext, int n, int nh, int dk, int dv, float q_scale,
                             hipStream_t stream) {
  GB_REQUIRE(n >= 0 && nh > 0 && dk > 0 && dv > 0, "mlstm_prep: bad sizes n=%d heads=%d dk=%d dv=%d", n, nh, dk, dv);
  GB_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && q_off + nh * dk <= stride && k_off + nh * dk <= stride &&
                 v_off + nh * dv <= stride, "mlstm_prep: heads beyond the row");
  const int longest = nh * dk > nh * (dv + 1) ? nh * dk : nh * (dv + 1);
  GB_REQUIRE((longest + kPiece - 1) / kPiece <= 65535, "mlstm_prep: rows too long for one launch");
  if (n == 0) return 0;
  const dim3 grid(n, (longest + kPiece - 1) / kPiece);
  const int threads = longest >= 512 ? 256 : 128;
  if (dtype == kF32)
    hipLaunchKernelGGL(mlstm_prep_kernel<float>, grid, dim3(threads), 0, stream, (const float*)proj, stride, q_off, k_off, v_off, coef,
                       q32, k32, decay, (float*)vext, nh, dk, dv, q_scale);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(mlstm_prep_kernel<bf16>, grid, dim3(threads), 0, stream, (const bf16*)proj, stride, q_off, k_off, v_off, coef,
                       q32, k32, decay, (bf16*)vext, nh, dk, dv, q_scale);
  else
    return fail("mlstm_prep: unknown dtype %d", dtype);
  return launched("mlstm_prep");
}

extern "C" int gb_mlstm_out(const float* o, const float* coef, const void* gate, int dtype, int gate_stride, const float* w,
                            void* out, int n, int nh, int dv, float eps, hipStream_t stream) {
  GB_REQUIRE(n >= 0 && nh > 0 && dv > 0 && gate_stride >= nh * dv, "mlstm_out: bad sizes n=%d heads=%d dv=%d", n, nh, dv);
  GB_REQUIRE((long long)n * nh < (1ll << 31), "mlstm_out: too many (token, head) pairs");
  if (n == 0) return 0;
  const dim3 grid((unsigned)((n * nh + 15) / 16));
  if (dtype == kF32)
    hipLaunchKernelGGL(mlstm_out_kernel<float>, grid, dim3(4 * kWave), 0, stream, o, coef, (const float*)gate, gate_stride, w,
                       (float*)out, nh, dv, eps, n * nh);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(mlstm_out_kernel<bf16>, grid, dim3(4 * kWave), 0, stream, o, coef, (const bf16*)gate, gate_stride, w,
                       (bf16*)out, nh, dv, eps, n * nh);
  else
    return fail("mlstm_out: unknown dtype %d", dtype);
  return launched("mlstm_out");
}

GB_TAPED(gb_linear_scan)
GB_TAPED(gb_retention_prep)
GB_TAPED(gb_gla_prep)
GB_TAPED(gb_head_norm_gate)
GB_TAPED(gb_mlstm_gates)
GB_TAPED(gb_mlstm_prep)
GB_TAPED(gb_mlstm_out)
