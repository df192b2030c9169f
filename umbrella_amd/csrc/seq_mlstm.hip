// Matrix memory with exponential gates (the mLSTM cell): per head a [D][Dv] fp32 state S and a normaliser n [D],
//     i_t = cap tanh(z_i / cap)        f_t = log sigmoid(cap tanh(z_f / cap))        m_t = max(f_t + m_(t-1), i_t)   (m_0 = 0)
//     S_t = e^(f_t + m_(t-1) - m_t) S_(t-1) + e^(i_t - m_t) k_t v_t^T          n_t the same with k_t alone
//     o_t = S_t^T q_t / (max(|n_t . q_t|, e^(-m_t)) + 1e-6)
// The running maximum m keeps every exponent non-positive.  With a_t = e^(f_t + m_(t-1) - m_t) and b_t = e^(i_t - m_t) this is the
// linear recurrence S <- a S + k (b v)^T with one decay per head, and n is the same recurrence with the value 1: the normaliser
// rides along as ONE EXTRA VALUE COLUMN (v' = [b v | b | 0 ..], Pp columns), so the scans of seq_gla.hip / seq_ssd.hip carry both
// and the read-out's column Dv is n . q.  This file holds what is special:
//   mscan   the gates and the running maximum of every (token, head): leaves log a, a, m and b for every token and the last m in
//           the sequence's slot (a sequence that starts at position 0 starts from m = 0 whatever its slot holds)
//   prep    scaled queries and the widened value rows
//   step    both for steps of one token per sequence, in one launch
// The stabilised division, the per-head norm and the output gate are head_gate of seq_retention.hip.  Everything is fp32.
#include "seq_common.h"

__device__ __forceinline__ float mlstm_gate_i(float z, float cap) { return cap * tanhf(z / cap); }
__device__ __forceinline__ float mlstm_gate_f(float z, float cap) { return log_sigmoidf_(cap * tanhf(z / cap)); }

// One wave per (sequence, head) walks the stretch in tiles of 64 tokens, lane = token.  The recurrence m <- max(f + m, i) is the
// composition of the maps m -> max(m + a, b); two of them compose to (a1 + a2, max(b1 + a2, b2)), so a tile is an inclusive scan
// over the lanes (six exchanges) applied to the maximum the tile inherits.  The gates are formed here (lane = token: tanh and
// log-sigmoid side by side), the next tile's projections are in flight while the current one is scanned.  Against the
// token-by-token order the sums f + f + .. are associated differently: the maxima agree to fp32 rounding, and since every
// decay and weight below is formed from the SAME maxima the recurrence they describe is the same.
__global__ __launch_bounds__(64) void mlstm_mscan_kernel(float* __restrict__ log_alpha, float* __restrict__ alpha,
                                                         float* __restrict__ mrun, float* __restrict__ bw,
                                                         float* __restrict__ mstate, const float* __restrict__ proj, int ld, int i_col,
                                                         int f_col, float cap, const int* __restrict__ seq_slot,
                                                         const int* __restrict__ seq_row0, const int* __restrict__ seq_pos0,
                                                         const int* __restrict__ seq_len, int H) {
  const int b = blockIdx.x / H, h = blockIdx.x - b * H, lane = threadIdx.x;
  const int n = seq_len[b];
  if (n <= 0) return;
  const long row0 = seq_row0[b];
  float* ms = mstate + (long)seq_slot[b] * H + h;
  float m_in = seq_pos0[b] == 0 ? 0.f : *ms;
  auto fetch = [&](int t0, float& zi, float& zf) {
    const long r = row0 + (t0 + lane < n ? t0 + lane : n - 1);        // clamped: never used past the stretch
    zi = proj[r * ld + i_col + h];
    zf = proj[r * ld + f_col + h];
  };
  float zi, zf;
  fetch(0, zi, zf);
  for (int t0 = 0; t0 < n; t0 += 64) {
    const float gi = mlstm_gate_i(zi, cap), gf = mlstm_gate_f(zf, cap);
    if (t0 + 64 < n) fetch(t0 + 64, zi, zf);
    const bool live = t0 + lane < n;
    float a = live ? gf : 0.f, bb = live ? gi : -INFINITY;           // past the stretch: the identity map
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const float pa = __shfl_up(a, o, 64), pb = __shfl_up(bb, o, 64);
      if (lane >= o) { bb = fmaxf(pb + a, bb); a = pa + a; }
    }
    const float m = fmaxf(a + m_in, bb);
    float mp = __shfl_up(m, 1, 64);
    if (lane == 0) mp = m_in;
    if (live) {
      const long r = row0 + t0 + lane;
      const float la = gf + mp - m;
      log_alpha[r * H + h] = la;
      alpha[r * H + h] = expf(la);
      mrun[r * H + h] = m;
      bw[r * H + h] = expf(gi - m);
    }
    m_in = __shfl(m, 63, 64);                                        // past the stretch the map is the identity: lane 63 holds the last m
  }
  if (lane == 0) *ms = m_in;
}

__global__ __launch_bounds__(256) void mlstm_prep_kernel(float* __restrict__ qs, float* __restrict__ vp, const float* __restrict__ proj,
                                                         int ld, int q_col, int v_col, const float* __restrict__ bw, int H, int D,
                                                         int Dv, int Pp, float qscale) {
  const int t = blockIdx.x, idx = blockIdx.y * 256 + threadIdx.x;
  const int nq = H * D;
  if (idx < nq) {
    qs[(long)t * nq + idx] = proj[(long)t * ld + q_col + idx] * qscale;
    return;
  }
  const int j = idx - nq;
  if (j >= H * Pp) return;
  const int h = j / Pp, c = j - h * Pp;
  const float w = bw[(long)t * H + h];
  vp[(long)t * H * Pp + j] = c < Dv ? w * proj[(long)t * ld + v_col + (long)h * Dv + c] : (c == Dv ? w : 0.f);
}

// one token per sequence: gates, maximum, decays, scaled query and widened value row of a (token, head) by one workgroup slice
__global__ __launch_bounds__(256) void mlstm_step_kernel(float* __restrict__ qs, float* __restrict__ vp, float* __restrict__ log_alpha,
                                                         float* __restrict__ alpha, float* __restrict__ mrun,
                                                         float* __restrict__ mstate, const float* __restrict__ proj, int ld, int q_col,
                                                         int v_col, int i_col, int f_col, const int* __restrict__ pos,
                                                         const int* __restrict__ slot_, int H, int D, int Dv, int Pp, float qscale,
                                                         float cap) {
  const int t = blockIdx.x, h = blockIdx.y;
  const float gi = mlstm_gate_i(proj[(long)t * ld + i_col + h], cap), gf = mlstm_gate_f(proj[(long)t * ld + f_col + h], cap);
  float* ms = mstate + (long)slot_[t] * H + h;
  const float m = pos[t] == 0 ? 0.f : *ms;               // every thread reads the old value before any writes the new one
  const float carried = gf + m;
  const float mn = fmaxf(carried, gi);
  const float la = carried - mn;
  const float bw = expf(gi - mn);
  __syncthreads();
  if (threadIdx.x == 0) {
    *ms = mn;
    log_alpha[(long)t * H + h] = la;
    alpha[(long)t * H + h] = expf(la);
    mrun[(long)t * H + h] = mn;
  }
  for (int d = threadIdx.x; d < D; d += 256) qs[(long)t * H * D + (long)h * D + d] = proj[(long)t * ld + q_col + (long)h * D + d] * qscale;
  for (int c = threadIdx.x; c < Pp; c += 256)
    vp[(long)t * H * Pp + (long)h * Pp + c] = c < Dv ? bw * proj[(long)t * ld + v_col + (long)h * Dv + c] : (c == Dv ? bw : 0.f);
}

extern "C" int umb_mlstm_mscan(float* log_alpha, float* alpha, float* mrun, float* bw, float* mstate, const float* proj, int ld,
                               int i_col, int f_col, float cap, const int* seq_slot, const int* seq_row0, const int* seq_pos0,
                               const int* seq_len, int B, int H, hipStream_t st) {
  if (B < 1 || H < 1 || !(cap > 0.f) || !log_alpha || !alpha || !mrun || !bw || !mstate || !proj || !seq_slot || !seq_row0 ||
      !seq_pos0 || !seq_len || i_col < 0 || f_col < 0 || ld < i_col + H || ld < f_col + H)
    return UMB_EINVAL;
  hipLaunchKernelGGL(mlstm_mscan_kernel, dim3(B * H), dim3(64), 0, st, log_alpha, alpha, mrun, bw, mstate, proj, ld, i_col, f_col, cap,
                     seq_slot, seq_row0, seq_pos0, seq_len, H);
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_mlstm_prep(float* qs, float* vp, const float* proj, int ld, int q_col, int v_col, const float* bw, int T, int H,
                              int D, int Dv, int Pp, float qscale, hipStream_t st) {
  if (T < 1 || H < 1 || D < 1 || Dv < 1 || Pp < Dv + 1 || !qs || !vp || !proj || !bw || q_col < 0 || v_col < 0 ||
      ld < q_col + H * D || ld < v_col + H * Dv)
    return UMB_EINVAL;
  hipLaunchKernelGGL(mlstm_prep_kernel, dim3(T, (H * (D + Pp) + 255) / 256), dim3(256), 0, st, qs, vp, proj, ld, q_col, v_col, bw, H, D,
                     Dv, Pp, qscale);
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_mlstm_step(float* qs, float* vp, float* log_alpha, float* alpha, float* mrun, float* mstate, const float* proj,
                              int ld, int q_col, int v_col, int i_col, int f_col, const int* pos, const int* slot, int T, int H, int D,
                              int Dv, int Pp, float qscale, float cap, hipStream_t st) {
  if (T < 1 || H < 1 || H > 65535 || D < 1 || Dv < 1 || Pp < Dv + 1 || !(cap > 0.f) || !qs || !vp || !log_alpha || !alpha || !mrun ||
      !mstate || !proj || !pos || !slot || q_col < 0 || v_col < 0 || i_col < 0 || f_col < 0 || ld < q_col + H * D ||
      ld < v_col + H * Dv || ld < i_col + H || ld < f_col + H)
    return UMB_EINVAL;
  hipLaunchKernelGGL(mlstm_step_kernel, dim3(T, H), dim3(256), 0, st, qs, vp, log_alpha, alpha, mrun, mstate, proj, ld, q_col, v_col,
                     i_col, f_col, pos, slot, H, D, Dv, Pp, qscale, cap);
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}
