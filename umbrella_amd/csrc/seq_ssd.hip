// Selective state-space layer with a scalar decay per head (the "state-space duality" form): per head a [N][Dv] fp32 state
//     S_t = exp(-exp(A_log) dt_t) S_(t-1) + dt_t B_t x_t^T          y_t = S_t^T C_t + D x_t
// where x, B, C come out of one input projection through a short causal convolution per channel and silu, dt = softplus(dt +
// bias) per head, and B / C are shared by the heads of a group.  The recurrence is the linear scan of seq_gla.hip with
// k = B, v = dt x, q = C and one decay per head; this file holds what surrounds it:
//   prep         convolution (inputs of earlier steps from the sequence's state ring) + bias + silu, dt, decay, dt x
//   conv_update  the step's last taps - 1 raw inputs into the state ring (after prep has read it); steps of one token per
//                sequence do this inside prep
//   gate         y = o + D x, times silu(z), unit RMS in equal parts of the row, times a weight and a constant, rounded
// Everything is fp32 (the convolution too); the only rounding is the gated, normed output that feeds the output projection.
// The convolution sums its taps oldest first whatever their source, so a position's value does not depend on where a prompt
// was cut.
#include "seq_common.h"

__device__ __forceinline__ float softplusf_(float z) { return fmaxf(z, 0.f) + log1pf(expf(-fabsf(z))); }

template <typename P>
__global__ __launch_bounds__(256) void ssd_prep_kernel(float* __restrict__ sx, int lds, float* __restrict__ alpha,
                                                       float* __restrict__ log_alpha, const float* __restrict__ proj, int ld, int col0,
                                                       const typename El<P>::type* __restrict__ conv_w,
                                                       const typename El<P>::type* __restrict__ conv_b,
                                                       float* __restrict__ conv_state, const float* __restrict__ dt_bias,
                                                       const float* __restrict__ a_log, const int* __restrict__ pos,
                                                       const int* __restrict__ slot_, int H, int Dv, int G, int N, int taps,
                                                       int update) {
  const int t = blockIdx.x, idx = blockIdx.y * 256 + threadIdx.x;
  const int inner = H * Dv, C = inner + 2 * G * N;
  const float* pr = proj + (long)t * ld + col0;
  const int dt_col = 2 * inner + 2 * G * N;
  if (idx >= C) {                                        // one thread per head: the decay
    const int h = idx - C;
    if (h < H) {
      const float la = -expf(a_log[h]) * softplusf_(pr[dt_col + h] + dt_bias[h]);
      alpha[(long)t * H + h] = expf(la);
      if (log_alpha) log_alpha[(long)t * H + h] = la;
    }
    return;
  }
  const int p = pos[t], slot = slot_[t];
  float acc = conv_b ? ldf<P>(conv_b + idx) : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int d = taps - 1 - j;                           // how far back the tap looks
    float in = 0.f;
    if (d <= p) {
      if (d == 0 || (t - d >= 0 && slot_[t - d] == slot)) in = proj[(long)(t - d) * ld + col0 + inner + idx];   // same step
      else in = conv_state[((long)slot * (taps - 1) + (p - d) % (taps - 1)) * C + idx];
    }
    acc += ldf<P>(conv_w + (long)idx * taps + j) * in;
  }
  // steps of one token per sequence: this thread is the only one that touches the ring of (slot, channel); the row of the
  // token's position held the oldest tap, which has been read above
  if (update && taps > 1) conv_state[((long)slot * (taps - 1) + p % (taps - 1)) * C + idx] = proj[(long)t * ld + col0 + inner + idx];
  const float v = siluf_(acc);
  if (idx < inner) {
    const int h = idx / Dv;
    sx[(long)t * lds + idx] = softplusf_(pr[dt_col + h] + dt_bias[h]) * v;
    sx[(long)t * lds + C + idx] = v;
  } else {
    sx[(long)t * lds + idx] = v;
  }
}

__global__ __launch_bounds__(256) void ssd_conv_update_kernel(float* __restrict__ conv_state, const float* __restrict__ proj, int ld,
                                                              int col0, const int* __restrict__ seq_slot,
                                                              const int* __restrict__ seq_row0, const int* __restrict__ seq_pos0,
                                                              const int* __restrict__ seq_len, int C, int taps) {
  const int c = blockIdx.x * 256 + threadIdx.x, b = blockIdx.y;
  if (c >= C) return;
  const int n = seq_len[b], keep = taps - 1;
  const int first = n > keep ? n - keep : 0;
  for (int i = first; i < n; ++i) {
    const int p = seq_pos0[b] + i;
    conv_state[((long)seq_slot[b] * keep + p % keep) * C + c] = proj[(long)(seq_row0[b] + i) * ld + col0 + c];
  }
}

template <typename P>
__global__ __launch_bounds__(256) void ssd_gate_kernel(typename El<P>::type* __restrict__ out, int ldo, const float* __restrict__ o,
                                                       const float* __restrict__ sx, int lds, int x_col,
                                                       const float* __restrict__ proj, int ld, int z_col,
                                                       const float* __restrict__ d_skip, const typename El<P>::type* __restrict__ w,
                                                       int H, int Dv, int norm_groups, float eps, float out_scale) {
  __shared__ float red[8];
  const int t = blockIdx.x, grp = blockIdx.y, inner = H * Dv, gs = inner / norm_groups;
  auto value = [&](int i) -> float {
    const float y = o[(long)t * inner + i] + (d_skip ? d_skip[i / Dv] : 0.f) * sx[(long)t * lds + x_col + i];
    return y * siluf_(proj[(long)t * ld + z_col + i]);
  };
  float ss = 0.f;
  for (int k = threadIdx.x; k < gs; k += 256) { const float v = value(grp * gs + k); ss += v * v; }
  ss = block_sum<256>(ss, red);
  const float f = out_scale / sqrtf(ss / (float)gs + eps);
  for (int k = threadIdx.x; k < gs; k += 256) {
    const int i = grp * gs + k;
    stf<P>(out + (long)t * ldo + i, value(i) * f * ldf<P>(w + i));
  }
}

extern "C" int umb_ssd_prep(float* sx, int lds, float* alpha, float* log_alpha, const float* proj, int ld, int col0, const void* conv_w,
                            const void* conv_b, float* conv_state, const float* dt_bias, const float* a_log, const int* pos,
                            const int* slot, int T, int H, int Dv, int G, int N, int taps, int update_state, int dtype,
                            hipStream_t st) {
  if (T < 1 || H < 1 || Dv < 1 || G < 1 || N < 1 || H % G || taps < 1 || !sx || !alpha || !proj || !conv_w || !dt_bias ||
      !a_log || !pos || !slot || (taps > 1 && !conv_state))
    return UMB_EINVAL;
  const int inner = H * Dv, C = inner + 2 * G * N;
  if (lds < C + inner || col0 < 0 || ld < col0 + 2 * inner + 2 * G * N + H) return UMB_EINVAL;
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    hipLaunchKernelGGL(ssd_prep_kernel<P>, dim3(T, (C + H + 255) / 256), dim3(256), 0, st, sx, lds, alpha, log_alpha, proj, ld, col0,
                       (const E*)conv_w, (const E*)conv_b, conv_state, dt_bias, a_log, pos, slot, H, Dv, G, N, taps, update_state);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_ssd_conv_update(float* conv_state, const float* proj, int ld, int col0, const int* seq_slot,
                                   const int* seq_row0, const int* seq_pos0, const int* seq_len, int B, int C, int taps,
                                   hipStream_t st) {
  if (taps <= 1) return UMB_OK;
  if (B < 1 || B > 65535 || C < 1 || !conv_state || !proj || !seq_slot || !seq_row0 || !seq_pos0 || !seq_len || col0 < 0 ||
      ld < col0 + C)
    return UMB_EINVAL;
  hipLaunchKernelGGL(ssd_conv_update_kernel, dim3((C + 255) / 256, B), dim3(256), 0, st, conv_state, proj, ld, col0, seq_slot,
                     seq_row0, seq_pos0, seq_len, C, taps);
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_ssd_gate(void* out, int ldo, const float* o, const float* sx, int lds, int x_col, const float* proj, int ld,
                            int z_col, const float* d_skip, const void* w, int T, int H, int Dv, int norm_groups, float eps,
                            float out_scale, int dtype, hipStream_t st) {
  if (T < 1 || H < 1 || Dv < 1 || norm_groups < 1 || norm_groups > 65535 || (H * Dv) % norm_groups || !out || !o || !sx || !proj ||
      !w || ldo < H * Dv)
    return UMB_EINVAL;
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    hipLaunchKernelGGL(ssd_gate_kernel<P>, dim3(T, norm_groups), dim3(256), 0, st, (E*)out, ldo, o, sx, lds, x_col, proj, ld, z_col,
                       d_skip, (const E*)w, H, Dv, norm_groups, eps, out_scale);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

// ---- the recurrence in chunks, for stretches of many tokens.  With ONE decay per head the recurrence of a chunk of Q tokens is
// a handful of small matrix products (l_t = log a_t, c_t = l_1 + .. + l_t inside the chunk):
//     S_end = exp(c_Q) S_start + sum_s exp(c_Q - c_s) k_s v_s^T                                   (chunk summary)
//     o_t   = exp(c_t) S_start^T q_t + sum_{s <= t} exp(c_t - c_s) (q_t . k_s) v_s                 (read-out)
// so all chunks of all sequences run side by side: (1) every chunk's summary from S_start = 0, (2) a pass over the chunks of a
// (sequence, head) that turns summaries into start states and leaves the final state in the slot, (3) every chunk's read-outs.
// Everything is fp32 on the vector pipe; exponents are of non-positive numbers.  Which tokens share a chunk depends on their place
// in the step only; against the token-by-token scan the sums are associated differently: equal to fp32 rounding.
constexpr int SC_Q = 64;         // tokens per chunk
constexpr int SC_PS = 64;        // value columns per workgroup of the read-out kernel (16 per thread quad)

struct ScArgs {
  const float *q, *k, *v, *la;   // rows [T][ld*]: q / k groups of N, v heads of P, la [T][H] log decays
  int ldq, ldk, ldv, H, hpg, N, P, max_chunks;
  const int *seq_slot, *seq_row0, *seq_pos0, *seq_len;
};

// inclusive prefix sums of the chunk's log decays into cum[SC_Q] (tokens past the stretch add nothing); one wave.  The sums are
// kept in double: a decay between two tokens of a chunk is the exponential of a DIFFERENCE of two prefix sums, and with strong
// decays (logarithms of -10 and below) fp32 prefix sums of a few hundred would leave that difference good to 1e-5 only, where
// the token-by-token recurrence multiplies by every decay itself.
__device__ __forceinline__ void sc_cumsum(double* cum, const ScArgs& a, long row0, int cnt, int h) {
  const int lane = threadIdx.x;
  if (lane < 64) {
    double v = lane < cnt ? (double)a.la[(row0 + lane) * a.H + h] : 0.0;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const double u = __shfl_up(v, o, 64);
      if (lane >= o) v += u;
    }
    cum[lane] = v;
  }
}

// (1) chunk summaries: grid (value-column slices of 16, chunks, sequences x heads); thread n owns row n of the slice
__global__ __launch_bounds__(256) void ssd_chunk_state_kernel(float* __restrict__ sc, float* __restrict__ ac, ScArgs a) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  const int b = blockIdx.z / a.H, h = blockIdx.z % a.H, c = blockIdx.y, p0 = blockIdx.x * 16;
  const int len = a.seq_len[b], t0 = c * SC_Q;
  if (t0 >= len) return;
  const int cnt = len - t0 < SC_Q ? len - t0 : SC_Q, N = a.N, P = a.P;
  const long row0 = a.seq_row0[b] + t0;
  double* cum = reinterpret_cast<double*>(sm);   // [64] doubles
  float* kw = sm + 128;                    // [Q][N]: k_s * exp(c_Q - c_s)
  float* vs = kw + SC_Q * N;               // [Q][16]
  sc_cumsum(cum, a, row0, cnt, h);
  __syncthreads();
  const double cend = cum[SC_Q - 1];
  const int g = h / a.hpg;
  for (int i = threadIdx.x; i < SC_Q * N; i += 256) {
    const int s = i / N, n = i % N;
    kw[i] = s < cnt ? a.k[(row0 + s) * a.ldk + (long)g * N + n] * expf((float)(cend - cum[s])) : 0.f;
  }
  for (int i = threadIdx.x; i < SC_Q * 16; i += 256) {
    const int s = i >> 4, p = p0 + (i & 15);
    vs[i] = (s < cnt && p < P) ? a.v[(row0 + s) * a.ldv + (long)h * P + p] : 0.f;
  }
  __syncthreads();
  const int n = threadIdx.x;
  if (n < N) {
    float acc[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[j] = 0.f;
    for (int s = 0; s < cnt; ++s) {
      const float kv = kw[s * N + n];
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[j] += kv * vs[s * 16 + j];
    }
    float* dst = sc + ((((long)b * a.H + h) * a.max_chunks + c) * N + n) * P + p0;
#pragma unroll
    for (int j = 0; j < 16; ++j)
      if (p0 + j < P) dst[j] = acc[j];
  }
  if (threadIdx.x == 0 && blockIdx.x == 0) ac[((long)b * a.H + h) * a.max_chunks + c] = expf((float)cend);
}

// (2) start states: thread per state element of a (sequence, head), chunks in order; sc[c] becomes the START state of chunk c
__global__ __launch_bounds__(256) void ssd_chunk_pass_kernel(float* __restrict__ sc, const float* __restrict__ ac,
                                                             float* __restrict__ state, ScArgs a) {
  const int b = blockIdx.z, h = blockIdx.y;
  const long e = (long)blockIdx.x * 256 + threadIdx.x, NP = (long)a.N * a.P;
  if (e >= NP) return;
  const int len = a.seq_len[b], nch = (len + SC_Q - 1) / SC_Q;
  float* sp = state + (((long)a.seq_slot[b] * a.H + h) * NP) + e;
  float S = a.seq_pos0[b] == 0 ? 0.f : *sp;
  const long base = ((long)b * a.H + h) * a.max_chunks;
  for (int c = 0; c < nch; ++c) {
    float* x = sc + (base + c) * NP + e;
    const float add = *x;
    *x = S;
    S = ac[base + c] * S + add;
  }
  *sp = S;
}

// (3) read-outs: grid (value-column slices of SC_PS, chunks, sequences x heads); thread (t = tid / 4, quarter = tid % 4)
__global__ __launch_bounds__(256) void ssd_chunk_out_kernel(float* __restrict__ o, const float* __restrict__ sc, ScArgs a) {
  extern __shared__ __attribute__((aligned(16))) float sm[];
  const int b = blockIdx.z / a.H, h = blockIdx.z % a.H, c = blockIdx.y, p0 = blockIdx.x * SC_PS;
  const int len = a.seq_len[b], t0 = c * SC_Q;
  if (t0 >= len) return;
  const int cnt = len - t0 < SC_Q ? len - t0 : SC_Q, N = a.N, P = a.P, NL = N + 1;
  const long row0 = a.seq_row0[b] + t0;
  double* cum = reinterpret_cast<double*>(sm);   // [64] doubles
  float* qs = sm + 128;                    // [Q][N + 1]
  float* kt = qs + SC_Q * NL;              // [N][Q] keys transposed; later the start state [N][SC_PS]
  float* vs = kt + (N * SC_Q > N * SC_PS ? N * SC_Q : N * SC_PS);   // [Q][SC_PS]
  float* ms = vs + SC_Q * SC_PS;           // [Q][Q + 1]: decayed, masked scores
  sc_cumsum(cum, a, row0, cnt, h);
  const int g = h / a.hpg;
  for (int i = threadIdx.x; i < SC_Q * N; i += 256) {
    const int s = i / N, n = i % N;
    const bool ok = s < cnt;
    qs[s * NL + n] = ok ? a.q[(row0 + s) * a.ldq + (long)g * N + n] : 0.f;
    kt[n * SC_Q + s] = ok ? a.k[(row0 + s) * a.ldk + (long)g * N + n] : 0.f;
  }
  for (int i = threadIdx.x; i < SC_Q * SC_PS; i += 256) {
    const int s = i / SC_PS, p = p0 + i % SC_PS;
    vs[i] = (s < cnt && p < P) ? a.v[(row0 + s) * a.ldv + (long)h * P + p] : 0.f;
  }
  __syncthreads();
  const int t = threadIdx.x >> 2, qd = threadIdx.x & 3;
  float acc[16];
#pragma unroll
  for (int j = 0; j < 16; ++j) acc[j] = 0.f;
  // scores of token t against keys 16 qd .. 16 qd + 15
  for (int n = 0; n < N; ++n) {
    const float qv = qs[t * NL + n];
    const f32x4* kr = reinterpret_cast<const f32x4*>(kt + n * SC_Q + 16 * qd);
#pragma unroll
    for (int j4 = 0; j4 < 4; ++j4) {
      const f32x4 kk = kr[j4];
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[4 * j4 + e] += qv * kk[e];
    }
  }
  const double ct = cum[t];
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    const int s = 16 * qd + j;
    ms[t * (SC_Q + 1) + s] = s <= t ? acc[j] * expf((float)(ct - cum[s])) : 0.f;
  }
  __syncthreads();                          // scores are in ms, kt is free: bring in the chunk's start state
  const float* s0 = sc + ((((long)b * a.H + h) * a.max_chunks + c) * N) * P;
  for (int i = threadIdx.x; i < N * SC_PS; i += 256) {
    const int n = i / SC_PS, p = p0 + i % SC_PS;
    kt[i] = p < P ? s0[(long)n * P + p] : 0.f;
  }
  __syncthreads();
  float y[16], y0[16];
#pragma unroll
  for (int j = 0; j < 16; ++j) { y[j] = 0.f; y0[j] = 0.f; }
  for (int s = 0; s <= t; ++s) {
    const float mv = ms[t * (SC_Q + 1) + s];
    const f32x4* vr = reinterpret_cast<const f32x4*>(vs + s * SC_PS + 16 * qd);
#pragma unroll
    for (int j4 = 0; j4 < 4; ++j4) {
      const f32x4 vv = vr[j4];
#pragma unroll
      for (int e = 0; e < 4; ++e) y[4 * j4 + e] += mv * vv[e];
    }
  }
  for (int n = 0; n < N; ++n) {
    const float qv = qs[t * NL + n];
    const f32x4* sr = reinterpret_cast<const f32x4*>(kt + n * SC_PS + 16 * qd);
#pragma unroll
    for (int j4 = 0; j4 < 4; ++j4) {
      const f32x4 sv = sr[j4];
#pragma unroll
      for (int e = 0; e < 4; ++e) y0[4 * j4 + e] += qv * sv[e];
    }
  }
  if (t < cnt) {
    const float et = expf((float)ct);
    float* dst = o + (row0 + t) * ((long)a.H * P) + (long)h * P + p0 + 16 * qd;
#pragma unroll
    for (int j = 0; j < 16; ++j)
      if (p0 + 16 * qd + j < P) dst[j] = y[j] + et * y0[j];
  }
}

static inline size_t sc_out_lds(int N) {
  const size_t kt = (size_t)N * (SC_Q > SC_PS ? SC_Q : SC_PS);
  return (128 + (size_t)SC_Q * (N + 1) + kt + (size_t)SC_Q * SC_PS + (size_t)SC_Q * (SC_Q + 1)) * sizeof(float);
}

// floats of scratch the chunked form needs for a step of B stretches, the longest max_len tokens; 0: the shape is not covered
extern "C" long umb_ssd_scan_chunked_floats(int B, int max_len, int H, int N, int P) {
  if (B < 1 || max_len < 1 || H < 1 || N < 1 || N > 256 || P < 1 || sc_out_lds(N) > 160 * 1024) return 0;
  const long chunks = (max_len + SC_Q - 1) / SC_Q;
  return (long)B * H * chunks * ((long)N * P + 1);
}

extern "C" int umb_ssd_scan_chunked(float* o, float* state, const float* q, int ldq, const float* k, int ldk, const float* v, int ldv,
                                    const float* log_alpha, int qk_heads, const int* seq_slot, const int* seq_row0,
                                    const int* seq_pos0, const int* seq_len, int B, int max_len, int H, int N, int P, float* scratch,
                                    long scratch_floats, hipStream_t st) {
  const long need = umb_ssd_scan_chunked_floats(B, max_len, H, N, P);
  if (need == 0 || need > scratch_floats || !o || !state || !q || !k || !v || !log_alpha || !scratch || qk_heads < 1 || H % qk_heads ||
      !seq_slot || !seq_row0 || !seq_pos0 || !seq_len || (long)B * H > 65535 || ldq < qk_heads * N || ldk < qk_heads * N || ldv < H * P)
    return UMB_EINVAL;
  const int chunks = (max_len + SC_Q - 1) / SC_Q;
  if (chunks > 65535) return UMB_EINVAL;
  ScArgs a{q, k, v, log_alpha, ldq, ldk, ldv, H, H / qk_heads, N, P, chunks, seq_slot, seq_row0, seq_pos0, seq_len};
  float* sc = scratch;
  float* ac = scratch + (long)B * H * chunks * N * P;
  const size_t lds1 = (128 + (size_t)SC_Q * N + SC_Q * 16) * sizeof(float), lds3 = sc_out_lds(N);
  if (ensure_dynamic_lds<ssd_chunk_state_kernel>(lds1) != UMB_OK || ensure_dynamic_lds<ssd_chunk_out_kernel>(lds3) != UMB_OK)
    return UMB_EHIP;
  hipLaunchKernelGGL(ssd_chunk_state_kernel, dim3((P + 15) / 16, chunks, B * H), dim3(256), lds1, st, sc, ac, a);
  hipLaunchKernelGGL(ssd_chunk_pass_kernel, dim3((unsigned)(((long)N * P + 255) / 256), H, B), dim3(256), 0, st, sc, ac, state, a);
  hipLaunchKernelGGL(ssd_chunk_out_kernel, dim3((P + SC_PS - 1) / SC_PS, chunks, B * H), dim3(256), lds3, st, o, sc, a);
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}
