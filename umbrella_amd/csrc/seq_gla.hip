// Gated linear attention: a [D][Dv] matrix state per (sequence, head), decayed per key channel and updated by an outer
// product at every token,
//     S_t = diag(alpha_t) S_(t-1) + k_t v_t^T        o_t = S_t^T q_t
// with alpha_t = sigmoid(W_a2 (W_a1 h_t) + b)^(1/tau) in (0, 1).  Everything here is fp32: the decay and its logarithm, the
// state, the products that enter it and the read-out.  The state lives in a slot array [slots][H][D][Dv] and is carried from
// step to step; a sequence whose first row is at position 0 starts from zero whatever its slot held before.
//
// scan kernel: one WAVE owns four value columns of one (sequence, head): lane (r = lane % 16, c = lane / 16) keeps NR
// consecutive rows (r NR ...) of column c in registers, so the update is register-local and the read-out sum over rows is a
// butterfly inside 16 lanes, and the order of every sum is fixed by (D) alone -- a token's output never depends on how the
// sequence was cut into steps.  The token loop is the only serial dimension; its inputs are independent of the recurrence and
// are staged ahead through LDS in chunks of 16 tokens.
#include "seq_common.h"
#include <type_traits>

template <typename P>
__global__ __launch_bounds__(256) void gla_decay_kernel(float* __restrict__ alpha, const float* __restrict__ proj, int ld,
                                                        int a_col, const typename El<P>::type* __restrict__ w_a2,
                                                        const typename El<P>::type* __restrict__ b_a2, int HD, int rank,
                                                        float inv_tau) {
  extern __shared__ float a_s[];
  const int t = blockIdx.x;
  for (int i = threadIdx.x; i < rank; i += 256) a_s[i] = proj[(long)t * ld + a_col + i];
  __syncthreads();
  for (int n = blockIdx.y * 256 + threadIdx.x; n < HD; n += gridDim.y * 256) {
    const typename El<P>::type* wr = w_a2 + (long)n * rank;
    float z = 0.f;
    for (int i = 0; i < rank; ++i) z += ldf<P>(wr + i) * a_s[i];
    if (b_a2) z += ldf<P>(b_a2 + n);
    alpha[(long)t * HD + n] = expf(log_sigmoidf_(z) * inv_tau);
  }
}

constexpr int GLA_MAXR = 16;     // rows per lane: D <= 256
constexpr int GLA_TC = 16;       // tokens per staged chunk
constexpr int GLA_COLS = 16;     // value columns per workgroup (4 per wave)

// Workgroup = (sequence, head, 16 value columns), 4 waves of 4 columns.  The token loop is serial, so its inputs must not
// cost a memory round trip per token: chunks of 16 tokens (alpha, k, q rows of the head and the 16 v columns) are staged
// through a double-buffered LDS tile -- the global loads of chunk c + 1 are in flight while chunk c is consumed from LDS.
// V4: D, Dv and the row stride of proj are multiples of 4 -> the staging moves 16-byte pieces (a quarter of the address
// arithmetic, which is what this issue-bound kernel spends its time on).
// Operand placement is general: q and k rows hold groups of D shared by `hpg` consecutive heads each (1: a group per head),
// and the decay is per key channel (alpha [T][H D]) or, with aph, one number per head (alpha [T][H]) that fills the staged
// row -- the state-space layers with a scalar decay per head run on the same kernel.
template <int NR, bool V4>
__global__ __launch_bounds__(256) void gla_scan_kernel(float* __restrict__ o, float* __restrict__ state,
                                                       const float* __restrict__ qp, int ldq, const float* __restrict__ kp,
                                                       int ldk, const float* __restrict__ vp, int ldv,
                                                       const float* __restrict__ alpha, int aph, int hpg,
                                                       const int* __restrict__ seq_slot, const int* __restrict__ seq_row0,
                                                       const int* __restrict__ seq_pos0, const int* __restrict__ seq_len, int H,
                                                       int D, int Dv, float qscale) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  constexpr int VW = V4 ? 4 : 1;                        // floats per staged piece
  constexpr int STG = (3 * NR + 1 + VW - 1) / VW;       // staged pieces per thread: TC (3 D + 16) / 256 <= 3 NR + 1 floats
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 15;
  const int cbase = blockIdx.x * GLA_COLS, cl = wave * 4 + (lane >> 4), c = cbase + cl;
  const int h = blockIdx.y, b = blockIdx.z, hq = h / hpg;
  const int n = seq_len[b];
  if (n <= 0) return;
  const bool c_ok = c < Dv;
  const int slot = seq_slot[b], row0 = seq_row0[b];
  float* sp = state + (((long)slot * H + h) * D) * Dv + (c_ok ? c : 0);
  float S[NR];
  const bool fresh = seq_pos0[b] == 0;
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int d = r * NR + i;
    S[i] = (!fresh && c_ok && d < D) ? sp[(long)d * Dv] : 0.f;
  }
  const int HD = H * D, rowlen = 3 * D + GLA_COLS, chunk = GLA_TC * rowlen;
  const int nch = (n + GLA_TC - 1) / GLA_TC;
  typedef typename std::conditional<V4, f32x4, float>::type piece;
  piece stage[STG];
  const int rowp = rowlen / VW, chunkp = chunk / VW;    // in pieces
  // chunk ch -> registers.  Every load is unconditional and lands on a valid address (indices are clamped): loads that sit in
  // divergent branches would each wait for their own round trip.  What a clamped load brings is never used: tokens past the
  // sequence are not consumed, columns past Dv are not written, indices past the chunk are not stashed.
  const int tt0 = tid / rowp, ci0 = (tid - tt0 * rowp) * VW;
  auto fetch = [&](int ch) {
    int tt = tt0, ci = ci0;                             // (token, column) of staged piece e * 256 + tid, kept incrementally
#pragma unroll
    for (int e = 0; e < STG; ++e) {
      if (e) {
        ci += 256 * VW;
        while (ci >= rowlen) { ci -= rowlen; ++tt; }
        if (tt >= GLA_TC) { tt = GLA_TC - 1; ci = rowlen - VW; }     // past the chunk: any valid address
      }
      int t = ch * GLA_TC + tt;
      t = t < n ? t : n - 1;
      const long row = row0 + t;
      int vc = cbase + ci - 3 * D;
      vc = vc + VW <= Dv ? vc : Dv - VW;
      const bool is_a = ci < D;
      const float* src = (is_a && !aph) ? alpha + row * HD + (long)h * D + ci
                       : ci < 2 * D ? kp + row * ldk + (long)hq * D + (is_a ? ci : ci - D)
                       : ci < 3 * D ? qp + row * ldq + (long)hq * D + (ci - 2 * D)
                                    : vp + row * ldv + (long)h * Dv + vc;
      stage[e] = *reinterpret_cast<const piece*>(src);
      if (aph) {                                        // uniform: one decay per head fills the alpha part of the row
        const float a = alpha[row * H + h];
        if (is_a) {
          if constexpr (V4) stage[e] = piece{a, a, a, a};
          else stage[e] = a;
        }
      }
    }
  };
  auto stash = [&](float* buf) {
#pragma unroll
    for (int e = 0; e < STG; ++e) {
      const int idx = e * 256 + tid;
      if (idx < chunkp) reinterpret_cast<piece*>(buf)[idx] = stage[e];
    }
  };
  fetch(0);
  stash(lds);
  __syncthreads();
  for (int ch = 0; ch < nch; ++ch) {
    const float* buf = lds + (ch & 1) * chunk;
    if (ch + 1 < nch) fetch(ch + 1);
    const int cnt = n - ch * GLA_TC < GLA_TC ? n - ch * GLA_TC : GLA_TC;
    float pt[GLA_TC];                                   // this lane's share (its rows) of every token's read-out
#pragma unroll
    for (int tt = 0; tt < GLA_TC; ++tt) {
      float acc = 0.f;
      if (tt < cnt) {
        const float* row = buf + tt * rowlen;
        const float v = row[3 * D + cl];
        float al[NR], kk[NR], qq[NR];
        bool got = false;
        if constexpr (NR % 4 == 0) {
          if ((D & 3) == 0) {                           // 16-byte LDS reads of the lane's NR consecutive rows
#pragma unroll
            for (int i = 0; i < NR; i += 4) {
              const f32x4 a4 = *reinterpret_cast<const f32x4*>(row + r * NR + i);
              const f32x4 k4 = *reinterpret_cast<const f32x4*>(row + D + r * NR + i);
              const f32x4 q4 = *reinterpret_cast<const f32x4*>(row + 2 * D + r * NR + i);
#pragma unroll
              for (int e = 0; e < 4; ++e) { al[i + e] = a4[e]; kk[i + e] = k4[e]; qq[i + e] = q4[e]; }
            }
            got = true;
          }
        }
        if (!got) {
#pragma unroll
          for (int i = 0; i < NR; ++i) {
            const int d = r * NR + i;
            al[i] = row[d]; kk[i] = row[D + d]; qq[i] = row[2 * D + d];
          }
        }
#pragma unroll
        for (int i = 0; i < NR; ++i) {
          if (r * NR + i < D) {
            S[i] = al[i] * S[i] + kk[i] * v;
            acc += S[i] * qq[i];
          }
        }
      }
      pt[tt] = acc;
    }
    // sum over the 16 row lanes, all 16 tokens at once: a transposing butterfly (15 exchanges instead of 64).  At the step with
    // mask m a lane keeps the half of its values whose token bit m equals its own lane bit and hands the other half to its
    // partner; lane r ends up with the whole sum of token r.  Every token's sum has the same tree (pairs by 8, 4, 2, 1).
    float p8[8], p4[4], p2[2];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const bool up = r & 8;
      p8[j] = (up ? pt[j + 8] : pt[j]) + __shfl_xor(up ? pt[j] : pt[j + 8], 8, 64);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bool up = r & 4;
      p4[j] = (up ? p8[j + 4] : p8[j]) + __shfl_xor(up ? p8[j] : p8[j + 4], 4, 64);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const bool up = r & 2;
      p2[j] = (up ? p4[j + 2] : p4[j]) + __shfl_xor(up ? p4[j] : p4[j + 2], 2, 64);
    }
    const bool up1 = r & 1;
    const float mine = ((up1 ? p2[1] : p2[0]) + __shfl_xor(up1 ? p2[0] : p2[1], 1, 64)) * qscale;
    if (r < cnt && c_ok) o[(long)(row0 + ch * GLA_TC + r) * (H * Dv) + (long)h * Dv + c] = mine;
    if (ch + 1 < nch) stash(lds + ((ch + 1) & 1) * chunk);
    __syncthreads();
  }
  if (c_ok) {
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int d = r * NR + i;
      if (d < D) sp[(long)d * Dv] = S[i];
    }
  }
}

template <typename P>
__global__ __launch_bounds__(256) void gla_gate_kernel(typename El<P>::type* __restrict__ out, const float* __restrict__ o,
                                                       const float* __restrict__ proj, int ld, int g_col,
                                                       const typename El<P>::type* __restrict__ w, int T, int H, int Dv, float eps) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const long th = (long)blockIdx.x * 4 + wave;           // (token, head)
  if (th >= (long)T * H) return;
  const int t = (int)(th / H), h = (int)(th % H);
  const float* orow = o + (long)t * H * Dv + (long)h * Dv;
  float ss = 0.f;
  for (int i = lane; i < Dv; i += 64) { const float v = orow[i]; ss += v * v; }
  ss = wave_sum(ss);
  const float f = 1.f / sqrtf(ss / (float)Dv + eps);
  const float* gr = proj + (long)t * ld + g_col + (long)h * Dv;
  for (int i = lane; i < Dv; i += 64)
    stf<P>(out + (long)t * H * Dv + (long)h * Dv + i, orow[i] * f * ldf<P>(w + i) * siluf_(gr[i]));
}

extern "C" int umb_gla_decay(float* alpha, const float* proj, int ld, int a_col, const void* w_a2, const void* b_a2, int T, int HD,
                             int rank, float tau, int dtype, hipStream_t st) {
  if (T < 1 || HD < 1 || rank < 1 || rank > 8192 || !(tau > 0.f) || !alpha || !proj || !w_a2) return UMB_EINVAL;
  const int gy = (HD + 255) / 256 > 64 ? 64 : (HD + 255) / 256;
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    hipLaunchKernelGGL(gla_decay_kernel<P>, dim3(T, gy), dim3(256), rank * sizeof(float), st, alpha, proj, ld, a_col,
                       (const E*)w_a2, (const E*)b_a2, HD, rank, 1.f / tau);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_lin_scan(float* o, float* state, const float* q, int ldq, const float* k, int ldk, const float* v, int ldv,
                            const float* alpha, int alpha_per_head, int qk_heads, const int* seq_slot, const int* seq_row0,
                            const int* seq_pos0, const int* seq_len, int B, int H, int D, int Dv, float qscale, hipStream_t st) {
  if (B < 1 || H < 1 || D < 1 || D > 16 * GLA_MAXR || Dv < 1 || qk_heads < 1 || H % qk_heads || !o || !state || !q || !k || !v ||
      !alpha || ldq < qk_heads * D || ldk < qk_heads * D || ldv < H * Dv)
    return UMB_EINVAL;
  const dim3 grid((Dv + GLA_COLS - 1) / GLA_COLS, H, B);
  const int nr = (D + 15) / 16, aph = alpha_per_head ? 1 : 0, hpg = H / qk_heads;
  const size_t lds = 2 * (size_t)GLA_TC * (3 * D + GLA_COLS) * sizeof(float);
  const bool v4 = D % 4 == 0 && Dv % 4 == 0 && ldq % 4 == 0 && ldk % 4 == 0 && ldv % 4 == 0 &&
                  ((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (aph ? 0 : (uintptr_t)alpha)) % 16 == 0;
#define GLA_SCAN_LAUNCH(NR, V4)                                                                                           \
  do {                                                                                                                    \
    if (ensure_dynamic_lds<gla_scan_kernel<NR, V4>>(lds) != UMB_OK) return UMB_EHIP;                                      \
    hipLaunchKernelGGL((gla_scan_kernel<NR, V4>), grid, dim3(256), lds, st, o, state, q, ldq, k, ldk, v, ldv, alpha, aph, \
                       hpg, seq_slot, seq_row0, seq_pos0, seq_len, H, D, Dv, qscale);                                      \
  } while (0)
#define GLA_SCAN_CASE(NR)                                                                                                 \
  case NR:                                                                                                                \
    if (v4) GLA_SCAN_LAUNCH(NR, true); else GLA_SCAN_LAUNCH(NR, false);                                                   \
    break;
  switch (nr) {
    GLA_SCAN_CASE(1) GLA_SCAN_CASE(2) GLA_SCAN_CASE(3) GLA_SCAN_CASE(4) GLA_SCAN_CASE(5) GLA_SCAN_CASE(6) GLA_SCAN_CASE(7)
    GLA_SCAN_CASE(8) GLA_SCAN_CASE(9) GLA_SCAN_CASE(10) GLA_SCAN_CASE(11) GLA_SCAN_CASE(12) GLA_SCAN_CASE(13)
    GLA_SCAN_CASE(14) GLA_SCAN_CASE(15) GLA_SCAN_CASE(16)
    default: return UMB_EINVAL;
  }
#undef GLA_SCAN_CASE
#undef GLA_SCAN_LAUNCH
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_gla_scan(float* o, float* state, const float* proj, int ld, const float* alpha, const int* seq_slot,
                            const int* seq_row0, const int* seq_pos0, const int* seq_len, int B, int H, int D, int Dv,
                            float qscale, hipStream_t st) {
  if (!proj || H < 1 || D < 1 || Dv < 1 || ld < 2 * H * D + H * Dv) return UMB_EINVAL;
  return umb_lin_scan(o, state, proj, ld, proj + (long)H * D, ld, proj + 2L * H * D, ld, alpha, 0, H, seq_slot, seq_row0, seq_pos0,
                      seq_len, B, H, D, Dv, qscale, st);
}

extern "C" int umb_gla_gate(void* out, const float* o, const float* proj, int ld, int g_col, const void* w, int T, int H, int Dv,
                            float eps, int dtype, hipStream_t st) {
  if (T < 1 || H < 1 || Dv < 1 || !out || !o || !proj || !w) return UMB_EINVAL;
  const long th = (long)T * H;
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    hipLaunchKernelGGL(gla_gate_kernel<P>, dim3((unsigned)((th + 3) / 4)), dim3(256), 0, st, (E*)out, o, proj, ld, g_col,
                       (const E*)w, T, H, Dv, eps);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}
