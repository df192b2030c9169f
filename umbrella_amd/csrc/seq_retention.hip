// Retention: linear attention with ONE FIXED decay per head and neither softmax nor denominator,
//     S_t = decay_h S_(t-1) + k_t v_t^T        o_t = S_t^T q_t
// with rotary positions on q and k and a constant on k.  The recurrence itself is the linear scan of seq_gla.hip (token by
// token) or the chunked form of seq_ssd.hip (stretches), both with one decay per head; this file holds what surrounds it:
//   rope_scale   rotary positions of either pair layout on the first rot_dims features of a run of heads, times a constant
//                (one for the first heads of the run, another for the rest: q and k in one launch)
//   decay_fill   the per-head constants as the [T][H] decay rows (and their logarithms) the scans read
//   head_gate    every head's read-out over its root mean square (optionally first divided by a stabilised normaliser that
//                the scan carried as an extra value column), times an optional weight, times silu or sigmoid of a gate
//                column, times a constant, rounded for the output projection
// Angles are fp32 (position times a tabulated fp32 frequency, full-range sincosf); everything here is fp32.
#include "seq_common.h"

// layout 0: feature i pairs with i + rot_dims / 2 ("rotate half"); 1: feature 2i pairs with 2i + 1 (interleaved)
__global__ __launch_bounds__(256) void rope_scale_kernel(float* __restrict__ out, int ldo, const float* __restrict__ in, int ld,
                                                         const int* __restrict__ pos, const float* __restrict__ freq, int heads,
                                                         int D, int rot_dims, int layout, int heads_a, float scale_a,
                                                         float scale_b) {
  const int t = blockIdx.x, idx = blockIdx.y * 256 + threadIdx.x;
  if (idx >= heads * D) return;
  const int h = idx / D, d = idx - h * D;
  const float* src = in + (long)t * ld + (long)h * D;
  float v = src[d];
  if (d < rot_dims) {
    const int half = rot_dims >> 1;
    int i, other;
    bool first;
    if (layout == 0) { first = d < half; i = first ? d : d - half; other = first ? d + half : d - half; }
    else { first = (d & 1) == 0; i = d >> 1; other = d ^ 1; }
    float sn, cs;
    sincosf((float)pos[t] * freq[i], &sn, &cs);
    const float w = src[other];
    v = first ? v * cs - w * sn : v * cs + w * sn;
  }
  out[(long)t * ldo + idx] = v * (h < heads_a ? scale_a : scale_b);
}

__global__ __launch_bounds__(256) void decay_fill_kernel(float* __restrict__ alpha, float* __restrict__ log_alpha,
                                                         const float* __restrict__ decay, long n, int H) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const float a = decay[i % H];
  alpha[i] = a;
  if (log_alpha) log_alpha[i] = logf(a);
}

// one wave per (token, head).  o rows are [H][P] with the head's Dv read-outs first; den_col >= 0: column den_col holds
// n . q and the read-outs are first divided by max(|n . q|, exp(-m)) + 1e-6 (m = mrun[t][h]).
// w: null, [Dv] shared by the heads (w_stride 0) or [H Dv] (w_stride Dv).  gate_kind 0: silu, 1: sigmoid.
template <typename P>
__global__ __launch_bounds__(256) void head_gate_kernel(typename El<P>::type* __restrict__ out, int ldo, const float* __restrict__ o,
                                                        int Pc, int den_col, const float* __restrict__ mrun,
                                                        const float* __restrict__ proj, int ld, int g_col,
                                                        const typename El<P>::type* __restrict__ w, int w_stride, int gate_kind,
                                                        int T, int H, int Dv, float eps, float out_scale) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const long th = (long)blockIdx.x * 4 + wave;
  if (th >= (long)T * H) return;
  const int t = (int)(th / H), h = (int)(th % H);
  const float* orow = o + ((long)t * H + h) * Pc;
  float inv = 1.f;
  if (den_col >= 0) inv = 1.f / (fmaxf(fabsf(orow[den_col]), expf(-mrun[(long)t * H + h])) + 1e-6f);
  float ss = 0.f;
  for (int i = lane; i < Dv; i += 64) { const float v = orow[i] * inv; ss += v * v; }
  ss = wave_sum(ss);
  const float f = out_scale / sqrtf(ss / (float)Dv + eps);
  const float* gr = proj + (long)t * ld + g_col + (long)h * Dv;
  for (int i = lane; i < Dv; i += 64) {
    const float g = gr[i];
    const float gv = gate_kind == 0 ? siluf_(g) : 1.f / (1.f + expf(-g));
    const float wv = w ? ldf<P>(w + (long)h * w_stride + i) : 1.f;
    stf<P>(out + (long)t * ldo + (long)h * Dv + i, orow[i] * inv * f * wv * gv);
  }
}

extern "C" int umb_rope_scale(float* out, int ldo, const float* in, int ld, const int* pos, const float* freq, int T, int heads,
                              int D, int rot_dims, int layout, int heads_a, float scale_a, float scale_b, hipStream_t st) {
  if (T < 1 || heads < 1 || D < 1 || rot_dims < 0 || rot_dims > D || (rot_dims & 1) || (rot_dims && !freq) || layout < 0 ||
      layout > 1 || !out || !in || !pos || ldo < heads * D || ld < heads * D)
    return UMB_EINVAL;
  hipLaunchKernelGGL(rope_scale_kernel, dim3(T, (heads * D + 255) / 256), dim3(256), 0, st, out, ldo, in, ld, pos, freq, heads, D,
                     rot_dims, layout, heads_a, scale_a, scale_b);
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_decay_fill(float* alpha, float* log_alpha, const float* decay, int T, int H, hipStream_t st) {
  if (T < 1 || H < 1 || !alpha || !decay) return UMB_EINVAL;
  const long n = (long)T * H;
  hipLaunchKernelGGL(decay_fill_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, alpha, log_alpha, decay, n, H);
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_head_gate(void* out, int ldo, const float* o, int P_cols, int den_col, const float* mrun, const float* proj,
                             int ld, int g_col, const void* w, int w_per_head, int gate_kind, int T, int H, int Dv, float eps,
                             float out_scale, int dtype, hipStream_t st) {
  if (T < 1 || H < 1 || Dv < 1 || P_cols < Dv || den_col >= P_cols || (den_col >= 0 && (den_col < Dv || !mrun)) || !out || !o ||
      !proj || ldo < H * Dv || ld < g_col + H * Dv || g_col < 0 || gate_kind < 0 || gate_kind > 1)
    return UMB_EINVAL;
  const long th = (long)T * H;
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    hipLaunchKernelGGL(head_gate_kernel<P>, dim3((unsigned)((th + 3) / 4)), dim3(256), 0, st, (E*)out, ldo, o, P_cols, den_col, mrun,
                       proj, ld, g_col, (const E*)w, w_per_head ? Dv : 0, gate_kind, T, H, Dv, eps, out_scale);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}
