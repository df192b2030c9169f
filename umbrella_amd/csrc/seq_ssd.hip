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
                                                       const float* __restrict__ proj, int ld, int col0,
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
    if (h < H) alpha[(long)t * H + h] = expf(-expf(a_log[h]) * softplusf_(pr[dt_col + h] + dt_bias[h]));
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

extern "C" int umb_ssd_prep(float* sx, int lds, float* alpha, const float* proj, int ld, int col0, const void* conv_w,
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
    hipLaunchKernelGGL(ssd_prep_kernel<P>, dim3(T, (C + H + 255) / 256), dim3(256), 0, st, sx, lds, alpha, proj, ld, col0,
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
