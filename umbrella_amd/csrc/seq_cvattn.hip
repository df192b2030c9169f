// Front end of a softmax-attention mixer whose projections pass a SHORT CAUSAL CONVOLUTION over time before anything else:
//     u_t[c] = sum_j w[c][j] raw_(t - taps + 1 + j)[c]          (zeros before the sequence's start; q, k and v channels alike)
//     q = rope(rms_norm_whole(u_q) * w_q)     k = rope(rms_norm_whole(u_k) * w_k)     v = u_v
// where the RMS norm runs over the WHOLE projection (all heads at once, plain weights of that size) and the rotary positions
// turn the first rot_dims features of every head (either pair layout, tabulated fp32 frequencies -- whatever frequency
// scaling a design has is in the table).  q goes out as fp32, k and v into the paged store.  The raw projections of the last
// taps - 1 positions are the sequence's state: a ring [slots][taps - 1][channels] fp32, position p in row p % (taps - 1); the
// ring is read here and refreshed afterwards (umb_ssd_conv_update; steps of one token per sequence refresh it here, by the thread
// that read it).  Taps are summed oldest first whatever their source.  The attention itself is seq_battn.hip.
// One workgroup per token; the convolved q | k row lives in LDS between the sum of squares and the rotation.  All fp32.
#include "seq_common.h"

constexpr int CVA_MAXT = 8;      // taps whose loads are issued together (more: a plain loop)

// NT threads per token: 256 when the step has many tokens, 1024 when it has few (a decoding step is a handful of workgroups
// that each walk thousands of channels).  The taps of a channel are loaded unconditionally from clamped addresses -- the
// same step's rows or the ring -- before any is used: a load that sits behind a per-tap branch waits for its own round trip.
template <typename P, int NT>
__global__ __launch_bounds__(NT) void cva_prep_kernel(float* __restrict__ q, UmbPagedKV kv, const float* __restrict__ proj, int ld,
                                                      const typename El<P>::type* __restrict__ conv_w, float* __restrict__ conv_state,
                                                      const typename El<P>::type* __restrict__ w_q,
                                                      const typename El<P>::type* __restrict__ w_k, const int* __restrict__ pos,
                                                      const int* __restrict__ slot_, const float* __restrict__ freq, int H, int G,
                                                      int D, int E, int taps, int rot_dims, int layout, int update, float eps) {
  typedef typename El<P>::type El_;
  extern __shared__ float row_s[];                      // [H D + G D]
  __shared__ float red[NT / 64];
  const int t = blockIdx.x, p = pos[t], slot = slot_[t];
  const int nq = H * D, nk = G * D, C = nq + nk + G * E;
  // where tap j (looking d = taps - 1 - j positions back) comes from: bit j of `same`: a row of this step; of `live`: not
  // before the sequence's start
  unsigned same = 0, live = 0;
  if (conv_w && taps <= CVA_MAXT) {
    for (int j = 0; j < taps; ++j) {
      const int d = taps - 1 - j;
      if (d <= p) {
        live |= 1u << j;
        if (d == 0 || (t - d >= 0 && slot_[t - d] == slot)) same |= 1u << j;
      }
    }
  }
  const long ring0 = (long)slot * (taps - 1);
  float ssq = 0.f, ssk = 0.f;
  // nothing is stored to global fp32 memory inside this loop (the ring is refreshed after it), so the loads of several
  // channels overlap
#pragma unroll 4
  for (int c = threadIdx.x; c < C; c += NT) {
    float acc;
    if (conv_w && taps <= CVA_MAXT) {
      float in[CVA_MAXT], wv[CVA_MAXT];
#pragma unroll
      for (int j = 0; j < CVA_MAXT; ++j) {
        if (j < taps) {
          const int d = taps - 1 - j;
          const bool sm = (same >> j) & 1u, lv = (live >> j) & 1u;
          const float* src = (sm || !lv) ? proj + (long)(t - (sm ? d : 0)) * ld + c
                                         : conv_state + (ring0 + (p - d) % (taps - 1)) * C + c;
          in[j] = *src;
          wv[j] = ldf<P>(conv_w + (long)c * taps + j);
        }
      }
      acc = 0.f;
#pragma unroll
      for (int j = 0; j < CVA_MAXT; ++j)
        if (j < taps) acc += wv[j] * (((live >> j) & 1u) ? in[j] : 0.f);      // oldest tap first
    } else if (conv_w) {
      acc = 0.f;
      for (int j = 0; j < taps; ++j) {
        const int d = taps - 1 - j;                       // how far back the tap looks
        float in = 0.f;
        if (d <= p) {
          if (d == 0 || (t - d >= 0 && slot_[t - d] == slot)) in = proj[(long)(t - d) * ld + c];        // same step
          else in = conv_state[(ring0 + (p - d) % (taps - 1)) * C + c];
        }
        acc += ldf<P>(conv_w + (long)c * taps + j) * in;
      }
    } else {
      acc = proj[(long)t * ld + c];
    }
    if (c < nq) { row_s[c] = acc; ssq += acc * acc; }
    else if (c < nq + nk) { row_s[c] = acc; ssk += acc * acc; }
    else {
      const int j = c - nq - nk, g = j / E, e = j - g * E;
      stf<P>(reinterpret_cast<El_*>(kv.v) + pkv_tok(kv, slot, p, g, G, E) + e, acc);
    }
  }
  // steps of one token per sequence: the ring row of this position held the oldest tap, which the same thread has read above
  if (update && conv_w && taps > 1)
    for (int c = threadIdx.x; c < C; c += NT) conv_state[(ring0 + p % (taps - 1)) * C + c] = proj[(long)t * ld + c];
  ssq = block_sum<NT>(ssq, red);
  ssk = block_sum<NT>(ssk, red);                         // its first barrier comes after every read of the first sum
  const float fq = 1.f / sqrtf(ssq / (float)nq + eps), fk = 1.f / sqrtf(ssk / (float)nk + eps);
  const int half = rot_dims >> 1;
  for (int c = threadIdx.x; c < nq + nk; c += NT) {
    const bool is_q = c < nq;
    const int cc = is_q ? c : c - nq;
    const int h = cc / D, d = cc - h * D;
    const float f = is_q ? fq : fk;
    const El_* w = is_q ? w_q : w_k;
    float v = row_s[c] * f * (w ? ldf<P>(w + cc) : 1.f);
    if (d < rot_dims) {
      int i, other;
      bool first;
      if (layout == 0) { first = d < half; i = first ? d : d - half; other = first ? d + half : d - half; }
      else { first = (d & 1) == 0; i = d >> 1; other = d ^ 1; }
      const int oc = c - d + other;
      const float u = row_s[oc] * f * (w ? ldf<P>(w + cc - d + other) : 1.f);
      float sn, cs;
      sincosf((float)p * freq[i], &sn, &cs);
      v = first ? v * cs - u * sn : v * cs + u * sn;
    }
    if (is_q) q[(long)t * nq + cc] = v;
    else stf<P>(reinterpret_cast<El_*>(kv.k) + pkv_tok(kv, slot, p, h, G, D) + d, v);
  }
}

extern "C" int umb_cva_prep(float* q, const UmbPagedKV* kv, const float* proj, int ld, const void* conv_w, float* conv_state,
                            const void* w_q, const void* w_k, const int* pos, const int* slot, const float* freq, int T, int H, int G,
                            int D, int E, int taps, int rot_dims, int layout, int update_state, float eps, int dtype,
                            hipStream_t st) {
  if (T < 1 || H < 1 || G < 1 || H % G || D < 1 || E < 1 || taps < 1 || rot_dims < 0 || rot_dims > D || (rot_dims & 1) ||
      (rot_dims && !freq) || layout < 0 || layout > 1 || !q || !kv || !kv->k || !kv->v || !kv->pages || kv->page < 1 || !proj ||
      !pos || !slot || ld < H * D + G * D + G * E || (conv_w && taps > 1 && !conv_state))
    return UMB_EINVAL;
  const size_t lds = (size_t)(H + G) * D * sizeof(float);
  if (lds > 160 * 1024 - 64) return UMB_EINVAL;
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type El_;
    if (T <= 64) {
      if (ensure_dynamic_lds<cva_prep_kernel<P, 1024>>(lds) != UMB_OK) return UMB_EHIP;
      hipLaunchKernelGGL((cva_prep_kernel<P, 1024>), dim3(T), dim3(1024), lds, st, q, *kv, proj, ld, (const El_*)conv_w, conv_state,
                         (const El_*)w_q, (const El_*)w_k, pos, slot, freq, H, G, D, E, taps, rot_dims, layout, update_state, eps);
    } else {
      if (ensure_dynamic_lds<cva_prep_kernel<P, 256>>(lds) != UMB_OK) return UMB_EHIP;
      hipLaunchKernelGGL((cva_prep_kernel<P, 256>), dim3(T), dim3(256), lds, st, q, *kv, proj, ld, (const El_*)conv_w, conv_state,
                         (const El_*)w_q, (const El_*)w_k, pos, slot, freq, H, G, D, E, taps, rot_dims, layout, update_state, eps);
    }
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}
