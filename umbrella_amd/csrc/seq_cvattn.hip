// Front end of a softmax-attention mixer whose projections pass a SHORT CAUSAL CONVOLUTION over time before anything else:
//     u_t[c] = sum_j w[c][j] raw_(t - taps + 1 + j)[c]          (zeros before the sequence's start; q, k and v channels alike)
//     q = rope(rms_norm_whole(u_q) * w_q)     k = rope(rms_norm_whole(u_k) * w_k)     v = u_v
// where the RMS norm runs over the WHOLE projection (all heads at once, plain weights of that size) and the rotary positions
// turn the first rot_dims features of every head (either pair layout, tabulated fp32 frequencies -- whatever frequency
// scaling a design has is in the table).  q goes out as fp32, k and v into the paged store.  The raw projections of the last
// taps - 1 positions are the sequence's state: a ring [slots][taps - 1][channels] fp32, position p in row p % (taps - 1); the
// ring is read here and refreshed afterwards (umb_ssd_conv_update; steps of one token per sequence refresh it here, by the thread
// that read it).  Taps are summed oldest first whatever their source.  The attention itself is seq_battn.hip.
// Steps of many tokens: one workgroup per token, the convolved q | k row in LDS between the sums of squares and the rotation;
// steps of few tokens: two launches over (token, 256 channels) with the row and the partial sums in scratch.  All fp32.
#include "seq_common.h"

constexpr int CVA_MAXT = 8;      // taps whose loads are issued together (more: a plain loop)

struct CvaTaps { unsigned same, live; };     // bit j: tap j comes from a row of this step / is not before the sequence's start

__device__ __forceinline__ CvaTaps cva_taps(const int* __restrict__ slot_, int t, int p, int slot, int taps) {
  CvaTaps m{0u, 0u};
  if (taps <= CVA_MAXT) {
    for (int j = 0; j < taps; ++j) {
      const int d = taps - 1 - j;                         // how far back the tap looks
      if (d <= p) {
        m.live |= 1u << j;
        if (d == 0 || (t - d >= 0 && slot_[t - d] == slot)) m.same |= 1u << j;
      }
    }
  }
  return m;
}

// the convolved value of channel c of token t.  The taps are loaded unconditionally from clamped addresses -- the same step's
// rows or the ring -- before any is used: a load that sits behind a per-tap branch waits for its own round trip.
template <typename P>
__device__ __forceinline__ float cva_channel(const float* __restrict__ proj, int ld, const typename El<P>::type* __restrict__ conv_w,
                                             const float* __restrict__ conv_state, const int* __restrict__ slot_, CvaTaps m, int t,
                                             int p, int slot, int c, int C, int taps) {
  if (!conv_w) return proj[(long)t * ld + c];
  const long ring0 = (long)slot * (taps - 1);
  float acc = 0.f;
  if (taps <= CVA_MAXT) {
    float in[CVA_MAXT], wv[CVA_MAXT];
#pragma unroll
    for (int j = 0; j < CVA_MAXT; ++j) {
      if (j < taps) {
        const int d = taps - 1 - j;
        const bool sm = (m.same >> j) & 1u, lv = (m.live >> j) & 1u;
        const float* src = (sm || !lv) ? proj + (long)(t - (sm ? d : 0)) * ld + c : conv_state + (ring0 + (p - d) % (taps - 1)) * C + c;
        in[j] = *src;
        wv[j] = ldf<P>(conv_w + (long)c * taps + j);
      }
    }
#pragma unroll
    for (int j = 0; j < CVA_MAXT; ++j)
      if (j < taps) acc += wv[j] * (((m.live >> j) & 1u) ? in[j] : 0.f);      // oldest tap first
  } else {
    for (int j = 0; j < taps; ++j) {
      const int d = taps - 1 - j;
      float in = 0.f;
      if (d <= p) {
        if (d == 0 || (t - d >= 0 && slot_[t - d] == slot)) in = proj[(long)(t - d) * ld + c];        // same step
        else in = conv_state[(ring0 + (p - d) % (taps - 1)) * C + c];
      }
      acc += ldf<P>(conv_w + (long)c * taps + j) * in;
    }
  }
  return acc;
}

// element c of the normed, rotated [q | k] row of token t from the convolved row `row` (LDS or global) -> q (fp32) or cache K
template <typename P>
__device__ __forceinline__ void cva_finish(float* __restrict__ q, const UmbPagedKV& kv, const float* row, int c, float fq, float fk,
                                           const typename El<P>::type* __restrict__ w_q, const typename El<P>::type* __restrict__ w_k,
                                           const float* __restrict__ freq, int t, int p, int slot, int nq, int G, int D, int rot_dims,
                                           int layout) {
  typedef typename El<P>::type El_;
  const bool is_q = c < nq;
  const int cc = is_q ? c : c - nq;
  const int h = cc / D, d = cc - h * D;
  const float f = is_q ? fq : fk;
  const El_* w = is_q ? w_q : w_k;
  float v = row[c] * f * (w ? ldf<P>(w + cc) : 1.f);
  if (d < rot_dims) {
    const int half = rot_dims >> 1;
    int i, other;
    bool first;
    if (layout == 0) { first = d < half; i = first ? d : d - half; other = first ? d + half : d - half; }
    else { first = (d & 1) == 0; i = d >> 1; other = d ^ 1; }
    const float u = row[c - d + other] * f * (w ? ldf<P>(w + cc - d + other) : 1.f);
    float sn, cs;
    sincosf((float)p * freq[i], &sn, &cs);
    v = first ? v * cs - u * sn : v * cs + u * sn;
  }
  if (is_q) q[(long)t * nq + cc] = v;
  else stf<P>(reinterpret_cast<El_*>(kv.k) + pkv_tok(kv, slot, p, h, G, D) + d, v);
}

// one workgroup per token (steps of many tokens): the convolved q | k row lives in LDS between the sums of squares and the rotation
template <typename P>
__global__ __launch_bounds__(256) void cva_prep_kernel(float* __restrict__ q, UmbPagedKV kv, const float* __restrict__ proj, int ld,
                                                       const typename El<P>::type* __restrict__ conv_w, float* __restrict__ conv_state,
                                                       const typename El<P>::type* __restrict__ w_q,
                                                       const typename El<P>::type* __restrict__ w_k, const int* __restrict__ pos,
                                                       const int* __restrict__ slot_, const float* __restrict__ freq, int H, int G,
                                                       int D, int E, int taps, int rot_dims, int layout, int update, float eps) {
  typedef typename El<P>::type El_;
  extern __shared__ float row_s[];                      // [H D + G D]
  __shared__ float red[4];
  const int t = blockIdx.x, p = pos[t], slot = slot_[t];
  const int nq = H * D, nk = G * D, C = nq + nk + G * E;
  const CvaTaps m = cva_taps(slot_, t, p, slot, conv_w ? taps : 0);
  float ssq = 0.f, ssk = 0.f;
  for (int c = threadIdx.x; c < C; c += 256) {
    const float acc = cva_channel<P>(proj, ld, conv_w, conv_state, slot_, m, t, p, slot, c, C, taps);
    if (c < nq) { row_s[c] = acc; ssq += acc * acc; }
    else if (c < nq + nk) { row_s[c] = acc; ssk += acc * acc; }
    else {
      const int j = c - nq - nk, g = j / E, e = j - g * E;
      stf<P>(reinterpret_cast<El_*>(kv.v) + pkv_tok(kv, slot, p, g, G, E) + e, acc);
    }
  }
  // steps of one token per sequence: the ring row of this position held the oldest tap, which the same thread has read above
  if (update && conv_w && taps > 1)
    for (int c = threadIdx.x; c < C; c += 256) conv_state[((long)slot * (taps - 1) + p % (taps - 1)) * C + c] = proj[(long)t * ld + c];
  ssq = block_sum<256>(ssq, red);
  ssk = block_sum<256>(ssk, red);                        // its first barrier comes after every read of the first sum
  const float fq = 1.f / sqrtf(ssq / (float)nq + eps), fk = 1.f / sqrtf(ssk / (float)nk + eps);
  for (int c = threadIdx.x; c < nq + nk; c += 256)
    cva_finish<P>(q, kv, row_s, c, fq, fk, w_q, w_k, freq, t, p, slot, nq, G, D, rot_dims, layout);
}

// Steps of few tokens (decoding): one workgroup per token would walk thousands of channels through several dependent round
// trips.  Two launches instead, both over (token, 256 channels): the convolution (+ ring refresh, + V append) leaves the
// convolved q | k row and every block's two partial sums of squares in scratch; the second sums the partials in block order
// (the same order in every thread and for every batch), norms, rotates and stores.
template <typename P>
__global__ __launch_bounds__(256) void cva_conv_kernel(float* __restrict__ u, float* __restrict__ part, UmbPagedKV kv,
                                                       const float* __restrict__ proj, int ld,
                                                       const typename El<P>::type* __restrict__ conv_w, float* __restrict__ conv_state,
                                                       const int* __restrict__ pos, const int* __restrict__ slot_, int H, int G, int D,
                                                       int E, int taps, int update) {
  typedef typename El<P>::type El_;
  __shared__ float red[4];
  const int t = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x, p = pos[t], slot = slot_[t];
  const int nq = H * D, nk = G * D, C = nq + nk + G * E;
  const CvaTaps m = cva_taps(slot_, t, p, slot, conv_w ? taps : 0);
  float sq = 0.f, sk = 0.f;
  if (c < C) {
    const float acc = cva_channel<P>(proj, ld, conv_w, conv_state, slot_, m, t, p, slot, c, C, taps);
    if (update && conv_w && taps > 1) conv_state[((long)slot * (taps - 1) + p % (taps - 1)) * C + c] = proj[(long)t * ld + c];
    if (c < nq + nk) {
      u[(long)t * (nq + nk) + c] = acc;
      if (c < nq) sq = acc * acc; else sk = acc * acc;
    } else {
      const int j = c - nq - nk, g = j / E, e = j - g * E;
      stf<P>(reinterpret_cast<El_*>(kv.v) + pkv_tok(kv, slot, p, g, G, E) + e, acc);
    }
  }
  sq = block_sum<256>(sq, red);
  sk = block_sum<256>(sk, red);
  if (threadIdx.x == 0) {
    float* pr = part + ((long)t * gridDim.y + blockIdx.y) * 2;
    pr[0] = sq;
    pr[1] = sk;
  }
}

template <typename P>
__global__ __launch_bounds__(256) void cva_finish_kernel(float* __restrict__ q, UmbPagedKV kv, const float* __restrict__ u,
                                                         const float* __restrict__ part, int nblk,
                                                         const typename El<P>::type* __restrict__ w_q,
                                                         const typename El<P>::type* __restrict__ w_k, const int* __restrict__ pos,
                                                         const int* __restrict__ slot_, const float* __restrict__ freq, int H, int G,
                                                         int D, int rot_dims, int layout, float eps) {
  const int t = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  const int nq = H * D, nk = G * D;
  float ssq = 0.f, ssk = 0.f;
  for (int b = 0; b < nblk; ++b) {                       // uniform: every thread forms the same two sums in the same order
    ssq += part[((long)t * nblk + b) * 2];
    ssk += part[((long)t * nblk + b) * 2 + 1];
  }
  if (c >= nq + nk) return;
  const float fq = 1.f / sqrtf(ssq / (float)nq + eps), fk = 1.f / sqrtf(ssk / (float)nk + eps);
  cva_finish<P>(q, kv, u + (long)t * (nq + nk), c, fq, fk, w_q, w_k, freq, t, pos[t], slot_[t], nq, G, D, rot_dims, layout);
}

extern "C" int umb_cva_prep(float* q, const UmbPagedKV* kv, const float* proj, int ld, const void* conv_w, float* conv_state,
                            const void* w_q, const void* w_k, const int* pos, const int* slot, const float* freq, int T, int H, int G,
                            int D, int E, int taps, int rot_dims, int layout, int update_state, float eps, float* scratch,
                            long scratch_floats, int dtype, hipStream_t st) {
  if (T < 1 || H < 1 || G < 1 || H % G || D < 1 || E < 1 || taps < 1 || rot_dims < 0 || rot_dims > D || (rot_dims & 1) ||
      (rot_dims && !freq) || layout < 0 || layout > 1 || !q || !kv || !kv->k || !kv->v || !kv->pages || kv->page < 1 || !proj ||
      !pos || !slot || ld < H * D + G * D + G * E || (conv_w && taps > 1 && !conv_state))
    return UMB_EINVAL;
  const int nqk = (H + G) * D, C = nqk + G * E, nblk = (C + 255) / 256;
  const bool split = T <= 64 && scratch && scratch_floats >= (long)T * nqk + (long)T * nblk * 2 && nblk <= 65535;
  const size_t lds = (size_t)nqk * sizeof(float);
  if (!split && lds > 160 * 1024 - 64) return UMB_EINVAL;
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type El_;
    if (split) {
      float* u = scratch;
      float* part = scratch + (long)T * nqk;
      hipLaunchKernelGGL(cva_conv_kernel<P>, dim3(T, nblk), dim3(256), 0, st, u, part, *kv, proj, ld, (const El_*)conv_w, conv_state, pos,
                         slot, H, G, D, E, taps, update_state);
      hipLaunchKernelGGL(cva_finish_kernel<P>, dim3(T, (nqk + 255) / 256), dim3(256), 0, st, q, *kv, u, part, nblk, (const El_*)w_q,
                         (const El_*)w_k, pos, slot, freq, H, G, D, rot_dims, layout, eps);
    } else {
      if (ensure_dynamic_lds<cva_prep_kernel<P>>(lds) != UMB_OK) return UMB_EHIP;
      hipLaunchKernelGGL(cva_prep_kernel<P>, dim3(T), dim3(256), lds, st, q, *kv, proj, ld, (const El_*)conv_w, conv_state,
                         (const El_*)w_q, (const El_*)w_k, pos, slot, freq, H, G, D, E, taps, rot_dims, layout, update_state, eps);
    }
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}
