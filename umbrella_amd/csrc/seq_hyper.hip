// Several residual streams ("hyper-connections").  A token's residual is S copies x_1 .. x_S of W fp32 values, stored
// [T][S][W].  A sublayer f reads ONE combination of them and writes back to ALL of them:
//     u = sum_s in[s] x_s            h = u / sqrt(mean(u^2) + eps) * (offset + w)          y = f(h)
//     x_t <- sum_s mix[s][t] x_s + m out[t] y          (all t from the OLD x_s)
// in / out / mix are small fp32 tables of the sublayer; S = 1 with in = out = mix = 1 is the plain residual x + m y.  The
// norm weight is stored around `offset` (0: a plain weight; 1: a weight that is zero for "no change").
//
// One workgroup owns one token row.  The seam kernel does the write of the sublayer behind it and the read of the one ahead
// in one pass over the row: thread i keeps the combined value u of its elements in registers (EPT each), the one sum of
// squares goes through LDS, and the row is normed from the registers.  Everything is fp32; only h is rounded.
#include "seq_common.h"

constexpr int HC_MAXS = 8;       // streams

struct HcTables {
  float in[HC_MAXS], out[HC_MAXS], mix[HC_MAXS][HC_MAXS];
};

// the sublayer's tables from device memory (null: trivial) into registers; every thread reads the same few words
__device__ __forceinline__ void hc_load(HcTables& t, const float* in, const float* out, const float* mix, int S) {
#pragma unroll
  for (int s = 0; s < HC_MAXS; ++s) {
    t.in[s] = s < S ? (in ? in[s] : 1.f) : 0.f;
    t.out[s] = s < S ? (out ? out[s] : 1.f) : 0.f;
#pragma unroll
    for (int u = 0; u < HC_MAXS; ++u) t.mix[s][u] = (s < S && u < S) ? (mix ? mix[s * S + u] : (s == u ? 1.f : 0.f)) : 0.f;
  }
}

// EPT > 0: the row's u values stay in registers (W <= 256 EPT); 0: they are formed again from x in the second pass
template <typename P, int NS, int EPT>
__global__ __launch_bounds__(256) void hc_seam_kernel(float* __restrict__ x, typename El<P>::type* __restrict__ h,
                                                      const float* __restrict__ y, const float* __restrict__ mix,
                                                      const float* __restrict__ out, float m, const float* __restrict__ in_next,
                                                      const typename El<P>::type* __restrict__ w_next, float offset, int W, int S,
                                                      float eps, int read) {
  __shared__ float red[8];
  HcTables tb;
  hc_load(tb, in_next, out, mix, S);
  const int t = blockIdx.x;
  float* xr = x + (long)t * S * W;
  const float* yr = y + (long)t * W;
  constexpr int NE = EPT > 0 ? EPT : 1;
  float uv[NE];
  float ss = 0.f;
  auto element = [&](int i) -> float {
    float xo[NS];
#pragma unroll
    for (int s = 0; s < NS; ++s) xo[s] = s < S ? xr[(long)s * W + i] : 0.f;
    const float yv = m * yr[i];
    float u = 0.f;
#pragma unroll
    for (int tt = 0; tt < NS; ++tt) {
      if (tt < S) {
        float a = 0.f;
#pragma unroll
        for (int s = 0; s < NS; ++s) a += tb.mix[s][tt] * xo[s];
        a += tb.out[tt] * yv;
        xr[(long)tt * W + i] = a;
        u += tb.in[tt] * a;
      }
    }
    return u;
  };
  if constexpr (EPT > 0) {
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const int i = threadIdx.x + 256 * e;
      uv[e] = i < W ? element(i) : 0.f;
      ss += uv[e] * uv[e];
    }
  } else {
    for (int i = threadIdx.x; i < W; i += 256) { const float u = element(i); ss += u * u; }
  }
  if (!read) return;
  ss = block_sum<256>(ss, red);
  const float f = 1.f / sqrtf(ss / (float)W + eps);
  if constexpr (EPT > 0) {
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const int i = threadIdx.x + 256 * e;
      if (i < W) stf<P>(h + (long)t * W + i, uv[e] * f * (offset + ldf<P>(w_next + i)));
    }
  } else {
    for (int i = threadIdx.x; i < W; i += 256) {
      float u = 0.f;
#pragma unroll
      for (int s = 0; s < NS; ++s) u += s < S ? tb.in[s] * xr[(long)s * W + i] : 0.f;
      stf<P>(h + (long)t * W + i, u * f * (offset + ldf<P>(w_next + i)));
    }
  }
}

// read alone (rows gathered): u = sum_s in[s] x_s -> u_out (fp32) and / or h = norm(u) * (offset + w)
template <typename P>
__global__ __launch_bounds__(256) void hc_read_kernel(float* __restrict__ u_out, typename El<P>::type* __restrict__ h,
                                                      const float* __restrict__ x, const int* __restrict__ rows,
                                                      const float* __restrict__ in, const typename El<P>::type* __restrict__ w,
                                                      float offset, int W, int S, float eps) {
  __shared__ float red[8];
  const int t = blockIdx.x;
  const float* xr = x + (long)(rows ? rows[t] : t) * S * W;
  float ss = 0.f;
  auto comb = [&](int i) -> float {
    float u = 0.f;
    for (int s = 0; s < S; ++s) u += (in ? in[s] : 1.f) * xr[(long)s * W + i];
    return u;
  };
  for (int i = threadIdx.x; i < W; i += 256) {
    const float u = comb(i);
    if (u_out) u_out[(long)t * W + i] = u;
    ss += u * u;
  }
  if (!h) return;
  ss = block_sum<256>(ss, red);
  const float f = 1.f / sqrtf(ss / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += 256) stf<P>(h + (long)t * W + i, comb(i) * f * (offset + ldf<P>(w + i)));
}

// every stream <- embed[token] * scale; h <- the first read.  With all streams equal u = (sum_s in[s]) e, formed as the
// same sum the read kernel forms, so a one-token step and a prompt give the same bits.
template <typename P>
__global__ __launch_bounds__(256) void hc_embed_kernel(float* __restrict__ x, typename El<P>::type* __restrict__ h,
                                                       const typename El<P>::type* __restrict__ embed,
                                                       const int* __restrict__ tokens, float scale, const float* __restrict__ in,
                                                       const typename El<P>::type* __restrict__ w, float offset, int W, int V,
                                                       int S, float eps) {
  __shared__ float red[8];
  const int t = blockIdx.x;
  int tok = tokens[t];
  tok = tok < 0 ? 0 : (tok >= V ? V - 1 : tok);
  const typename El<P>::type* er = embed + (long)tok * W;
  float* xr = x + (long)t * S * W;
  float ss = 0.f;
  auto comb = [&](float e) -> float {
    float u = 0.f;
    for (int s = 0; s < S; ++s) u += (in ? in[s] : 1.f) * e;
    return u;
  };
  for (int i = threadIdx.x; i < W; i += 256) {
    const float e = ldf<P>(er + i) * scale;
    for (int s = 0; s < S; ++s) xr[(long)s * W + i] = e;
    const float u = comb(e);
    ss += u * u;
  }
  if (!h) return;
  ss = block_sum<256>(ss, red);
  const float f = 1.f / sqrtf(ss / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += 256) stf<P>(h + (long)t * W + i, comb(ldf<P>(er + i) * scale) * f * (offset + ldf<P>(w + i)));
}

extern "C" int umb_hc_embed(float* x, void* h, const void* embed, const int* tokens, float scale, const float* in, const void* w,
                            float offset, int T, int W, int V, int S, float eps, int dtype, hipStream_t st) {
  if (T < 1 || W < 1 || V < 1 || S < 1 || S > HC_MAXS || !x || !embed || !tokens || (h && !w)) return UMB_EINVAL;
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    hipLaunchKernelGGL(hc_embed_kernel<P>, dim3(T), dim3(256), 0, st, x, (E*)h, (const E*)embed, tokens, scale, in, (const E*)w,
                       offset, W, V, S, eps);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

template <typename P, int NS>
static int hc_seam_launch(float* x, void* h, const float* y, const float* mix, const float* out, float m, const float* in_next,
                          const void* w_next, float offset, int T, int W, int S, float eps, hipStream_t st) {
  typedef typename El<P>::type E;
  const int read = w_next != nullptr;
#define HC_SEAM(EPT)                                                                                                        \
  hipLaunchKernelGGL((hc_seam_kernel<P, NS, EPT>), dim3(T), dim3(256), 0, st, x, (E*)h, y, mix, out, m, in_next, (const E*)w_next, \
                     offset, W, S, eps, read)
  if (W <= 256) HC_SEAM(1);
  else if (W <= 1024) HC_SEAM(4);
  else if (W <= 2048) HC_SEAM(8);
  else if (W <= 4096) HC_SEAM(16);
  else HC_SEAM(0);
#undef HC_SEAM
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_hc_seam(float* x, void* h, const float* y, const float* mix, const float* out, float m, const float* in_next,
                           const void* w_next, float offset, int T, int W, int S, float eps, int dtype, hipStream_t st) {
  if (T < 1 || W < 1 || S < 1 || S > HC_MAXS || !x || !y || (w_next && !h)) return UMB_EINVAL;
  DISPATCH_SEQ_DTYPE(dtype, {
    if (S == 1) return hc_seam_launch<P, 1>(x, h, y, mix, out, m, in_next, w_next, offset, T, W, S, eps, st);
    if (S == 2) return hc_seam_launch<P, 2>(x, h, y, mix, out, m, in_next, w_next, offset, T, W, S, eps, st);
    if (S <= 4) return hc_seam_launch<P, 4>(x, h, y, mix, out, m, in_next, w_next, offset, T, W, S, eps, st);
    return hc_seam_launch<P, HC_MAXS>(x, h, y, mix, out, m, in_next, w_next, offset, T, W, S, eps, st);
  })
}

extern "C" int umb_hc_read(float* u_out, void* h, const float* x, const int* rows, const float* in, const void* w, float offset,
                           int R, int W, int S, float eps, int dtype, hipStream_t st) {
  if (R < 1 || W < 1 || S < 1 || S > HC_MAXS || !x || (!u_out && !h) || (h && !w)) return UMB_EINVAL;
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    hipLaunchKernelGGL(hc_read_kernel<P>, dim3(R), dim3(256), 0, st, u_out, (E*)h, x, rows, in, (const E*)w, offset, W, S, eps);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}
