// Layers whose two sublayers read the SAME residual:  x <- x + (mixer(norm1(x)) + ff(norm2(x))).
// The seam between two such layers adds both outputs into the fp32 residual stream and leaves the next layer's two normed
// inputs, one launch per layer; the same kernel starts a step from the embedding table, and adds the embedding row back in
// where a stack runs a span of layers again (the row is read from the table again: storage -> fp32 is exact, so nothing is kept).
// Norm weights are stored around `offset` (factor offset + w).  One workgroup owns one token row; everything is fp32, only
// h1 / h2 are rounded.
#include "seq_common.h"

// mode 0: x += y1 + y2; 1: x = embed[token] * escale; 2: x += (y1 + y2) + embed[token] * escale.  y1 / y2 may be null.
template <typename P, int EPT>
__global__ __launch_bounds__(256) void blk_seam_kernel(float* __restrict__ x, typename El<P>::type* __restrict__ h1,
                                                       typename El<P>::type* __restrict__ h2, const float* __restrict__ y1,
                                                       const float* __restrict__ y2, const typename El<P>::type* __restrict__ embed,
                                                       const int* __restrict__ tokens, int mode, float escale,
                                                       const typename El<P>::type* __restrict__ w1,
                                                       const typename El<P>::type* __restrict__ w2, float offset, int W, int V,
                                                       float eps) {
  __shared__ float red[8];
  const int t = blockIdx.x;
  float* xr = x + (long)t * W;
  const typename El<P>::type* er = nullptr;
  if (mode) {
    int tok = tokens[t];
    tok = tok < 0 ? 0 : (tok >= V ? V - 1 : tok);
    er = embed + (long)tok * W;
  }
  auto element = [&](int i) -> float {
    float v;
    if (mode == 1) {
      v = ldf<P>(er + i) * escale;
    } else {
      v = xr[i];
      if (y1 || y2) {
        float y = y1 ? y1[(long)t * W + i] : 0.f;
        if (y2) y += y2[(long)t * W + i];
        v += y;                                         // x + (mixer + feed-forward)
      }
      if (mode == 2) v += ldf<P>(er + i) * escale;
    }
    xr[i] = v;
    return v;
  };
  constexpr int NE = EPT > 0 ? EPT : 1;
  float keep[NE];
  float ss = 0.f;
  if constexpr (EPT > 0) {
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const int i = threadIdx.x + 256 * e;
      keep[e] = i < W ? element(i) : 0.f;
      ss += keep[e] * keep[e];
    }
  } else {
    for (int i = threadIdx.x; i < W; i += 256) { const float v = element(i); ss += v * v; }
  }
  if (!w1 && !w2) return;
  ss = block_sum<256>(ss, red);
  const float f = 1.f / sqrtf(ss / (float)W + eps);
  auto store = [&](int i, float v) {
    if (w1) stf<P>(h1 + (long)t * W + i, v * f * (offset + ldf<P>(w1 + i)));
    if (w2) stf<P>(h2 + (long)t * W + i, v * f * (offset + ldf<P>(w2 + i)));
  };
  if constexpr (EPT > 0) {
#pragma unroll
    for (int e = 0; e < EPT; ++e) {
      const int i = threadIdx.x + 256 * e;
      if (i < W) store(i, keep[e]);
    }
  } else {
    for (int i = threadIdx.x; i < W; i += 256) store(i, xr[i]);       // the thread's own stores
  }
}

extern "C" int umb_blk_seam(float* x, void* h1, void* h2, const float* y1, const float* y2, const void* embed, const int* tokens,
                            int embed_mode, float embed_scale, const void* w1, const void* w2, float offset, int T, int W, int V,
                            float eps, int dtype, hipStream_t st) {
  if (T < 1 || W < 1 || !x || embed_mode < 0 || embed_mode > 2 || (embed_mode && (!embed || !tokens || V < 1)) || (w1 && !h1) ||
      (w2 && !h2))
    return UMB_EINVAL;
#define BLK_SEAM(EPT)                                                                                                          \
  hipLaunchKernelGGL((blk_seam_kernel<P, EPT>), dim3(T), dim3(256), 0, st, x, (E*)h1, (E*)h2, y1, y2, (const E*)embed, tokens, \
                     embed_mode, embed_scale, (const E*)w1, (const E*)w2, offset, W, V, eps)
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    if (W <= 256) BLK_SEAM(1);
    else if (W <= 1024) BLK_SEAM(4);
    else if (W <= 2048) BLK_SEAM(8);
    else if (W <= 4096) BLK_SEAM(16);
    else BLK_SEAM(0);
  })
#undef BLK_SEAM
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

__global__ __launch_bounds__(256) void seq_scale_kernel(float* __restrict__ buf, long n, float scale) {
  const long i = (long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) buf[i] *= scale;
}

extern "C" int umb_seq_scale(float* buf, long n, float scale, hipStream_t st) {
  if (n < 1 || !buf) return UMB_EINVAL;
  hipLaunchKernelGGL(seq_scale_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, buf, n, scale);
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}
