// Feed-forward pieces beyond the gated SiLU layer that the linear kernel's epilogue covers: the PolyNorm activation and the
// routing of tokens to experts.
//
// PolyNorm: act(z) = a N(z) + b N(z^2) + c N(z^3) + e, powers element by element, N(v) = v / sqrt(mean(v^2) + eps) over the
// token's row -- three sums (z^2, z^4, z^6) in one pass, everything fp32.
//
// Routed experts: score = sigmoid(router logit) in fp32; a token keeps its `top` largest scores (ties go to the lower
// index) and uses the scores themselves, not renormalised, as weights.  The weight multiplies the expert's INPUT (the gated
// expert is not linear, so this differs from weighting its output).  The (token, choice) pairs are brought into expert order on
// the device -- a counting sort inside one workgroup -- and cut into tiles of at most 64 rows of one expert, which the grouped
// linear kernel walks; the host never sees a count.  Every pair's row is computed on its own (an output's summation order
// depends on K alone), so the order of rows inside an expert, which the sort does not fix, does not reach the results; the
// pairs of a token are added back in choice order.
#include "seq_common.h"

template <typename P>
__global__ __launch_bounds__(256) void polynorm_kernel(typename El<P>::type* __restrict__ out, const float* __restrict__ z,
                                                       const typename El<P>::type* __restrict__ coef, int F, float eps) {
  __shared__ float red[3][4];
  const int t = blockIdx.x, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const float* zr = z + (long)t * F;
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  const bool vec = (F & 3) == 0;
  if (vec) {                                     // 16-byte loads, four in flight per thread
#pragma unroll 4
    for (int i = 4 * threadIdx.x; i < F; i += 1024) {
      const f32x4 v = *reinterpret_cast<const f32x4*>(zr + i);
#pragma unroll
      for (int e = 0; e < 4; ++e) { const float v2 = v[e] * v[e]; s2 += v2; s4 += v2 * v2; s6 += v2 * v2 * v2; }
    }
  } else {
    for (int i = threadIdx.x; i < F; i += 256) {
      const float v = zr[i], v2 = v * v;
      s2 += v2; s4 += v2 * v2; s6 += v2 * v2 * v2;
    }
  }
  s2 = wave_sum(s2); s4 = wave_sum(s4); s6 = wave_sum(s6);
  if (lane == 0) { red[0][wave] = s2; red[1][wave] = s4; red[2][wave] = s6; }
  __syncthreads();
  s2 = red[0][0] + red[0][1] + red[0][2] + red[0][3];
  s4 = red[1][0] + red[1][1] + red[1][2] + red[1][3];
  s6 = red[2][0] + red[2][1] + red[2][2] + red[2][3];
  const float a = ldf<P>(coef) / sqrtf(s2 / (float)F + eps), b = ldf<P>(coef + 1) / sqrtf(s4 / (float)F + eps),
              c = ldf<P>(coef + 2) / sqrtf(s6 / (float)F + eps), e = ldf<P>(coef + 3);
  if (vec) {
#pragma unroll 4
    for (int i = 4 * threadIdx.x; i < F; i += 1024) {
      const f32x4 v = *reinterpret_cast<const f32x4*>(zr + i);
#pragma unroll
      for (int k = 0; k < 4; ++k) stf<P>(out + (long)t * F + i + k, a * v[k] + b * (v[k] * v[k]) + c * (v[k] * v[k] * v[k]) + e);
    }
  } else {
    for (int i = threadIdx.x; i < F; i += 256) {
      const float v = zr[i];
      stf<P>(out + (long)t * F + i, a * v + b * (v * v) + c * (v * v * v) + e);
    }
  }
}

// one wave per token; lane l looks at experts l, l + 64, ...; `top` rounds of arg-max over the experts not yet taken.  The
// order is taken on the logits: the sigmoid is monotonic, and where it saturates in fp32 (two scores both rounding to 1) the
// logits still tell the experts apart.
__global__ __launch_bounds__(256) void moe_route_kernel(int* __restrict__ sel, float* __restrict__ wt,
                                                        const float* __restrict__ logits, int T, int E, int top) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + wave;
  if (t >= T) return;
  const float* z = logits + (long)t * E;
  int prev_i = -1;
  float prev_z = INFINITY;
  for (int k = 0; k < top; ++k) {
    // candidates come after (prev_z, prev_i) in the order "logit descending, index ascending"
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float v = z[e];
      const bool after = v < prev_z || (v == prev_z && e > prev_i);
      if (after && (v > best || (v == best && e < bi))) { best = v; bi = e; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
    }
    if (bi >= E) { bi = 0; best = -INFINITY; }      // no candidate left (logits that are not numbers): keep indices in range
    if (lane == 0) { sel[(long)t * top + k] = bi; wt[(long)t * top + k] = 1.f / (1.f + expf(-best)); }
    prev_z = best; prev_i = bi;
  }
}

// Softmax routing: scores = softmax(logits) over ALL experts (fp32, expf); the choice is made on score + correction (a bias
// that steers the load and never reaches the weights; ties go to the lower index); the weights are the chosen experts'
// scores over their sum.  One wave per token; lane l looks at experts l, l + 64, ...
__global__ __launch_bounds__(256) void moe_route_softmax_kernel(int* __restrict__ sel, float* __restrict__ wt,
                                                                const float* __restrict__ logits,
                                                                const float* __restrict__ correction, int T, int E, int top) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + wave;
  if (t >= T) return;
  const float* z = logits + (long)t * E;
  float mx = -INFINITY;
  for (int e = lane; e < E; e += 64) mx = fmaxf(mx, z[e]);
  mx = wave_max(mx);
  float den = 0.f;
  for (int e = lane; e < E; e += 64) den += expf(z[e] - mx);
  den = wave_sum(den);
  int prev_i = -1;
  float prev_c = INFINITY, tot = 0.f;
  for (int k = 0; k < top; ++k) {
    // candidates come after (prev_c, prev_i) in the order "choice score descending, index ascending"
    float best = -INFINITY, best_s = 0.f;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float s = expf(z[e] - mx) / den;
      const float c = s + (correction ? correction[e] : 0.f);
      const bool after = c < prev_c || (c == prev_c && e > prev_i);
      if (after && (c > best || (c == best && e < bi))) { best = c; bi = e; best_s = s; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, 64), os = __shfl_xor(best_s, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; best_s = os; }
    }
    if (bi >= E) { bi = 0; best = -INFINITY; best_s = 0.f; }      // no candidate left (scores that are not numbers)
    if (lane == 0) { sel[(long)t * top + k] = bi; wt[(long)t * top + k] = best_s; }
    tot += best_s;
    prev_c = best; prev_i = bi;
  }
  __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
  __builtin_amdgcn_wave_barrier();
  if (lane == 0)
    for (int k = 0; k < top; ++k) wt[(long)t * top + k] = wt[(long)t * top + k] / (tot + 1e-20f);
}

// single workgroup: counts per expert (LDS atomics), row offsets, tile list, then every pair's row
__global__ __launch_bounds__(1024) void moe_plan_kernel(int* __restrict__ pos_of, int* __restrict__ tiles,
                                                        const int* __restrict__ sel, int pairs, int E, int max_tiles, int TR) {
  extern __shared__ int sm[];                 // [E] counts, [E] offsets / cursors
  int* cnt = sm;
  int* cur = sm + E;
  for (int e = threadIdx.x; e < E; e += 1024) cnt[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < pairs; i += 1024) atomicAdd(&cnt[min(max(sel[i], 0), E - 1)], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int off = 0, nt = 0;
    for (int e = 0; e < E; ++e) {
      cur[e] = off;
      for (int r = 0; r < cnt[e]; r += TR) {
        if (nt < max_tiles) { tiles[3 * nt] = e; tiles[3 * nt + 1] = off + r; tiles[3 * nt + 2] = cnt[e] - r < TR ? cnt[e] - r : TR; }
        ++nt;
      }
      off += cnt[e];
    }
    for (; nt < max_tiles; ++nt) { tiles[3 * nt] = 0; tiles[3 * nt + 1] = 0; tiles[3 * nt + 2] = 0; }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < pairs; i += 1024) pos_of[i] = atomicAdd(&cur[min(max(sel[i], 0), E - 1)], 1);
}

template <typename P>
__global__ __launch_bounds__(256) void moe_scatter_kernel(typename El<P>::type* __restrict__ xs,
                                                          const typename El<P>::type* __restrict__ h, const float* __restrict__ wt,
                                                          const int* __restrict__ pos_of, int W, int top) {
  const int pr = blockIdx.x, t = pr / top;
  const float wv = wt ? wt[pr] : 1.f;
  const long dst = (long)pos_of[pr] * W;
  for (int c = threadIdx.x; c < W; c += 256) stf<P>(xs + dst + c, wv * ldf<P>(h + (long)t * W + c));
}

__global__ __launch_bounds__(256) void moe_combine_kernel(float* __restrict__ y, const float* __restrict__ ye,
                                                          const int* __restrict__ pos_of, int W, int top, int add) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < W; c += 256) {
    float a = add ? y[(long)t * W + c] : 0.f;
    for (int k = 0; k < top; ++k) a += ye[(long)pos_of[(long)t * top + k] * W + c];
    y[(long)t * W + c] = a;
  }
}

__global__ __launch_bounds__(256) void moe_combine_weighted_kernel(float* __restrict__ y, const float* __restrict__ ye,
                                                                   const float* __restrict__ wt, const int* __restrict__ pos_of,
                                                                   int W, int top, int add) {
  const int t = blockIdx.x;
  for (int c = threadIdx.x; c < W; c += 256) {
    float a = add ? y[(long)t * W + c] : 0.f;
    for (int k = 0; k < top; ++k) a += wt[(long)t * top + k] * ye[(long)pos_of[(long)t * top + k] * W + c];
    y[(long)t * W + c] = a;
  }
}

extern "C" int umb_polynorm(void* out, const float* z, const void* coef, int T, int F, float eps, int dtype, hipStream_t st) {
  if (T < 1 || F < 1 || !out || !z || !coef) return UMB_EINVAL;
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    hipLaunchKernelGGL(polynorm_kernel<P>, dim3(T), dim3(256), 0, st, (E*)out, z, (const E*)coef, F, eps);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_moe_route(int* sel, float* wt, const float* logits, int T, int E, int top, hipStream_t st) {
  if (T < 1 || E < 1 || top < 1 || top > E || !sel || !wt || !logits) return UMB_EINVAL;
  hipLaunchKernelGGL(moe_route_kernel, dim3((T + 3) / 4), dim3(256), 0, st, sel, wt, logits, T, E, top);
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_moe_plan(int* pos_of, int* tiles, const int* sel, int T, int E, int top, int max_tiles, int tile_rows,
                            hipStream_t st) {
  const long pairs = (long)T * top;
  if (T < 1 || E < 1 || E > 4096 || top < 1 || pairs > 0x7fffffffL || tile_rows < 1 ||
      max_tiles < (pairs + tile_rows - 1) / tile_rows + E || !pos_of || !tiles || !sel)
    return UMB_EINVAL;
  hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(1024), 2 * E * sizeof(int), st, pos_of, tiles, sel, (int)pairs, E, max_tiles,
                     tile_rows);
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_moe_scatter(void* xs, const void* h, const float* wt, const int* pos_of, int T, int W, int top, int dtype,
                               hipStream_t st) {
  if (T < 1 || W < 1 || top < 1 || !xs || !h || !pos_of) return UMB_EINVAL;
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    hipLaunchKernelGGL(moe_scatter_kernel<P>, dim3(T * top), dim3(256), 0, st, (E*)xs, (const E*)h, wt, pos_of, W, top);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_moe_combine(float* y, const float* ye, const int* pos_of, int T, int W, int top, int add, hipStream_t st) {
  if (T < 1 || W < 1 || top < 1 || !y || !ye || !pos_of) return UMB_EINVAL;
  hipLaunchKernelGGL(moe_combine_kernel, dim3(T), dim3(256), 0, st, y, ye, pos_of, W, top, add);
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_moe_route_softmax(int* sel, float* wt, const float* logits, const float* correction, int T, int E, int top,
                                     hipStream_t st) {
  if (T < 1 || E < 1 || top < 1 || top > E || !sel || !wt || !logits) return UMB_EINVAL;
  hipLaunchKernelGGL(moe_route_softmax_kernel, dim3((T + 3) / 4), dim3(256), 0, st, sel, wt, logits, correction, T, E, top);
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_moe_combine_weighted(float* y, const float* ye, const float* wt, const int* pos_of, int T, int W, int top,
                                        int add, hipStream_t st) {
  if (T < 1 || W < 1 || top < 1 || !y || !ye || !wt || !pos_of) return UMB_EINVAL;
  hipLaunchKernelGGL(moe_combine_weighted_kernel, dim3(T), dim3(256), 0, st, y, ye, wt, pos_of, W, top, add);
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

// Routing on the logits themselves: the `top` largest logits of a token (ties: the lower index) are chosen and their weights are
// the softmax over JUST the chosen logits (fp32, expf).  logits rows are ld apart (other columns may follow the E logits).
__global__ __launch_bounds__(256) void moe_route_top_kernel(int* __restrict__ sel, float* __restrict__ wt,
                                                            const float* __restrict__ logits, int ld, int T, int E, int top) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + wave;
  if (t >= T) return;
  const float* z = logits + (long)t * ld;
  int prev_i = -1;
  float prev_z = INFINITY, first = 0.f, tot = 0.f;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      const float v = z[e];
      const bool after = v < prev_z || (v == prev_z && e > prev_i);
      if (after && (v > best || (v == best && e < bi))) { best = v; bi = e; }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
    }
    if (bi >= E) { bi = 0; best = -INFINITY; }      // no candidate left (logits that are not numbers): keep indices in range
    if (k == 0) first = best;                       // the largest logit: every exponent below is <= 0
    const float ev = expf(best - first);
    tot += ev;
    if (lane == 0) { sel[(long)t * top + k] = bi; wt[(long)t * top + k] = ev; }
    prev_z = best; prev_i = bi;
  }
  __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
  __builtin_amdgcn_wave_barrier();
  if (lane == 0)
    for (int k = 0; k < top; ++k) wt[(long)t * top + k] = wt[(long)t * top + k] / tot;
}

// y[t] = sigmoid(gate[t ldg]) * ys[t] + sum_k wt[t top + k] * ye[pos_of[t top + k]]   (ys null: no shared part; gate null: 1)
__global__ __launch_bounds__(256) void moe_combine_gated_kernel(float* y, const float* ys, const float* __restrict__ ye,
                                                                const float* __restrict__ wt, const int* __restrict__ pos_of,
                                                                const float* __restrict__ gate, int ldg, int W, int top) {
  const int t = blockIdx.x;
  const float gs = gate ? 1.f / (1.f + expf(-gate[(long)t * ldg])) : 1.f;
  for (int c = threadIdx.x; c < W; c += 256) {
    float a = 0.f;
    for (int k = 0; k < top; ++k) a += wt[(long)t * top + k] * ye[(long)pos_of[(long)t * top + k] * W + c];
    y[(long)t * W + c] = ys ? a + gs * ys[(long)t * W + c] : a;
  }
}

extern "C" int umb_moe_route_top(int* sel, float* wt, const float* logits, int ld, int T, int E, int top, hipStream_t st) {
  if (T < 1 || E < 1 || top < 1 || top > E || ld < E || !sel || !wt || !logits) return UMB_EINVAL;
  hipLaunchKernelGGL(moe_route_top_kernel, dim3((T + 3) / 4), dim3(256), 0, st, sel, wt, logits, ld, T, E, top);
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_moe_combine_gated(float* y, const float* ys, const float* ye, const float* wt, const int* pos_of,
                                     const float* gate, int ldg, int T, int W, int top, hipStream_t st) {
  if (T < 1 || W < 1 || top < 1 || !y || !ye || !wt || !pos_of) return UMB_EINVAL;
  hipLaunchKernelGGL(moe_combine_gated_kernel, dim3(T), dim3(256), 0, st, y, ys, ye, wt, pos_of, gate, ldg, W, top);
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}
