// Causal softmax attention with a learned bias by distance, grouped query heads, over the paged key/value store.
//     q_i = unit_rms(W_q h_i) * w_q * temp(i)       k_j = unit_rms(W_k h_j) * w_k       v_j = unit_rms(W_v h_j)
//     score(i, j, h) = q_i . k_j * scale + bias[h][min(i - j, n_dist - 1)]      (j <= i, i - j < window)
//     out_i = c * sigmoid(gate_i[h]) * softmax_j(score) . v
// temp(i) = 1 + coef ln(floor((i + 1) / every) + 1) sharpens the queries of long contexts; the bias table is indexed by the
// clamped distance itself (whatever bucketing a design uses is expanded into it at load).  Keys and values are cached as
// normed (storage dtype); queries, scores, weights, maxima and sums are fp32 (expf, not the fast intrinsic).
//
// prep: one wave per (token, head slot): query heads -> fp32 q, key heads -> cache K, value heads -> cache V.
// attend (vector pipe, any dtype and head size): workgroup = (token, RH query heads of ONE key/value head, so one pass over
// the keys serves them all); waves take 64-key rounds by round number; score phase lane = key, value phase lane = value
// column with eight keys' rows in flight; per-wave running maximum / denominator, merged through LDS in wave order.  Which
// keys land in which wave and round depends on the query's position alone -- never on the batch or on how a prompt was cut.
#include "seq_common.h"

static inline bool bsa_kv_ok(const UmbPagedKV* kv) { return kv && kv->k && kv->v && kv->pages && kv->page >= 1 && kv->max_pages >= 1; }

template <typename P>
__global__ __launch_bounds__(256) void bsa_prep_kernel(float* __restrict__ q, UmbPagedKV kv, const float* __restrict__ proj, int ld,
                                                       const typename El<P>::type* __restrict__ w_q,
                                                       const typename El<P>::type* __restrict__ w_k, const int* __restrict__ pos,
                                                       const int* __restrict__ slot, int T, int H, int G, int D, int E,
                                                       float temp_coef, int temp_every, float eps) {
  typedef typename El<P>::type El_;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int per = H + 2 * G;
  const long item = (long)blockIdx.x * 4 + wave;
  if (item >= (long)T * per) return;
  const int t = (int)(item / per), hs = (int)(item % per);
  const int n = hs < H + G ? D : E;
  const int col = hs < H ? hs * D : (hs < H + G ? H * D + (hs - H) * D : H * D + G * D + (hs - H - G) * E);
  const float* src = proj + (long)t * ld + col;
  float ss = 0.f;
  for (int i = lane; i < n; i += 64) { const float v = src[i]; ss += v * v; }
  ss = wave_sum(ss);
  const float f = 1.f / sqrtf(ss / (float)n + eps);
  const int p = pos[t];
  if (hs < H) {
    const float temp = temp_every > 0 ? 1.f + temp_coef * logf((float)((p + 1) / temp_every + 1)) : 1.f;
    for (int i = lane; i < n; i += 64) q[(long)t * H * D + (long)hs * D + i] = src[i] * f * (w_q ? ldf<P>(w_q + i) : 1.f) * temp;
  } else if (hs < H + G) {
    El_* row = reinterpret_cast<El_*>(kv.k) + pkv_tok(kv, slot[t], p, hs - H, G, D);
    for (int i = lane; i < n; i += 64) stf<P>(row + i, src[i] * f * (w_k ? ldf<P>(w_k + i) : 1.f));
  } else {
    El_* row = reinterpret_cast<El_*>(kv.v) + pkv_tok(kv, slot[t], p, hs - H - G, G, E);
    for (int i = lane; i < n; i += 64) stf<P>(row + i, src[i] * f);
  }
}

constexpr int BSA_MAXC = 4;      // value columns per lane: E <= 256

template <typename P, int RH, int NC, int NW>
__global__ __launch_bounds__(NW * 64) void bsa_attend_kernel(typename El<P>::type* __restrict__ out, int ldo,
                                                             const float* __restrict__ q, UmbPagedKV kv,
                                                             const float* __restrict__ proj, int ld, int gate_col,
                                                             const float* __restrict__ bias, int n_dist,
                                                             const int* __restrict__ pos, const int* __restrict__ slot_, int H,
                                                             int G, int D, int E, int window, float scale, float out_scale) {
  typedef typename El<P>::type El_;
  extern __shared__ float lds[];
  constexpr int KB = 8;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int Dp = (D + 3) & ~3, Ep = (E + 3) & ~3, Mp = Dp > Ep ? Dp : Ep;
  // [RH][Dp] queries (later [NW][RH][Ep] partial sums), [NW][2 RH] maxima and denominators, per wave [RH][64] weights + offsets
  float* q_s = lds;
  float* ml_s = lds + NW * RH * Mp;
  float* w_s = ml_s + NW * 2 * RH + wave * (RH * 64 + 128);
  long* off_s = reinterpret_cast<long*>(w_s + RH * 64);
  const int t = blockIdx.x, hpg = H / G;
  const int h0 = blockIdx.y * RH, g = h0 / hpg;           // RH divides H / G: the block's heads share key/value head g
  const int i = pos[t], slot = slot_[t];
  for (int x = threadIdx.x; x < RH * D; x += NW * 64) {
    const int r = x / D, d = x % D;
    q_s[r * Dp + d] = q[((long)t * H + h0 + r) * D + d];
  }
  __syncthreads();
  const int j_lo = i - window + 1 > 0 ? i - window + 1 : 0;
  const int n_keys = i - j_lo + 1;
  const bool vec = (D & 7) == 0 && sizeof(El_) == 2;
  float acc[RH][NC], m_run[RH], l_run[RH];
#pragma unroll
  for (int r = 0; r < RH; ++r) {
    m_run[r] = -INFINITY;
    l_run[r] = 0.f;
#pragma unroll
    for (int c = 0; c < NC; ++c) acc[r][c] = 0.f;
  }
  int dcl[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) dcl[c] = lane + 64 * c < E ? lane + 64 * c : E - 1;
  for (int base = wave * 64; base < n_keys; base += NW * 64) {
    const int kx = base + lane;
    float s[RH];
#pragma unroll
    for (int r = 0; r < RH; ++r) s[r] = 0.f;
    long off = 0;
    int dist = 0;
    if (kx < n_keys) {
      const int j = j_lo + kx;
      dist = i - j;
      const El_* kr = reinterpret_cast<const El_*>(kv.k) + pkv_tok(kv, slot, j, g, G, D);
      off = pkv_tok(kv, slot, j, g, G, E);
      bool done = false;
      if constexpr (sizeof(El_) == 2) {
        if (vec) {
          for (int d = 0; d < D; d += 64) {              // eight 16-byte loads in flight, then their 64 x RH products
            u32x4 kk[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) kk[u] = *reinterpret_cast<const u32x4*>(kr + (d + 8 * u < D ? d + 8 * u : 0));
#pragma unroll
            for (int u = 0; u < 8; ++u) {
              if (d + 8 * u >= D) break;
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                const float k0 = lo_f<P>(kk[u][e]), k1 = hi_f<P>(kk[u][e]);
                const int dd = d + 8 * u + 2 * e;
#pragma unroll
                for (int r = 0; r < RH; ++r) s[r] += q_s[r * Dp + dd] * k0 + q_s[r * Dp + dd + 1] * k1;
              }
            }
          }
          done = true;
        }
      }
      if (!done) {
        for (int d = 0; d < D; ++d) {
          const float kd = ldf<P>(kr + d);
#pragma unroll
          for (int r = 0; r < RH; ++r) s[r] += q_s[r * Dp + d] * kd;
        }
      }
    }
    const int bi = dist < n_dist ? dist : n_dist - 1;
#pragma unroll
    for (int r = 0; r < RH; ++r) {
      const float sv = kx < n_keys ? s[r] * scale + (bias ? bias[(long)(h0 + r) * n_dist + bi] : 0.f) : -INFINITY;
      const float m_new = fmaxf(m_run[r], wave_max(sv));          // finite: every round has at least one key
      const float fac = expf(m_run[r] - m_new);                   // 0 on the first round (m_run = -inf)
      const float pw = kx < n_keys ? expf(sv - m_new) : 0.f;
      l_run[r] = l_run[r] * fac + wave_sum(pw);
      m_run[r] = m_new;
#pragma unroll
      for (int c = 0; c < NC; ++c) acc[r][c] *= fac;
      w_s[r * 64 + lane] = pw;
    }
    off_s[lane] = off;
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
    const int cnt = n_keys - base < 64 ? n_keys - base : 64;
    for (int j0 = 0; j0 < cnt; j0 += KB) {
      float vv[KB][NC];
#pragma unroll
      for (int u = 0; u < KB; ++u) {
        const long oj = off_s[j0 + u < cnt ? j0 + u : cnt - 1];
#pragma unroll
        for (int c = 0; c < NC; ++c) vv[u][c] = ldf<P>(reinterpret_cast<const El_*>(kv.v) + oj + dcl[c]);
      }
#pragma unroll
      for (int u = 0; u < KB; ++u) {
#pragma unroll
        for (int r = 0; r < RH; ++r) {
          const float wj = j0 + u < cnt ? w_s[r * 64 + j0 + u] : 0.f;
#pragma unroll
          for (int c = 0; c < NC; ++c) acc[r][c] += wj * vv[u][c];
        }
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "wavefront");
    __builtin_amdgcn_wave_barrier();
  }
  __syncthreads();                                  // every wave is done with the queries: their LDS becomes the partials
#pragma unroll
  for (int r = 0; r < RH; ++r) {
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int d = lane + 64 * c;
      if (d < E) lds[(wave * RH + r) * Ep + d] = acc[r][c];
    }
    if (lane == 0) { ml_s[(wave * RH + r) * 2] = m_run[r]; ml_s[(wave * RH + r) * 2 + 1] = l_run[r]; }
  }
  __syncthreads();
  for (int x = threadIdx.x; x < RH * E; x += NW * 64) {
    const int r = x / E, d = x % E;
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < NW; ++w) M = fmaxf(M, ml_s[(w * RH + r) * 2]);
    float o = 0.f, L = 0.f;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const float mw = ml_s[(w * RH + r) * 2];
      const float f = mw == -INFINITY ? 0.f : expf(mw - M);
      o += lds[(w * RH + r) * Ep + d] * f;
      L += ml_s[(w * RH + r) * 2 + 1] * f;
    }
    const float gt = gate_col >= 0 ? 1.f / (1.f + expf(-proj[(long)t * ld + gate_col + h0 + r])) : 1.f;
    stf<P>(out + (long)t * ldo + (long)(h0 + r) * E + d, out_scale * gt * (o / L));
  }
}

extern "C" int umb_bsa_prep(float* q, const UmbPagedKV* kv, const float* proj, int ld, const void* w_q, const void* w_k,
                            const int* pos, const int* slot, int T, int H, int G, int D, int E, float temp_coef, int temp_every,
                            float eps, int dtype, hipStream_t st) {
  if (T < 1 || H < 1 || G < 1 || H % G || D < 1 || E < 1 || !q || !bsa_kv_ok(kv) || !proj || !pos || !slot ||
      ld < H * D + G * D + G * E)
    return UMB_EINVAL;
  const long items = (long)T * (H + 2 * G);
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type El_;
    hipLaunchKernelGGL(bsa_prep_kernel<P>, dim3((unsigned)((items + 3) / 4)), dim3(256), 0, st, q, *kv, proj, ld, (const El_*)w_q,
                       (const El_*)w_k, pos, slot, T, H, G, D, E, temp_coef, temp_every, eps);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

extern "C" int umb_bsa_attend(void* out, int ldo, const float* q, const UmbPagedKV* kv, const float* proj, int ld, int gate_col,
                              const float* bias, int n_dist, const int* pos, const int* slot, int T, int H, int G, int D, int E,
                              int window, float scale, float out_scale, int dtype, hipStream_t st) {
  if (T < 1 || H < 1 || G < 1 || H % G || D < 1 || E < 1 || E > 64 * BSA_MAXC || window < 1 || !out || !q || !bsa_kv_ok(kv) ||
      !pos || !slot || ldo < H * E || (bias && n_dist < 1) || (gate_col >= 0 && (!proj || ld < gate_col + H)))
    return UMB_EINVAL;
  const int hpg = H / G, nc = (E + 63) / 64;
  const int Dp = (D + 3) & ~3, Ep = (E + 3) & ~3, Mp = Dp > Ep ? Dp : Ep;
  // heads of one workgroup: query heads of one key/value head, as many as divide the group and fit the register budget
  int rh = nc <= 2 ? 8 : 4;
  while (rh > 1 && hpg % rh) rh >>= 1;
  const dim3 grid(T, H / rh);
  int nw = (long)T * (H / rh) < 1024 ? 16 : 4;
  auto lds_of = [&](int w) { return ((size_t)w * rh * Mp + (size_t)w * 2 * rh + (size_t)w * (rh * 64 + 128)) * sizeof(float); };
  if (nw == 16 && lds_of(16) > 128 * 1024) nw = 4;
  if (lds_of(nw) > 160 * 1024) return UMB_EINVAL;
  const size_t lds = lds_of(nw);
#define BSA_LAUNCH(RH, NC, NW)                                                                                              \
  do {                                                                                                                      \
    if (ensure_dynamic_lds<bsa_attend_kernel<P, RH, NC, NW>>(lds) != UMB_OK) return UMB_EHIP;                               \
    hipLaunchKernelGGL((bsa_attend_kernel<P, RH, NC, NW>), grid, dim3(NW * 64), lds, st, (El_*)out, ldo, q, *kv, proj, ld,  \
                       gate_col, bias, n_dist, pos, slot, H, G, D, E, window, scale, out_scale);                            \
  } while (0)
#define BSA_NW(RH, NC)                                                                                                      \
  if (nw == 16) BSA_LAUNCH(RH, NC, 16); else BSA_LAUNCH(RH, NC, 4)
#define BSA_RH(NC)                                                                                                          \
  if (rh == 8) { BSA_NW(8, NC); } else if (rh == 4) { BSA_NW(4, NC); } else if (rh == 2) { BSA_NW(2, NC); } else { BSA_NW(1, NC); }
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type El_;
    if (nc <= 1) { BSA_RH(1) }
    else if (nc <= 2) { BSA_RH(2) }
    else { if (rh == 4) { BSA_NW(4, 4); } else if (rh == 2) { BSA_NW(2, 4); } else { BSA_NW(1, 4); } }
  })
#undef BSA_RH
#undef BSA_NW
#undef BSA_LAUNCH
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

// the matrix-pipe prompt kernel is declared in the header; until a shape is covered the forward takes the kernel above
extern "C" int umb_bsa_attend_tiled_ok(int H, int G, int D, int E, int dtype) {
  (void)H; (void)G; (void)D; (void)E; (void)dtype;
  return 0;
}

extern "C" int umb_bsa_attend_tiled(void* out, int ldo, const float* q, const UmbPagedKV* kv, const float* proj, int ld,
                                    int gate_col, const float* bias, int n_dist, const int* seq_slot, const int* seq_row0,
                                    const int* seq_pos0, const int* seq_len, int B, int max_len, int H, int G, int D, int E,
                                    int window, float scale, float out_scale, int dtype, hipStream_t st) {
  (void)out; (void)ldo; (void)q; (void)kv; (void)proj; (void)ld; (void)gate_col; (void)bias; (void)n_dist; (void)seq_slot;
  (void)seq_row0; (void)seq_pos0; (void)seq_len; (void)B; (void)max_len; (void)H; (void)G; (void)D; (void)E; (void)window;
  (void)scale; (void)out_scale; (void)dtype; (void)st;
  return UMB_EINVAL;
}
