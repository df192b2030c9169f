// Causal softmax attention with a learned bias by distance, grouped query heads, over the paged key/value store.
//     q_i = unit_rms(W_q h_i) * w_q * temp(i)       k_j = unit_rms(W_k h_j) * w_k       v_j = unit_rms(W_v h_j)
//     score(i, j, h) = q_i . k_j * scale + bias[h][min(i - j, n_dist - 1)]      (j <= i, i - j < window)
//     out_i = c * sigmoid(gate_i[h]) * softmax_j(score) . v
// With softcap > 0 the scaled product is capped before the bias joins it: softcap tanh(q . k scale / softcap).
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

constexpr int BSA_MAXC = 8;      // value columns per lane: E <= 512

template <typename P, int RH, int NC, int NW>
__global__ __launch_bounds__(NW * 64) void bsa_attend_kernel(typename El<P>::type* __restrict__ out, int ldo,
                                                             const float* __restrict__ q, UmbPagedKV kv,
                                                             const float* __restrict__ proj, int ld, int gate_col,
                                                             const float* __restrict__ bias, int n_dist,
                                                             const int* __restrict__ pos, const int* __restrict__ slot_, int H,
                                                             int G, int D, int E, int window, float scale, float out_scale,
                                                             float softcap, float* __restrict__ part, int nsplit) {
  typedef typename El<P>::type El_;
  extern __shared__ float lds[];
  constexpr int KB = 8;
  const int split = blockIdx.z;                         // nsplit > 1: the workgroup takes every nsplit-th group of NW rounds
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
  for (int base = (split * NW + wave) * 64; base < n_keys; base += nsplit * NW * 64) {
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
      float sc = s[r] * scale;
      if (softcap > 0.f) sc = softcap * tanhf(sc / softcap);          // capped score; the bias (if any) is added to the capped value
      const float sv = kx < n_keys ? sc + (bias ? bias[(long)(h0 + r) * n_dist + bi] : 0.f) : -INFINITY;
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
    if (nsplit > 1) {                                  // partial result of this split: [t][h][split][E + 2] = o.., M, L
      float* pr = part + (((long)t * H + h0 + r) * nsplit + split) * (E + 2);
      pr[d] = o;
      if (d == 0) { pr[E] = M; pr[E + 1] = L; }
      continue;
    }
    const float gt = gate_col >= 0 ? 1.f / (1.f + expf(-proj[(long)t * ld + gate_col + h0 + r])) : 1.f;
    stf<P>(out + (long)t * ldo + (long)(h0 + r) * E + d, out_scale * gt * (o / L));
  }
}

// the splits of one (token, head) merged: lane s holds split s's maximum and denominator (a split that had no key carries
// M = -inf, L = 0), the factors go round by shuffles, every sum runs over the splits in order
template <typename P>
__global__ __launch_bounds__(64) void bsa_merge_kernel(typename El<P>::type* __restrict__ out, int ldo, const float* __restrict__ part,
                                                       const float* __restrict__ proj, int ld, int gate_col, int H, int E,
                                                       int nsplit, float out_scale) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* pr = part + ((long)t * H + h) * nsplit * (E + 2);
  const float ms = lane < nsplit ? pr[lane * (E + 2) + E] : -INFINITY;
  const float ls = lane < nsplit ? pr[lane * (E + 2) + E + 1] : 0.f;
  const float gt = gate_col >= 0 ? 1.f / (1.f + expf(-proj[(long)t * ld + gate_col + h])) : 1.f;
  const float M = wave_max(ms);
  const float fs = ms == -INFINITY ? 0.f : expf(ms - M);
  float L = 0.f, f[16];
#pragma unroll
  for (int s = 0; s < 16; ++s) {
    f[s] = __shfl(fs, s, 64);
    L += __shfl(ls * fs, s, 64);
  }
  const float c = out_scale * gt / L;
  for (int d = lane; d < E; d += 64) {
    float v[16];
#pragma unroll
    for (int s = 0; s < 16; ++s) v[s] = pr[(s < nsplit ? s : nsplit - 1) * (E + 2) + d];
    float o = 0.f;
#pragma unroll
    for (int s = 0; s < 16; ++s) o += s < nsplit ? v[s] * f[s] : 0.f;
    stf<P>(out + (long)t * ldo + (long)h * E + d, o * c);
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
                              int window, float scale, float out_scale, float softcap, float* scratch, long scratch_floats,
                              int dtype, hipStream_t st) {
  if (T < 1 || H < 1 || G < 1 || H % G || D < 1 || E < 1 || E > 64 * BSA_MAXC || window < 1 || !out || !q || !bsa_kv_ok(kv) ||
      !pos || !slot || ldo < H * E || (bias && n_dist < 1) || (gate_col >= 0 && (!proj || ld < gate_col + H)))
    return UMB_EINVAL;
  const int hpg = H / G, nc = (E + 63) / 64;
  const int Dp = (D + 3) & ~3, Ep = (E + 3) & ~3, Mp = Dp > Ep ? Dp : Ep;
  // heads of one workgroup: query heads of one key/value head, as many as divide the group and fit the register budget
  int rh = nc <= 2 ? 8 : (nc <= 4 ? 4 : 2);
  while (rh > 1 && hpg % rh) rh >>= 1;
  // A handful of (token, head block) items leaves most of the chip idle while each walks all its keys: with scratch for the
  // partial results the keys of an item are dealt to several workgroups (whole groups of four 64-key rounds by number, so the
  // order of every sum is a function of the position and of the step's row count only) and merged by a second launch.
  const long items = (long)T * (H / rh);
  int nsplit = 1;
  if (scratch && items <= 64) {                          // fewer than ~2048 waves in all with sixteen waves per item
    nsplit = (int)(512 / items) < 16 ? (int)(512 / items) : 16;
    while (nsplit > 1 && (long)T * H * nsplit * (E + 2) > scratch_floats) nsplit >>= 1;
  }
  const dim3 grid(T, H / rh, nsplit);
  int nw = (nsplit > 1 || items >= 1024) ? 4 : 16;
  auto lds_of = [&](int w) { return ((size_t)w * rh * Mp + (size_t)w * 2 * rh + (size_t)w * (rh * 64 + 128)) * sizeof(float); };
  if (nw == 16 && lds_of(16) > 128 * 1024) nw = 4;
  if (lds_of(nw) > 160 * 1024) return UMB_EINVAL;
  const size_t lds = lds_of(nw);
#define BSA_LAUNCH(RH, NC, NW)                                                                                              \
  do {                                                                                                                      \
    if (ensure_dynamic_lds<bsa_attend_kernel<P, RH, NC, NW>>(lds) != UMB_OK) return UMB_EHIP;                               \
    hipLaunchKernelGGL((bsa_attend_kernel<P, RH, NC, NW>), grid, dim3(NW * 64), lds, st, (El_*)out, ldo, q, *kv, proj, ld,  \
                       gate_col, bias, n_dist, pos, slot, H, G, D, E, window, scale, out_scale, softcap, scratch, nsplit);           \
  } while (0)
#define BSA_NW(RH, NC)                                                                                                      \
  if (nw == 16) BSA_LAUNCH(RH, NC, 16); else BSA_LAUNCH(RH, NC, 4)
#define BSA_RH(NC)                                                                                                          \
  if (rh == 8) { BSA_NW(8, NC); } else if (rh == 4) { BSA_NW(4, NC); } else if (rh == 2) { BSA_NW(2, NC); } else { BSA_NW(1, NC); }
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type El_;
    if (nc <= 1) { BSA_RH(1) }
    else if (nc <= 2) { BSA_RH(2) }
    else if (nc <= 4) { if (rh == 4) { BSA_NW(4, 4); } else if (rh == 2) { BSA_NW(2, 4); } else { BSA_NW(1, 4); } }
    else { if (rh == 2) { BSA_NW(2, 8); } else { BSA_NW(1, 8); } }
    if (nsplit > 1)
      hipLaunchKernelGGL(bsa_merge_kernel<P>, dim3(T, H), dim3(64), 0, st, (El_*)out, ldo, scratch, proj, ld, gate_col, H, E, nsplit,
                         out_scale);
  })
#undef BSA_RH
#undef BSA_NW
#undef BSA_LAUNCH
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

// ---- prompt attention on the matrix pipe (16-bit storage; D a multiple of 8, E a multiple of 16).
// Workgroup = (16 consecutive positions of one sequence, one key/value head, a block of 4 HPW of its query heads); wave w owns
// HPW heads.  The tile's keys -- from the first position's window start to the last position -- are walked in steps of 32 by
// the whole workgroup: the step's 32 cached key rows and value rows are staged ONCE into LDS (keys as cached: the A operand of
// S^T = K Q^T; values transposed: the A operand of O^T += V^T P^T) and serve every head of the workgroup; the next step's rows
// are in flight in registers while the current one is used.  Per step and head: two 16-key score tiles; the bias of the
// lane's eight (query, key) pairs, fetched by distance before the products are issued; online softmax in fp32 with base-2
// exponents, accumulators rescaled only when a maximum moved; the lane's eight weights ARE its share of the B operand of the
// value product.  Scores and weights keep fp32 accuracy on the 16-bit pipe: the fp32 queries and the fp32 weights enter as
// high + low 16-bit halves (two products each, 2^-17 relative).
constexpr float BSA_LOG2E = 1.4426950408889634f;

template <typename P> __device__ __forceinline__ void split2(float a, float b, unsigned& hi, unsigned& lo) {
  const u16 ah = P::from_f(a), bh = P::from_f(b);
  hi = (unsigned)ah | ((unsigned)bh << 16);
  lo = pack2<P>(a - P::to_f(ah), b - P::to_f(bh));
}

template <typename P, int NSM, int NVM, int HPW>
__global__ __launch_bounds__(256) void bsa_attend_mfma_kernel(u16* __restrict__ out, int ldo, const float* __restrict__ q,
                                                              UmbPagedKV kv, const float* __restrict__ proj, int ld, int gate_col,
                                                              const float* __restrict__ bias, int n_dist,
                                                              const int* __restrict__ seq_slot, const int* __restrict__ seq_row0,
                                                              const int* __restrict__ seq_pos0, const int* __restrict__ seq_len,
                                                              int H, int G, int D, int E, int window, float scale, float out_scale,
                                                              float softcap) {
  extern __shared__ __attribute__((aligned(16))) u16 bsa_lds[];
  constexpr int NLK = (NSM * 4 + 7) / 8, NLV = (NVM * 2 + 7) / 8;     // 16-byte chunks of a key / value row per staging thread
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, j = lane & 15, g4 = lane >> 4;
  const int LD = D + 8;                               // LDS row stride of the key tile: 16 bytes of padding spread the banks
  const int ns = (D + 31) >> 5, nv = E >> 4, nck = D >> 3, ncv = E >> 3;
  constexpr int LT = 36;                              // row stride of the transposed value tile: 32 keys + 8 bytes of padding
  u16* k_s = bsa_lds;                                 // [32][LD]
  u16* v_t = bsa_lds + 32 * LD;                       // [E][LT]
  const int b = blockIdx.y;
  const int n = seq_len[b], q0 = blockIdx.x * 16;
  if (q0 >= n) return;                                // the whole workgroup
  const int hpg = H / G, hblocks = (hpg + 4 * HPW - 1) / (4 * HPW);
  const int g = blockIdx.z / hblocks;
  const int hl0 = ((blockIdx.z % hblocks) * 4 + wave) * HPW;         // first of the wave's heads inside the group
  const bool active = hl0 < hpg;                      // a wave without heads still stages rows and meets the barriers
  const int slot = seq_slot[b], row0 = seq_row0[b], pos0 = seq_pos0[b];
  const int nq = n - q0 < 16 ? n - q0 : 16;
  const int i_first = pos0 + q0, i_last = i_first + nq - 1;
  const bool q_ok = j < nq;
  const int i_j = i_first + (q_ok ? j : nq - 1);
  const long qrow = row0 + q0 + (q_ok ? j : nq - 1);
  const int j_lo = i_first - window + 1 > 0 ? i_first - window + 1 : 0;
  const int total = i_last - j_lo + 1;
  const float scale2 = scale * BSA_LOG2E;
  const u16* kbase = reinterpret_cast<const u16*>(kv.k);
  const u16* vbase = reinterpret_cast<const u16*>(kv.v);
  u32x4 qh[HPW][NSM], ql[HPW][NSM];
  f32x4 o[HPW][NVM];
  float m_run[HPW], l_run[HPW];
  bool h_ok[HPW];
  int hd[HPW];
#pragma unroll
  for (int hh = 0; hh < HPW; ++hh) {
    h_ok[hh] = hl0 + hh < hpg;
    hd[hh] = g * hpg + (h_ok[hh] ? hl0 + hh : hpg - 1);
    const float* qr = q + (qrow * H + hd[hh]) * D;
#pragma unroll
    for (int s = 0; s < NSM; ++s) {
      const int d = 32 * s + 8 * g4;
      qh[hh][s] = u32x4{0u, 0u, 0u, 0u};
      ql[hh][s] = u32x4{0u, 0u, 0u, 0u};
      if (s < ns && d < D) {
        const f32x4 a = *reinterpret_cast<const f32x4*>(qr + d), c = *reinterpret_cast<const f32x4*>(qr + d + 4);
        unsigned hi[4], lo[4];
        split2<P>(a[0], a[1], hi[0], lo[0]);
        split2<P>(a[2], a[3], hi[1], lo[1]);
        split2<P>(c[0], c[1], hi[2], lo[2]);
        split2<P>(c[2], c[3], hi[3], lo[3]);
        qh[hh][s] = u32x4{hi[0], hi[1], hi[2], hi[3]};
        ql[hh][s] = u32x4{lo[0], lo[1], lo[2], lo[3]};
      }
    }
#pragma unroll
    for (int dt = 0; dt < NVM; ++dt) o[hh][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    m_run[hh] = -INFINITY;
    l_run[hh] = 0.f;
  }
  // staging role of a thread: key row sm of the step, 16-byte chunks sc, sc + 8, ... of that row (keys and values)
  const int sm = threadIdx.x & 31, sc = threadIdx.x >> 5;
  u32x4 stk[NLK], stv[NLV];
  auto fetch = [&](int base) {
    const int kx = base + sm;
    const bool ok = kx < total;
    const long offk = ok ? pkv_tok(kv, slot, j_lo + kx, g, G, D) : 0;
    const long offv = ok ? pkv_tok(kv, slot, j_lo + kx, g, G, E) : 0;
#pragma unroll
    for (int u = 0; u < NLK; ++u) {
      const int ch = sc + 8 * u;
      stk[u] = (ok && ch < nck) ? *reinterpret_cast<const u32x4*>(kbase + offk + 8 * ch) : u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int u = 0; u < NLV; ++u) {
      const int ch = sc + 8 * u;
      stv[u] = (ok && ch < ncv) ? *reinterpret_cast<const u32x4*>(vbase + offv + 8 * ch) : u32x4{0u, 0u, 0u, 0u};
    }
  };
  fetch(0);
  for (int base = 0; base < total; base += 32) {
    __syncthreads();                                  // every wave is done with the previous tile
#pragma unroll
    for (int u = 0; u < NLK; ++u) {
      const int ch = sc + 8 * u;
      if (ch < nck) *reinterpret_cast<u32x4*>(k_s + sm * LD + 8 * ch) = stk[u];
    }
#pragma unroll
    for (int u = 0; u < NLV; ++u) {
      const int ch = sc + 8 * u;
      if (ch < ncv) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          v_t[(8 * ch + 2 * e) * LT + sm] = (u16)(stv[u][e] & 0xffffu);
          v_t[(8 * ch + 2 * e + 1) * LT + sm] = (u16)(stv[u][e] >> 16);
        }
      }
    }
    __syncthreads();
    if (base + 32 < total) fetch(base + 32);          // in flight while this step is used
    if (!active) continue;
    // which of the lane's eight keys this query sees, and at what distance: the same for every head
    bool vis[8];
    int di[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int jt = j_lo + base + 16 * (e >> 2) + 4 * g4 + (e & 3);
      vis[e] = q_ok && jt <= i_j && jt > i_j - window;
      const int dd = i_j - jt;
      di[e] = dd < 0 ? 0 : (dd < n_dist ? dd : n_dist - 1);
    }
    float bv[HPW][8];
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh)
#pragma unroll
      for (int e = 0; e < 8; ++e) bv[hh][e] = bias ? bias[(long)hd[hh] * n_dist + di[e]] : 0.f;
    f32x4 sc2[HPW][2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
#pragma unroll
      for (int hh = 0; hh < HPW; ++hh) sc2[hh][u] = f32x4{0.f, 0.f, 0.f, 0.f};
      const u16* kr = k_s + (16 * u + j) * LD;
#pragma unroll
      for (int s = 0; s < NSM; ++s) {
        const int d = 32 * s + 8 * g4;
        if (s < ns) {
          const u32x4 kf = d < D ? *reinterpret_cast<const u32x4*>(kr + d) : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
          for (int hh = 0; hh < HPW; ++hh) {
            sc2[hh][u] = P::mfma(kf, ql[hh][s], sc2[hh][u]);
            sc2[hh][u] = P::mfma(kf, qh[hh][s], sc2[hh][u]);
          }
        }
      }
    }
    u32x4 ph[HPW], pl[HPW];
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
      // maxima and exponents in base 2 (scale2 = scale log2 e): one v_exp_f32 per weight
      float sv[8], mx = -INFINITY;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float raw = sc2[hh][e >> 2][e & 3] * scale2;
        if (softcap > 0.f) raw = softcap * tanhf(sc2[hh][e >> 2][e & 3] * scale / softcap) * BSA_LOG2E;      // capped, then to base 2
        sv[e] = vis[e] ? raw + bv[hh][e] * BSA_LOG2E : -INFINITY;
        mx = fmaxf(mx, sv[e]);
      }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m_run[hh], mx);
      const float m_ref = m_new == -INFINITY ? 0.f : m_new;          // a row that has seen no key yet: all weights 0
      const float fac = __builtin_amdgcn_exp2f(m_run[hh] - m_ref);
      float w[8], sum = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        w[e] = __builtin_amdgcn_exp2f(sv[e] - m_ref);
        sum += w[e];
      }
      sum += __shfl_xor(sum, 16, 64);
      sum += __shfl_xor(sum, 32, 64);
      l_run[hh] = l_run[hh] * fac + sum;
      m_run[hh] = m_new;
      if (__ballot(fac != 1.f)) {                                    // the maximum moved for some row of the tile
#pragma unroll
        for (int dt = 0; dt < NVM; ++dt) {
          if (dt < nv) { o[hh][dt][0] *= fac; o[hh][dt][1] *= fac; o[hh][dt][2] *= fac; o[hh][dt][3] *= fac; }
        }
      }
      unsigned hi[4], lo[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) split2<P>(w[2 * e], w[2 * e + 1], hi[e], lo[e]);
      ph[hh] = u32x4{hi[0], hi[1], hi[2], hi[3]};
      pl[hh] = u32x4{lo[0], lo[1], lo[2], lo[3]};
    }
    // O^T[d][query] += V^T[d][keys] P^T[keys][query]: lane (d row j of tile dt, quad g4) reads its 8 keys' values
#pragma unroll
    for (int dt = 0; dt < NVM; ++dt) {
      if (dt < nv) {
        const u16* vr = v_t + (16 * dt + j) * LT + 4 * g4;
        const u32x2 t0 = *reinterpret_cast<const u32x2*>(vr), t1 = *reinterpret_cast<const u32x2*>(vr + 16);
        const u32x4 va = u32x4{t0[0], t0[1], t1[0], t1[1]};
#pragma unroll
        for (int hh = 0; hh < HPW; ++hh) {
          o[hh][dt] = P::mfma(va, pl[hh], o[hh][dt]);
          o[hh][dt] = P::mfma(va, ph[hh], o[hh][dt]);
        }
      }
    }
  }
  // lane holds O^T[d = 16 dt + 4 g4 + rr][query j]
  if (q_ok && active) {
#pragma unroll
    for (int hh = 0; hh < HPW; ++hh) {
      if (!h_ok[hh]) continue;
      const float gt = gate_col >= 0 ? 1.f / (1.f + expf(-proj[qrow * ld + gate_col + hd[hh]])) : 1.f;
      const float inv = out_scale * gt / l_run[hh];
      u16* orow = out + qrow * ldo + (long)hd[hh] * E;
#pragma unroll
      for (int dt = 0; dt < NVM; ++dt) {
        if (dt < nv) {
#pragma unroll
          for (int rr = 0; rr < 4; ++rr) orow[16 * dt + 4 * g4 + rr] = P::from_f(o[hh][dt][rr] * inv);
        }
      }
    }
  }
}

extern "C" int umb_bsa_attend_tiled_ok(int H, int G, int D, int E, int dtype) {
  return H >= 1 && G >= 1 && H % G == 0 && (dtype == UMB_SEQ_BF16 || dtype == UMB_SEQ_F16) && D >= 8 && D % 8 == 0 && D <= 256 &&
         E >= 16 && E % 16 == 0 && E <= 256;
}

extern "C" int umb_bsa_attend_tiled(void* out, int ldo, const float* q, const UmbPagedKV* kv, const float* proj, int ld,
                                    int gate_col, const float* bias, int n_dist, const int* seq_slot, const int* seq_row0,
                                    const int* seq_pos0, const int* seq_len, int B, int max_len, int H, int G, int D, int E,
                                    int window, float scale, float out_scale, float softcap, int dtype, hipStream_t st) {
  if (B < 1 || B > 65535 || max_len < 1 || window < 1 || !out || !q || !bsa_kv_ok(kv) || !seq_slot || !seq_row0 || !seq_pos0 ||
      !seq_len || ldo < H * E || (bias && n_dist < 1) || (gate_col >= 0 && (!proj || ld < gate_col + H)) ||
      !umb_bsa_attend_tiled_ok(H, G, D, E, dtype))
    return UMB_EINVAL;
  if (!bias) n_dist = 1;
  const int hpg = H / G;
  const size_t lds = ((size_t)32 * (D + 8) + (size_t)E * 36) * sizeof(u16);
#define BSA_MFMA(NSM, NVM, HPW)                                                                                            \
  do {                                                                                                                     \
    const int hblocks = (hpg + 4 * HPW - 1) / (4 * HPW);                                                                   \
    if ((long)G * hblocks > 65535) return UMB_EINVAL;                                                                      \
    const dim3 grid((max_len + 15) / 16, B, G * hblocks);                                                                  \
    if (ensure_dynamic_lds<bsa_attend_mfma_kernel<P, NSM, NVM, HPW>>(lds) != UMB_OK) return UMB_EHIP;                      \
    hipLaunchKernelGGL((bsa_attend_mfma_kernel<P, NSM, NVM, HPW>), grid, dim3(256), lds, st, (u16*)out, ldo, q, *kv, proj, \
                       ld, gate_col, bias, n_dist, seq_slot, seq_row0, seq_pos0, seq_len, H, G, D, E, window, scale,       \
                       out_scale, softcap);                                                                                \
  } while (0)
#define BSA_MFMA_SHAPE()                                                                                                   \
  if (D <= 128 && E <= 128) { if (hpg > 4) BSA_MFMA(4, 8, 2); else BSA_MFMA(4, 8, 1); }                                    \
  else BSA_MFMA(8, 16, 1)
  if (dtype == UMB_SEQ_BF16) { using P = BF16; BSA_MFMA_SHAPE(); }
  else { using P = F16; BSA_MFMA_SHAPE(); }
#undef BSA_MFMA_SHAPE
#undef BSA_MFMA
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}
