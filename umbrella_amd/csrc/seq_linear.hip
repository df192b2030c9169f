// General linear layer for the sequence-mixer models: out[T][N] = x[T][K] . W[N][K]^T + bias for ANY T, N, K, weights as
// stored (row-major [out][in], no repacking), 16-bit or fp32 storage, fp32 accumulation on the matrix pipe.
//
// Both operands are K-contiguous, so a lane's 8 consecutive K-elements of "its" row ARE its share of an MFMA operand:
//   v_mfma_f32_16x16x32_{bf16,f16}: A 16 rows x 32 k, lane (j = lane % 16, g = lane / 16) supplies row j, k 8g .. 8g+7
//   v_mfma_f32_16x16x4_f32 (true fp32, x8): the same 8 elements feed instruction i with element i of every lane, i.e. step i
//   multiplies k = 8g + i of A with k = 8g + i of B -- the pairing is what matters, the order inside the 32-k step is free.
// Weights are the A operand (rows = output features), tokens the B operand: lane l ends up with outputs
// (n = 4 (l / 16) + r, token = l % 16), r = 0..3.  Weights go HBM -> VGPR (every weight element is used by exactly one wave of
// a <= 64-token launch), as in the skinny GEMM of gemm.hip.
//
// A workgroup owns one 16-row output tile and up to 64 tokens; its four waves split K (wave w takes the 32-k steps w, w+4, ...)
// and their partial tiles are summed through LDS in wave order: the summation order of an output is a function of K alone,
// never of T or of the row's place in the batch.  K % 8 != 0 (or a tail) falls back to guarded element loads.
#include "seq_common.h"

template <typename P> struct Frag8 { u32x4 v; };
template <> struct Frag8<F32> { f32x4 lo, hi; };

template <typename P, bool VEC>
__device__ __forceinline__ Frag8<P> load8(const typename El<P>::type* __restrict__ row, bool ok, int k, int K) {
  Frag8<P> f;
  if constexpr (VEC) {                      // K % 8 == 0: k < K means the whole 8-group is inside, 16-byte aligned
    const bool in = ok && k < K;
    if constexpr (sizeof(typename El<P>::type) == 2) {
      f.v = in ? *reinterpret_cast<const u32x4*>(row + k) : u32x4{0u, 0u, 0u, 0u};
    } else {
      f.lo = in ? *reinterpret_cast<const f32x4*>(row + k) : f32x4{0.f, 0.f, 0.f, 0.f};
      f.hi = in ? *reinterpret_cast<const f32x4*>(row + k + 4) : f32x4{0.f, 0.f, 0.f, 0.f};
    }
  } else {
    if constexpr (sizeof(typename El<P>::type) == 2) {
      unsigned e[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) e[i] = (ok && k + i < K) ? (unsigned)row[k + i] : 0u;
      f.v = u32x4{e[0] | (e[1] << 16), e[2] | (e[3] << 16), e[4] | (e[5] << 16), e[6] | (e[7] << 16)};
    } else {
      float e[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) e[i] = (ok && k + i < K) ? row[k + i] : 0.f;
      f.lo = f32x4{e[0], e[1], e[2], e[3]};
      f.hi = f32x4{e[4], e[5], e[6], e[7]};
    }
  }
  return f;
}

template <typename P> __device__ __forceinline__ f32x4 mma8(const Frag8<P>& a, const Frag8<P>& b, f32x4 c) {
  return P::mfma(a.v, b.v, c);
}
template <> __device__ __forceinline__ f32x4 mma8<F32>(const Frag8<F32>& a, const Frag8<F32>& b, f32x4 c) {
#pragma unroll
  for (int i = 0; i < 4; ++i) c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.lo[i], b.lo[i], c, 0, 0, 0);
#pragma unroll
  for (int i = 0; i < 4; ++i) c = __builtin_amdgcn_mfma_f32_16x16x4f32(a.hi[i], b.hi[i], c, 0, 0, 0);
  return c;
}

enum { EPI_F32 = 0, EPI_DT = 1, EPI_SILU_MUL = 2, EPI_GATE = 3, EPI_RELU2 = 4, EPI_CLAMP_GLU = 5 };
// the two stacked-halves epilogues: silu(gate) * up, or the capped form g sigmoid(alpha g) (u + 1) with g = min(gate, limit),
// u = clamp(up, -limit, limit)
static inline bool epi_dual(int epi) { return epi == EPI_SILU_MUL || epi == EPI_CLAMP_GLU; }
__device__ __forceinline__ float glu_pair(int epi, float g, float u, float limit, float alpha) {
  if (epi == EPI_CLAMP_GLU) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    return g / (1.f + expf(-alpha * g)) * (u + 1.f);
  }
  return siluf_(g) * u;
}

// Where a launch departs from the dense [T][K] x [N][K] problem: row strides of x and out, a batch of independent problems
// along blockIdx.z (element strides sx / sw / so), or token tiles read from device memory (grouped: tile blockIdx.y is
// {group, first row, rows}; its weights start at w + group * gs).  EPI_GATE multiplies by sigmoid(gate[t ldg + z sg + n]).
struct LinExt {
  int ldx, ldo;
  long sx, sw, so, gs;
  const int* tiles;
  const float* gate;
  int ldg, sg;
  float limit, alpha;      // EPI_CLAMP_GLU
};
static inline LinExt lin_dense(int N, int K) { return LinExt{K, N, 0, 0, 0, 0, nullptr, nullptr, 0, 0}; }

// NT output tiles x TT token tiles of 16 per workgroup (each wave holds all NT x TT accumulator tiles of its K share: one weight
// fragment meets TT token fragments and one token fragment NT weight fragments, so a launch of many tokens moves
// 1 / NT + 1 / TT fragment loads per MFMA instead of 1 + 1 / TT); DUAL: a second weight matrix W2 = W + N * K (the "up" half)
// with its own accumulators (NT <= 2: the partial tiles of both halves share the 64 KiB of LDS).
template <typename P, int NT, int TT, bool VEC, bool DUAL>
__global__ __launch_bounds__(256) void seq_linear_kernel(void* __restrict__ out_, const typename El<P>::type* __restrict__ x,
                                                         const typename El<P>::type* __restrict__ w,
                                                         const typename El<P>::type* __restrict__ bias, int T, int N, int K,
                                                         int epi, LinExt ext) {
  typedef typename El<P>::type E;
  static_assert(!DUAL || NT <= 2, "gate and up partials of NT x TT tiles must fit the LDS");
  __shared__ float red[DUAL ? 2 : 1][4][NT * TT][256];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int j = lane & 15, g = lane >> 4;
  int t0 = blockIdx.y * (TT * 16);
  const int ldx = ext.ldx, ldo = ext.ldo;
  long obase = (long)blockIdx.z * ext.so;
  const float* gate = ext.gate ? ext.gate + (long)blockIdx.z * ext.sg : nullptr;
  x += (long)blockIdx.z * ext.sx;
  w += (long)blockIdx.z * ext.sw;
  if (ext.tiles) {                         // grouped: this workgroup's rows and weights come from the tile list
    const int* td = ext.tiles + 3 * blockIdx.y;
    const int rows = td[2];
    if (rows <= 0) return;
    w += (long)td[0] * ext.gs;
    x += (long)td[1] * ldx;
    obase += (long)td[1] * ldo;
    T = rows;
    t0 = 0;
  }
  const E* wrow[NT];
  bool n_ok[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int n_row = (blockIdx.x * NT + nt) * 16 + j;
    n_ok[nt] = n_row < N;
    wrow[nt] = w + (long)(n_ok[nt] ? n_row : 0) * K;
  }
  const long half = DUAL ? (long)N * K : 0;
  const E* xrow[TT];
  bool t_ok[TT];
#pragma unroll
  for (int tt = 0; tt < TT; ++tt) {
    const int t = t0 + tt * 16 + j;
    t_ok[tt] = t < T;
    xrow[tt] = x + (long)(t_ok[tt] ? t : 0) * ldx;
  }
  f32x4 acc[NT][TT], acc2[NT][TT];
#pragma unroll
  for (int tt = 0; tt < TT; ++tt) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) { acc[nt][tt] = f32x4{0.f, 0.f, 0.f, 0.f}; acc2[nt][tt] = f32x4{0.f, 0.f, 0.f, 0.f}; }
  }

  constexpr int UN = (NT * TT == 1) ? (DUAL ? 8 : 16) : 2;        // 32-k steps in flight per wave (a single-tile launch is latency-bound:
                                                    // K = 2048 is two round trips per wave instead of four)
  for (int k0 = wave * 32; k0 < K; k0 += 128 * UN) {
    Frag8<P> a[UN][NT], a2[UN][NT], b[UN][TT];
#pragma unroll
    for (int u = 0; u < UN; ++u) {
      const int k = k0 + u * 128 + g * 8;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        a[u][nt] = load8<P, VEC>(wrow[nt], n_ok[nt], k, K);
        if constexpr (DUAL) a2[u][nt] = load8<P, VEC>(wrow[nt] + half, n_ok[nt], k, K);
      }
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) b[u][tt] = load8<P, VEC>(xrow[tt], t_ok[tt], k, K);
    }
#pragma unroll
    for (int u = 0; u < UN; ++u) {
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          acc[nt][tt] = mma8<P>(a[u][nt], b[u][tt], acc[nt][tt]);
          if constexpr (DUAL) acc2[nt][tt] = mma8<P>(a2[u][nt], b[u][tt], acc2[nt][tt]);
        }
      }
    }
  }
#pragma unroll
  for (int tt = 0; tt < TT; ++tt) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      *reinterpret_cast<f32x4*>(&red[0][wave][nt * TT + tt][lane * 4]) = acc[nt][tt];
      if constexpr (DUAL) *reinterpret_cast<f32x4*>(&red[1][wave][nt * TT + tt][lane * 4]) = acc2[nt][tt];
    }
  }
  __syncthreads();
  // thread (l = tid / 4, r = tid % 4) finishes output (n = 4 (l / 16) + r, token = l % 16) of every tile
  const int l = threadIdx.x >> 2, r = threadIdx.x & 3;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int n = (blockIdx.x * NT + nt) * 16 + 4 * (l >> 4) + r;
    if (n >= N) continue;
    const float bv = bias ? ldf<P>(bias + n) : 0.f;
    const float bv2 = (DUAL && bias) ? ldf<P>(bias + N + n) : 0.f;
#pragma unroll
    for (int tt = 0; tt < TT; ++tt) {
      const int t = t0 + tt * 16 + (l & 15);
      if (t >= T) continue;
      float s = red[0][0][nt * TT + tt][threadIdx.x];
#pragma unroll
      for (int ww = 1; ww < 4; ++ww) s += red[0][ww][nt * TT + tt][threadIdx.x];
      s += bv;
      if constexpr (DUAL) {
        float u = red[1][0][nt * TT + tt][threadIdx.x];
#pragma unroll
        for (int ww = 1; ww < 4; ++ww) u += red[1][ww][nt * TT + tt][threadIdx.x];
        u += bv2;
        stf<P>(reinterpret_cast<E*>(out_) + obase + (long)t * ldo + n, glu_pair(epi, s, u, ext.limit, ext.alpha));
      } else if (epi == EPI_DT) {
        stf<P>(reinterpret_cast<E*>(out_) + obase + (long)t * ldo + n, s);
      } else if (epi == EPI_RELU2) {
        const float rl = fmaxf(s, 0.f);
        stf<P>(reinterpret_cast<E*>(out_) + obase + (long)t * ldo + n, rl * rl);
      } else if (epi == EPI_GATE) {
        stf<P>(reinterpret_cast<E*>(out_) + obase + (long)t * ldo + n, s / (1.f + expf(-gate[(long)t * ext.ldg + n])));
      } else {
        reinterpret_cast<float*>(out_)[obase + (long)t * ldo + n] = s;
      }
    }
  }
}

// ---- many tokens (T > 64), 16-bit storage: a 128 x 128 output tile per workgroup, operands staged through LDS.
// The skinny kernel above streams every weight once per 64 tokens and every token fragment once per 16 (or 64) output rows
// straight from L2: right when weights dominate, wasteful when both operands are re-used 128 times.  Here a stage of 64 k
// (A: 128 output rows, B: 128 tokens, 16 KiB each) is fetched with 16-byte loads into registers while the previous stage is
// consumed, written to the other half of a double-buffered 64 KiB LDS tile, and each of the four waves (2 x 2) reads the
// fragments of its 64 x 64 sub-tile from there: 8 fragment reads per 16 MFMAs, every read a contiguous KiB (the tile is
// stored as two [128 rows][32 k] halves so that a fragment's 16 rows x 64 B are adjacent: no bank conflict).
// K is summed in order inside one accumulator (no K split): results differ from the skinny kernel by rounding only.
// DUAL (gate/up): the 128 staged weight rows are 64 gate rows and the 64 up rows of the same outputs.
template <typename P, bool DUAL>
__global__ __launch_bounds__(256) void seq_linear_wide_kernel(void* __restrict__ out_, const u16* __restrict__ x,
                                                              const u16* __restrict__ w, const u16* __restrict__ bias, int T,
                                                              int N, int K, int epi, LinExt ext) {
  __shared__ __attribute__((aligned(16))) u16 tile[2][2][2][128 * 32];      // [buffer][A | B][k half][row][32 k]
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, j = lane & 15, g = lane >> 4;
  const int wm = wave >> 1, wn = wave & 1;
  int t0 = blockIdx.y * 128;
  long obase = 0;
  if (ext.tiles) {                         // grouped: a tile of up to 128 rows of one group
    const int* td = ext.tiles + 3 * blockIdx.y;
    if (td[2] <= 0) return;
    w += (long)td[0] * ext.gs;
    x += (long)td[1] * K;
    obase = (long)td[1] * N;
    T = td[2];
    t0 = 0;
  }
  const int n0 = blockIdx.x * (DUAL ? 64 : 128);
  // staging: thread owns chunks c = tid + 256 i (i < 4) of each operand's 128 x 8 chunk grid: row c / 8, 16-byte chunk c % 8
  const u16* asrc[4];
  const u16* bsrc[4];
  bool aok[4], bok[4];
  int soff[4], kc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = tid + 256 * i, row = c >> 3, ch = c & 7;
    int n = DUAL ? (row < 64 ? n0 + row : N + n0 + (row - 64)) : n0 + row;
    aok[i] = DUAL ? (n0 + (row & 63) < N) : (n < N);
    asrc[i] = w + (long)(aok[i] ? n : 0) * K + ch * 8;
    bok[i] = t0 + row < T;
    bsrc[i] = x + (long)(bok[i] ? t0 + row : 0) * K + ch * 8;
    kc[i] = ch * 8;
    soff[i] = (ch >> 2) * (128 * 32) + row * 32 + (ch & 3) * 8;
  }
  u32x4 ra[4], rb[4];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool in = k0 + kc[i] < K;
      ra[i] = (aok[i] && in) ? *reinterpret_cast<const u32x4*>(asrc[i] + k0) : u32x4{0u, 0u, 0u, 0u};
      rb[i] = (bok[i] && in) ? *reinterpret_cast<const u32x4*>(bsrc[i] + k0) : u32x4{0u, 0u, 0u, 0u};
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      *reinterpret_cast<u32x4*>(&tile[buf][0][0][0] + soff[i]) = ra[i];
      *reinterpret_cast<u32x4*>(&tile[buf][1][0][0] + soff[i]) = rb[i];
    }
  };
  int arow[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) arow[i] = DUAL ? ((i >> 1) * 64 + wm * 32 + (i & 1) * 16) : (wm * 64 + i * 16);
  f32x4 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int tt = 0; tt < 4; ++tt) acc[i][tt] = f32x4{0.f, 0.f, 0.f, 0.f};
  fetch(0);
  stash(0);
  __syncthreads();
  const int nst = (K + 63) / 64;
  for (int st = 0; st < nst; ++st) {
    const int buf = st & 1;
    if (st + 1 < nst) fetch((st + 1) * 64);
#pragma unroll
    for (int kh = 0; kh < 2; ++kh) {
      u32x4 fa[4], fb[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        fa[i] = *reinterpret_cast<const u32x4*>(&tile[buf][0][kh][(arow[i] + j) * 32 + g * 8]);
        fb[i] = *reinterpret_cast<const u32x4*>(&tile[buf][1][kh][(wn * 64 + i * 16 + j) * 32 + g * 8]);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) acc[i][tt] = P::mfma(fa[i], fb[tt], acc[i][tt]);
    }
    if (st + 1 < nst) stash(buf ^ 1);
    __syncthreads();
  }
  // lane holds outputs (row = 4 g + r of its A tile, token = j of its B tile)
#pragma unroll
  for (int tt = 0; tt < 4; ++tt) {
    const int t = t0 + wn * 64 + tt * 16 + j;
    if (t >= T) continue;
#pragma unroll
    for (int i = 0; i < (DUAL ? 2 : 4); ++i) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int n = n0 + (DUAL ? wm * 32 + i * 16 : arow[i]) + 4 * g + r;
        if (n >= N) continue;
        float sv = acc[i][tt][r] + (bias ? P::to_f(bias[n]) : 0.f);
        if constexpr (DUAL) {
          const float uv = acc[i + 2][tt][r] + (bias ? P::to_f(bias[N + n]) : 0.f);
          reinterpret_cast<u16*>(out_)[obase + (long)t * N + n] = P::from_f(glu_pair(epi, sv, uv, ext.limit, ext.alpha));
        } else if (epi == EPI_DT) {
          reinterpret_cast<u16*>(out_)[obase + (long)t * N + n] = P::from_f(sv);
        } else if (epi == EPI_RELU2) {
          const float rl = fmaxf(sv, 0.f);
          reinterpret_cast<u16*>(out_)[obase + (long)t * N + n] = P::from_f(rl * rl);
        } else {
          reinterpret_cast<float*>(out_)[obase + (long)t * N + n] = sv;
        }
      }
    }
  }
}

template <typename P>
static int launch_wide(void* out, const void* x, const void* w, const void* bias, int T, int N, int K, int epi, hipStream_t st,
                       const LinExt& ext = LinExt{0, 0, 0, 0, 0, 0, nullptr, nullptr, 0, 0}, int gy = 0) {
  if constexpr (sizeof(typename El<P>::type) == 2) {
    const unsigned ty = gy > 0 ? gy : (T + 127) / 128;
    if (epi_dual(epi))
      hipLaunchKernelGGL((seq_linear_wide_kernel<P, true>), dim3((N + 63) / 64, ty), dim3(256), 0, st, out,
                         (const u16*)x, (const u16*)w, (const u16*)bias, T, N, K, epi, ext);
    else
      hipLaunchKernelGGL((seq_linear_wide_kernel<P, false>), dim3((N + 127) / 128, ty), dim3(256), 0, st, out,
                         (const u16*)x, (const u16*)w, (const u16*)bias, T, N, K, epi, ext);
    UMB_LAUNCH_CHECK();
    return UMB_OK;
  } else {
    return UMB_EINVAL;
  }
}

// gy > 0: the number of token tiles is given (grouped launches); gz: independent problems
template <typename P, int NT, int TT, bool VEC>
static int launch_tt(void* out, const void* x, const void* w, const void* bias, int T, int N, int K, int epi, hipStream_t st,
                     const LinExt& ext, int gy = 0, int gz = 1) {
  typedef typename El<P>::type E;
  constexpr int NTD = NT > 2 ? 2 : NT;             // gate/up: two tile pairs at most
  const dim3 grid((N + NT * 16 - 1) / (NT * 16), gy > 0 ? gy : (T + TT * 16 - 1) / (TT * 16), gz);
  if (epi_dual(epi))
    hipLaunchKernelGGL((seq_linear_kernel<P, NTD, TT, VEC, true>), dim3((N + NTD * 16 - 1) / (NTD * 16), grid.y, gz), dim3(256), 0,
                       st, out, (const E*)x, (const E*)w, (const E*)bias, T, N, K, epi, ext);
  else
    hipLaunchKernelGGL((seq_linear_kernel<P, NT, TT, VEC, false>), grid, dim3(256), 0, st, out, (const E*)x, (const E*)w,
                       (const E*)bias, T, N, K, epi, ext);
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}

template <typename P, bool VEC>
static int launch_vec(void* out, const void* x, const void* w, const void* bias, int T, int N, int K, int epi, hipStream_t st,
                      const LinExt& ext, int gz = 1) {
  if (T <= 16) return launch_tt<P, 1, 1, VEC>(out, x, w, bias, T, N, K, epi, st, ext, 0, gz);
  if (T <= 32) return launch_tt<P, 1, 2, VEC>(out, x, w, bias, T, N, K, epi, st, ext, 0, gz);
  // many tokens: the launch is bound by fragment loads per MFMA, not by weight bytes -> four output tiles per workgroup
  // (the K order of every output is unchanged: a row's value does not depend on which variant computed it)
  const bool dense = gz == 1 && ext.ldx == K && ext.ldo == N && epi != EPI_GATE;
  if (T > 64 && N >= 64 && sizeof(typename El<P>::type) == 2) {
    if (VEC && dense && T >= 256 && N >= 128) return launch_wide<P>(out, x, w, bias, T, N, K, epi, st, LinExt{0, 0, 0, 0, 0, 0, nullptr, nullptr, 0, 0, ext.limit, ext.alpha});      // both operands re-used
    return launch_tt<P, 4, 4, VEC>(out, x, w, bias, T, N, K, epi, st, ext, 0, gz);
  }
  return launch_tt<P, 1, 4, VEC>(out, x, w, bias, T, N, K, epi, st, ext, 0, gz);
}

static int seq_linear_any(void* out, const void* x, const void* w, const void* bias, int T, int N, int K, int epi, float limit,
                          float alpha, int dtype, hipStream_t st) {
  if (T < 1 || N < 1 || K < 1 || epi < 0 || (epi > 2 && epi != EPI_RELU2 && epi != EPI_CLAMP_GLU) || !out || !x || !w) return UMB_EINVAL;
  if (epi_dual(epi)) {
    if (N & 1) return UMB_EINVAL;
    N >>= 1;                                   // rows of each half
  }
  LinExt ext = lin_dense(N, K);
  ext.limit = limit;
  ext.alpha = alpha;
  DISPATCH_SEQ_DTYPE(dtype, {
    if (K % 8 == 0) return launch_vec<P, true>(out, x, w, bias, T, N, K, epi, st, ext);
    return launch_vec<P, false>(out, x, w, bias, T, N, K, epi, st, ext);
  })
}

extern "C" int umb_seq_linear(void* out, const void* x, const void* w, const void* bias, int T, int N, int K, int epi, int dtype,
                              hipStream_t st) {
  if (epi == EPI_CLAMP_GLU) return UMB_EINVAL;              // that epilogue has constants: umb_seq_linear_glu
  return seq_linear_any(out, x, w, bias, T, N, K, epi, 0.f, 0.f, dtype, st);
}

extern "C" int umb_seq_linear_glu(void* out, const void* x, const void* w, const void* bias, int T, int N, int K, float limit,
                                  float alpha, int dtype, hipStream_t st) {
  if (!(limit > 0.f)) return UMB_EINVAL;
  return seq_linear_any(out, x, w, bias, T, N, K, EPI_CLAMP_GLU, limit, alpha, dtype, st);
}

extern "C" int umb_seq_linear_batched(void* out, const void* x, const void* w, int T, int N, int K, int ldx, int ldo, int batch,
                                      long sx, long sw, long so, int epi, const float* gate, int ldg, int sg, int dtype,
                                      hipStream_t st) {
  if (T < 1 || N < 1 || K < 1 || batch < 1 || batch > 65535 || ldx < K || ldo < N || !out || !x || !w ||
      !(epi == EPI_F32 || epi == EPI_DT || epi == EPI_GATE) || (epi == EPI_GATE && !gate))
    return UMB_EINVAL;
  const LinExt ext{ldx, ldo, sx, sw, so, 0, nullptr, gate, ldg, sg};
  // 16-byte loads need every row start aligned: the strides as well as K
  const bool vec = K % 8 == 0 && ldx % 8 == 0 && sx % 8 == 0 && sw % 8 == 0;
  DISPATCH_SEQ_DTYPE(dtype, {
    if (vec) return launch_vec<P, true>(out, x, w, nullptr, T, N, K, epi, st, ext, batch);
    return launch_vec<P, false>(out, x, w, nullptr, T, N, K, epi, st, ext, batch);
  })
}

static int seq_linear_grouped_any(void* out, const void* x, const void* w, const int* tiles, int max_tiles, int tile_rows, long gs,
                                  int N, int K, int epi, float limit, float alpha, int dtype, hipStream_t st) {
  if (max_tiles < 1 || max_tiles > 65535 || N < 1 || K < 1 || epi < 0 || (epi > 2 && epi != EPI_RELU2 && epi != EPI_CLAMP_GLU) || !out ||
      !x || !w || !tiles ||
      (tile_rows != 16 && tile_rows != 64 && tile_rows != 128))
    return UMB_EINVAL;
  if (epi_dual(epi)) {
    if (N & 1) return UMB_EINVAL;
    N >>= 1;
  }
  const LinExt ext{K, N, 0, 0, 0, gs, tiles, nullptr, 0, 0, limit, alpha};
  if (tile_rows == 128) {                  // many rows per group: both operands staged through LDS (16-bit storage only)
    if (dtype == UMB_SEQ_F32 || K % 8 || gs % 8) return UMB_EINVAL;
    if (dtype == UMB_SEQ_BF16) return launch_wide<BF16>(out, x, w, nullptr, 128, N, K, epi, st, ext, max_tiles);
    return launch_wide<F16>(out, x, w, nullptr, 128, N, K, epi, st, ext, max_tiles);
  }
  if (tile_rows == 16) {                   // a few rows in all (decoding): one 16-row output tile per workgroup, many workgroups
    DISPATCH_SEQ_DTYPE(dtype, {
      if (K % 8 == 0 && gs % 8 == 0) return launch_tt<P, 1, 1, true>(out, x, w, nullptr, 16, N, K, epi, st, ext, max_tiles);
      return launch_tt<P, 1, 1, false>(out, x, w, nullptr, 16, N, K, epi, st, ext, max_tiles);
    })
  }
  DISPATCH_SEQ_DTYPE(dtype, {
    if (K % 8 == 0 && gs % 8 == 0) {
      if (N >= 64 && sizeof(typename El<P>::type) == 2) return launch_tt<P, 4, 4, true>(out, x, w, nullptr, 64, N, K, epi, st, ext, max_tiles);
      return launch_tt<P, 1, 4, true>(out, x, w, nullptr, 64, N, K, epi, st, ext, max_tiles);
    }
    return launch_tt<P, 1, 4, false>(out, x, w, nullptr, 64, N, K, epi, st, ext, max_tiles);
  })
}

extern "C" int umb_seq_linear_grouped(void* out, const void* x, const void* w, const int* tiles, int max_tiles, int tile_rows,
                                      long gs, int N, int K, int epi, int dtype, hipStream_t st) {
  if (epi == EPI_CLAMP_GLU) return UMB_EINVAL;
  return seq_linear_grouped_any(out, x, w, tiles, max_tiles, tile_rows, gs, N, K, epi, 0.f, 0.f, dtype, st);
}

extern "C" int umb_seq_linear_grouped_glu(void* out, const void* x, const void* w, const int* tiles, int max_tiles, int tile_rows,
                                          long gs, int N, int K, float limit, float alpha, int dtype, hipStream_t st) {
  if (!(limit > 0.f)) return UMB_EINVAL;
  return seq_linear_grouped_any(out, x, w, tiles, max_tiles, tile_rows, gs, N, K, EPI_CLAMP_GLU, limit, alpha, dtype, st);
}
