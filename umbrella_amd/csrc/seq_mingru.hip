// Minimal gated recurrence (minGRU): the gates read only the current token, so the recurrence is linear in the state and
// runs element by element,
//     z_t = sigmoid(zr_t)      c_t = ur_t + 1/2 (ur_t >= 0) | sigmoid(ur_t) (ur_t < 0)      S_t = (1 - z_t) S_(t-1) + z_t c_t
//     out_t = S_t * silu(gr_t)
// with zr / ur / gr three column blocks of the fused input projection (fp32, biases already added).  Everything is fp32;
// only the gated output that feeds the output projection is rounded.  The state is one fp32 per (sequence slot, channel).
//
// One thread owns one channel of one sequence; consecutive threads own consecutive channels, so every load of the token loop
// is coalesced.  The loop's inputs do not depend on the recurrence: CH tokens' worth are loaded and turned into (a, b) =
// (1 - z, z c) and the output gate before the dependent chain of fused multiply-adds runs, so a long prompt costs one memory
// round trip per CH tokens, not one per token.  Steps of one token per sequence launch one thread per (sequence, channel).
//
// Long stretches (prompts) are cut into pieces of MG_PIECE tokens that run side by side: S_end = A S_start + B with
// A = prod a_t and B the piece's own scan from zero (kernel 1, one thread per (piece, channel)); a piece then folds the (A, B)
// of the pieces before it, in order, into its start state and runs its tokens (kernel 2).  The cut positions are a function
// of the position inside the step only, the arithmetic is the same fused multiply-adds in another association: results agree
// with the token-by-token form to fp32 rounding.
#include "seq_common.h"

constexpr int MG_CH = 8;
constexpr int MG_PIECE = 32;     // tokens per piece of a long stretch
constexpr int MG_LONG = 128;     // stretches from this length on are cut into pieces

template <typename P>
__global__ __launch_bounds__(256) void mingru_scan_kernel(typename El<P>::type* __restrict__ out, float* __restrict__ state,
                                                          const float* __restrict__ proj, int ld, int z_col, int u_col, int g_col,
                                                          const int* __restrict__ seq_slot, const int* __restrict__ seq_row0,
                                                          const int* __restrict__ seq_pos0, const int* __restrict__ seq_len,
                                                          int Wm) {
  const int c = blockIdx.x * 256 + threadIdx.x, b = blockIdx.y;
  if (c >= Wm) return;
  const int n = seq_len[b];
  if (n <= 0) return;
  const long row0 = seq_row0[b];
  float* sp = state + (long)seq_slot[b] * Wm + c;
  float S = seq_pos0[b] == 0 ? 0.f : *sp;
  for (int t0 = 0; t0 < n; t0 += MG_CH) {
    float zr[MG_CH], ur[MG_CH], gr[MG_CH];
#pragma unroll
    for (int e = 0; e < MG_CH; ++e) {
      const long row = row0 + (t0 + e < n ? t0 + e : n - 1);       // clamped: what it brings past the end is not used
      const float* pr = proj + row * ld + c;
      zr[e] = pr[z_col]; ur[e] = pr[u_col]; gr[e] = pr[g_col];
    }
#pragma unroll
    for (int e = 0; e < MG_CH; ++e) {
      const float z = 1.f / (1.f + expf(-zr[e]));
      const float cand = ur[e] >= 0.f ? ur[e] + 0.5f : 1.f / (1.f + expf(-ur[e]));
      zr[e] = 1.f - z;
      ur[e] = z * cand;
      gr[e] = siluf_(gr[e]);
    }
#pragma unroll
    for (int e = 0; e < MG_CH; ++e) {
      if (t0 + e < n) {
        S = zr[e] * S + ur[e];
        stf<P>(out + (row0 + t0 + e) * Wm + c, S * gr[e]);
      }
    }
  }
  *sp = S;
}

// (a_t, b_t, gate_t) of CH tokens from row `row`, clamped at `last`
__device__ __forceinline__ void mg_load(const float* __restrict__ proj, int ld, int z_col, int u_col, int g_col, long row, long last,
                                        int c, float* a, float* b, float* g, bool want_g) {
  float zr[MG_CH], ur[MG_CH], gr[MG_CH];
#pragma unroll
  for (int e = 0; e < MG_CH; ++e) {
    const float* pr = proj + (row + e < last ? row + e : last) * ld + c;
    zr[e] = pr[z_col]; ur[e] = pr[u_col]; gr[e] = want_g ? pr[g_col] : 0.f;
  }
#pragma unroll
  for (int e = 0; e < MG_CH; ++e) {
    const float z = 1.f / (1.f + expf(-zr[e]));
    const float cand = ur[e] >= 0.f ? ur[e] + 0.5f : 1.f / (1.f + expf(-ur[e]));
    a[e] = 1.f - z;
    b[e] = z * cand;
    g[e] = want_g ? siluf_(gr[e]) : 0.f;
  }
}

// kernel 1 of the long form: (A, B) of every piece; grid (channels / 256, pieces of the longest stretch, sequences);
// ab [sequence][piece][2][Wm]
// The first piece starts from the carried state (zero for a sequence at position 0) and leaves a copy of it in init [B][Wm]:
// the second kernel, whose last piece overwrites the state while others still start, never reads the state array.
__global__ __launch_bounds__(256) void mingru_piece_kernel(float* __restrict__ ab, float* __restrict__ init,
                                                           const float* __restrict__ state, const float* __restrict__ proj, int ld,
                                                           int z_col, int u_col, const int* __restrict__ seq_slot,
                                                           const int* __restrict__ seq_row0, const int* __restrict__ seq_pos0,
                                                           const int* __restrict__ seq_len, int Wm) {
  const int c = blockIdx.x * 256 + threadIdx.x, pc = blockIdx.y, b = blockIdx.z;
  const int t0 = pc * MG_PIECE, len = seq_len[b];
  if (c >= Wm || t0 >= len) return;
  const int n = len - t0 < MG_PIECE ? len - t0 : MG_PIECE;
  const long row0 = seq_row0[b] + t0, last = row0 + n - 1;
  float A = 1.f, Bv = 0.f;
  if (pc == 0) {
    Bv = seq_pos0[b] == 0 ? 0.f : state[(long)seq_slot[b] * Wm + c];
    init[(long)b * Wm + c] = Bv;
  }
  for (int i = 0; i < n; i += MG_CH) {
    float a[MG_CH], bb[MG_CH], g[MG_CH];
    mg_load(proj, ld, z_col, u_col, 0, row0 + i, last, c, a, bb, g, false);
#pragma unroll
    for (int e = 0; e < MG_CH; ++e)
      if (i + e < n) { A *= a[e]; Bv = a[e] * Bv + bb[e]; }
  }
  const long q = (long)b * gridDim.y + pc;
  ab[(q * 2) * Wm + c] = A;
  ab[(q * 2 + 1) * Wm + c] = Bv;
}

// kernel 2: a piece's start state from the pieces before it, in order, then its tokens; the last piece stores the state
template <typename P>
__global__ __launch_bounds__(256) void mingru_long_kernel(typename El<P>::type* __restrict__ out, float* __restrict__ state,
                                                          const float* __restrict__ ab, const float* __restrict__ init,
                                                          const float* __restrict__ proj, int ld, int z_col, int u_col, int g_col,
                                                          const int* __restrict__ seq_slot,
                                                          const int* __restrict__ seq_row0, const int* __restrict__ seq_pos0,
                                                          const int* __restrict__ seq_len, int Wm) {
  const int c = blockIdx.x * 256 + threadIdx.x, pc = blockIdx.y, b = blockIdx.z;
  const int t0 = pc * MG_PIECE, len = seq_len[b];
  if (c >= Wm || t0 >= len) return;
  const int n = len - t0 < MG_PIECE ? len - t0 : MG_PIECE;
  float* sp = state + (long)seq_slot[b] * Wm + c;
  float S = pc == 0 ? init[(long)b * Wm + c] : 0.f;       // piece 0's summary already starts from the carried state
  for (int k = 0; k < pc; ++k) {
    const long q = (long)b * gridDim.y + k;
    S = ab[(q * 2) * Wm + c] * S + ab[(q * 2 + 1) * Wm + c];
  }
  const long row0 = seq_row0[b] + t0, last = row0 + n - 1;
  for (int i = 0; i < n; i += MG_CH) {
    float a[MG_CH], bb[MG_CH], g[MG_CH];
    mg_load(proj, ld, z_col, u_col, g_col, row0 + i, last, c, a, bb, g, true);
#pragma unroll
    for (int e = 0; e < MG_CH; ++e) {
      if (i + e < n) {
        S = a[e] * S + bb[e];
        stf<P>(out + (row0 + i + e) * Wm + c, S * g[e]);
      }
    }
  }
  if (t0 + n == len) *sp = S;
}

extern "C" long umb_mingru_scratch_floats(int T, int B, int Wm) {
  return ((long)(T / MG_PIECE) + B) * 2 * Wm + (long)B * Wm;      // the piece summaries of a step of T rows in B stretches + start states
}

extern "C" int umb_mingru_scan(void* out, float* state, const float* proj, int ld, int z_col, int u_col, int g_col,
                               const int* seq_slot, const int* seq_row0, const int* seq_pos0, const int* seq_len, int B, int Wm,
                               int max_len, float* scratch, long scratch_floats, int dtype, hipStream_t st) {
  if (B < 1 || B > 65535 || Wm < 1 || ld < 1 || z_col < 0 || u_col < 0 || g_col < 0 || z_col + Wm > ld || u_col + Wm > ld ||
      g_col + Wm > ld || !out || !state || !proj || !seq_slot || !seq_row0 || !seq_pos0 || !seq_len)
    return UMB_EINVAL;
  const int pieces = (max_len + MG_PIECE - 1) / MG_PIECE;
  if (max_len >= MG_LONG && scratch && pieces <= 65535 && ((long)B * pieces * 2 + B) * Wm <= scratch_floats) {
    const dim3 grid((Wm + 255) / 256, pieces, B);
    float* init = scratch + (long)B * pieces * 2 * Wm;
    hipLaunchKernelGGL(mingru_piece_kernel, grid, dim3(256), 0, st, scratch, init, state, proj, ld, z_col, u_col, seq_slot, seq_row0,
                       seq_pos0, seq_len, Wm);
    DISPATCH_SEQ_DTYPE(dtype, {
      typedef typename El<P>::type E;
      hipLaunchKernelGGL(mingru_long_kernel<P>, grid, dim3(256), 0, st, (E*)out, state, scratch, init, proj, ld, z_col, u_col, g_col,
                         seq_slot, seq_row0, seq_pos0, seq_len, Wm);
    })
    UMB_LAUNCH_CHECK();
    return UMB_OK;
  }
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    hipLaunchKernelGGL(mingru_scan_kernel<P>, dim3((Wm + 255) / 256, B), dim3(256), 0, st, (E*)out, state, proj, ld, z_col, u_col,
                       g_col, seq_slot, seq_row0, seq_pos0, seq_len, Wm);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}
