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
#include "seq_common.h"

constexpr int MG_CH = 8;

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

extern "C" int umb_mingru_scan(void* out, float* state, const float* proj, int ld, int z_col, int u_col, int g_col,
                               const int* seq_slot, const int* seq_row0, const int* seq_pos0, const int* seq_len, int B, int Wm,
                               int dtype, hipStream_t st) {
  if (B < 1 || B > 65535 || Wm < 1 || ld < 1 || z_col < 0 || u_col < 0 || g_col < 0 || z_col + Wm > ld || u_col + Wm > ld ||
      g_col + Wm > ld || !out || !state || !proj || !seq_slot || !seq_row0 || !seq_pos0 || !seq_len)
    return UMB_EINVAL;
  DISPATCH_SEQ_DTYPE(dtype, {
    typedef typename El<P>::type E;
    hipLaunchKernelGGL(mingru_scan_kernel<P>, dim3((Wm + 255) / 256, B), dim3(256), 0, st, (E*)out, state, proj, ld, z_col, u_col,
                       g_col, seq_slot, seq_row0, seq_pos0, seq_len, Wm);
  })
  UMB_LAUNCH_CHECK();
  return UMB_OK;
}
