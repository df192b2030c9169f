// Forward pass of a sequence-mixer stack: walks the layer list of a UmbSeqModel and launches the kernels of
// seq_linear / seq_norm / seq_gla / seq_pwattn on one stream.  A layer is
//     x <- x + norm1b(mixer(norm1(x)))      x <- x + norm2b(ff(norm2(x)))    (the second only where the layer has one)
// with every norm a grouped RMS norm.  The seam kernel (resid_norm) adds a sublayer's normed output into the fp32 residual
// stream and produces the next sublayer's normed input in one pass, so a layer is
//     attention: proj GEMM | rope + unit-norm + append | pool | attend (matrix pipe for prompts) | out GEMM | seam | gate-up GEMM (SiLU*up epilogue) |
//                down GEMM | seam
//     GLA:       proj GEMM | decay | scan | head norm * SiLU gate | out GEMM | seam (| feed-forward as above)
//     minGRU:    proj GEMM ([z | x | g], biases in the GEMM) | scan with the output gate | out GEMM | seam
//     attention beside a state-space layer (both read the same input, one fused proj GEMM, one out GEMM over [a | b]):
//                norms + temperature + append | attend  ||  convolution + dt + decay | state ring | scan | gate + norm
//     retention: proj GEMM ([q | k | v | g]) | rotary + constants | decay rows | scan | per-head unit RMS * SiLU gate | out GEMM
//     convolved attention beside a matrix memory (one fused proj GEMM, one out GEMM over [a | b]):
//                convolution + whole-row norms + rotary + append | ring | attend (capped scores)  ||  gates + running maximum |
//                scaled queries + widened values | scan | stabilised division + per-head norm + sigmoid gate
// Stacks whose two sublayers read the SAME residual (UmbSeqModel.block = UMB_BLOCK_PARALLEL) run mixer and feed-forward from two
// normed inputs and meet in one seam per layer; a layer may ask for the embedding row to be added again in front of it.
// Models with several residual streams (UmbSeqModel.streams >= 1) use the stream seam instead: write of the sublayer behind
// it and read (combination + norm) of the one ahead in one launch.
// Nothing here depends on the host between launches: a step can be captured into a hipGraph.
#include "seq_common.h"

#define SEQ_TRY(call)            \
  do {                           \
    const int rc__ = (call);     \
    if (rc__ != UMB_OK) return rc__; \
  } while (0)

static inline int lin(const UmbSeqLinear& l, void* out, const void* x, int T, int epi, int dtype, hipStream_t st) {
  return umb_seq_linear(out, x, l.w, l.bias, T, l.N, l.K, epi, dtype, st);
}

static const void* first_norm_of(const UmbSeqModel* m, int l) { return l < m->L ? m->layers[l].norm1 : nullptr; }

// What a sublayer reads.  With a pre-norm the seam kernel has already left norm(x) * w in ws->h.  Without one the sublayer
// reads the residual stream itself through the causal convolution x + conv(x), whose last inputs are the sequence's state.
static int sublayer_input(const UmbSeqModel* m, const UmbSeqWork* ws, const UmbSeqStep* s, const void* pre_norm, const void* canon,
                          float* canon_state, bool h_ready, hipStream_t st) {
  const int T = s->T, W = m->W, dt = m->dtype;
  if (pre_norm) return canon ? UMB_EINVAL : UMB_OK;           // a convolution on normed inputs is not implemented
  if (h_ready) return UMB_OK;                                 // the seam before it has already run the convolution
  if (!canon) return UMB_EINVAL;                              // every design so far has one of the two
  if (s->max_len == 1) return umb_canon_step(ws->h, ws->x, canon, canon_state, s->pos, s->slot, T, W, m->canon_taps, dt, st);
  SEQ_TRY(umb_canon_conv(ws->h, ws->x, canon, canon_state, s->pos, s->slot, T, W, m->canon_taps, dt, st));
  return umb_canon_update(canon_state, ws->x, s->seq_slot, s->seq_row0, s->seq_pos0, s->seq_len, s->B, W, m->canon_taps, st);
}

// The seam behind a sublayer: x <- x + norm(y) * w_post, and what the NEXT sublayer reads.  With a pre-norm that is
// norm(x) * w_next (same kernel).  Without one, a step of one token per sequence also runs the next sublayer's convolution
// and state update here (*h_ready); longer steps leave it to sublayer_input, where a token's neighbours are complete.
static int seam(const UmbSeqModel* m, const UmbSeqWork* ws, const UmbSeqStep* s, const void* w_post, const void* w_next,
                const void* next_canon, float* next_state, bool* h_ready, hipStream_t st) {
  const int T = s->T, W = m->W;
  *h_ready = false;
  if (!w_next && next_canon && s->max_len == 1 && umb_seq_resid_canon_step_ok(W, m->groups)) {
    *h_ready = true;
    return umb_seq_resid_canon_step(ws->x, ws->h, ws->y, w_post, next_canon, next_state, s->pos, s->slot, T, W, m->groups,
                                    m->canon_taps, m->eps, m->dtype, st);
  }
  return umb_seq_resid_norm(ws->x, ws->h, ws->y, w_post, w_next, T, W, m->groups, m->eps, m->dtype, st);
}

// the first product of a feed-forward with its activation as epilogue: silu(gate) * up or the capped form over stacked
// [gate; up], or relu(up)^2
static int lin_act(const UmbSeqLayer& ly, const UmbSeqLinear& l, float limit, void* out, const void* x, int T, int dt, hipStream_t st) {
  if (ly.act_kind == UMB_ACT_CLAMP_GLU) return umb_seq_linear_glu(out, x, l.w, l.bias, T, l.N, l.K, limit, ly.act_alpha, dt, st);
  return lin(l, out, x, T, ly.act_kind == UMB_ACT_RELU2 ? 4 : 2, dt, st);
}

// feed-forward of h_in (dtype [T][W]) into y_out (fp32 [T][W])
static int feed_forward(const UmbSeqModel* m, const UmbSeqLayer& ly, const UmbSeqWork* ws, const UmbSeqStep* s, const void* h_in,
                        float* y_out, hipStream_t st) {
  const int T = s->T, W = m->W, dt = m->dtype;
  const int epi = ly.act_kind == UMB_ACT_RELU2 ? 4 : 2, stack = ly.act_kind == UMB_ACT_RELU2 ? 1 : 2;
  if (ly.ff_kind == UMB_FF_GATED) {
    SEQ_TRY(lin_act(ly, ly.gu, ly.act_limit, ws->act, h_in, T, dt, st));
    return lin(ly.down, y_out, ws->act, T, 0, dt, st);
  }
  if (ly.ff_kind == UMB_FF_POLYNORM) {
    if (!ly.act || ly.gu.N != ly.ff) return UMB_EINVAL;
    SEQ_TRY(lin(ly.gu, ws->proj, h_in, T, 0, dt, st));                         // "up" alone
    SEQ_TRY(umb_polynorm(ws->act, ws->proj, ly.act, T, ly.ff, m->eps, dt, st));
    return lin(ly.down, y_out, ws->act, T, 0, dt, st);
  }
  if (ly.ff_kind == UMB_FF_MOE) {
    const int E = ly.experts, top = ly.top, F = ly.expert_ff;
    if (E < 1 || top < 1 || top > E || F < 1 || !ly.e_gu || !ly.e_down || !ws->moe_sel || !ws->moe_wt || !ws->moe_pos ||
        !ws->moe_tiles || !ws->moe_xs || !ws->moe_act || !ws->moe_y || ly.router.N != E + (ly.shared_gate ? 1 : 0))
      return UMB_EINVAL;
    const bool top_logits = ly.route_kind == UMB_ROUTE_TOP_LOGITS;
    if (ly.shared_gate && (!top_logits || !ly.s_gu.w)) return UMB_EINVAL;      // the gated shared expert comes with that routing
    const long pairs = (long)T * top;
    // many rows per expert (prompts): tiles of 128 rows on the LDS-staged kernel; few (decoding): tiles of 64, weights streamed
    // a handful of rows in all: tiles of 16, one output tile per workgroup
    const int tr = (dt != UMB_SEQ_F32 && pairs >= 64L * E && W % 8 == 0 && F % 8 == 0) ? 128 : (pairs <= 64 ? 16 : 64);
    const int max_tiles = (int)((pairs + tr - 1) / tr) + E;
    if (max_tiles > ws->moe_max_tiles) return UMB_EINVAL;
    if (ly.s_gu.w) {                                                           // the shared expert sees every token
      SEQ_TRY(lin_act(ly, ly.s_gu, ly.shared_limit, ws->act, h_in, T, dt, st));
      SEQ_TRY(lin(ly.s_down, y_out, ws->act, T, 0, dt, st));
    }
    SEQ_TRY(lin(ly.router, ws->proj, h_in, T, 0, dt, st));
    // sigmoid routing weighs the expert's input, the softmax kinds its output
    const bool w_out = ly.route_kind != UMB_ROUTE_SIGMOID_IN;
    if (top_logits) SEQ_TRY(umb_moe_route_top(ws->moe_sel, ws->moe_wt, ws->proj, ly.router.N, T, E, top, st));
    else if (w_out) SEQ_TRY(umb_moe_route_softmax(ws->moe_sel, ws->moe_wt, ws->proj, ly.correction, T, E, top, st));
    else SEQ_TRY(umb_moe_route(ws->moe_sel, ws->moe_wt, ws->proj, T, E, top, st));
    SEQ_TRY(umb_moe_plan(ws->moe_pos, ws->moe_tiles, ws->moe_sel, T, E, top, max_tiles, tr, st));
    SEQ_TRY(umb_moe_scatter(ws->moe_xs, h_in, w_out ? nullptr : ws->moe_wt, ws->moe_pos, T, W, top, dt, st));
    if (ly.act_kind == UMB_ACT_CLAMP_GLU)
      SEQ_TRY(umb_seq_linear_grouped_glu(ws->moe_act, ws->moe_xs, ly.e_gu, ws->moe_tiles, max_tiles, tr, 2L * F * W, 2 * F, W,
                                         ly.act_limit, ly.act_alpha, dt, st));
    else
      SEQ_TRY(umb_seq_linear_grouped(ws->moe_act, ws->moe_xs, ly.e_gu, ws->moe_tiles, max_tiles, tr, (long)stack * F * W, stack * F, W,
                                     epi, dt, st));
    SEQ_TRY(umb_seq_linear_grouped(ws->moe_y, ws->moe_act, ly.e_down, ws->moe_tiles, max_tiles, tr, (long)W * F, W, F, 0, dt, st));
    if (top_logits)                                       // the shared expert's output times the sigmoid of the extra router row
      return umb_moe_combine_gated(y_out, ly.s_gu.w ? y_out : nullptr, ws->moe_y, ws->moe_wt, ws->moe_pos,
                                   ly.shared_gate ? ws->proj + E : nullptr, ly.router.N, T, W, top, st);
    if (w_out) return umb_moe_combine_weighted(y_out, ws->moe_y, ws->moe_wt, ws->moe_pos, T, W, top, ly.s_gu.w ? 1 : 0, st);
    return umb_moe_combine(y_out, ws->moe_y, ws->moe_pos, T, W, top, ly.s_gu.w ? 1 : 0, st);
  }
  return UMB_EINVAL;
}

// minGRU: proj = [z | x | g] with the biases of z and x added by the product; the scan applies the output gate
static int mix_mingru(const UmbSeqModel* m, const UmbSeqLayer& ly, const UmbSeqWork* ws, const UmbSeqStep* s, hipStream_t st) {
  const int Wm = ly.dim;
  if (ly.proj.N != 3 * Wm || !ly.state || ly.out.K != Wm) return UMB_EINVAL;
  // ws->aux holds the piece summaries of long stretches (sized by the runtime: umb_mingru_scratch_floats of Tmax rows)
  return umb_mingru_scan(ws->mix, ly.state, ws->proj, 3 * Wm, 0, Wm, 2 * Wm, s->seq_slot, s->seq_row0, s->seq_pos0, s->seq_len, s->B,
                         Wm, s->max_len, ws->aux, umb_mingru_scratch_floats(s->T, s->B, Wm), m->dtype, st);
}

// softmax attention with a distance bias beside a state-space layer; both read the projection of the same input and write
// their halves of the row that the one output projection reads: [scale_a * attention | scale_b * state space]
static int mix_attn_ssd(const UmbSeqModel* m, const UmbSeqLayer& ly, const UmbSeqWork* ws, const UmbSeqStep* s, hipStream_t st) {
  const int T = s->T, dt = m->dtype, ld = ly.proj.N;
  const int H = ly.heads, G = ly.kv_heads, D = ly.dim, E = ly.vdim;
  const int sH = ly.s_heads, sDv = ly.s_vdim, N = ly.s_state, sG = ly.s_groups;
  if (H < 1 || G < 1 || sH < 1 || sG < 1) return UMB_EINVAL;
  const int gate_col = H * D + G * D + G * E, col0 = gate_col + H;
  const int inner = sH * sDv, C = inner + 2 * sG * N, lds = C + inner, ldo = H * E + inner;
  if (ld != col0 + 2 * inner + 2 * sG * N + sH || ly.out.K != ldo || !ly.state) return UMB_EINVAL;
  float* q = ws->aux;                                        // [T][H D] | [T][lds] | [T][sH] | [T][sH] | scratch
  float* sx = q + (size_t)T * H * D;
  float* alpha = sx + (size_t)T * lds;
  float* log_alpha = alpha + (size_t)T * sH;
  float* spare2 = log_alpha + (size_t)T * sH;
  const long spare2_floats = ws->aux_floats - (long)(spare2 - ws->aux);
  SEQ_TRY(umb_bsa_prep(q, &ly.kv, ws->proj, ld, ly.q_norm, ly.k_norm, s->pos, s->slot, T, H, G, D, E, ly.temp_coef, ly.temp_every,
                       m->eps, dt, st));
  if (s->max_len >= 16 && umb_bsa_attend_tiled_ok(H, G, D, E, dt))
    SEQ_TRY(umb_bsa_attend_tiled(ws->mix, ldo, q, &ly.kv, ws->proj, ld, gate_col, ly.dist_bias, ly.n_dist, s->seq_slot, s->seq_row0,
                                 s->seq_pos0, s->seq_len, s->B, s->max_len, H, G, D, E, ly.window, ly.scale, ly.mix_scale_a, 0.f, dt, st));
  else {
    // what the step leaves free of aux holds the partial results of split keys (the state-space part below uses sx / alpha
    // after the attention is done, so its region may be used too, but the queries may not)
    float* spare = q + (size_t)T * H * D;
    const long spare_floats = ws->aux_floats - (long)T * H * D;
    SEQ_TRY(umb_bsa_attend(ws->mix, ldo, q, &ly.kv, ws->proj, ld, gate_col, ly.dist_bias, ly.n_dist, s->pos, s->slot, T, H, G, D, E,
                           ly.window, ly.scale, ly.mix_scale_a, 0.f, spare_floats > 0 ? spare : nullptr, spare_floats, dt, st));
  }
  const int single = s->max_len == 1;                       // one token per sequence: the ring is updated inside prep
  SEQ_TRY(umb_ssd_prep(sx, lds, alpha, log_alpha, ws->proj, ld, col0, ly.s_conv, ly.s_conv_b, ly.s_conv_state, ly.s_dt_bias, ly.s_a_log, s->pos,
                       s->slot, T, sH, sDv, sG, N, ly.s_taps, single, dt, st));
  if (!single)
    SEQ_TRY(umb_ssd_conv_update(ly.s_conv_state, ws->proj, ld, col0 + inner, s->seq_slot, s->seq_row0, s->seq_pos0, s->seq_len,
                                s->B, C, ly.s_taps, st));
  // stretches of many tokens: the recurrence in chunks side by side, where the shape is covered and the scratch suffices
  const long need = s->max_len >= 64 ? umb_ssd_scan_chunked_floats(s->B, s->max_len, sH, N, sDv) : 0;
  if (need > 0 && need <= spare2_floats && (long)s->B * sH <= 65535)
    SEQ_TRY(umb_ssd_scan_chunked(ws->o, ly.state, sx + inner + sG * N, lds, sx + inner, lds, sx, lds, log_alpha, sG, s->seq_slot,
                                 s->seq_row0, s->seq_pos0, s->seq_len, s->B, s->max_len, sH, N, sDv, spare2, spare2_floats, st));
  else
    SEQ_TRY(umb_lin_scan(ws->o, ly.state, sx + inner + sG * N, lds, sx + inner, lds, sx, lds, alpha, 1, sG, s->seq_slot, s->seq_row0,
                         s->seq_pos0, s->seq_len, s->B, sH, N, sDv, 1.f, st));
  void* right = static_cast<char*>(ws->mix) + (size_t)H * E * seq_elem_bytes(dt);
  return umb_ssd_gate(right, ldo, ws->o, sx, lds, C, ws->proj, ld, col0, ly.s_d, ly.s_norm, T, sH, sDv, ly.s_norm_groups, m->eps,
                      ly.mix_scale_b, dt, st);
}

static inline long al4(long n) { return (n + 3) & ~3L; }

// the recurrence S <- a S + k v^T, o = S^T q with one decay per head: chunks side by side for stretches of many tokens where the
// shape is covered and the scratch suffices, token by token otherwise
static int scan_per_head(float* o, float* state, const float* q, int ldq, const float* k, int ldk, const float* v, int ldv,
                         const float* alpha, const float* log_alpha, const UmbSeqStep* s, int H, int D, int P, float* scratch,
                         long scratch_floats, hipStream_t st) {
  const long need = s->max_len >= 64 ? umb_ssd_scan_chunked_floats(s->B, s->max_len, H, D, P) : 0;
  if (need > 0 && need <= scratch_floats && (long)s->B * H <= 65535)
    return umb_ssd_scan_chunked(o, state, q, ldq, k, ldk, v, ldv, log_alpha, H, s->seq_slot, s->seq_row0, s->seq_pos0, s->seq_len, s->B,
                                s->max_len, H, D, P, scratch, scratch_floats, st);
  return umb_lin_scan(o, state, q, ldq, k, ldk, v, ldv, alpha, 1, H, s->seq_slot, s->seq_row0, s->seq_pos0, s->seq_len, s->B, H, D, P,
                      1.f, st);
}

// retention: proj = [q | k | v | g]; rotary on q and k (k times its constant), the scan with the heads' fixed decays, per-head
// unit RMS times silu(g)
static int mix_retention(const UmbSeqModel* m, const UmbSeqLayer& ly, const UmbSeqWork* ws, const UmbSeqStep* s, hipStream_t st) {
  const int T = s->T, dt = m->dtype, ld = ly.proj.N, H = ly.heads, D = ly.dim, Dv = ly.vdim, HD = H * D;
  if (H < 1 || ld != 2 * HD + 2 * H * Dv || !ly.state || !ly.decay || ly.out.K != H * Dv) return UMB_EINVAL;
  float* qk = ws->aux;                                       // [T][2 H D] | alpha [T][H] | log alpha [T][H] | scratch
  float* alpha = qk + al4((long)T * 2 * HD);
  float* log_alpha = alpha + al4((long)T * H);
  float* spare = log_alpha + al4((long)T * H);
  const long spare_floats = ws->aux_floats - (long)(spare - ws->aux);
  if (spare_floats < 0) return UMB_EINVAL;
  SEQ_TRY(umb_rope_scale(qk, 2 * HD, ws->proj, ld, s->pos, ly.rot_freq, T, 2 * H, D, ly.rot_dims, ly.rot_layout, H, 1.f, ly.qscale, st));
  SEQ_TRY(umb_decay_fill(alpha, log_alpha, ly.decay, T, H, st));
  SEQ_TRY(scan_per_head(ws->o, ly.state, qk, 2 * HD, qk + HD, 2 * HD, ws->proj + 2 * HD, ld, alpha, log_alpha, s, H, D, Dv, spare,
                        spare_floats, st));
  return umb_head_gate(ws->mix, H * Dv, ws->o, Dv, -1, nullptr, ws->proj, ld, 2 * HD + H * Dv, nullptr, 0, 0, T, H, Dv, m->eps, 1.f, dt,
                       st);
}

// softmax attention behind a short convolution beside a matrix memory with exponential gates; both read the projection of the
// same input and write their halves of the row that the one output projection reads: [scale_a * attention | scale_b * memory]
static int mix_attn_mlstm(const UmbSeqModel* m, const UmbSeqLayer& ly, const UmbSeqWork* ws, const UmbSeqStep* s, hipStream_t st) {
  const int T = s->T, dt = m->dtype, ld = ly.proj.N;
  const int H = ly.heads, G = ly.kv_heads, D = ly.dim, E = ly.vdim;
  const int Hm = ly.m_heads, Dm = ly.m_dim, Em = ly.m_vdim, Pp = ly.m_pad;
  if (H < 1 || G < 1 || Hm < 1 || Pp <= Em) return UMB_EINVAL;
  const int C = H * D + G * D + G * E;                       // convolved channels
  const int mq = C, mk = mq + Hm * Dm, mv = mk + Hm * Dm, mg = mv + Hm * Em, ic = mg + Hm * Em, fc = ic + Hm;
  const int ldo = H * E + Hm * Em;
  if (ld != fc + Hm || ly.out.K != ldo || !ly.state || !ly.m_max || ly.c_taps < 1) return UMB_EINVAL;
  float* q = ws->aux;                                        // [T][H D] | qs | vp | input weights | alpha | log alpha | m | scratch
  float* qs = q + al4((long)T * H * D);
  float* vp = qs + al4((long)T * Hm * Dm);
  float* bw = vp + al4((long)T * Hm * Pp);
  float* alpha = bw + al4((long)T * Hm);
  float* log_alpha = alpha + al4((long)T * Hm);
  float* mrun = log_alpha + al4((long)T * Hm);
  float* spare2 = mrun + al4((long)T * Hm);
  const long spare2_floats = ws->aux_floats - (long)(spare2 - ws->aux);
  if (spare2_floats < 0) return UMB_EINVAL;
  const int single = s->max_len == 1;                        // one token per sequence: the ring is refreshed inside prep
  // (what lies behind the queries is scratch until the memory's part begins: the convolved row of few-token steps, split keys)
  SEQ_TRY(umb_cva_prep(q, &ly.kv, ws->proj, ld, ly.c_conv, ly.c_conv_state, ly.q_norm, ly.k_norm, s->pos, s->slot, ly.rot_freq, T, H, G,
                       D, E, ly.c_taps, ly.rot_dims, ly.rot_layout, single, m->eps, qs, ws->aux_floats - (long)(qs - ws->aux), dt, st));
  if (!single && ly.c_conv)
    SEQ_TRY(umb_ssd_conv_update(ly.c_conv_state, ws->proj, ld, 0, s->seq_slot, s->seq_row0, s->seq_pos0, s->seq_len, s->B, C, ly.c_taps, st));
  if (s->max_len >= 16 && umb_bsa_attend_tiled_ok(H, G, D, E, dt))
    SEQ_TRY(umb_bsa_attend_tiled(ws->mix, ldo, q, &ly.kv, ws->proj, ld, -1, nullptr, 0, s->seq_slot, s->seq_row0, s->seq_pos0, s->seq_len,
                                 s->B, s->max_len, H, G, D, E, ly.window, ly.scale, ly.mix_scale_a, ly.softcap, dt, st));
  else                                                       // the memory's regions are written after the attention: scratch now
    SEQ_TRY(umb_bsa_attend(ws->mix, ldo, q, &ly.kv, ws->proj, ld, -1, nullptr, 0, s->pos, s->slot, T, H, G, D, E, ly.window, ly.scale,
                           ly.mix_scale_a, ly.softcap, qs, ws->aux_floats - (long)(qs - ws->aux), dt, st));
  const float qscale = 1.f / sqrtf((float)Dm);
  if (single)
    SEQ_TRY(umb_mlstm_step(qs, vp, log_alpha, alpha, mrun, ly.m_max, ws->proj, ld, mq, mv, ic, fc, s->pos, s->slot, T, Hm, Dm, Em, Pp,
                           qscale, ly.gate_cap, st));
  else {
    SEQ_TRY(umb_mlstm_mscan(log_alpha, alpha, mrun, bw, ly.m_max, ws->proj, ld, ic, fc, ly.gate_cap, s->seq_slot, s->seq_row0, s->seq_pos0,
                            s->seq_len, s->B, Hm, st));
    SEQ_TRY(umb_mlstm_prep(qs, vp, ws->proj, ld, mq, mv, bw, T, Hm, Dm, Em, Pp, qscale, st));
  }
  SEQ_TRY(scan_per_head(ws->o, ly.state, qs, Hm * Dm, ws->proj + mk, ld, vp, Hm * Pp, alpha, log_alpha, s, Hm, Dm, Pp, spare2,
                        spare2_floats, st));
  void* right = static_cast<char*>(ws->mix) + (size_t)H * E * seq_elem_bytes(dt);
  return umb_head_gate(right, ldo, ws->o, Pp, Em, mrun, ws->proj, ld, mg, ly.m_norm, 1, 1, T, Hm, Em, m->eps, ly.mix_scale_b, dt, st);
}

// the mixer of one layer: from the fused projection in ws->proj to the row ws->mix that the output projection reads
static int run_mixer(const UmbSeqModel* m, const UmbSeqLayer& ly, const UmbSeqWork* ws, const UmbSeqStep* s, hipStream_t st) {
  const int T = s->T, dt = m->dtype, ld = ly.proj.N;
  const float eps = m->eps;
  if (ly.kind == UMB_MIX_POOLED_WINDOW) {
    const int H = ly.heads, G = ly.kv_heads, D = ly.dim;
    if (ly.vdim != D || ld != H * D + G * D + H) return UMB_EINVAL;
    SEQ_TRY(umb_pwa_prep(ws->aux, &ly.kv, ws->proj, ld, s->pos, s->slot, ly.rot_freq, T, H, G, D, ly.rot_dims, eps, dt, st));
    SEQ_TRY(umb_pwa_pool(&ly.kv, s->seq_slot, s->seq_pos0, s->seq_len, s->B, s->max_len, G, D, ly.pool, dt, st));
    // steps that bring stretches of a sequence (prompts) take the matrix-pipe kernel where the shape allows it
    if (dt != UMB_SEQ_F32 && D % 32 == 0 && D <= 256 && s->max_len >= 16)
      SEQ_TRY(umb_pwa_attend_tiled(ws->mix, ws->aux, &ly.kv, ws->proj, ld, H * D + G * D, ly.pos_bias, s->seq_slot, s->seq_row0,
                                   s->seq_pos0, s->seq_len, s->B, s->max_len, H, G, D, ly.window, ly.pool, ly.scale, dt, st));
    else
      SEQ_TRY(umb_pwa_attend(ws->mix, ws->aux, &ly.kv, ws->proj, ld, H * D + G * D, ly.pos_bias, s->pos, s->slot, T, H, G, D,
                             ly.window, ly.pool, ly.scale, dt, st));
  } else if (ly.kind == UMB_MIX_GLA) {
    const int H = ly.heads, D = ly.dim, Dv = ly.vdim, HD = H * D;
    if (ld != 2 * HD + 2 * H * Dv + ly.rank || !ly.state) return UMB_EINVAL;
    SEQ_TRY(umb_gla_decay(ws->aux, ws->proj, ld, 2 * HD + 2 * H * Dv, ly.a2.w, ly.a2.bias, T, HD, ly.rank, ly.tau, dt, st));
    SEQ_TRY(umb_gla_scan(ws->o, ly.state, ws->proj, ld, ws->aux, s->seq_slot, s->seq_row0, s->seq_pos0, s->seq_len, s->B, H, D,
                         Dv, ly.qscale, st));
    SEQ_TRY(umb_gla_gate(ws->mix, ws->o, ws->proj, ld, 2 * HD + H * Dv, ly.head_norm, T, H, Dv, eps, dt, st));
  } else if (ly.kind == UMB_MIX_LATENT) {
    // proj = [dq | dkv (latent + rotated key part) | gate]; the query latent goes up to the heads, its unrotated parts are
    // carried into the key/value latent space (W_uk^T, one product per head), attention runs against the cached rows, the
    // value up-projection W_uv follows the weighted sum, with the sigmoid gate as its epilogue
    const int H = ly.heads, D = ly.dim, R = ly.rot_dim, Dv = ly.vdim, Rq = ly.q_rank, Rc = ly.kv_rank, Dk = Rc + R;
    if (ld != Rq + Dk + H * Dv || ly.uq.N != H * (D + R) || ly.uq.K != Rq || !ly.uk_t || !ly.uv || !ly.dq_norm || !ly.dkv_norm)
      return UMB_EINVAL;
    SEQ_TRY(umb_lat_prep(ws->act, &ly.kv, ws->proj, ld, ly.dq_norm, ly.dkv_norm, s->pos, s->slot, ly.rot_freq, T, Rq, Rc, R,
                         ly.rot_dims, eps, dt, st));
    SEQ_TRY(lin(ly.uq, ws->o, ws->act, T, 0, dt, st));
    SEQ_TRY(umb_lat_qsplit(ws->mix, ws->aux, ws->o, s->pos, ly.rot_freq, T, H, D, R, Rc, ly.rot_dims, dt, st));
    SEQ_TRY(umb_seq_linear_batched(ws->aux, ws->mix, ly.uk_t, T, Rc, D, H * D, H * Dk, H, D, (long)Rc * D, Dk, 0, nullptr, 0, 0,
                                   dt, st));
    if (s->max_len >= 16 && umb_lat_attend_tiled_ok(H, Rc, R, dt))
      SEQ_TRY(umb_lat_attend_tiled(ws->act, ws->aux, &ly.kv, ly.sink, s->seq_slot, s->seq_row0, s->seq_pos0, s->seq_len, s->B,
                                   s->max_len, H, Rc, R, ly.window, ly.scale, dt, st));
    else
      SEQ_TRY(umb_lat_attend(ws->act, ws->aux, &ly.kv, ly.sink, s->pos, s->slot, T, H, Rc, R, ly.window, ly.scale, dt, st));
    SEQ_TRY(umb_seq_linear_batched(ws->mix, ws->act, ly.uv, T, Dv, Rc, H * Rc, H * Dv, H, Rc, (long)Dv * Rc, Dv, 3,
                                   ws->proj + Rq + Dk, ld, Dv, dt, st));
  } else if (ly.kind == UMB_MIX_MINGRU) {
    SEQ_TRY(mix_mingru(m, ly, ws, s, st));
  } else if (ly.kind == UMB_MIX_ATTN_SSD) {
    SEQ_TRY(mix_attn_ssd(m, ly, ws, s, st));
  } else if (ly.kind == UMB_MIX_RETENTION) {
    SEQ_TRY(mix_retention(m, ly, ws, s, st));
  } else if (ly.kind == UMB_MIX_ATTN_MLSTM) {
    SEQ_TRY(mix_attn_mlstm(m, ly, ws, s, st));
  } else {
    return UMB_EINVAL;
  }
  return UMB_OK;
}

// Layers whose sublayers both read the same residual: x <- x + (mixer(norm1 x) + ff(norm2 x)); one seam launch per layer adds
// both outputs (and, in front of a span that runs again, the embedding row) and norms for the next layer.
static int forward_parallel_blocks(const UmbSeqModel* m, const UmbSeqWork* ws, const UmbSeqStep* s, hipStream_t st) {
  const int T = s->T, W = m->W, dt = m->dtype;
  if (!ws->h2 || !ws->y2 || !m->layers[0].norm1 || m->layers[0].add_embed) return UMB_EINVAL;
  const UmbSeqLayer& l0 = m->layers[0];
  SEQ_TRY(umb_blk_seam(ws->x, ws->h, ws->h2, nullptr, nullptr, m->embed, s->tokens, 1, m->embed_scale, l0.norm1,
                       l0.has_mlp ? l0.norm2 : nullptr, m->norm_offset, T, W, m->V, m->eps, dt, st));
  for (int l = 0; l < m->L; ++l) {
    const UmbSeqLayer& ly = m->layers[l];
    const UmbSeqLayer* nl = l + 1 < m->L ? &m->layers[l + 1] : nullptr;
    if (!ly.norm1 || (ly.has_mlp && !ly.norm2)) return UMB_EINVAL;
    SEQ_TRY(lin(ly.proj, ws->proj, ws->h, T, 0, dt, st));
    SEQ_TRY(run_mixer(m, ly, ws, s, st));
    SEQ_TRY(lin(ly.out, ws->y, ws->mix, T, 0, dt, st));
    if (ly.has_mlp) SEQ_TRY(feed_forward(m, ly, ws, s, ws->h2, ws->y2, st));
    const float* y2 = ly.has_mlp ? ws->y2 : nullptr;
    const void* w1 = nl ? nl->norm1 : nullptr;
    const void* w2 = nl && nl->has_mlp ? nl->norm2 : nullptr;
    const int add = nl && nl->add_embed ? 2 : 0;
    if (s->trace && add) {                                   // the trace shows the layer's own result: the embedding joins after it
      SEQ_TRY(umb_blk_seam(ws->x, nullptr, nullptr, ws->y, y2, nullptr, nullptr, 0, 0.f, nullptr, nullptr, 0.f, T, W, m->V, m->eps, dt, st));
      if (hipMemcpyAsync(s->trace + (long)l * T * W, ws->x, (size_t)T * W * sizeof(float), hipMemcpyDeviceToDevice, st) != hipSuccess)
        return UMB_EHIP;
      SEQ_TRY(umb_blk_seam(ws->x, ws->h, ws->h2, nullptr, nullptr, m->embed, s->tokens, 2, m->embed_scale, w1, w2, m->norm_offset, T, W,
                           m->V, m->eps, dt, st));
      continue;
    }
    SEQ_TRY(umb_blk_seam(ws->x, ws->h, ws->h2, ws->y, y2, m->embed, s->tokens, add, m->embed_scale, w1, w2, m->norm_offset, T, W, m->V,
                         m->eps, dt, st));
    if (s->trace && hipMemcpyAsync(s->trace + (long)l * T * W, ws->x, (size_t)T * W * sizeof(float), hipMemcpyDeviceToDevice, st) != hipSuccess)
      return UMB_EHIP;
  }
  if (s->R > 0) {
    // the final norm of the wanted rows only (a single stream read through the offset norm), then the head
    SEQ_TRY(umb_hc_read(nullptr, ws->h, ws->x, s->logit_rows, nullptr, m->final_norm, m->norm_offset, s->R, W, 1, m->eps, dt, st));
    SEQ_TRY(lin(m->head, ws->logits, ws->h, s->R, 0, dt, st));
    if (m->logit_scale != 0.f && m->logit_scale != 1.f) SEQ_TRY(umb_seq_scale(ws->logits, (long)s->R * m->V, m->logit_scale, st));
  }
  return UMB_OK;
}

extern "C" int umb_seq_forward(const UmbSeqModel* m, const UmbSeqWork* ws, const UmbSeqStep* s, hipStream_t st) {
  if (!m || !ws || !s || m->L < 1 || !m->layers || s->T < 1 || s->T > ws->Tmax || s->B < 1 || s->R < 0 || s->R > ws->Rmax)
    return UMB_EINVAL;
  if (m->block == UMB_BLOCK_PARALLEL) return forward_parallel_blocks(m, ws, s, st);
  const int T = s->T, W = m->W, dt = m->dtype, groups = m->groups;
  const float eps = m->eps;
  const bool hyper = m->streams >= 1;          // several residual streams: norms in front only, stream seams
  const int S = m->streams;
  if (hyper) {
    if (!m->layers[0].norm1) return UMB_EINVAL;
    SEQ_TRY(umb_hc_embed(ws->x, ws->h, m->embed, s->tokens, m->embed_scale, m->layers[0].hc1_in, m->layers[0].norm1,
                         m->norm_offset, T, W, m->V, S, eps, dt, st));
  } else if (m->layers[0].norm1)
    SEQ_TRY(umb_seq_embed_norm(ws->x, ws->h, m->embed, s->tokens, m->layers[0].norm1, T, W, m->V, groups, eps, dt, st));
  else
    SEQ_TRY(umb_seq_embed(ws->x, m->embed, s->tokens, m->embed_scale, T, W, m->V, dt, st));
  bool h_ready = false;
  for (int l = 0; l < m->L; ++l) {
    const UmbSeqLayer& ly = m->layers[l];
    const UmbSeqLayer* nl = l + 1 < m->L ? &m->layers[l + 1] : nullptr;
    if (!hyper) SEQ_TRY(sublayer_input(m, ws, s, ly.norm1, ly.canon1, ly.canon_state1, h_ready, st));
    SEQ_TRY(lin(ly.proj, ws->proj, ws->h, T, 0, dt, st));
    SEQ_TRY(run_mixer(m, ly, ws, s, st));
    SEQ_TRY(lin(ly.out, ws->y, ws->mix, T, 0, dt, st));
    if (hyper) {
      // write of this sublayer and read of the next one (the feed-forward, the next layer's mixer, or nothing) in one launch
      const float* in2 = ly.has_mlp ? ly.hc2_in : (nl ? nl->hc1_in : nullptr);
      const void* w2 = ly.has_mlp ? ly.norm2 : (nl ? nl->norm1 : nullptr);
      if ((ly.has_mlp || nl) && !w2) return UMB_EINVAL;
      SEQ_TRY(umb_hc_seam(ws->x, ws->h, ws->y, ly.hc1_mix, ly.hc1_out, m->resid_mult, in2, w2, m->norm_offset, T, W, S, eps, dt, st));
      if (ly.has_mlp) {
        SEQ_TRY(feed_forward(m, ly, ws, s, ws->h, ws->y, st));
        if (nl && !nl->norm1) return UMB_EINVAL;
        SEQ_TRY(umb_hc_seam(ws->x, ws->h, ws->y, ly.hc2_mix, ly.hc2_out, m->resid_mult, nl ? nl->hc1_in : nullptr,
                            nl ? nl->norm1 : nullptr, m->norm_offset, T, W, S, eps, dt, st));
      }
      if (s->trace) SEQ_TRY(umb_hc_read(s->trace + (long)l * T * W, nullptr, ws->x, nullptr, nullptr, nullptr, 0.f, T, W, S, eps, dt, st));
      continue;
    }
    const void* next = ly.has_mlp ? ly.norm2 : first_norm_of(m, l + 1);
    SEQ_TRY(seam(m, ws, s, ly.norm1b, next, ly.has_mlp ? ly.canon2 : (nl ? nl->canon1 : nullptr),
                 ly.has_mlp ? ly.canon_state2 : (nl ? nl->canon_state1 : nullptr), &h_ready, st));
    if (ly.has_mlp) {
      SEQ_TRY(sublayer_input(m, ws, s, ly.norm2, ly.canon2, ly.canon_state2, h_ready, st));
      SEQ_TRY(feed_forward(m, ly, ws, s, ws->h, ws->y, st));
      SEQ_TRY(seam(m, ws, s, ly.norm2b, first_norm_of(m, l + 1), nl ? nl->canon1 : nullptr, nl ? nl->canon_state1 : nullptr,
                   &h_ready, st));
    }
    if (s->trace) {
      if (hipMemcpyAsync(s->trace + (long)l * T * W, ws->x, (size_t)T * W * sizeof(float), hipMemcpyDeviceToDevice, st) != hipSuccess)
        return UMB_EHIP;
    }
  }
  if (s->R > 0) {
    // final norm of the wanted rows only (of the sum of the streams, where there are several), then the head
    if (hyper)
      SEQ_TRY(umb_hc_read(nullptr, ws->h, ws->x, s->logit_rows, nullptr, m->final_norm, m->norm_offset, s->R, W, S, eps, dt, st));
    else
      SEQ_TRY(umb_seq_group_norm(nullptr, ws->h, ws->x, s->logit_rows, m->final_norm, s->R, W, groups, eps, dt, st));
    SEQ_TRY(lin(m->head, ws->logits, ws->h, s->R, 0, dt, st));
  }
  return UMB_OK;
}

extern "C" const char* umb_seq_version(void) { return "umbrella_seq 0.1 (gfx950)"; }
