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

// feed-forward of ws->h into ws->y (fp32)
static int feed_forward(const UmbSeqModel* m, const UmbSeqLayer& ly, const UmbSeqWork* ws, const UmbSeqStep* s, hipStream_t st) {
  const int T = s->T, W = m->W, dt = m->dtype;
  // the activation lives in the first product's epilogue: silu(gate) * up over stacked [gate; up], or relu(up)^2
  const int epi = ly.act_kind == UMB_ACT_RELU2 ? 4 : 2, stack = ly.act_kind == UMB_ACT_RELU2 ? 1 : 2;
  if (ly.ff_kind == UMB_FF_GATED) {
    SEQ_TRY(lin(ly.gu, ws->act, ws->h, T, epi, dt, st));
    return lin(ly.down, ws->y, ws->act, T, 0, dt, st);
  }
  if (ly.ff_kind == UMB_FF_POLYNORM) {
    if (!ly.act || ly.gu.N != ly.ff) return UMB_EINVAL;
    SEQ_TRY(lin(ly.gu, ws->proj, ws->h, T, 0, dt, st));                        // "up" alone
    SEQ_TRY(umb_polynorm(ws->act, ws->proj, ly.act, T, ly.ff, m->eps, dt, st));
    return lin(ly.down, ws->y, ws->act, T, 0, dt, st);
  }
  if (ly.ff_kind == UMB_FF_MOE) {
    const int E = ly.experts, top = ly.top, F = ly.expert_ff;
    if (E < 1 || top < 1 || top > E || F < 1 || !ly.e_gu || !ly.e_down || !ws->moe_sel || !ws->moe_wt || !ws->moe_pos ||
        !ws->moe_tiles || !ws->moe_xs || !ws->moe_act || !ws->moe_y || ly.router.N != E)
      return UMB_EINVAL;
    const long pairs = (long)T * top;
    // many rows per expert (prompts): tiles of 128 rows on the LDS-staged kernel; few (decoding): tiles of 64, weights streamed
    // a handful of rows in all: tiles of 16, one output tile per workgroup
    const int tr = (dt != UMB_SEQ_F32 && pairs >= 64L * E && W % 8 == 0 && F % 8 == 0) ? 128 : (pairs <= 64 ? 16 : 64);
    const int max_tiles = (int)((pairs + tr - 1) / tr) + E;
    if (max_tiles > ws->moe_max_tiles) return UMB_EINVAL;
    if (ly.s_gu.w) {                                                           // the shared expert sees every token
      SEQ_TRY(lin(ly.s_gu, ws->act, ws->h, T, epi, dt, st));
      SEQ_TRY(lin(ly.s_down, ws->y, ws->act, T, 0, dt, st));
    }
    SEQ_TRY(lin(ly.router, ws->proj, ws->h, T, 0, dt, st));
    // sigmoid routing weighs the expert's input, softmax routing its output
    const bool w_out = ly.route_kind == UMB_ROUTE_SOFTMAX_OUT;
    if (w_out) SEQ_TRY(umb_moe_route_softmax(ws->moe_sel, ws->moe_wt, ws->proj, ly.correction, T, E, top, st));
    else SEQ_TRY(umb_moe_route(ws->moe_sel, ws->moe_wt, ws->proj, T, E, top, st));
    SEQ_TRY(umb_moe_plan(ws->moe_pos, ws->moe_tiles, ws->moe_sel, T, E, top, max_tiles, tr, st));
    SEQ_TRY(umb_moe_scatter(ws->moe_xs, ws->h, w_out ? nullptr : ws->moe_wt, ws->moe_pos, T, W, top, dt, st));
    SEQ_TRY(umb_seq_linear_grouped(ws->moe_act, ws->moe_xs, ly.e_gu, ws->moe_tiles, max_tiles, tr, (long)stack * F * W, stack * F, W,
                                   epi, dt, st));
    SEQ_TRY(umb_seq_linear_grouped(ws->moe_y, ws->moe_act, ly.e_down, ws->moe_tiles, max_tiles, tr, (long)W * F, W, F, 0, dt, st));
    if (w_out) return umb_moe_combine_weighted(ws->y, ws->moe_y, ws->moe_wt, ws->moe_pos, T, W, top, ly.s_gu.w ? 1 : 0, st);
    return umb_moe_combine(ws->y, ws->moe_y, ws->moe_pos, T, W, top, ly.s_gu.w ? 1 : 0, st);
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
                                 s->seq_pos0, s->seq_len, s->B, s->max_len, H, G, D, E, ly.window, ly.scale, ly.mix_scale_a, dt, st));
  else {
    // what the step leaves free of aux holds the partial results of split keys (the state-space part below uses sx / alpha
    // after the attention is done, so its region may be used too, but the queries may not)
    float* spare = q + (size_t)T * H * D;
    const long spare_floats = ws->aux_floats - (long)T * H * D;
    SEQ_TRY(umb_bsa_attend(ws->mix, ldo, q, &ly.kv, ws->proj, ld, gate_col, ly.dist_bias, ly.n_dist, s->pos, s->slot, T, H, G, D, E,
                           ly.window, ly.scale, ly.mix_scale_a, spare_floats > 0 ? spare : nullptr, spare_floats, dt, st));
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

extern "C" int umb_seq_forward(const UmbSeqModel* m, const UmbSeqWork* ws, const UmbSeqStep* s, hipStream_t st) {
  if (!m || !ws || !s || m->L < 1 || !m->layers || s->T < 1 || s->T > ws->Tmax || s->B < 1 || s->R < 0 || s->R > ws->Rmax)
    return UMB_EINVAL;
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
    const int ld = ly.proj.N;
    if (!hyper) SEQ_TRY(sublayer_input(m, ws, s, ly.norm1, ly.canon1, ly.canon_state1, h_ready, st));
    SEQ_TRY(lin(ly.proj, ws->proj, ws->h, T, 0, dt, st));
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
    } else {
      return UMB_EINVAL;
    }
    SEQ_TRY(lin(ly.out, ws->y, ws->mix, T, 0, dt, st));
    if (hyper) {
      // write of this sublayer and read of the next one (the feed-forward, the next layer's mixer, or nothing) in one launch
      const float* in2 = ly.has_mlp ? ly.hc2_in : (nl ? nl->hc1_in : nullptr);
      const void* w2 = ly.has_mlp ? ly.norm2 : (nl ? nl->norm1 : nullptr);
      if ((ly.has_mlp || nl) && !w2) return UMB_EINVAL;
      SEQ_TRY(umb_hc_seam(ws->x, ws->h, ws->y, ly.hc1_mix, ly.hc1_out, m->resid_mult, in2, w2, m->norm_offset, T, W, S, eps, dt, st));
      if (ly.has_mlp) {
        SEQ_TRY(feed_forward(m, ly, ws, s, st));
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
      SEQ_TRY(feed_forward(m, ly, ws, s, st));
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
