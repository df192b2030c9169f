/* libumbrella_seq.so -- C ABI of the sequence-mixer model family on MI355X (gfx950).
 *
 * Decoder stacks whose layers mix tokens with something other than the dense tree-masked softmax attention of
 * libumbrella_hip.so: gated linear attention (a per-head matrix state carried from token to token) and sliding-window
 * attention over a paged key/value store with mean-pooled blocks behind the window and sigmoid (un-normalised) weights;
 * latent attention; a minimal gated recurrence; softmax attention with a bias by distance beside a state-space layer with a
 * scalar decay per head; residuals of one or several streams; dense, PolyNorm and routed-expert feed-forwards.
 * The layer list, every size and every constant are data (UmbSeqLayer); one forward entry point walks the list.
 *
 * Conventions are those of umbrella_hip.h: extern "C", plain pointers and sizes, 0 or a negative errno-style code,
 * nothing allocated, every call asynchronous on `stream`, all run-time indices read from device memory.
 *
 * dtype: 0 = fp16, 1 = bf16, 2 = fp32 -- the type of weights, of activations that feed a matrix product and of cached
 * keys / values.  Whatever the dtype, these are fp32: the residual stream, every norm, rotary angles, attention scores
 * and weights, decays, the recurrent state and everything that enters the recurrence, all matrix-product accumulators.
 *
 * A step is a RAGGED batch: T rows, the rows of one sequence contiguous and at consecutive positions.  Nothing is padded.
 */
#ifndef UMBRELLA_SEQ_H
#define UMBRELLA_SEQ_H
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct ihipStream_t* umb_stream_t;   /* == hipStream_t */

enum { UMB_SEQ_F16 = 0, UMB_SEQ_BF16 = 1, UMB_SEQ_F32 = 2 };
enum { UMB_MIX_POOLED_WINDOW = 0, UMB_MIX_GLA = 1, UMB_MIX_LATENT = 2, UMB_MIX_MINGRU = 3, UMB_MIX_ATTN_SSD = 4,
       UMB_MIX_RETENTION = 5, UMB_MIX_ATTN_MLSTM = 6 };
/* feed-forward kinds: gated SiLU (W_down (silu(W_gate h) * W_up h)), PolyNorm (W_down polynorm(W_up h)), routed experts */
enum { UMB_FF_GATED = 0, UMB_FF_POLYNORM = 1, UMB_FF_MOE = 2 };
/* activation of a feed-forward / expert: silu(W_gate h) * (W_up h) over stacked [gate; up], relu(W_up h)^2 (no gate), or the
 * capped form g sigmoid(alpha g) (u + 1) with g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit) over stacked [gate; up] */
enum { UMB_ACT_SILU_GATED = 0, UMB_ACT_RELU2 = 1, UMB_ACT_CLAMP_GLU = 2 };
/* routing of experts: sigmoid scores that multiply the expert's input; or softmax scores, chosen with a correction added,
 * renormalised over the chosen ones, that multiply the expert's output */
enum { UMB_ROUTE_SIGMOID_IN = 0, UMB_ROUTE_SOFTMAX_OUT = 1, UMB_ROUTE_TOP_LOGITS = 2 };
/* UMB_ROUTE_TOP_LOGITS: the largest logits are chosen, the weights are the softmax over the chosen logits alone and multiply
 * the experts' outputs */
/* how a layer's sublayers meet the residual: one after the other (x + f(..) then x + g(..), the forms below), or BOTH reading the
 * same x: x <- x + (mixer(norm1(x)) + ff(norm2(x))) */
enum { UMB_BLOCK_SEQUENTIAL = 0, UMB_BLOCK_PARALLEL = 1 };

/* W [N][K] row-major (as stored: out x in), optional bias [N]; applied as W x + b */
typedef struct UmbSeqLinear { const void* w; const void* bias; int32_t N, K; } UmbSeqLinear;

/* ------------------------------------------------------------------ stand-alone ops (each is also a step of the forward) */

/* out[T][N] = x[T][K] . W^T + bias, fp32 accumulation in a fixed order that depends on (N, K) only.
 * epi 0: out fp32; epi 1: out in `dtype`; epi 2: W stacks [gate; up] (N = 2 N'), out[T][N'] in `dtype` =
 * silu(gate) * up; epi 4: out in `dtype` = relu(acc)^2.  x and W in `dtype`. */
int umb_seq_linear(void* out, const void* x, const void* w, const void* bias, int T, int N, int K, int epi, int dtype,
                   umb_stream_t stream);

/* The same product for `batch` independent problems (blockIdx.z): problem b reads x + b sx (rows ldx apart), weights
 * w + b sw ([N][K]) and writes out + b so (rows ldo apart); strides in elements; no bias.  epi 0 / 1 as above;
 * epi 3: out in `dtype` = acc * sigmoid(gate[t ldg + b sg + n]) (gate fp32).  The K order of an output is that of
 * umb_seq_linear. */
int umb_seq_linear_batched(void* out, const void* x, const void* w, int T, int N, int K, int ldx, int ldo, int batch, long sx,
                           long sw, long so, int epi, const float* gate, int ldg, int sg, int dtype, umb_stream_t stream);
/* Grouped product over row ranges read from device memory: tile i (blockIdx.y, i < max_tiles) is {group, first row, rows}
 * (3 int32, rows <= tile_rows, rows == 0: nothing); its rows of x [*][K] meet w + group * gs ([N][K], or the stacked
 * [2N'][K] of epi 2) and land in the same rows of out.  No bias.  tile_rows 64: weights streamed per tile (few rows per
 * group); 128: both operands staged through LDS (16-bit storage, K and gs multiples of 8). */
int umb_seq_linear_grouped(void* out, const void* x, const void* w, const int* tiles, int max_tiles, int tile_rows, long gs,
                           int N, int K, int epi, int dtype, umb_stream_t stream);

/* RMS norm in `groups` equal consecutive parts of a row: part / sqrt(mean(part^2) + eps), whole row times w.
 * x fp32 [*][W]; rows: optional gather (row i of out comes from row rows[i] of x); out_f32 and/or out_dt may be given. */
int umb_seq_group_norm(float* out_f32, void* out_dt, const float* x, const int* rows, const void* w, int T, int W, int groups,
                       float eps, int dtype, umb_stream_t stream);
/* x[t] <- embed[tokens[t]] (fp32); h[t] <- group_norm(x[t]) * w in `dtype` */
int umb_seq_embed_norm(float* x, void* h, const void* embed, const int* tokens, const void* w, int T, int W, int V, int groups,
                       float eps, int dtype, umb_stream_t stream);
/* x <- x + group_norm(y) * w_post ; if w_next: h <- group_norm(x) * w_next in `dtype`   (y fp32 [T][W]) */
int umb_seq_resid_norm(float* x, void* h, const float* y, const void* w_post, const void* w_next, int T, int W, int groups,
                       float eps, int dtype, umb_stream_t stream);

/* x[t] <- embed[tokens[t]] * scale (fp32) */
int umb_seq_embed(float* x, const void* embed, const int* tokens, float scale, int T, int W, int V, int dtype,
                  umb_stream_t stream);

/* ---- causal convolution over time in front of a sublayer ("canon"): h[t] = x[t] + sum_j w[c][j] x(p - taps + 1 + j), the
 * sum over the `taps` positions up to and including the token's own position p; positions before the sequence's start are
 * zero, positions of earlier steps come from the sequence's state.  x fp32 [T][W]; w [W][taps]; h in `dtype`.
 * state fp32 [slots][taps - 1][W]: the input at position p lives in row p % (taps - 1).  The convolution reads the state;
 * `umb_canon_update`, launched after it, stores the step's last inputs. taps == 1 needs no state. */
int umb_canon_conv(void* h, const float* x, const void* w, const float* state, const int* pos, const int* slot, int T, int W,
                   int taps, int dtype, umb_stream_t stream);
int umb_canon_update(float* state, const float* x, const int* seq_slot, const int* seq_row0, const int* seq_pos0,
                     const int* seq_len, int B, int W, int taps, umb_stream_t stream);
/* one launch for steps of one token per sequence: convolution and state update by the same thread */
int umb_canon_step(void* h, const float* x, const void* w, float* state, const int* pos, const int* slot, int T, int W,
                   int taps, int dtype, umb_stream_t stream);

/* The seam x <- x + group_norm(y) * w_post followed by that convolution, for steps of one token per sequence, in one
 * launch: h = canon(x), the state row of the token's position is overwritten with the new x.  Covers groups == 1 and
 * groups whose length is a multiple of 256 (umb_seq_resid_canon_step_ok: 1 / 0, no stream). */
int umb_seq_resid_canon_step_ok(int W, int groups);
int umb_seq_resid_canon_step(float* x, void* h, const float* y, const void* w_post, const void* canon, float* state,
                             const int* pos, const int* slot, int T, int W, int groups, int taps, float eps, int dtype,
                             umb_stream_t stream);

/* ---- PolyNorm activation: out[t] = a N(z) + b N(z^2) + c N(z^3) + e with powers element by element and
 * N(v) = v / sqrt(mean(v^2) + eps) over the row; coef = {a, b, c, e} in `dtype`; z fp32 [T][F], out in `dtype`. */
int umb_polynorm(void* out, const float* z, const void* coef, int T, int F, float eps, int dtype, umb_stream_t stream);

/* ---- routed experts.  logits fp32 [T][E]; scores = sigmoid(logits); each token keeps its `top` largest (compared on the
 * logits, so scores that saturate to the same fp32 value are still told apart; ties: the lower index), weight = the score
 * itself.  sel [T][top] expert ids, wt [T][top] fp32. */
int umb_moe_route(int* sel, float* wt, const float* logits, int T, int E, int top, umb_stream_t stream);
/* orders the T*top (token, choice) pairs by expert: pos_of [T*top] = row of the pair in the expert-ordered list,
 * tiles [max_tiles][3] = {expert, first row, rows} covering every expert's rows in pieces of at most tile_rows
 * (max_tiles >= ceil(T top / tile_rows) + E; unused entries get rows = 0). */
int umb_moe_plan(int* pos_of, int* tiles, const int* sel, int T, int E, int top, int max_tiles, int tile_rows,
                 umb_stream_t stream);
/* xs[pos_of[t top + k]] = wt[t][k] * h[t]  (the weight multiplies the expert's INPUT; wt null: 1); h, xs in `dtype` */
int umb_moe_scatter(void* xs, const void* h, const float* wt, const int* pos_of, int T, int W, int top, int dtype,
                    umb_stream_t stream);
/* y[t] = (add ? y[t] : 0) + sum_k ye[pos_of[t top + k]]  (k ascending) */
int umb_moe_combine(float* y, const float* ye, const int* pos_of, int T, int W, int top, int add, umb_stream_t stream);

/* ---- gated linear attention.  proj fp32 [T][ld]: columns [q (H D) | k (H D) | v (H Dv) | g (H Dv) | a (rank)].
 * decay: alpha[t][H D] = sigmoid(W_a2 a + b)^(1/tau), fp32 */
int umb_gla_decay(float* alpha, const float* proj, int ld, int a_col, const void* w_a2, const void* b_a2, int T, int HD, int rank,
                  float tau, int dtype, umb_stream_t stream);
/* per sequence and head: S <- diag(alpha_t) S + k_t v_t^T ; o_t = S^T (q_t * qscale).  state fp32 [slots][H][D][Dv]; a
 * sequence whose first position is 0 starts from S = 0 whatever its slot holds.  o fp32 [T][H Dv]. */
int umb_gla_scan(float* o, float* state, const float* proj, int ld, const float* alpha, const int* seq_slot, const int* seq_row0,
                 const int* seq_pos0, const int* seq_len, int B, int H, int D, int Dv, float qscale, umb_stream_t stream);
/* out[t][h] = rms_norm(o[t][h]) * w (w [Dv], shared by heads) * silu(g[t][h]) in `dtype` */
int umb_gla_gate(void* out, const float* o, const float* proj, int ld, int g_col, const void* w, int T, int H, int Dv, float eps,
                 int dtype, umb_stream_t stream);

/* ---- sliding-window attention with pooled blocks over a paged store.
 * Pages hold `page` tokens; page table pages[slot][max_pages].  Per layer: K and V [pages][G][page][D] in `dtype`, and
 * the pooled K / V [pages][G][ceil(page / pool)][D] in fp32: block b (positions b pool .. b pool + pool - 1) lives in the
 * page of its LAST position e, at entry (e % page) / pool. */
typedef struct UmbPagedKV {
  void* k; void* v; float* kp; float* vp;
  const int32_t* pages; int32_t max_pages, page, n_pages, pad_;
} UmbPagedKV;
/* proj fp32 [T][ld]: columns [q (H D) | k (G D) | gate (H)] with the projection biases already added.
 * q <- unit_rms(rope(q)) fp32 [T][H D]; cache K <- unit_rms(rope(k)), cache V <- k as projected; interleaved pairs
 * (2i, 2i+1) of the first rot_dims features turn by pos * freq[i]. */
int umb_pwa_prep(float* q, const UmbPagedKV* kv, const float* proj, int ld, const int* pos, const int* slot, const float* freq,
                 int T, int H, int G, int D, int rot_dims, float eps, int dtype, umb_stream_t stream);
/* pooled entries of every block whose last position this step wrote: the fp32 mean of the `pool` cached keys / values */
int umb_pwa_pool(const UmbPagedKV* kv, const int* seq_slot, const int* seq_pos0, const int* seq_len, int B, int max_len, int G,
                 int D, int pool, int dtype, umb_stream_t stream);
/* out[t][h] = sigmoid(gate[t][h]) * sum over visible keys of sigmoid(q.k * scale + pos_bias[h]) * v, in `dtype`.
 * Visible to position i: tokens j with 0 <= i - j < window, and blocks b with b pool + pool - 1 <= i - window. */
int umb_pwa_attend(void* out, const float* q, const UmbPagedKV* kv, const float* proj, int ld, int gate_col, const void* pos_bias,
                   const int* pos, const int* slot, int T, int H, int G, int D, int window, int pool, float scale, int dtype,
                   umb_stream_t stream);

/* The same attention for steps that bring whole stretches of a sequence (prompts), on the matrix pipe: 16-bit storage only,
 * D a multiple of 32 (<= 256); workgroups own 16 consecutive positions of one sequence.  Scores and weights keep fp32
 * accuracy: the fp32 factors (q, pooled means, weights) enter as high + low 16-bit halves. */
int umb_pwa_attend_tiled(void* out, const float* q, const UmbPagedKV* kv, const float* proj, int ld, int gate_col,
                         const void* pos_bias, const int* seq_slot, const int* seq_row0, const int* seq_pos0, const int* seq_len,
                         int B, int max_len, int H, int G, int D, int window, int pool, float scale, int dtype,
                         umb_stream_t stream);

/* ---- latent attention: queries and keys/values go through low-rank latents; the cache holds, per token, the normed
 * key/value latent c [kv_rank] and one rotated key part [rot_dim] shared by all heads (one row of kv_rank + rot_dim in
 * `dtype`; pages as above, UmbPagedKV.k only, one "head").  Scores and values are taken against c itself:
 *   score(i, j, h) = (q_lat[i][h] . c[j] + q_rot[i][h] . k_rot[j]) * scale,   q_lat = W_uk[h]^T q_nope
 *   out[i][h]      = W_uv[h] (sum_j p[i][j][h] c[j]),
 * which equals attention over per-head keys W_uk[h] c and values W_uv[h] c without ever forming them.
 * lat_prep: proj fp32 [T][ld] = [dq (q_rank) | dkv (kv_rank + rot_dim) | ...]; cq = rms_norm(dq) * w_q in `dtype`;
 * cache row = [rms_norm(dkv[:kv_rank]) * w_kv | rope(dkv[kv_rank:])]. */
int umb_lat_prep(void* cq, const UmbPagedKV* kv, const float* proj, int ld, const void* w_q, const void* w_kv, const int* pos,
                 const int* slot, const float* freq, int T, int q_rank, int kv_rank, int rot_dim, int rot_dims, float eps,
                 int dtype, umb_stream_t stream);
/* q fp32 [T][H (D + R)] head by head [unrotated D | rotated R] -> qn [T][H D] in `dtype` (unrotated parts) and
 * qa[t][h][kv_rank ..] = rope(rotated part) fp32 (qa fp32 [T][H][kv_rank + R]; the first kv_rank come from the
 * batched product with W_uk^T) */
int umb_lat_qsplit(void* qn, float* qa, const float* q, const int* pos, const float* freq, int T, int H, int D, int R,
                   int kv_rank, int rot_dims, int dtype, umb_stream_t stream);
/* softmax attention of qa over the cached rows of the window (0 <= i - j < window) with a sink per head in the
 * denominator (exp(sink[h]): no key, no value, not scaled; sink may be null); out [T][H][kv_rank] in `dtype`. */
int umb_lat_attend(void* out, const float* qa, const UmbPagedKV* kv, const void* sink, const int* pos, const int* slot, int T,
                   int H, int kv_rank, int rot_dim, int window, float scale, int dtype, umb_stream_t stream);
/* the same for steps that bring stretches of a sequence, on the matrix pipe: workgroups own 16 consecutive positions of
 * one sequence.  umb_lat_attend_tiled_ok says (1 / 0) whether the kernel covers a shape and dtype; it has no stream. */
int umb_lat_attend_tiled(void* out, const float* qa, const UmbPagedKV* kv, const void* sink, const int* seq_slot,
                         const int* seq_row0, const int* seq_pos0, const int* seq_len, int B, int max_len, int H, int kv_rank,
                         int rot_dim, int window, float scale, int dtype, umb_stream_t stream);

/* ---- several residual streams ("hyper-connections").  The residual is S copies per token, x fp32 [T][S][W].  A sublayer
 * reads u = sum_s in[s] x_s through an RMS norm whose weight is stored around `offset` (h = u / rms(u) * (offset + w));
 * its output y is written back to all streams at once from the old ones: x_t <- sum_s mix[s][t] x_s + m out[t] y.
 * in / out / mix are fp32 and may be null (all ones / all ones / identity); S = 1 with nulls is the plain x + m y.
 * embed: every stream <- embed[token] * scale, h <- first read.  seam: write of the sublayer behind, read of the one ahead
 * (in_next null and w_next null: no read).  read: rows gathered through `rows` (null: all), u_out (fp32 [R][W]) and / or
 * h may be given; in null sums the streams. */
int umb_hc_embed(float* x, void* h, const void* embed, const int* tokens, float scale, const float* in, const void* w,
                 float offset, int T, int W, int V, int S, float eps, int dtype, umb_stream_t stream);
int umb_hc_seam(float* x, void* h, const float* y, const float* mix, const float* out, float m, const float* in_next,
                const void* w_next, float offset, int T, int W, int S, float eps, int dtype, umb_stream_t stream);
int umb_hc_read(float* u_out, void* h, const float* x, const int* rows, const float* in, const void* w, float offset, int R,
                int W, int S, float eps, int dtype, umb_stream_t stream);

/* ---- minimal gated recurrence, element by element over `Wm` channels: with the projections zr / ur / gr (fp32, biases
 * added, columns z_col / u_col / g_col of proj [T][ld]), z = sigmoid(zr), candidate = ur + 1/2 where ur >= 0, else
 * sigmoid(ur); S_t = (1 - z) S_(t-1) + z candidate; out[t] = S_t * silu(gr) in `dtype`.  state fp32 [slots][Wm]; a
 * sequence that starts at position 0 starts from S = 0 whatever its slot holds.  max_len: the longest stretch of the step;
 * long stretches run as pieces side by side (piece summaries, then a fold) when scratch (fp32, at least
 * umb_mingru_scratch_floats(T, B, Wm) floats; no stream argument) is given, else token by token. */
long umb_mingru_scratch_floats(int T, int B, int Wm);
int umb_mingru_scan(void* out, float* state, const float* proj, int ld, int z_col, int u_col, int g_col, const int* seq_slot,
                    const int* seq_row0, const int* seq_pos0, const int* seq_len, int B, int Wm, int max_len, float* scratch,
                    long scratch_floats, int dtype, umb_stream_t stream);

/* ---- linear recurrence with a matrix state per head, general operand placement (umb_gla_scan is one case of it):
 * S <- a_t S + k_t v_t^T, o_t = S^T (q_t * qscale); q and k rows [T][ldq / ldk] hold qk_heads groups of D (head h reads
 * group h / (H / qk_heads)), v rows H heads of Dv; the decay is per key channel (alpha [T][H D], alpha_per_head 0) or one
 * number per head (alpha [T][H], alpha_per_head 1).  state fp32 [slots][H][D][Dv]. */
int umb_lin_scan(float* o, float* state, const float* q, int ldq, const float* k, int ldk, const float* v, int ldv,
                 const float* alpha, int alpha_per_head, int qk_heads, const int* seq_slot, const int* seq_row0,
                 const int* seq_pos0, const int* seq_len, int B, int H, int D, int Dv, float qscale, umb_stream_t stream);

/* ---- selective state space with a scalar decay per head (state-space duality).  proj fp32 [T][ld]; from column col0:
 * [z (H Dv) | x (H Dv) | B (G N) | C (G N) | dt (H)].  prep: x, B, C through a causal convolution per channel (w [C][taps],
 * last column the token's own, bias b, inputs of earlier steps from conv_state fp32 [slots][taps - 1][C], the input of
 * position p in row p % (taps - 1)) and silu; dt = softplus(dt + dt_bias[h]); sx fp32 [T][lds] = [dt x | B | C | x],
 * alpha [T][H] = exp(-exp(a_log[h]) dt), log_alpha [T][H] (may be null) its logarithm.  conv_update, launched after prep, stores the step's last raw inputs; with
 * update_state (steps of ONE token per sequence only) prep stores the token's input itself and conv_update is not needed.
 * The recurrence itself is umb_lin_scan (k = B, v = dt x, q = C).
 * gate: y = o + d_skip[h] x, times silu(z), unit RMS in `norm_groups` equal parts of the H Dv row, times w, times
 * out_scale, in `dtype` at out[t ldo + ...]. */
int umb_ssd_prep(float* sx, int lds, float* alpha, float* log_alpha, const float* proj, int ld, int col0, const void* conv_w,
                 const void* conv_b,
                 float* conv_state, const float* dt_bias, const float* a_log, const int* pos, const int* slot, int T, int H,
                 int Dv, int G, int N, int taps, int update_state, int dtype, umb_stream_t stream);
int umb_ssd_conv_update(float* conv_state, const float* proj, int ld, int col0, const int* seq_slot, const int* seq_row0,
                        const int* seq_pos0, const int* seq_len, int B, int C, int taps, umb_stream_t stream);
/* The recurrence of umb_lin_scan with one decay per head (given as its logarithm), for stretches of many tokens: chunks of 64
 * tokens run side by side -- chunk summaries, a pass over the chunks that leaves every chunk's start state and the final state
 * in the slot, then all read-outs (qscale 1).  scratch fp32 of at least umb_ssd_scan_chunked_floats(..) floats (0: the shape is
 * not covered; no stream argument).  Equal to the token-by-token scan to fp32 rounding. */
long umb_ssd_scan_chunked_floats(int B, int max_len, int H, int N, int P);
int umb_ssd_scan_chunked(float* o, float* state, const float* q, int ldq, const float* k, int ldk, const float* v, int ldv,
                         const float* log_alpha, int qk_heads, const int* seq_slot, const int* seq_row0, const int* seq_pos0,
                         const int* seq_len, int B, int max_len, int H, int N, int P, float* scratch, long scratch_floats,
                         umb_stream_t stream);
int umb_ssd_gate(void* out, int ldo, const float* o, const float* sx, int lds, int x_col, const float* proj, int ld, int z_col,
                 const float* d_skip, const void* w, int T, int H, int Dv, int norm_groups, float eps, float out_scale, int dtype,
                 umb_stream_t stream);

/* ---- causal softmax attention with a bias by distance over a paged store (UmbPagedKV: k [pages][G][page][D],
 * v [pages][G][page][E] in `dtype`; kp / vp unused).  proj fp32 [T][ld] = [q (H D) | k (G D) | v (G E) | gate (H)].
 * prep: q <- unit_rms(q) * w_q * (1 + temp_coef ln(floor((pos + 1) / temp_every) + 1)), fp32 [T][H D] (w_q, w_k [D], shared by
 * the heads; null: 1); cache K <- unit_rms(k) * w_k; cache V <- unit_rms(v) (no weight).
 * attend: score(i, j, h) = q_i . k_j * scale + bias[h][min(i - j, n_dist - 1)] over j <= i with i - j < window (bias fp32
 * [H][n_dist], null: none); softmax; out[t ldo + h E ..] = out_scale * sigmoid(gate[t][h]) * sum_j p_j v_j in `dtype`
 * (gate_col < 0: no gate).  softcap > 0: the scaled product is capped, softcap tanh(q . k scale / softcap), before the bias
 * joins it.  scratch (fp32, may be null): with it, steps of few rows deal each row's keys to several workgroups
 * (as many as T H 16 (E + 2) floats allow, at most 16) and merge the partial results in a second launch. */
int umb_bsa_prep(float* q, const UmbPagedKV* kv, const float* proj, int ld, const void* w_q, const void* w_k, const int* pos,
                 const int* slot, int T, int H, int G, int D, int E, float temp_coef, int temp_every, float eps, int dtype,
                 umb_stream_t stream);
int umb_bsa_attend(void* out, int ldo, const float* q, const UmbPagedKV* kv, const float* proj, int ld, int gate_col,
                   const float* bias, int n_dist, const int* pos, const int* slot, int T, int H, int G, int D, int E, int window,
                   float scale, float out_scale, float softcap, float* scratch, long scratch_floats, int dtype,
                   umb_stream_t stream);
/* the same for steps that bring stretches of a sequence, on the matrix pipe (16-bit storage; umb_bsa_attend_tiled_ok says
 * 1 / 0 whether the kernel covers a shape and dtype; it has no stream): workgroups own 16 consecutive positions */
int umb_bsa_attend_tiled_ok(int H, int G, int D, int E, int dtype);
int umb_bsa_attend_tiled(void* out, int ldo, const float* q, const UmbPagedKV* kv, const float* proj, int ld, int gate_col,
                         const float* bias, int n_dist, const int* seq_slot, const int* seq_row0, const int* seq_pos0,
                         const int* seq_len, int B, int max_len, int H, int G, int D, int E, int window, float scale,
                         float out_scale, float softcap, int dtype, umb_stream_t stream);

/* ---- routed experts, softmax form: scores = softmax(logits) over all experts; the `top` largest of score + correction
 * (correction fp32 [E], null: none; ties: the lower index) are chosen; wt = the chosen scores over (their sum + 1e-20). */
int umb_moe_route_softmax(int* sel, float* wt, const float* logits, const float* correction, int T, int E, int top,
                          umb_stream_t stream);
/* y[t] = (add ? y[t] : 0) + sum_k wt[t top + k] * ye[pos_of[t top + k]]  (k ascending) */
int umb_moe_combine_weighted(float* y, const float* ye, const float* wt, const int* pos_of, int T, int W, int top, int add,
                             umb_stream_t stream);

/* ---- the capped gated epilogue over stacked [gate; up] (N = 2 N'): out[T][N'] in `dtype` = g sigmoid(alpha g) (u + 1) with
 * g = min(gate, limit), u = clamp(up, -limit, limit); dense and grouped forms of umb_seq_linear / umb_seq_linear_grouped */
int umb_seq_linear_glu(void* out, const void* x, const void* w, const void* bias, int T, int N, int K, float limit, float alpha,
                       int dtype, umb_stream_t stream);
int umb_seq_linear_grouped_glu(void* out, const void* x, const void* w, const int* tiles, int max_tiles, int tile_rows, long gs,
                               int N, int K, float limit, float alpha, int dtype, umb_stream_t stream);

/* ---- layers whose two sublayers read the same residual.  One launch between two layers:
 *   embed_mode 0: x += y1 + y2;  1: x = embed[token] * embed_scale;  2: x += (y1 + y2) + embed[token] * embed_scale
 * (y1 / y2 fp32 [T][W], either may be null), then h1 = x / rms(x) * (offset + w1) and h2 likewise with w2, in `dtype` (w1 / w2
 * null: that output is not written). */
int umb_blk_seam(float* x, void* h1, void* h2, const float* y1, const float* y2, const void* embed, const int* tokens,
                 int embed_mode, float embed_scale, const void* w1, const void* w2, float offset, int T, int W, int V, float eps,
                 int dtype, umb_stream_t stream);
/* buf[i] *= scale, i < n */
int umb_seq_scale(float* buf, long n, float scale, umb_stream_t stream);

/* ---- rotary positions on a run of heads: in fp32 [T][ld] holds `heads` heads of D; the first rot_dims features of every head
 * turn by pos * freq[i] (layout 0: feature i pairs with i + rot_dims / 2; 1: feature 2i with 2i + 1), the rest pass; the first
 * heads_a heads are then multiplied by scale_a, the others by scale_b.  out fp32 [T][ldo]. */
int umb_rope_scale(float* out, int ldo, const float* in, int ld, const int* pos, const float* freq, int T, int heads, int D,
                   int rot_dims, int layout, int heads_a, float scale_a, float scale_b, umb_stream_t stream);
/* alpha[t][h] = decay[h], log_alpha[t][h] = log(decay[h]) (log_alpha may be null): the rows the linear scans read */
int umb_decay_fill(float* alpha, float* log_alpha, const float* decay, int T, int H, umb_stream_t stream);
/* Behind a linear scan: o fp32 [T][H][P_cols], the head's Dv read-outs first.  den_col >= 0: column den_col holds n . q and the
 * read-outs are divided by max(|n . q|, exp(-mrun[t][h])) + 1e-6 first.  Then each head over its root mean square (eps), times
 * w ([Dv] shared by the heads, [H Dv] with w_per_head, or null), times silu (gate_kind 0) or sigmoid (1) of
 * proj[t][g_col + h Dv + i], times out_scale, in `dtype` at out[t ldo + h Dv + i]. */
int umb_head_gate(void* out, int ldo, const float* o, int P_cols, int den_col, const float* mrun, const float* proj, int ld,
                  int g_col, const void* w, int w_per_head, int gate_kind, int T, int H, int Dv, float eps, float out_scale,
                  int dtype, umb_stream_t stream);

/* ---- softmax attention behind a short causal convolution.  proj fp32 [T][ld] = [q (H D) | k (G D) | v (G E) | ...] (biases
 * added): every channel passes u_t = sum_j w[c][j] raw_(t - taps + 1 + j) (conv_w [C][taps] in `dtype`, null: none; earlier
 * steps' inputs from conv_state fp32 [slots][taps - 1][C], position p in row p % (taps - 1)); q and k are RMS-normed over their
 * WHOLE rows (weights w_q [H D], w_k [G D], null: 1) and rotated (rot_dims, layout and freq as umb_rope_scale); q -> fp32
 * [T][H D], k and v -> the paged store.  The ring is refreshed by umb_ssd_conv_update (col0 0) afterwards, or here with
 * update_state (steps of ONE token per sequence only).  scratch (fp32, may be null): with T (H D + G D + 2 ceil(C / 256)) floats
 * of it, steps of at most 64 tokens run as two launches over (token, 256 channels) instead of one workgroup per token.  The
 * attention is umb_bsa_attend with a softcap. */
int umb_cva_prep(float* q, const UmbPagedKV* kv, const float* proj, int ld, const void* conv_w, float* conv_state, const void* w_q,
                 const void* w_k, const int* pos, const int* slot, const float* freq, int T, int H, int G, int D, int E, int taps,
                 int rot_dims, int layout, int update_state, float eps, float* scratch, long scratch_floats, int dtype,
                 umb_stream_t stream);

/* ---- matrix memory with exponential gates.  Per (token, head), from columns i_col / f_col of proj: i = cap tanh(z_i / cap),
 * f = log sigmoid(cap tanh(z_f / cap)).  mscan: the running maximum m_t = max(f_t + m_(t-1), i_t) of every stretch (tiles of 64 tokens
 * scanned side by side; mstate fp32 [slots][H]; a sequence that starts at position 0 starts from m = 0); log_alpha[t][h] =
 * f_t + m_(t-1) - m_t, alpha its exponential, mrun[t][h] = m_t, bw[t][h] = e^(i_t - m_t).  prep: qs fp32 [T][H D] = q * qscale;
 * vp fp32 [T][H][Pp] = [bw v | bw | 0 ..] (Pp > Dv): a linear scan over (qs, k, vp, alpha) carries the matrix state and, as value
 * column Dv, the normaliser.  step: both for steps of one token per sequence. */
int umb_mlstm_mscan(float* log_alpha, float* alpha, float* mrun, float* bw, float* mstate, const float* proj, int ld, int i_col,
                    int f_col, float cap, const int* seq_slot, const int* seq_row0, const int* seq_pos0, const int* seq_len, int B,
                    int H, umb_stream_t stream);
int umb_mlstm_prep(float* qs, float* vp, const float* proj, int ld, int q_col, int v_col, const float* bw, int T, int H, int D,
                   int Dv, int Pp, float qscale, umb_stream_t stream);
int umb_mlstm_step(float* qs, float* vp, float* log_alpha, float* alpha, float* mrun, float* mstate, const float* proj, int ld,
                   int q_col, int v_col, int i_col, int f_col, const int* pos, const int* slot, int T, int H, int D, int Dv, int Pp,
                   float qscale, float cap, umb_stream_t stream);

/* ---- routed experts chosen on the logits: the `top` largest of logits[t ld ..E] (ties: the lower index); wt = softmax over
 * the chosen logits alone */
int umb_moe_route_top(int* sel, float* wt, const float* logits, int ld, int T, int E, int top, umb_stream_t stream);
/* y[t] = sigmoid(gate[t ldg]) * ys[t] + sum_k wt[t top + k] * ye[pos_of[t top + k]]  (ys null: none; gate null: 1; y may be ys) */
int umb_moe_combine_gated(float* y, const float* ys, const float* ye, const float* wt, const int* pos_of, const float* gate,
                          int ldg, int T, int W, int top, umb_stream_t stream);

/* ------------------------------------------------------------------ the model */
typedef struct UmbSeqLayer {
  int32_t kind, has_mlp;
  int32_t heads, kv_heads, dim, vdim;
  int32_t window, pool, rot_dims, rank;
  int32_t ff, pad_;
  float scale, tau, qscale, pad2_;
  UmbSeqLinear proj;      /* fused input projection: [q | k | gate] or [q | k | v | g | a] */
  UmbSeqLinear a2;        /* GLA: decay up-projection [heads dim][rank] + bias */
  UmbSeqLinear out;       /* output projection */
  UmbSeqLinear gu, down;  /* feed-forward: stacked [gate; up], down */
  const void* pos_bias;   /* attention: [heads] */
  const void* head_norm;  /* GLA: [vdim] */
  /* x <- x + norm1b(mixer(norm1(x))), x <- x + norm2b(ff(norm2(x))); norm1 / norm2 null: the sublayer reads the
   * residual stream itself (through the convolution below) */
  const void *norm1, *norm1b, *norm2, *norm2b;
  const float* rot_freq;  /* [rot_dims / 2] fp32 */
  UmbPagedKV kv;          /* attention layers */
  float* state;           /* GLA layers: [slots][heads][dim][vdim] fp32 */
  /* latent attention (proj = [dq | dkv | gate]) */
  int32_t q_rank, kv_rank, rot_dim, ff_kind;
  /* routed experts */
  int32_t experts, top, expert_ff, shared_ff;
  UmbSeqLinear uq;        /* [heads (dim + rot_dim)][q_rank] */
  const void* uk_t;       /* [heads][kv_rank][dim]: W_uk of every head, transposed */
  const void* uv;         /* [heads vdim][kv_rank] */
  const void *dq_norm, *dkv_norm, *sink;
  /* convolution in front of the sublayers: weights [W][taps], state [slots][taps - 1][W] fp32 (null: none) */
  const void *canon1, *canon2;
  float *canon_state1, *canon_state2;
  const void* act;        /* PolyNorm: {a, b, c, e} */
  UmbSeqLinear router;    /* [experts][W] */
  const void* e_gu;       /* [experts][2 expert_ff][W]: every expert's stacked [gate; up] */
  const void* e_down;     /* [experts][W][expert_ff] */
  UmbSeqLinear s_gu, s_down;   /* shared expert (s_gu.w null: none) */
  /* act: UMB_ACT_* of the dense feed-forward, the experts and the shared expert (relu^2: gu / e_gu / s_gu hold the
   * up-projection alone); route: UMB_ROUTE_*; correction fp32 [experts] (softmax routing, may be null) */
  int32_t act_kind, route_kind;
  const float* correction;
  /* several residual streams (model.streams >= 1): read / write / mix weights of the two sublayers, fp32, null = trivial */
  const float *hc1_in, *hc1_out, *hc1_mix, *hc2_in, *hc2_out, *hc2_mix;
  /* minGRU (kind 3): proj = [z | x | g], each `dim` wide; state [slots][dim] fp32.
   * attention beside a state-space layer (kind 4), both reading the same input: proj = [q | k | v | gate | z | x | B | C | dt];
   * attention: heads / kv_heads / dim / vdim / scale / window, q_norm / k_norm [dim], dist_bias fp32 [heads][n_dist],
   * query temperature; state space: s_heads x s_vdim, state size s_state, s_groups groups of B / C, s_taps convolution taps;
   * the output projection reads [mix_scale_a * attention | mix_scale_b * state space] */
  const void *q_norm, *k_norm;
  const float* dist_bias;
  int32_t n_dist, temp_every;
  float temp_coef, mix_scale_a, mix_scale_b, pad3_;
  int32_t s_heads, s_vdim, s_state, s_groups, s_norm_groups, s_taps;
  const void *s_conv, *s_conv_b, *s_norm;
  const float *s_dt_bias, *s_a_log, *s_d;
  float* s_conv_state;        /* [slots][s_taps - 1][channels] fp32 */
  /* retention (kind 5): proj = [q | k | v | g], heads x dim (q, k) and heads x vdim (v, g); decay fp32 [heads], one fixed decay
   * per head; rotary (rot_layout 0: halves, 1: interleaved; rot_dims, rot_freq) on q and k, k times qscale after it; each head's
   * read-out over its root mean square, times silu(g); state [slots][heads][dim][vdim].
   * convolved attention beside a matrix memory (kind 6), both reading the same input: proj = [q | k | v | mq | mk | mv | mg | i | f];
   * attention: heads / kv_heads / dim / vdim / scale / softcap, c_taps-tap convolution c_conv [(heads + kv_heads) dim + kv_heads
   * vdim][c_taps] with ring c_conv_state, whole-row norms q_norm [heads dim] / k_norm [kv_heads dim], rotary as above; memory:
   * m_heads x m_dim keys, m_vdim values, gates capped at gate_cap, m_norm [m_heads m_vdim], state [slots][m_heads][m_dim][m_pad]
   * (value column m_vdim carries the normaliser) and the running maximum m_max [slots][m_heads]; the output projection reads
   * [mix_scale_a * attention | mix_scale_b * memory] */
  const float* decay;
  int32_t rot_layout, c_taps;
  float softcap, gate_cap;
  const void* c_conv;
  float* c_conv_state;
  int32_t m_heads, m_dim, m_vdim, m_pad;
  const void* m_norm;
  float* m_max;
  /* UMB_ACT_CLAMP_GLU: limits of the experts (or the dense feed-forward) and of the shared expert, the sigmoid's factor;
   * shared_gate: the router's product has one more row, whose sigmoid multiplies the shared expert's output */
  float act_limit, shared_limit, act_alpha;
  int32_t shared_gate;
  /* the embedding row is added to x once more right before this layer (a span of layers that runs again) */
  int32_t add_embed, pad4_;
} UmbSeqLayer;

typedef struct UmbSeqModel {
  int32_t dtype, L, W, V, groups, canon_taps;
  float eps, embed_scale;    /* embed_scale: the embedding row is multiplied by it (1: as stored) */
  const void* embed; const void* final_norm; UmbSeqLinear head;
  const UmbSeqLayer* layers;
  /* streams >= 1: the residual is `streams` copies per token (ws.x is [Tmax][streams][W]), a sublayer is
   * x <- mix x + resid_mult * out * f(norm(in . x)) with norm weights stored around norm_offset, and the model ends with
   * the norm of the sum of the streams; 0: the single-stream forms above */
  int32_t streams, block;    /* block: UMB_BLOCK_* (parallel: norms stored around norm_offset, ws.h2 / ws.y2 in use) */
  float resid_mult, norm_offset;
  float logit_scale, pad2_;  /* the logits are multiplied by it (0 or 1: as they are) */
} UmbSeqModel;

/* activations of one step (caller-owned, sized for Tmax rows) */
typedef struct UmbSeqWork {
  float* x;        /* residual stream [Tmax][W] fp32 ([Tmax][streams][W] with several streams) */
  void* h;         /* normed input of the current sublayer [Tmax][W] dtype */
  float* proj;     /* fused projection output [Tmax][max proj N] fp32 */
  float* aux;      /* q / alpha [Tmax][max heads*dim] fp32 */
  float* o;        /* GLA scan output [Tmax][max heads*vdim] fp32 */
  void* mix;       /* mixer output before the output projection [Tmax][max heads*vdim] dtype */
  void* act;       /* feed-forward activation [Tmax][max ff] dtype */
  float* y;        /* sublayer output [Tmax][W] fp32 */
  float* logits;   /* [Rmax][V] fp32 */
  int32_t Tmax, Rmax;
  /* routed experts (null when no layer has any): pairs = Tmax * max top */
  int32_t* moe_sel;   /* [pairs] */
  float* moe_wt;      /* [pairs] */
  int32_t* moe_pos;   /* [pairs] */
  int32_t* moe_tiles; /* [moe_max_tiles][3] */
  void* moe_xs;       /* [pairs][W] dtype */
  void* moe_act;      /* [pairs][max expert_ff] dtype */
  float* moe_y;       /* [pairs][W] fp32 */
  int64_t moe_max_tiles;
  int64_t aux_floats;  /* floats in aux (what a step does not use of it serves as scratch) */
  void* h2;            /* parallel blocks: normed input of the feed-forward [Tmax][W] dtype */
  float* y2;           /* parallel blocks: feed-forward output [Tmax][W] fp32 */
} UmbSeqWork;

typedef struct UmbSeqStep {
  int32_t T, B, R, max_len;
  const int32_t *tokens, *pos, *slot;                       /* [T] */
  const int32_t *seq_slot, *seq_row0, *seq_pos0, *seq_len;  /* [B] */
  const int32_t* logit_rows;                                /* [R] rows whose logits are wanted */
  float* trace;                                             /* optional [L][T][W]: the residual stream after every layer (the sum of the streams) */
} UmbSeqStep;

int umb_lat_attend_tiled_ok(int H, int kv_rank, int rot_dim, int dtype);

int umb_seq_forward(const UmbSeqModel* m, const UmbSeqWork* ws, const UmbSeqStep* s, umb_stream_t stream);

/* sampling on fp32 logits rows (the same kernels as libumbrella_hip.so) */
int umb_argmax_rows(int* out, const float* logits, int rows, int V, umb_stream_t stream);
int umb_sample_rows(int* sampled, float* logits, int rows, int V, const int* tokens_all, const int* n_ptr,
                    float penalty, float temperature, int topk, float topp, const void* seed, int dbg_k,
                    int* dbg_idx, float* dbg_p, umb_stream_t stream);

const char* umb_seq_version(void);

#ifdef __cplusplus
}
#endif
#endif
