// lm_kernels.h — launchers of the layered-model tier (api_lm.hip): a decoder stack whose layers are described by data (which
// mixer, which feed-forward, which sizes), served for ragged batches of sequences that each own a state slot.
//
// Conventions shared by every launcher below
//   * Activations are fp32 rows in device memory; weights are bf16 [out][in] row-major (K contiguous), vectors fp32.
//   * A step carries M token rows (all entries of the batch back to back).  Per-row metadata lives in device arrays:
//     row_pos (position of the token in its sequence), row_slot (state slot of its sequence), row_prev (row index of the token
//     in front of it when that token is part of the same step, -1 when it is held by the slot's state).
//   * `f32` selects true 32-bit products (fp32 MFMA / fp32 FMA) instead of bf16 x bf16 products with fp32 accumulation.
//     Norms, softmax, gates, recurrent state, positions and the residual are fp32 in both modes.
#pragma once
#include "zg_common.h"

namespace zg {
namespace lm {

// ------------------------------------------------------------------------------------------------ linear maps
enum { ACT_NONE = 0, ACT_RELU2 = 1, ACT_GELU_ERF = 2, ACT_SCALE_SOFTCAP = 3 /* v <- v act_a, then act_b tanh(v / act_b) when act_b > 0 */ };
// Gated activations of rows [gate (F) | up (F)] (GLU_CLIPPED: also a row factor and the clip `limit`)
enum { GLU_SILU = 0 /* silu(gate) up */, GLU_CLIPPED = 1 /* g sigmoid(1.702 g) (u + 1), g = min(s gate, limit), u = clamp(s up, -limit, limit) */ };

// C[m][n] = act( sum_k A[arow(m)][k] * B[n][k] )      for m < M, n < N
//   arow(m) = a_rows ? a_rows[m] / a_div : m          (row gather: a token's row feeds each of its expert assignments)
//   nz > 1: grid.z batches with element offsets a_zoff / b_zoff / c_zoff per z (one matrix per head)
//   z_group != null: batch z reads the matrix B + z_group[z] * b_zoff instead (the expert an assignment was routed to)
//   grp_off != null (n_groups > 0): rows [grp_off[e], grp_off[e + 1]) of A / C use the matrix B + e * b_zoff (rows sorted by
//   expert); M is then the total row count, an upper bound for the tile list
struct Linear {
    const float* A = nullptr;
    int lda = 0;
    const int* a_rows = nullptr;
    int a_div = 1;
    const bf16_t* B = nullptr;
    int ldb = 0;
    float* C = nullptr;
    int ldc = 0;
    int M = 0, N = 0, K = 0;
    int act = ACT_NONE;
    float act_a = 1.0f, act_b = 0.0f;  // constants of ACT_SCALE_SOFTCAP
    int a_glu = 0;  // > 0 (row-vector kernel only): A rows are [gate (a_glu) | up (a_glu)] and enter through their gated activation, K = a_glu
    int glu_kind = GLU_SILU;
    float glu_limit = 0.0f;            // GLU_CLIPPED
    const float* glu_scale = nullptr;  // GLU_CLIPPED, batched one-row form: factor of batch z's row (null: 1)
    int glu_gate_col = -1;             // >= 0: the activated row is multiplied by sigmoid(A row[glu_gate_col]) (a gate logit behind gate | up)
    int nz = 1;
    long long a_zoff = 0, b_zoff = 0, c_zoff = 0;
    const int* z_group = nullptr;
    const int* grp_off = nullptr;
    int n_groups = 0;
};
// Picks the row-vector kernel (few rows: decode) or the tiled matrix-core kernel (prompt portions).
int launch_linear(const Linear& L, bool f32, hipStream_t s);
constexpr int kGemvMaxRows = 8;
// Two products of one-row batches (M == 1 each) in ONE launch of the row-vector kernel; whatever does not fit that form runs as two
// launches.  Neither product may read what the other writes.
int launch_linear_pair(const Linear& a, const Linear& b, bool f32, hipStream_t s);

// ------------------------------------------------------------------------------------------------ norms, embedding, shift
// x[m] = table[ids[m]] (bf16 -> fp32); an id outside [0, vocab) raises *flag (pinned or device int) and yields a zero row.
// scale multiplies the row; x_copy (may be null) receives the same rows.
// pos_freq != null: the position's sinusoid vector is added: entry 2i = sin(row_pos[m] * pos_freq[i]), entry 2i + 1 = cos of that
// angle (an fp32 product; pos_freq[i] = 10000^(-2i/W), rounded once on the host).
int launch_embed(const bf16_t* table, const int* ids, float* x, float* x_copy, float scale, int M, int W, int vocab, int* flag, const int* row_pos,
                 const float* pos_freq, hipStream_t s);
// RMS norm with a weight stored as an offset from one, then the token shift:
//   h[m] = x[m] / rms(x[m]) * (1 + w);   out[m] = h[m] + (h[prev(m)] - h[m]) * mu
// prev(m) = row_prev[m] when >= 0, else the row kept for the slot: shift_state[row_slot[m]] (zeros for a new sequence).
// Rows listed in last_rows (the last token of every entry) also store their UNSHIFTED h into last_out[entry] — committed to
// the slots' state by launch_commit_rows once the step has run, so that no row of this launch reads a state another row wrote.
// mu == null: no shift (out = h).
int launch_norm_shift(const float* x, const float* w, const float* mu, float eps, float* out, int M, int W, const int* row_prev,
                      const int* row_slot, const float* shift_state, size_t slot_stride, const int* row_entry_if_last, float* last_out,
                      hipStream_t s);
// dst[slots[e]] = src[e] for every entry e; rows of `width` floats (dst rows slot_stride apart, src rows src_stride apart)
int launch_commit_rows(float* dst, size_t slot_stride, const float* src, size_t src_stride, const int* slots, int n_entries, int width,
                       int n_sets, size_t dst_set_stride, size_t src_set_stride, hipStream_t s);
// x[m] += y[m] / rms(y[m]) * (1 + w)            (the norm behind a sublayer, then the residual sum)
int launch_norm_add(float* x, const float* y, const float* w, float eps, int M, int W, hipStream_t s);
// x[m] += y[m] / rms(y[m]) * (1 + wb);  h[m] = x[m] / rms(x[m]) * (1 + wn)   (the two above in one launch)
int launch_norm_add_norm(float* x, const float* y, const float* wb, const float* wn, float eps, float* h, int M, int W, hipStream_t s);
// Steps of one row per entry: the sum behind a pass's last sublayer (y, or the weighted sum of the chosen experts' rows yexp) and
// the next pass's norm + shift in one launch.  *taken = false for rows too wide for its registers (nothing launched).
int launch_sum_norm_shift(float* x, const float* y, const float* yexp, const float* weight, int top, const float* wb, const float* wn, const float* mu,
                          float eps, float* out, int M, int W, const int* row_slot, const float* shift_state, size_t slot_stride,
                          const int* row_entry_if_last, float* last_out, hipStream_t s, bool* taken);
// out[j] = x[rows[j]] / rms * (1 + w)            (the model's last norm on the rows whose logits are asked for; plain: * w)
int launch_norm_gather(const float* x, const int* rows, const float* w, float eps, float* out, int n_rows, int W, bool plain, hipStream_t s);
// Side-by-side sublayers: both read the same x through norms with plain weights, so one pass serves both:
//   [x[m] += add.a[m] + add.b[m] + add.w * add.bias + sum_k (add.exp_w ? add.exp_w[m top + k] : 1) add.exp[m top + k]
//    (what the layer before left open; any part may be null)]
//   ha[m] = x[m] / rms(x[m]) * wa;   hb[m] = x[m] / rms(x[m]) * wb   (hb / wb may be null)
struct OpenSums {
    const float *a = nullptr, *b = nullptr, *bias = nullptr;
    float w = 0.0f;
    const float *exp = nullptr, *exp_w = nullptr;  // rows of the chosen experts in assignment order, `top` per token
    int top = 0;
    __host__ __device__ bool any() const { return a || b || bias || exp; }
};
int launch_norm_two(float* x, const OpenSums& add, const float* wa, const float* wb, float eps, float* ha, float* hb, int M, int W, hipStream_t s);
// x[m] += the same sums
int launch_add_two(float* x, const OpenSums& add, int M, int W, hipStream_t s);
// In place over `rows` rows of `width` floats with row stride ld: v / rms(v) * w  (a plain weight; per-head norms)
int launch_norm_plain(float* v, int ld, int rows_per_m, int width, int M, const float* w, float eps, hipStream_t s);

// Norms without statistics: n(v) = tanh(alpha v) * w + b.  A norm's tensors lie together, nw = [w (W) | b (W) | alpha (1)].
// out[j] = n(x[rows ? rows[j] : j]);  pre != null (rows == null): x[j] <- pre(x[j]) first, in place (a norm behind the embedding).
int launch_tanh_norm(float* x, const float* pre, const float* nw, const int* rows, float* out, int n_rows, int W, hipStream_t s);
// What a sublayer left, summed in a fixed order:  a[m] + sum_k exp_w[m top + k] * exp[inv ? inv[m top + k] : m top + k] + b[m]
// (any part may be null; the experts' rows in choice order).
struct SumParts {
    const float *a = nullptr, *exp = nullptr, *exp_w = nullptr;
    const int* inv = nullptr;
    int top = 0;
    const float* b = nullptr;
};
// x[m] += mult * nb(sum of the parts);  h[m] = nn(x[m])   (nn / h may be null): the norm behind a sublayer, the residual sum and
// the norm in front of the next sublayer in one launch.
int launch_tanh_sum_norm(float* x, const SumParts& y, const float* nb, float mult, const float* nn, float* h, int M, int W, hipStream_t s);

// ------------------------------------------------------------------------------------------------ gated linear recurrence (HGRN2)
// proj rows are [q (H D) | f (H D) | v (H V)] as the fused projection left them; the gates are activated where the scan stages
// them:  q <- silu(q);   f <- low + (1 - low) * sigmoid(f + bias)
// Per entry e (rows ent_start[e] .. + ent_len[e]) and head: S <- diag(f_t) S + (1 - f_t) v_t^T, o_t = S^T q_t, token by token,
// S = state[ent_slot[e]] ([H][D][V] fp32) read at the start and written back at the end.  out rows [H V], row stride ldo.
// M: rows of the step.  ws (may be null): workspace for the chunk-parallel form of long steps, (M / 64 + n_entries) * (H D V + H D) floats.
// decay != null: linear attention with one fixed decay per head on the same machinery — proj rows [q (H D) | k (H D) | v (H V)], all
// three through silu on their way in:  S <- decay[h] S + k_t v_t^T, o_t = S^T q_t   (bias / low unused).
// gla != null: gated linear attention with a decay per key channel on the same machinery — proj rows [q (H D) | k (H D) | v (H V)]
// taken as they are, q times q_scale;  f = sigmoid(z + z_bias)^inv_tau, z rows [H D] with stride ldz (fp32 logarithm and
// exponential);  S <- diag(f) S + k_t v_t^T, o_t = S^T q_t.
struct GlaGate {
    const float* z = nullptr;
    int ldz = 0;
    const float* z_bias = nullptr;
    float inv_tau = 1.0f, q_scale = 1.0f;
};
int launch_hgrn2_scan(const float* proj, int ld, float* out, int ldo, float* state, size_t slot_stride, const int* ent_start,
                      const int* ent_len, const int* ent_slot, int n_entries, int M, int H, int D, int V, const float* bias, const float* low,
                      float* ws, size_t ws_floats, hipStream_t s, const float* decay = nullptr, const GlaGate* gla = nullptr);

// ------------------------------------------------------------------------------------------------ latent attention
// Rotary table of one layer: freq[i] for the rot_dims / 2 pairs (YaRN blend applied on the host) and the amplitude factor.
// proj rows: [dq (q_rank) | dkv latent (KR) | rotated key part (R)].  Writes cq[m] = norm(dq) * wq, and the token's cache row
// (latent = norm(dkv latent) * wkv | rotary(key part)) at its position: cache row of (slot, pos) = page_table[slot][pos / P] * P + pos % P.
struct Rotary {
    const float* freq;  // [dims / 2]
    int dims;           // rotated dimensions (the first `dims` of the part; the rest pass)
    float amp;
};
int launch_latent_prep(const float* proj, int ld, int M, int q_rank, int KR, int R, const float* wq, const float* wkv, float eps, Rotary rot,
                       const int* row_pos, const int* row_slot, const int* page_table, int max_pages, int page_tokens, float* cq,
                       float* cache, hipStream_t s);
// qa[m][h][KR ..] = rotary(q[m][h][D ..]) — the rotated query part moved behind the absorbed part (which a batched Linear wrote).
int launch_q_rotary(const float* q, int ldq, float* qa, int ldqa, int M, int H, int D, int R, int KR, Rotary rot, const int* row_pos, hipStream_t s);
// ctx[m][h][:KR] = sum_j softmax_j( scale * qa[m][h] . cacherow(j) ) latent(j) over the keys j <= row_pos[m] of the row's sequence.
// ws: fp32 workspace for the partials of split key ranges (steps of at most kGemvMaxRows rows: M * H * kAttnSplits * (KR + 2)
// floats; without it whole key rows per workgroup).
constexpr int kAttnSplits = 16;
int launch_latent_attention(const float* qa, float* ctx, int M, int H, int KR, int R, float scale, const int* row_pos, const int* row_slot,
                            const int* page_table, int max_pages, int page_tokens, const float* cache, float* ws, size_t ws_floats, hipStream_t s);

// The same for prompt portions on the matrix cores (bf16 operands, fp32 scores / softmax / accumulation): 32 queries of one entry
// and four heads per workgroup.  *taken = false when the latent is larger than the kernel's tiles hold (nothing launched).
int launch_latent_attention_tiles(const float* qa, float* ctx, int M, int H, int KR, int R, float scale, const int* ent_start, const int* ent_len,
                                  const int* ent_slot, int n_entries, const int* row_pos, const int* page_table, int max_pages, int page_tokens,
                                  const float* cache, hipStream_t s, bool* taken);

// ------------------------------------------------------------------------------------------------ causal convolutions with a tail
// out[m][c] = act( bias[c] + sum_j w[c][j] * in(m - (taps - 1) + j)[c]  (+ in(m)[c] with CONV_RESIDUAL) ),  in(.) = in[.] + pre_bias;
// inputs in front of the step come from the slot's tail ([taps - 1][C] floats at tail + slot * slot_stride, oldest first; zeros
// for a new sequence), which a second launch then moves on by the entry's tokens.  row_off[m]: place of row m inside its entry.
enum { CONV_RESIDUAL = 1, CONV_SILU = 2 };
struct ConvArgs {
    const float* in = nullptr;
    int ld_in = 0;
    float* out = nullptr;
    int ld_out = 0;
    int C = 0, taps = 1;
    const float* w = nullptr;         // [C][taps] fp32, last column = the current token
    const float* bias = nullptr;      // [C] or null
    const float* pre_bias = nullptr;  // [C] or null: a bias of the input rows (the tail holds inputs with it)
    int flags = 0;
    float* tail = nullptr;
    size_t slot_stride = 0;
};
// one_row_each: every entry brings exactly one row (decode steps): the convolution's own threads move the tails on, no second launch.
int launch_causal_conv(const ConvArgs& a, int M, int n_entries, bool one_row_each, const int* row_off, const int* row_slot, const int* ent_start,
                       const int* ent_len, const int* ent_slot, hipStream_t s);
// Steps of one row per entry: [x += x0] or [x += norm(y) * (1 + wb), y = yl or the mean of the two normed branches yl, yr with
// plain weights wl, wr], then h = norm(x) * (1 + wn), out = h + conv(h) over the slot's tail, the tail moved on — one launch.
// *taken = false for rows too wide for its registers (nothing launched).
int launch_norm_conv_single(float* x, const float* x0, const float* yl, const float* yr, const float* wl, const float* wr, const float* wb,
                            const float* wn, float eps, int M, int W, int taps, const float* cw, float* tail, size_t slot_stride,
                            const int* row_slot, float* out, hipStream_t s, bool* taken);
// x[m] += y[m]
int launch_add_rows(float* x, const float* y, int M, int W, hipStream_t s);

// ------------------------------------------------------------------------------------------------ windowed attention (sink, mixed heads, rotated values)
// proj rows [q (H D) | k (G D) | v (G V)]: q rotated in place; the rotated key and the value rotated over all V channels (pair i by
// pos * vfreq[i]) written to the token's cache row [G D | G V]; the page of (slot, pos) is page_table[slot][(pos / P) % max_pages]:
// a ring, so that a sequence whose old pages have been given back can grow beyond max_pages * P positions.
int launch_window_prep(float* proj, int ld, int M, int H, int G, int D, int V, Rotary rot, const float* vfreq, const int* row_pos,
                       const int* row_slot, const int* page_table, int max_pages, int page_tokens, float* cache, hipStream_t s);
// out[m][h] = turn_back_pos( sum_j w_h(j) value_(h / (H/G))(j) ),  w_h = sum_g talk[h][g] p_g,
// p_g(j) = exp(s_g(j)) / (exp(sink_g) + sum_j' exp(s_g(j'))),  s_g(j) = scale q_g . k(j),  over the keys pos - window < j <= pos
// (window 0: all j <= pos).  sink / talk may be null (no sink / no mix).
// keep_first > 0: beyond the window the first keep_first positions of the sequence stay visible (a row's keys are then numbered
// kept tokens first, then the window).  vfreq == null: values are cached unrotated and nothing is turned back.
// shape: what becomes of a scaled score before the softmax — capped (cap > 0: cap tanh(s / cap)), then less slope[h] per position
// of distance between the query and the key (slope != null).
struct ScoreShape {
    float cap = 0.0f;
    const float* slope = nullptr;  // [H]
};
int launch_window_attention(const float* q, int ldq, float* out, int ldo, int M, int H, int G, int D, int V, float scale, int window,
                            int keep_first, const float* sink, const float* talk, const float* vfreq, const int* row_pos, const int* row_slot,
                            const int* page_table, int max_pages, int page_tokens, const float* cache, hipStream_t s,
                            ScoreShape shape = ScoreShape());
// The prep of attention whose q and k are divided by their root mean square PER HEAD (no weight) and whose values are the
// un-normalised key heads: rows qk [q (H D) | k (G D)]; q <- q / rms(q) * (1 + qt_coef ln(floor((pos + 1) / qt_every) + 1)) in place (qt_every 0:
// no factor); the token's cache row [G D | G D] receives k / rms(k) and, behind it, k itself.
int launch_head_norm_prep(float* qk, int ld, int M, int H, int G, int D, float eps, float qt_coef, int qt_every, const int* row_pos,
                          const int* row_slot, const int* page_table, int max_pages, int page_tokens, float* cache, hipStream_t s);
// The prep of attention without rotation whose q and k are normed over the whole projection: rows qkv [q (H D) | k (G D) | v (G V)];
// q <- q / rms(q) * wq in place (rms over all H D entries), k / rms(k) * wk and v into the token's cache row [G D | G V].
// Steps of one row per entry: the convolution `a` over the channels q | k | v (its tails moved on) and the prep below in one launch,
// q written normed to qout.  *taken = false (nothing launched) for rows beyond its registers.
int launch_conv_norm_prep_single(const ConvArgs& a, float* qout, int ld_q, int M, int HD, int GD, int GV, const float* wq, const float* wk, float eps,
                                 const int* row_pos, const int* row_slot, const int* page_table, int max_pages, int page_tokens, float* cache,
                                 hipStream_t s, bool* taken);
int launch_whole_norm_prep(float* qkv, int ld, int M, int HD, int GD, int GV, const float* wq, const float* wk, float eps, const int* row_pos,
                           const int* row_slot, const int* page_table, int max_pages, int page_tokens, float* cache, hipStream_t s);

// The same with a row's keys split over up to kWinSplits workgroups and the scores kept in a workspace (three launches): what
// steps of few rows need to fill the chip, and prompt portions to compute every score once.  key_capacity: the most keys a row
// can see (the window, or the longest sequence).  ws: window_split_workspace(rows, ...) floats.  *taken = false (nothing
// launched) when the workspace is too small or a size is beyond the kernels' limits.  Portions (more than kGemvMaxRows rows, heads
// of at most 128 channels) take their scores from 32 x 32 tiles on the matrix cores in true fp32 (rows of an entry are consecutive
// rows with consecutive positions: ent_start / ent_len).
constexpr int kWinSplits = 64;
size_t window_split_workspace(int rows, int H, int V, int key_capacity, int* n_split_out);
int launch_window_attention_split(const float* q, int ldq, float* out, int ldo, int M, int H, int G, int D, int V, float scale, int window,
                                  int keep_first, const float* sink, const float* talk, const float* vfreq, const int* row_pos, const int* row_slot,
                                  const int* page_table, int max_pages, int page_tokens, const float* cache, int key_capacity, float* ws,
                                  size_t ws_floats, const int* ent_start, const int* ent_len, int n_entries, hipStream_t s, bool* taken,
                                  const float* out_gate = nullptr, int ld_gate = 0, float out_factor = 1.0f, ScoreShape shape = ScoreShape());
// (out_gate != null: a taken step multiplies the result by sigmoid(out_gate[m][.]) * out_factor where the shares are added)

// ------------------------------------------------------------------------------------------------ real-gated linear recurrent unit
// Per entry and channel c: r = sigmoid(gr + br), i = sigmoid(gi + bi), a = exp(-8 r softplus(lam)), S = a S + sqrt(1 - a^2) i u,
// out = S * gelu_tanh(y + by); S = state[slot][c], read at the start of the entry and written back at its end.
int launch_rglru_scan(const float* u, int ldu, const float* gr, const float* gi, int ldg, const float* br, const float* bi, const float* lam,
                      const float* y, int ldy, const float* by, float* out, int ldo, int C, float* state, size_t slot_stride, const int* ent_start,
                      const int* ent_len, const int* ent_slot, int n_entries, hipStream_t s);
// y[m] = (l[m] / rms(l[m]) * wl + r[m] / rms(r[m]) * wr) / 2
int launch_pair_norm_mean(const float* l, const float* r, const float* wl, const float* wr, float eps, float* y, int M, int W, hipStream_t s);

// ------------------------------------------------------------------------------------------------ gated delta rule, decay per key channel
// In place: the G query heads and G key heads of qk rows ([q (G D) | k (G D)]) to unit length (q also times D^-1/2);
// beta <- sigmoid(beta);  dec[h][d] <- exp(-exp(a_log[h]) * softplus(dec[h][d] + dt_bias[h][d])).
int launch_delta_prep(float* qk, int ldqk, int G, int D, float* beta, int ldb, int H, float* dec, int ldd, const float* a_log,
                      const float* dt_bias, int M, hipStream_t s);
// Per entry and head h (query / key head h / (H / G)), token by token on S = state[slot][h] ([D][V] fp32):
//   S <- diag(dec) S;  u = beta (v - S^T k);  S <- S + k u^T;  out = S^T q.
int launch_delta_scan(const float* qk, int ldqk, const float* v, int ldv, const float* beta, int ldb, const float* dec, int ldd, float* out,
                      int ldo, int H, int G, int D, int V, float* state, size_t slot_stride, const int* ent_start, const int* ent_len,
                      const int* ent_slot, int n_entries, hipStream_t s);
// In place over M * rows_per_m vectors of `width` floats: v / rms(v) * w * sigmoid(gate) * factor (gate laid out like v, row stride
// ldg).  w == null: no norm, the gate and the factor only.
// gate_silu: the gate is silu(gate) instead of sigmoid(gate).
int launch_norm_gate(float* v, int ld, int rows_per_m, int width, int M, const float* w, float eps, const float* gate, int ldg, hipStream_t s,
                     float factor = 1.0f, bool gate_silu = false);

// ------------------------------------------------------------------------------------------------ mixture of experts
// Per row: z = router . g (fp32), s = softmax(z), the `top` experts by s + correction (lowest index wins a tie), weights s.
// top_logits: z += correction (a bias), the `top` largest z (lowest index wins a tie), weights = softmax over the chosen z.
// rule ZG_LM_ROUTE_SIGMOID_INPUT: the `top` largest z (= the largest sigmoid scores; lowest index wins a tie), weights sigmoid(z).
// rule ZG_LM_ROUTE_SIGMOID_GROUPS: s = sigmoid(z), experts ranked by r = s + correction; the expert list is cut into `groups`
// contiguous blocks of equal size, a block ranks by r of its best plus r of its second-best expert, experts outside the `keep`
// top-ranked blocks get r = -inf; the `top` highest r win (lowest index wins a tie); weights s / (sum of the winners' s + 1e-20)
// * out_scale.
// pre != null (norms without statistics, widths up to kRouteFuseWidth): the routing workgroup of a row first does what
// launch_tanh_sum_norm would — x[m] += mult * nb(sum of y's parts), h[m] = nn(x[m]) with h == g — and routes on the result.
struct RoutePre {
    float* x = nullptr;
    SumParts y;
    const float* nb = nullptr;
    float mult = 1.0f;
    const float* nn = nullptr;
    float* h = nullptr;
};
constexpr int kRouteFuseWidth = 8192;
int launch_route(const float* g, int M, int W, const bf16_t* router, const float* correction, int E, int top, int* pick, float* weight,
                 int rule, hipStream_t s, int groups = 1, int keep = 1, float out_scale = 1.0f, const RoutePre* pre = nullptr);
// Sort the M * top assignments by expert: grp_off[E + 1], sorted[p] = assignment at sorted position p, inv[a] = position of a.
int launch_group(const int* pick, int n_assign, int E, int* grp_off, int* sorted, int* inv, hipStream_t s);
// h[p][j] = silu(gu[p][j]) * gu[p][F + j]
int launch_glu(const float* gu, float* h, int rows, int F, hipStream_t s);
// h[p][j] = act(s gu[p][j], s gu[p][F + j]) * t,  act(g, u) = g' sigmoid(1.702 g') (u' + 1), g' = min(g, limit), u' = clamp(u, -limit, limit)
//   s = row_scale ? row_scale[row_of ? row_of[p] : p] : 1   (the router's score of the assignment that sits at sorted place p)
//   t = gate_col >= 0 ? sigmoid(gu[p][gate_col]) : 1        (a gate logit that the same product left in the row)
// gu rows ld floats apart.
int launch_glu_clipped(const float* gu, int ld, float* h, int rows, int F, float limit, const float* row_scale, const int* row_of, int gate_col,
                       hipStream_t s);
// y[m] = sum_k (weight ? weight[m top + k] : 1) * yexp[inv ? inv[m top + k] : m top + k] (+ ys[m]), in choice order
int launch_expert_sum(float* y, const float* yexp, const int* inv, const float* weight, int top, const float* ys, int M, int W, hipStream_t s);
// y = sum_k weight[m][k] * yexp[inv ? inv[m top + k] : m top + k];   x[m] += y / rms(y) * (1 + w)
int launch_moe_combine(float* x, const float* yexp, const int* inv, const float* weight, int top, const float* w, float eps, int M, int W,
                       hipStream_t s);

// ------------------------------------------------------------------------------------------------ sampling support
// Per row: the maximum of its logits and the index of the first element that reaches it.  part_val / part_idx: workspace of
// rows * kArgmaxParts elements each (the row is scanned in slices by that many workgroups, a second launch combines them).
constexpr int kArgmaxParts = 64;
int launch_row_argmax(const float* logits, int rows, int n, float* max_out, int* idx_out, float* part_val, int* part_idx, hipStream_t s);

}  // namespace lm
}  // namespace zg
