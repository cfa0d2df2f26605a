// layered.h — launchers of the kernels that models described as a LIST OF LAYERS use (csrc/layered_model.cpp): a residual stream kept in
// f32, scalar-gain RMS norms with a short causal convolution in front of every sublayer, softmax attention with a logarithmic distance
// penalty and a sink term, retention (linear attention with a fixed decay per head, f32 state), a clamped gated feed-forward.
//
// One build serves both operand types: `bf16` selects 16-bit (bfloat16 bits) or f32 storage of GEMM operands, K/V cache rows and
// weights.  Norms, angles, scores, softmax weights, the recurrence and the residual sum are f32 in both.  Every mechanism's constants
// are arguments, none is baked in.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace nvr { namespace kl {

// One step's batch: row t of the step belongs to sequence row_seq[t]; the rows of sequence b are cu[b] .. cu[b+1]-1 and sit at
// positions start[b], start[b]+1, ... of that sequence.  slot[b] is its state slot, par[b] the half of the double-buffered
// convolution history that holds its state BEFORE this step (the step writes the other half).  Device pointers.
struct Batch {
    const int64_t *ids;
    const int32_t *row_seq, *cu, *start, *slot, *par, *block_tables;
    int32_t max_blocks, block_size, T, B, max_ctx;      // max_ctx: upper bound of start[b] + rows of b (host side)
    int32_t max_rows;                                   // longest chunk of the step
};

int prepare();                                          // LDS opt-ins (call once, outside captures)

// x[t] = E[ids[t]] * scale (f32 residual stream)
int embed_scale(const void *E, bool bf16, const int64_t *ids, int64_t T, int64_t W, float scale, float *x, hipStream_t s);

// u = x / sqrt(mean(x^2) + eps); for each of up to two consumers c: h = g_c * u, out_c[t] = h_t + sum_j w_c[:, j] * h_(t - taps + 1 + j), rows before
// position 0 are zero and rows before the chunk come from the history hist[par][slot] ([taps-1][W] f32 rows of u); the last row of every
// chunk writes the other half.  hist: [2][slots][taps-1][W].  out2 / w2 may be null (one consumer).  taps >= 1.
int norm_canon(const float *x, const Batch &b, int64_t W, float eps, int taps, float g1, const float *w1, void *out1, float g2, const float *w2, void *out2,
               bool bf16, float *hist, int64_t slots, hipStream_t s);

// rows of K ([G][D]) and V ([G][Dv]) out of the projection rows (operand type) (row stride ld; column offsets kcol / vcol) into the paged caches
// [blocks][block_size][G][D] / [..][Dv] at the rows' positions
int kv_store(const void *proj, int64_t ld, int64_t kcol, int64_t vcol, const Batch &b, int64_t G, int64_t D, int64_t Dv, void *kc, void *vc, bool bf16,
             bool v_grouped, hipStream_t s);   // v_grouped: the value page layout of the tiled attention, [block][block_size / 8][G][Dv][8 keys]

// Causal softmax attention through the block tables: query row t at position i sees keys j <= i of its sequence;
// score = q.k * scale - r1[h] * ln(1 + r2[h] * (i - j)); the denominator also holds exp(sink[h]) (no key, no value).  r1 / r2 / sink may be null (plain
// softmax attention).  q: rows of the operand type (stride ldq, heads [H][D]); out rows (stride ldo elements, heads [H][Dv]) of the operand type.
struct SinkAttnArgs {
    const void *q; int64_t ldq;             // operand type
    const void *kc, *vc;
    const float *r1, *r2, *sink;
    int32_t H, G, D, Dv; float scale;
    void *out; int64_t ldo;
    const float *pen; int32_t pen_n;         // tiled form: penalty_table of this layer ([H][pen_n]; null: no penalty)
    int32_t v_grouped;                       // tiled form: value pages in groups of 8 keys per column (kv_store's v_grouped), else row-major [.][G][Dv]
    int64_t vld;                             // general form: elements between the value rows of consecutive key/value heads (0: Dv); with vc = kc and vld = D the values
                                             // are the first Dv numbers of the key rows (one cached row per token serves as key and value)
    const float *slope;                      // a linear distance penalty instead of the logarithmic one: score -= slope[h] * (i - j) (null: none; not together with r1 / r2).
                                             // The tiled form takes it as its table (linear_penalty_table)
    int32_t window;                          // > 0: position i sees only the keys j with i - j < window (itself and the window - 1 before it); 0: every key j <= i
    int32_t chunk;                           // > 0: position i sees only the keys j <= i of its own chunk, floor(j / chunk) == floor(i / chunk), chunks counted from position 0
    float softcap;                           // > 0: score <- softcap * tanh(score / softcap) (after the scale, before any bias)
    const float *gate_bias;                  // not null: no softmax — the weight of a visible key is sigmoid(score + gate_bias[h]), not normalised over the keys
                                             // (both forms; not together with a penalty or a sink)
};
int sink_attention(const SinkAttnArgs &a, const Batch &b, bool bf16, hipStream_t s);     // any shape; a context that fits the LDS score buffer
// The same on the matrix cores (bf16 operands, D % 32 == 0, Dv % 16 == 0, both <= 256, H / G <= 16).  tiles (device, built by the host): tile i covers the
// rows row0 .. row0 + 64 / (H / G) - 1 of sequence seq's chunk, for all H / G query heads of a key/value head.  nsplit > 1 spreads a tile's keys over that many
// workgroups (decode-sized steps over long contexts) and merges their partials; workspace: sink_attention_workspace_bytes(ntiles * G * nsplit).
struct AttnTile { int32_t seq, row0; };
bool sink_attention_tiled_ok(const SinkAttnArgs &a, bool bf16, int block_size);   // (pages of a multiple of 8 tokens)
// tab[h][d] = r1[h] * ln(1 + r2[h] * d) * log2(e) for d < n: the penalty the tiled form subtracts in the base-2 domain
int penalty_table(const float *r1, const float *r2, int64_t H, int64_t n, float *tab, hipStream_t s);
// tab[h][d] = slope[h] * d * log2(e): the same table for a linear penalty
int linear_penalty_table(const float *slope, int64_t H, int64_t n, float *tab, hipStream_t s);
size_t sink_attention_workspace_bytes(int max_workgroups);
int sink_attention_tiled(const SinkAttnArgs &a, const Batch &b, const AttnTile *tiles, int ntiles, int nsplit, void *workspace, size_t workspace_bytes, hipStream_t s);

// Retention over the rows of a step: per head S <- decay[h] * S + k v^T, o = S^T q, with q and k rotated (first rot_dims coordinates, pairs (i, i + rot_dims/2),
// angle = position * freq[i], cosines and sines from a table) and k scaled by kscale after the rotation.  state: [slots][H][D][Dv] f32, zero at position 0.  proj: rows of the operand type (stride ld) holding
// q at column qcol ([H][D]), k at kcol, v at vcol ([H][Dv]).  o: f32 [T][H*Dv].
struct RetentionArgs {
    const void *proj; int64_t ld, qcol, kcol, vcol;
    const float *decay, *cos_t, *sin_t; int32_t rot_dims; float kscale;   // cos_t / sin_t: [positions][rot_dims / 2] of angle = position * freq[i]
    int32_t H, D, Dv;
    float *state; float *o;
    // gated form (az not null): the decay of token t and key channel d of head h is sigmoid(az[t][h * D + d] + abias[h * D + d])^inv_tau, all in f32 from rows of
    // the operand type (stride ldz), instead of decay[h]; q is scaled by qscale
    const void *az; int64_t ldz; const float *abias; float inv_tau, qscale;
    // token-gated form (tok_gate not null): S <- keep S + take k v^T with the two f32 numbers (keep, take) of token t and head h at tok_gate[(t * H + h) * 2]
    // (instead of decay[h]); q is scaled by qscale.  v_ones: the last v_ones of the Dv value columns are not read from proj (whose value rows hold Dv - v_ones
    // numbers per head): their value is 1 for every token, so that the state's column is the gated running sum of the keys and o's column its product with q.
    const float *tok_gate; int32_t v_ones;
    // qk_share > 1: that many consecutive heads read the same q and k (head h those of group h / qk_share; proj holds H / qk_share of each): a state-space layer's
    // input and output maps B and C shared by a group of heads
    int32_t qk_share;
    // gated form, decay_exp: the decay is exp(-exp(az + abias)) instead of a power of the sigmoid.  bonus (gated form, [H][D] f32): the output is read BEFORE the update
    // and sees the current token through the bonus alone, o = (S_(t-1) + diag(bonus_h) k v^T)^T q, then S_t = diag(decay) S_(t-1) + k v^T
    bool decay_exp; const float *bonus;
};
int retention(const RetentionArgs &a, const Batch &b, bool bf16, hipStream_t s);
// out[t][h*Dv + c] = o[t][h][c] / rms(o[t][h][:]) * w[c] * silu(gate[t][h*Dv + c]); gate: rows of the operand type (stride ldg) from column gcol; w (one weight per
// value column, shared by the heads) may be null; w_heads: w holds a weight per head and column ([H * Dv])
int head_norm_gate(const float *o, const void *gate, int64_t ldg, int64_t gcol, int64_t T, int64_t H, int64_t Dv, float eps, const float *w, void *out, int64_t ldo,
                   bool bf16, hipStream_t s, bool w_heads = false);

// g = min(gate, limit), u = clamp(up, -limit, limit): out = g * sigmoid(alpha * g) * (u + 1); gu: rows [T][2*F] of the operand type (gate columns, then up columns)
int clamped_glu(const void *gu, int64_t T, int64_t F, float limit, float alpha, void *out, int64_t ldo, bool bf16, hipStream_t s);

// x += mult * y (x f32, y of the operand type, [n])
int axpy(float *x, const void *y, bool bf16, float mult, int64_t n, hipStream_t s);

// out[r] = x[rows[r]] / sqrt(mean^2 + eps) * g, in the operand type
int norm_rows(const float *x, const int32_t *rows, int64_t R, int64_t W, float eps, float g, void *out, bool bf16, hipStream_t s);

// y[T][N] (f32, or the operand type) = a[T][K] . w[N][K]^T for shapes the tiled GEMMs do not take (any T, K, N)
int gemm_any(const void *a, int64_t lda, const void *w, int64_t T, int64_t K, int64_t N, void *y, bool y_f32, bool bf16, hipStream_t s);

// ---------------------------------------------------------------------------------------------------------------------------------------------------
// Further blocks (layered_blocks.hip)
int prepare_blocks();                                   // LDS opt-ins (call once, outside captures)

// x[t] = E[ids[t]] (f32), and the same rows into kept (the first of the kept streams) when not null
int embed_keep(const void *E, bool bf16, const int64_t *ids, int64_t T, int64_t W, float *x, float *kept, hipStream_t s);

// RMS norm in groups: a row of W numbers is split into `groups` equal consecutive parts, each divided by its own sqrt(mean^2 + eps), the whole times w.
//   xres null: out rows (operand type, stride ldo) = norm(in rows); in: f32 (in_f32) or operand type, stride ldi; rows (may be null) selects input rows.
//   xres not null: xres[r] += norm(in[r]) (in: operand type), and with w2 also out[r] = norm(xres[r]) * w2 — the sublayer's output joins the stream and the next
//   sublayer's input leaves in the same pass; with out_plain (and no w2) out[r] = xres[r] itself, in the operand type.
struct GroupNormArgs {
    const void *in; int64_t ldi; bool in_f32; const int32_t *rows; int64_t rows_n, W; int32_t groups; float eps; const float *w;
    float *xres; const float *w2; void *out; int64_t ldo; bool out_plain;
};
int group_norm(const GroupNormArgs &a, bool bf16, hipStream_t s);

// Latent attention caches ONE row per token: `rank` numbers of the latent (proj columns col ..., divided by their root mean square, times w) and `rot` numbers of a
// key part shared by the heads, rotated in pairs (2i, 2i+1) by position * freq[i].  pages: [blocks][block_size][rank + rot] of the operand type; rows (may be null):
// the same rows in step order, [T][rank + rot].
int latent_store(const void *proj, int64_t ld, int64_t col, const Batch &b, int64_t rank, int64_t rot, float eps, const float *w, const float *freq, void *pages, void *rows,
                 bool bf16, hipStream_t s);
// y[t][c] *= sigmoid(g[t][c]) (c < N; rows of y / g with strides ldy / ldg)
int sigmoid_gate(void *y, int64_t ldy, const void *g, int64_t ldg, int64_t T, int64_t N, bool bf16, hipStream_t s);
// The rotated part of the queries: q[t][h * qstride + qcol ...] (rot numbers, pairs (2i, 2i+1)) -> out[t][h * ostride + ocol ...]
int rotate_heads(const void *q, int64_t ldq, int64_t qstride, int64_t qcol, const Batch &b, int64_t H, int64_t rot, const float *freq, void *out, int64_t ldo, int64_t ostride,
                 int64_t ocol, bool bf16, hipStream_t s);

// y[t][h * hy + n] = sum_k a[t][h * ha + k] * w[h][n][k] (n < N, k < K; rows of a / y / gate with strides lda / ldy / ldg), times sigmoid(gate[t][h * hg + n]) when gate is not null.
// One matrix per head: the key expansion folded into the queries (w[h] = Wuk_h^T), the value expansion of the attended latent (w[h] = Wuv_h).
struct HeadLinearArgs { const void *a; int64_t lda, ha; const void *w; void *y; int64_t ldy, hy; const void *gate; int64_t ldg, hg; int32_t T, H, K, N; };
int head_linear(const HeadLinearArgs &a, bool bf16, hipStream_t s);

// Rows grouped by expert: y[r] = w[e] a[r] for off[e] <= r < off[e+1] (w: [groups][N][K]).  With src, row r of a is row src[r] / src_div of the array times rscale[src[r]]
// (the router's weight on the expert's input).  max_rows: an upper bound of off[groups] known to the host (the offsets stay on the device).
struct GroupedLinearArgs { const void *a; int64_t lda; const void *w; void *y; int64_t ldy; const int32_t *off; int32_t groups, K, N, max_rows; const int32_t *src; const float *rscale; int32_t src_div; };
int grouped_linear(const GroupedLinearArgs &a, bool bf16, hipStream_t s);

// out = c0 N(z) + c1 N(z^2) + c2 N(z^3) + c3, N(v) = v / sqrt(mean(v^2) + eps) over the F numbers of a row; coef: 4 floats on the device
int poly_norm(const void *z, int64_t ldz, int64_t T, int64_t F, float eps, const float *coef, void *out, int64_t ldo, bool bf16, hipStream_t s);
// out = silu(gate) * up; gu: rows [2 F] (gate columns, then up columns)
int silu_mul(const void *gu, int64_t T, int64_t F, void *out, int64_t ldo, bool bf16, hipStream_t s);

// Router of a mixture of experts: logits wr h in f32 (wr: [E][W] f32), the top largest per token -> sel / score (= sigmoid of the logit) [T][top]; then the rows
// grouped by expert: off [E + 1], order [T top] (place -> token * top + choice), place_of (its inverse).  With pad > 1 every expert's rows start at a multiple of pad
// (places then run up to (T top / pad + E) pad) and row_w[block] names the expert of each of the nblocks blocks of pad rows: the form a tiled product over whole
// row blocks wants, with the rows brought together by moe_gather (xs[place] = h[token] * score).
// softmax: score is the chosen experts' share of the softmax over ALL experts, divided by the sum of the chosen shares (+ 1e-20), instead of the sigmoid.
// extra > 0: rows E .. E + extra - 1 of wr are further f32 projections of h that leave as they are in extra_out[t * extra + i] (a shared expert's gate).
int moe_route(const void *h, int64_t ldh, int64_t T, int64_t W, const float *wr, int64_t E, int64_t top, int32_t *sel, float *score, int32_t *off, int32_t *order,
              int32_t *place_of, int64_t pad, int32_t *row_w, int64_t nblocks, bool bf16, hipStream_t s, bool softmax = false, int64_t extra = 0, float *extra_out = nullptr,
              const float *logits = nullptr, int64_t ldl = 0);   // logits (f32 rows of E + extra numbers, stride ldl): the products wr h formed beforehand (wr is then not read)
int moe_gather(const void *h, int64_t ldh, int64_t T, int64_t W, int64_t top, const int32_t *place_of, const float *score, void *xs, bool bf16, hipStream_t s);
// out[t] = sum_k y[place_of[t * top + k]] + shared[t] (shared may be null).  With score ([T][top] f32) choice k is weighted by score[t * top + k]; with shared_gate
// ([T] f32, stride gate_ld) the shared row is multiplied by sigmoid(shared_gate[t * gate_ld]).
int moe_combine(const void *y, const int32_t *place_of, int64_t T, int64_t top, const void *shared, int64_t W, void *out, bool bf16, hipStream_t s,
                const float *score = nullptr, const float *shared_gate = nullptr, int64_t gate_ld = 1);

// The per-layer token input is y = Wp (gelu_tanh(Wg x) * E[id][ecol .. ecol + dim)), x += y / rms(y) * wn: two ordinary products with this between them
// (z = Wg x rows of dim numbers -> g), and its last step inside layer_tail.
int side_gate(const void *z, const int64_t *ids, const void *E, int64_t lde, int64_t ecol, int64_t dim, int64_t T, void *g, bool bf16, hipStream_t s);

// The end of a layer, per row and each part optional: the token input's last step (x += side_y / rms(side_y) * side_norm; side_y rows of the operand type), the weighted
// average over depth (this x becomes kept stream nx - 1; x <- sum_j mix[j] kept[j], kept: [streams][kept_rows][W] f32), and the next layer's first norm of the new x.
struct LayerTailArgs {
    float *x; int32_t T, W; float eps;
    const void *side_y; const float *side_norm;
    float *kept; int64_t kept_rows; int32_t nx; const float *mix;
    const float *wnext; int32_t groups; void *out;
};
int layer_tail(const LayerTailArgs &a, bool bf16, hipStream_t s);

// ---------------------------------------------------------------------------------------------------------------------------------------------------
// Blocks of pre-norm layers with a layer scale (layered_gates.hip): learned positions, an exponentially gated matrix memory, a windowed attention with
// normed queries / keys / values, an elementwise gated recurrence, and the residual joins.

// x[t] = E[ids[t]] * scale + P[position of row t] (f32 residual stream; P: [positions][W] of the operand type, null: none)
int embed_pos(const void *E, const void *P, bool bf16, const Batch &b, int64_t W, float scale, float *x, hipStream_t s);

// Exponential gates of a matrix memory, per token and head, from the f32 pre-activations zi = pre[t][h], zf = pre[t][H + h] (row stride ldp) and their biases:
//   i = cap tanh((zi + bi[h]) / cap), f = log_sigmoid(cap tanh((zf + bf[h]) / cap)), m_t = max(f + m_(t-1), i) with m = 0 before a sequence's first token;
//   tok_gate[(t * H + h) * 2] = (e^(f + m_(t-1) - m_t), e^(i - m_t)) — retention's token-gated form takes these — and floor[t * H + h] = e^(-m_t).
// mstate: [slots][H] f32, the running maximum after each sequence's last token so far.
int exp_gates(const float *pre, int64_t ldp, const float *bi, const float *bf, float cap, const Batch &b, int64_t H, float *mstate, float *tok_gate, float *floor_out,
              hipStream_t s);
// The matrix memory's read-out: o rows [T][H][Dv + 1] f32 (retention's output with one column of ones: the last number of a head is n . q);
//   y = o[:Dv] / (max(|n . q|, floor) + 1e-6), y / rms(y) * w[h * Dv + c] * sigmoid(gate[t][h * Dv + c]) -> out rows (operand type, stride ldo)
int memory_readout(const float *o, const float *floor_in, const void *gate, int64_t ldg, int64_t gcol, int64_t T, int64_t H, int64_t Dv, float eps, const float *w, void *out,
                   int64_t ldo, bool bf16, hipStream_t s);

// Queries, keys and values of an attention whose norms span the projections: in row t of proj (operand type, stride ld)
//   q (H D numbers at qcol) <- q / rms(q) * wq * (1 + coef ln(floor((p + 1) / every) + 1)), in place (p the row's position; every 0: no temperature);
//   k (G D numbers at kcol) / rms(k) * wk -> the K page row of the position; v (G heads of Dv at vcol), each head / rms(head) -> the V page row.
// wq / wk null: that projection is stored as it is.  v_unit false: values as they are.  Page layouts as kv_store.
struct QkvNormArgs {
    void *proj; int64_t ld, qcol, kcol, vcol; int32_t H, G, D, Dv; float eps;
    const float *wq, *wk; bool v_unit; float temp_coef; int32_t temp_every;
    void *kc, *vc; bool v_grouped;
};
int qkv_norm_store(const QkvNormArgs &a, const Batch &b, bool bf16, hipStream_t s);

// Elementwise gated recurrence over the rows of a step: z = sigmoid(proj[zcol + c] + bz[c]), u = proj[ucol + c] + bu[c], cand = u + 1/2 (u >= 0) or sigmoid(u) (u < 0),
// S <- (1 - z) S + z cand, out[t][c] = S * silu(proj[gcol + c]) (operand type, stride ldo).  state: [slots][N] f32, zero before a sequence's first token.
int gated_unit(const void *proj, int64_t ld, int64_t zcol, int64_t ucol, int64_t gcol, const float *bz, const float *bu, const Batch &b, int64_t N, float *state, void *out, int64_t ldo,
               bool bf16, hipStream_t s);

// A sublayer's result joins the stream: x[t][c] += ls[c] * r, r = y1 (y2 null) or (y1 / rms(y1) * w1 + y2 / rms(y2) * w2) / 2 (two branches, each normed over the row);
// with wn also out[t] = x[t] / rms(x[t]) * wn in the operand type (the next sublayer's input).  y rows of the operand type, strides ld1 / ld2; ls may be null (ones).
// add (rows of the operand type, stride lda; may be null) is a further addend that joins as it is: x += ls * r + add (a feed-forward that read the same input as the mixer).
struct JoinArgs { float *x; int64_t T, W; float eps; const float *ls; const void *y1; int64_t ld1; const float *w1; const void *y2; int64_t ld2; const float *w2; const float *wn; void *out; int64_t ldo;
                  const void *add; int64_t lda; };
int residual_join(const JoinArgs &a, bool bf16, hipStream_t s);

// out = max(z, 0)^2 (rows of F numbers, strides ldz / ldo)
int relu_squared(const void *z, int64_t ldz, int64_t T, int64_t F, void *out, int64_t ldo, bool bf16, hipStream_t s);
// y[i] *= c (f32, n numbers)
int scale_f32(float *y, int64_t n, float c, hipStream_t s);

// ---------------------------------------------------------------------------------------------------------------------------------------------------
// Blocks of layers whose two sublayers read ONE norm, with a token shift in front of the mixer (layered_ssm.hip): a state-space mixer (causal convolution, step
// sizes, gated group norm; its recurrence is retention's token-gated form with shared input / output maps), rotated keys on their way into the pages, an
// attention without softmax over chunks of positions (SinkAttnArgs::gate_bias, chunk, softcap in both attention forms), the mixes of a time-mixing recurrence (retention's gated form with a bonus), the input of a pass over a
// looped range of layers.

// h = x / sqrt(mean(x^2) + eps) * w -> out_h (may be null); m_t = h_t + (h_(t-1) - h_t) * shift -> out_m (operand type; h_(-1) = 0; the row before a chunk comes from
// hist[par][slot], the chunk's last h goes to hist[par ^ 1][slot]).  hist: [2][slots][W] f32.
int norm_shift(const float *x, const Batch &b, int64_t W, float eps, const float *w, const float *shift, void *out_h, void *out_m, float *hist, int64_t slots, bool bf16, hipStream_t s);

// out[t] = [x[t] | x0[t]] in the operand type (rows of 2 W numbers): the input of the product that starts a pass over a looped range of layers
int pair_rows(const float *x, const float *x0, int64_t T, int64_t W, void *out, bool bf16, hipStream_t s);

// The front of a state-space mixer.  In row t of proj (operand type, stride ld) the C channels from column ccol pass a causal convolution per channel over `taps`
// rows (w: [C][taps] f32, the last column is the current row's; bias [C]) and silu -> out (operand type, stride ldo); rows before position 0 are zero, the taps - 1 rows
// before a chunk come from hist[par][slot] ([2][slots][taps - 1][C] f32) and the chunk's last taps - 1 inputs go to the other half.  The H step sizes at column dcol:
// dt = softplus(z + dt_bias[h]); tok_gate[(t * H + h) * 2] = (exp(-exp(a_log[h]) * dt), dt): retention's token-gated form takes them.
struct ConvGateArgs { const void *proj; int64_t ld, ccol, dcol; int32_t C, taps, H; const float *w, *bias, *dt_bias, *a_log; float *hist; int64_t slots; void *out; int64_t ldo; float *tok_gate; };
int conv_gates(const ConvGateArgs &a, const Batch &b, bool bf16, hipStream_t s);

// The end of a state-space mixer: y[t][h][c] = o[t][h][c] + skip[h] * xs[t][h * Dv + c] (o f32 [T][H * Dv], xs rows of the operand type, stride ldx); y *= silu(z) (z rows,
// stride ldz); y is RMS-normed in `groups` equal consecutive parts of the H * Dv numbers, times w -> out (operand type, stride ldo).
struct StateReadoutArgs { const float *o; const void *xs; int64_t ldx; const void *z; int64_t ldz; const float *skip, *w; int32_t T, H, Dv, groups; float eps; void *out; int64_t ldo; };
int state_readout(const StateReadoutArgs &a, bool bf16, hipStream_t s);

// Rotated queries and keys ('rotate half': coordinate i < rot / 2 of a head pairs with i + rot / 2, angle = position * freq[i], f32) for an attention over pages: q rotated in
// place in proj, k rotated -> the K page row of the position, v -> the V page row (layouts as kv_store).  freq: [rot / 2] f32 on the device.
struct RopeStoreArgs { void *proj; int64_t ld, qcol, kcol, vcol; int32_t H, G, D, Dv, rot; const float *freq; void *kc, *vc; bool v_grouped; };
int rope_store(const RopeStoreArgs &a, const Batch &b, bool bf16, hipStream_t s);

// out[t][i * W ...] = m_t + (m_(t-1) - m_t) * mu[i] for i < n (mu: [n][W] f32; m rows of the operand type, stride ldm; m_(-1) = 0; history as norm_shift, hist [2][slots][W] f32
// of m): the inputs of a time-mixing layer's projections, side by side in rows of n W numbers
int shift_mixes(const void *m, int64_t ldm, const Batch &b, int64_t W, int32_t n, const float *mu, void *out, float *hist, int64_t slots, bool bf16, hipStream_t s);

// y = tanh(y) in place (rows of N numbers, stride ld)
int tanh_rows(void *y, int64_t ld, int64_t T, int64_t N, bool bf16, hipStream_t s);

}}  // namespace nvr::kl
