/* libi64hip_dense.so - C ABI of the gfx950 (MI355X) kernels for decoder models with bf16 weights and a 32-bit residual:
 * tiled Linear on the bf16 / f32 matrix cores with fused epilogues, scaled embedding, gated post-norm residual with
 * grouped RMS norm and depth mixing, latent (low-rank, shared-key) attention over a paged cache with a sliding window,
 * multi-stream and sandwich-norm residuals, causal convolutions with carried inputs, state-space / gated / gated-linear recurrences,
 * attention with a distance bias (keys as values, or separate keys and values in one cached row), rotated attention (query / key norms,
 * two pair layouts, rotated values, capped scores, gated heads), learned attention sinks, the gated delta rule, expert routing with
 * grouped Linears over device-side row groups, row sampling.  A library of its own so that a process that serves such a model builds and
 * loads nothing else.
 *
 * Conventions are those of libi64hip.so (include/i64h.h): raw device pointers, caller-allocated outputs, no allocation
 * and no synchronisation inside, 0 on success, the reason of a failure in i64h_last_error() of THIS library.
 * Descriptor structs are passed by host pointer and read before the call returns.
 */
#ifndef I64H_DENSE_H
#define I64H_DENSE_H
#include <stdint.h>
#ifdef __cplusplus
extern "C" {
#endif

const char* i64h_last_error(void);
int i64h_version(void);
int i64h_device_check(void);

/* ---- Linear ------------------------------------------------------------------------------------------------------------
 * C[b][m, n] = epilogue( sum_k A[b][row(m), k] * W[b][n, k] ),  b < batch (one launch; blockIdx.z is the batch index).
 *   A fp32, row stride lda, batch b starts a_batch * b elements further (a column block of a wider matrix);
 *   row(m) = a_rows ? a_rows[m] : m;  W bf16 [N, K] row-major, batch stride w_batch elements;  C fp32, row stride ldc,
 *   batch stride c_batch.
 * exact = 0: A is rounded to bf16 (nearest even) while it is staged, products on v_mfma_f32_16x16x32_bf16, fp32 sums.
 * exact = 1: W is widened to fp32 while it is staged, products on v_mfma_f32_16x16x4_f32: true 32-bit arithmetic.
 * epilogue: I64H_EPI_STORE; I64H_EPI_GELU_MUL: gelu_tanh(A W^T) * (A W2^T) with W2 = W + N * K (gate rows, then up rows);
 *   I64H_EPI_MUL_SIGMOID: * sigmoid(E[b][m, n]) (E fp32, row stride lde, batch stride e_batch);
 *   I64H_EPI_SOFTCAP: cap * tanh(. / cap);  I64H_EPI_GELU_ERF: 0.5 v (1 + erf(v / sqrt 2));  I64H_EPI_SCALE: v * scale;
 *   I64H_EPI_SILU_MUL: silu(A W^T) * (A W2^T), laid out as I64H_EPI_GELU_MUL;
 *   I64H_EPI_XIELU: v > 0 ? act_a v^2 + v / 2 : act_b (exp(v) - 1 - v) + v / 2  (the caller passes act_a = softplus(p), act_b = 1/2 + softplus(q)).
 *   I64H_EPI_RELU_SQ: max(v, 0)^2.
 *   bias (may be NULL; fp32 [N], batch stride bias_batch) is added to the sum before any epilogue but the two gate / up ones.
 * group_off (may be NULL; device int32 [batch + 1], ascending): batch b takes the rows [group_off[b], group_off[b + 1]) of a_rows
 *   (of A itself without a_rows) and of C instead of all M rows; M is then the most rows any batch may have (it sizes the launch,
 *   workgroups past a batch's rows leave at once), and the launch needs no count on the host.  Such launches take the 64 x 64 tile form,
 *   or with M <= 64 the fragment-streaming form.
 * Any M, N, K >= 1; 16-byte loads are used where strides and addresses allow, element loads otherwise.
 * Launches with M <= I64H_SKINNY_ROWS take a weight-streaming form (one wave per output column group). */
#define I64H_EPI_STORE 0
#define I64H_EPI_GELU_MUL 1
#define I64H_EPI_MUL_SIGMOID 2
#define I64H_EPI_SOFTCAP 3
#define I64H_EPI_GELU_ERF 4
#define I64H_EPI_SCALE 5
#define I64H_EPI_SILU_MUL 6
#define I64H_EPI_XIELU 7
#define I64H_EPI_RELU_SQ 8
#define I64H_SKINNY_ROWS 8
typedef struct {
    const float* A;
    int64_t lda;
    const int32_t* a_rows;
    const void* W;
    float* C;
    int64_t ldc;
    int64_t M;
    int32_t N, K;
    int32_t batch;
    int64_t a_batch, w_batch, c_batch;
    int32_t exact;
    int32_t epilogue;
    const float* E;
    int64_t lde, e_batch;
    float softcap;
    const float* bias;
    int64_t bias_batch;
    float scale;
    float act_a, act_b;
    const int32_t* group_off;
} i64h_linear;
int i64h_linear_run(const i64h_linear* d, void* stream);

/* out[t, :] = float(table[ids[t], :]) * scale; table bf16 [V, W]; ids outside [0, V) are clamped. */
int i64h_embed_scaled(const int64_t* ids, const void* table_bf16, float scale, float* out, int64_t n, int32_t W, int64_t V, void* stream);

/* ---- gated post-norm residual + grouped RMS norm + depth mix, one launch per sublayer --------------------------------------
 * v = alpha * x[row(m)] + g * y[m],  g = gate_pre ? sigmoid(gate_pre[m] + gate_bias) : 1,  y == NULL: v = alpha * x;
 * out[m] = v / sqrt(mean over the group of v^2 + eps) * norm_w, the W columns cut into `groups` equal consecutive parts;
 * with mix_w != NULL the row is also stored at hist[hist_index][m] and
 *   mix_out[m] = sum_{j < hist_index} mix_w[j] * hist[j][m] + mix_w[hist_index] * out[m]        (hist fp32 [*, n, W]).
 * x_rows (may be NULL) gathers input rows (the final norm of the rows whose logits are wanted).  All math fp32. */
typedef struct {
    const float* x;
    const int32_t* x_rows;
    const float* y;
    int64_t ldy;
    const float* gate_pre;
    int64_t ldg;
    const float* gate_bias;
    float alpha;
    const float* norm_w;
    int32_t groups;
    float eps;
    float* out;
    float* hist;
    int32_t hist_index;
    const float* mix_w;
    float* mix_out;
    int64_t n;
    int32_t W;
} i64h_postnorm;
int i64h_gated_postnorm(const i64h_postnorm* d, void* stream);

/* ---- latent attention ----------------------------------------------------------------------------------------------------
 * One cached row per token and layer: [kv_rank latent values | rot_dim rotated key values], shared by all heads, in a paged
 * cache (num_blocks, block_size, kv_rank + rot_dim) of fp32 (cache_dtype 0) or bf16 (2); the row of (slot, position) is
 * block_table[slot * max_blocks_per_seq + position / block_size] * block_size + position % block_size.
 *
 * i64h_latent_prep, per token t of the projection rows P (fp32, row stride ldp):
 *   latent = P[t, dkv_off : +kv_rank] / sqrt(mean^2 + eps) * c_norm_w           -> cache row, columns [0, kv_rank)
 *   key    = rotate(P[t, dkv_off + kv_rank : +rot_dim], position)               -> cache row, columns [kv_rank, +rot_dim)
 *   Q[t, h, kv_rank : +rot_dim] = rotate(P[t, q_off + h * (dim + rot_dim) + dim : +rot_dim], position)   for every head h
 * rotate: the first rot_dims values in interleaved pairs (2i, 2i+1) by the angle position * inv_freq[i] (fp32 product,
 * full-range sine / cosine), the rest unchanged.  Q fp32 [n, heads, kv_rank + rot_dim]; its first kv_rank columns per head
 * (the query carried into latent space) are written by the caller's Linear. */
typedef struct {
    const float* P;
    int64_t ldp;
    int32_t q_off, dkv_off;
    int32_t heads, dim, rot_dim, kv_rank, rot_dims;
    const float* c_norm_w;
    float eps;
    const float* inv_freq;
    const int32_t* positions;
    const int32_t* slot_ids;
    const int32_t* block_table;
    int32_t max_blocks_per_seq, block_size;
    void* cache;
    int32_t cache_dtype;
    float* Q;
    int64_t n;
} i64h_latent_prep_args;
int i64h_latent_prep(const i64h_latent_prep_args* d, void* stream);

/* i64h_latent_attn: row t (sequence slot_ids[t], position p = positions[t]) sees the cached rows j of its sequence with
 * 0 <= p - j < window (window <= 0: every j <= p);  s_j = scale * Q[t, h, :] . row_j;  ordinary softmax over the visible j;
 * out[t, h, :kv_rank] = sum_j w_j * row_j[:kv_rank].  Scores, weights and sums in fp32.  out fp32 [n, heads, kv_rank].
 * With sink the denominator also holds exp(sink_w[h]) (exp(0) without sink_w): a term without a key and without a value, not scaled.
 * mode 1: one wave per (row, head), fp32 products, any sizes and cache type (of the options below it knows the sink).  Modes 0 / 2 / 3 take the matrix-core form when the cache
 * is bf16, kv_rank % 16 == 0 and <= 256, (kv_rank + rot_dim) % 8 == 0 and <= 320 (the row form otherwise): 2 (and 0) one wave per token
 * and group of 16 heads (rows that are one per sequence), 3 one wave per 16 consecutive rows and head (portions of prompts; rows of
 * different sequences in one tile are handled run by run). */
typedef struct {
    const float* Q;
    const void* cache;
    int32_t cache_dtype;
    const int32_t* block_table;
    int32_t max_blocks_per_seq, block_size;
    const int32_t* slot_ids;
    const int32_t* positions;
    int32_t window;
    float scale;
    float* out;
    int64_t n;
    int32_t heads, kv_rank, rot_dim;
    int32_t mode;
    int32_t splits;      /* mode 2: every token's keys are dealt to this many waves (tiles of 32 keys in turn) and merged by a second launch */
    float* workspace;    /* i64h_latent_attn_workspace_floats(n, heads, kv_rank, splits) floats when splits > 1 (NULL: no split) */
    /* the same matrix-core kernel under key-valued attention (i64h_kattn below); all zero / NULL: latent attention as described */
    int32_t row_stride;  /* values per cached row (0: kv_rank + rot_dim) */
    int32_t kv_groups;   /* key heads side by side in a cached row, kv_rank + rot_dim values each; head h reads number h / (heads / kv_groups) */
    int32_t chunk;       /* > 0: position p sees j <= p with j / chunk == p / chunk (the window is not used then) */
    const float* kscale; /* per cached row: multiplies Q . row */
    const float* bias;   /* fp32 [bias_rows, heads]: bias[min(p - j, bias_rows - 1), h] is added to the score */
    int32_t bias_rows;
    int32_t sink;        /* one more score of zero, without a value, in the softmax's denominator */
    int32_t key_off;     /* the first key_off columns of a cached row part carry values only: the caller's query is zero there, and the score
                            products over 32-column steps that lie wholly inside them are left out */
    const float* sink_w; /* with sink: fp32 [heads], the extra score of head h is sink_w[h] instead of zero (NULL: zero) */
    float softcap;       /* > 0: a score s (after scale and key scale, before any bias) becomes softcap * tanh(s / softcap) */
} i64h_latent_attn_args;
int i64h_set_latent_attn_decode_form(int32_t on); /* tuning / test knob: 1 (default) = mode 2 launches run the kernel that requests a tile's fragments a tile ahead; 0 = the general matrix-core kernel; same results up to summation order */
int64_t i64h_latent_attn_workspace_floats(int64_t n, int32_t heads, int32_t kv_rank, int32_t splits);
int i64h_latent_attn(const i64h_latent_attn_args* d, void* stream);

/* ==== recurrent and hybrid layers ==========================================================================================
 * Rows of a step are in sequence order: the rows of one sequence are consecutive and carry consecutive positions.  Row t
 * continues row t - 1 iff slot_ids[t - 1] == slot_ids[t] and positions[t - 1] + 1 == positions[t].  A sequence's state lives in
 * its slot; a row at position 0 starts from the empty state whatever the slot held before (a slot that is used again needs no
 * clearing).  seg_start [nseg + 1] lists the first row of every run of consecutive rows of one sequence (seg_start[nseg] = n). */

/* ---- token embedding + hashed bigram embedding ----------------------------------------------------------------------------------
 * out[c][t, :] = table[ids[t]] * scale + bigram[row(t)] for c < copies (out fp32 [copies, n, W]);  row(t) = buckets at position 0, else
 * (previous * mul_prev + ids[t] * mul_cur) mod buckets, previous = the token of the row before in the same sequence, or
 * prev_token[slot] (the last token of the sequence's earlier steps).  A second launch stores every sequence's last token of
 * this step in prev_token.  bigram == NULL: the token embedding alone.  pos_table (may be NULL; bf16 [pos_rows, W]): the row of the
 * token's position is added (positions past the table take its last row; callers bound positions by pos_rows).  Tables bf16. */
typedef struct {
    const int64_t* ids;
    const int32_t* positions;
    const int32_t* slot_ids;
    const void* table;
    int64_t V;
    int32_t W;
    const void* bigram;
    int64_t buckets, mul_prev, mul_cur;
    int64_t* prev_token;
    float* out;
    int32_t copies;
    int64_t n;
    const void* pos_table;
    int64_t pos_rows;
    float scale;         /* multiplies the token row only (not the bigram or position rows) */
} i64h_embed_bigram_args;
int i64h_embed_bigram(const i64h_embed_bigram_args* d, void* stream);

/* ---- multi-stream residual (hyper-connections) with the next sublayer's RMS norm -------------------------------------------------
 * streams fp32 [S, n, W], updated in place, one workgroup per row:
 *   write (y != NULL):  v = y2 ? 0.5 * (rms(y) * yn_w + rms(y2) * y2n_w) : (yn_w ? rms(y) * yn_w : y)
 *                       (rms over the W columns with y_eps; weights [W]; a single normed result is the post-norm of a sandwich layer)
 *                       post_w != NULL: v <- norm(v) * post_w, over the W columns with y_eps - the root mean square, or with post_center the
 *                       centred norm (v - mean) / sqrt(mean((v - mean)^2) + y_eps): a norm on a sublayer's result, whatever it is made of
 *                       new_t = sum_s mix[s * S + t] * old_s + out_w[t] * v          (mix == NULL: new_t = old_t + out_w[t] * v)
 *   read  (h != NULL):  u = sum_s in_w[s] * x_s  (in_w == NULL: the plain sum);  h = u / sqrt(mean(u^2) + eps) * norm_w[c % norm_w_len],
 *                       or with h_center the centred norm (u - mean) / sqrt(mean((u - mean)^2) + eps) * norm_w
 * rows (may be NULL, read only launches): h[m] is computed from row rows[m] of the streams (the rows whose logits are wanted). */
typedef struct {
    float* streams;
    int32_t S;
    int64_t n;
    int32_t W;
    const float* y;
    int64_t ldy;
    const float* y2;
    int64_t ldy2;
    const float* yn_w;
    const float* y2n_w;
    float y_eps;
    const float* mix;
    const float* out_w;
    const float* in_w;
    const float* norm_w;
    int32_t norm_w_len;
    float eps;
    float* h;
    const int32_t* rows;
    int64_t m_rows;
    const float* post_w;
    int32_t post_center;
    int32_t h_center;
} i64h_streams_args;
int i64h_streams_step(const i64h_streams_args* d, void* stream);

/* ---- causal per-channel convolution with carried inputs + silu ---------------------------------------------------------------------
 * out[t, c] = silu(bias[c] + sum_k w[c, k] * in(t, taps - 1 - k)),  in(t, d) = the input of channel c d positions before row t:
 * zero before position 0, a row of this step where the sequence has one there, else the carried inputs state fp32
 * [slots, taps - 1, channels] (the last taps - 1 inputs of the sequence's earlier steps, oldest first).  Inputs are the columns
 * [off, off + channels) of P.  A second launch stores the new carried inputs.  w fp32 [channels, taps].
 * mode 1: out[t, c] = in(t, 0) + bias[c] + sum_k ... without the activation (a convolution added to its own input). */
typedef struct {
    const float* P;
    int64_t ldp;
    int32_t off, channels, taps;
    const float* w;
    const float* bias;
    const int32_t* positions;
    const int32_t* slot_ids;
    float* state;
    float* out;
    int64_t ldo;
    int64_t n;
    int32_t mode;
    int32_t single_rows; /* 1: every row is the only row of its sequence in this launch: the launch that computes a row also stores its
                            sequence's new carried inputs (no second launch) */
} i64h_causal_conv_args;
int i64h_causal_conv(const i64h_causal_conv_args* d, void* stream);

/* ---- selective state-space recurrence (scalar decay per head) ---------------------------------------------------------------------
 * Per sequence and head a (state x vdim) matrix S in fp32:  dt = softplus(dt_raw + dt_bias[a]),
 *   S <- exp(-exp(A_log[a]) * dt) * S + dt * B_t x_t^T,   y_t = S^T C_t + Dskip[a] * x_t,
 * x_t = xbc[t, a * vdim : +vdim], B_t = xbc[t, heads * vdim + g * state : +state], C_t = xbc[t, heads * vdim + (groups + g) * state : +state],
 * g = a / (heads / groups), dt_raw = dt[t, a].  ssm_state fp32 [slots, heads, vdim, state] (S transposed; state <= 256).  All arithmetic fp32,
 * the tokens of a sequence strictly in their order. */
typedef struct {
    const float* xbc;
    int64_t ldx;
    const float* dt;
    int64_t lddt;
    const float* dt_bias;
    const float* A_log;
    const float* Dskip;
    int32_t heads, vdim, state, groups;
    const int32_t* seg_start;
    int32_t nseg;
    const int32_t* positions;
    const int32_t* slot_ids;
    float* ssm_state;
    float* y;
    int64_t ldy;
    int64_t n;
} i64h_ssm_scan_args;
int i64h_ssm_scan(const i64h_ssm_scan_args* d, void* stream);

/* out[t, :] = rms_groups(y[t, :] * silu(z[t, :])) * w: the `width` columns in `groups` equal consecutive parts, each divided by
 * sqrt(mean(part^2) + eps).  z == NULL: no gate.  gate_after: out = rms_groups(y) * w * silu(z), the gate behind the norm.
 * w_len (0: width) values of w, repeated over the columns (a head norm whose weights all heads share). */
typedef struct {
    const float* y;
    int64_t ldy;
    const float* z;
    int64_t ldz;
    const float* w;
    int32_t width, groups;
    float eps;
    float* out;
    int64_t ldo;
    int64_t n;
    int32_t gate_after;
    int32_t w_len;
} i64h_gate_norm_args;
int i64h_gate_norm(const i64h_gate_norm_args* d, void* stream);

/* ---- minimal gated recurrence ------------------------------------------------------------------------------------------------------
 * Per sequence and channel c < width, fp32:  z = sigmoid(P[t, z_off + c]),  u = P[t, x_off + c],
 *   cand = u >= 0 ? u + 0.5 : sigmoid(u),   S <- (1 - z) * S + z * cand,   out[t, c] = S * silu(P[t, g_off + c]).
 * state fp32 [slots, width]. */
typedef struct {
    const float* P;
    int64_t ldp;
    int32_t z_off, x_off, g_off, width;
    const int32_t* seg_start;
    int32_t nseg;
    const int32_t* positions;
    const int32_t* slot_ids;
    float* state;
    float* out;
    int64_t ldo;
    int64_t n;
} i64h_mingru_scan_args;
int i64h_mingru_scan(const i64h_mingru_scan_args* d, void* stream);

/* ---- attention whose values are the keys ---------------------------------------------------------------------------------------------
 * One cached row per token and layer: the kv_heads * dim key values as projected (fp32, cache_dtype 0, or bf16, 2), plus one fp32
 * number per token, kscale = 1 / sqrt(mean(row^2) + eps); paged as the latent cache above.
 * i64h_kattn_prep, per row t of the projections P:  q = P[t, q_off : + heads * dim], k = P[t, k_off : + kv_heads * dim];
 *   Q[t, h, d] = q[h, d] / sqrt(mean(q^2) + eps) * q_norm_w[h * dim + d] * k_norm_w[g * dim + d] * scale * temp[h]
 *   (means over the whole row; g = h / (heads / kv_heads); temp may be NULL), cache row <- k, kscale <- 1 / sqrt(mean(k^2) + eps).
 * With these a score against the normed key is Q[t, h] . k_j * kscale_j. */
typedef struct {
    const float* P;
    int64_t ldp;
    int32_t q_off, k_off;
    int32_t heads, kv_heads, dim;
    const float* q_norm_w;
    const float* k_norm_w;
    const float* temp;
    float scale, eps;
    const int32_t* positions;
    const int32_t* slot_ids;
    const int32_t* block_table;
    int32_t max_blocks_per_seq, block_size;
    void* cache;
    int32_t cache_dtype;
    float* kscale;
    float* Q;
    int64_t n;
} i64h_kattn_prep_args;
int i64h_kattn_prep(const i64h_kattn_prep_args* d, void* stream);

/* i64h_kattn: row t (position p) sees the cached positions j <= p of its sequence with j / chunk == p / chunk (chunk <= 0: all);
 *   s_j = Q[t, h] . k_j * kscale_j + bias[min(p - j, bias_rows - 1) * heads + h]      (bias fp32 [bias_rows, heads], may be NULL)
 *   w_j = exp(s_j) / (sink + sum_i exp(s_i))    (sink = 1: one more score of zero that carries no value; 0: the ordinary softmax)
 *   out[t, h, :] = sum_j w_j * k_j[g, :].   Scores, weights and sums fp32.  out fp32 [n, heads, dim].
 * The matrix-core form carries query and weights as two bf16 terms each (16 mantissa bits; products with the bf16 keys are exact). */
typedef struct {
    const float* Q;
    const void* cache;
    int32_t cache_dtype;
    const float* kscale;
    const int32_t* block_table;
    int32_t max_blocks_per_seq, block_size;
    const int32_t* slot_ids;
    const int32_t* positions;
    int32_t chunk;
    const float* bias;
    int32_t bias_rows;
    int32_t sink;
    float* out;
    int64_t n;
    int32_t heads, kv_heads, dim;
    int32_t mode;        /* 1: one wave per (row, head), fp32 products, any sizes and cache type; otherwise, where the cache is bf16 and dim % 16 == 0
                            and <= 256, the matrix-core kernel of the latent attention: 3 a wave per 16 consecutive rows and head (portions of
                            prompts), 0 / 2 a wave per token and 16 query heads of one key head (rows that are one per sequence) */
    int32_t splits;      /* mode 0 / 2: every token's keys are dealt to this many waves and merged by a second launch */
    float* workspace;    /* i64h_kattn_workspace_floats(n, heads, kv_heads, dim, splits) floats when splits > 1 */
    int32_t vdim;        /* > 0: keys and values are separate (see i64h_kv_prep): a cached row holds per key head [vdim values | dim key values], Q is
                            [n, heads, vdim + dim] with the query in the last dim columns of a head, out [n, heads, vdim], kscale may be NULL;
                            the workspace is then i64h_kattn_workspace_floats(n, heads, kv_heads, vdim, splits) floats */
    float softcap;       /* > 0: the score Q . k * kscale becomes softcap * tanh(. / softcap) before the bias is added */
} i64h_kattn_args;
int64_t i64h_kattn_workspace_floats(int64_t n, int32_t heads, int32_t kv_heads, int32_t dim, int32_t splits);
int i64h_kattn(const i64h_kattn_args* d, void* stream);

/* ---- attention with separate keys and values over one cached row per token --------------------------------------------------------------
 * i64h_kv_prep, per row t of the projections P:  q = P[t, q_off : + heads * dim], k = P[t, k_off : + kv_heads * dim], v = P[t, v_off : + kv_heads * vdim];
 *   cache row (slot, position) <- per key head g: [v_g (vdim) | k_g (dim)]   (cache == NULL: nothing is written - a layer that attends over
 *   the rows another layer cached);   Q[t, h, :] = [0 (vdim) | q_h * scale (dim)].
 * With these i64h_kattn (vdim > 0) computes softmax_j(Q . k_j + bias) v_j: the zeros make the value columns drop out of the score. */
typedef struct {
    const float* P;
    int64_t ldp;
    int32_t q_off, k_off, v_off;
    int32_t heads, kv_heads, dim, vdim;
    float scale;
    const int32_t* positions;
    const int32_t* slot_ids;
    const int32_t* block_table;
    int32_t max_blocks_per_seq, block_size;
    void* cache;
    int32_t cache_dtype;
    float* Q;
    int64_t n;
} i64h_kv_prep_args;
int i64h_kv_prep(const i64h_kv_prep_args* d, void* stream);

/* ---- gated linear recurrence (linear attention with a decay per key channel) ----------------------------------------------------------------
 * Per sequence and head a (dim x vdim) matrix S in fp32:   S <- diag(f_t) S + k_t v_t^T,   o_t = S^T q_t,
 * q_t = P[t, q_off + a * dim : + dim], f_t likewise at f_off, v_t = P[t, v_off + a * vdim : + vdim];  k_t = P[...k_off...] or, with k_off < 0,
 * k_t = 1 - f_t (the forget gate also decides what is written).  state fp32 [slots, heads, vdim, dim] (S transposed; dim <= 256).
 * i64h_gla_gates prepares q and f in place:  q <- q_act ? silu(q) : q;   f <- lower + (1 - lower) * sigmoid(f)   (lower fp32 [heads * dim] or NULL = 0).
 * All arithmetic fp32, the tokens of a sequence strictly in their order. */
typedef struct {
    float* P;
    int64_t ldp;
    int32_t q_off, f_off, k_off, v_off;
    int32_t heads, dim, vdim;
    const float* lower;
    int32_t q_act;
    const int32_t* seg_start;
    int32_t nseg;
    const int32_t* positions;
    const int32_t* slot_ids;
    float* state;
    float* out;          /* fp32 [n, heads * vdim], row stride ldo */
    int64_t ldo;
    int64_t n;
} i64h_gla_args;
int i64h_gla_gates(const i64h_gla_args* d, void* stream);
int i64h_gla_scan(const i64h_gla_args* d, void* stream);

/* ---- attention with rotated queries, keys and (optionally) values over [values | keys] rows ---------------------------------------------
 * i64h_rot_prep, per row t of the projections P (position pos):  q = P[t, q_off : + heads * dim], k = P[t, k_off : + kv_heads * dim],
 * v = P[t, v_off : + kv_heads * vdim];
 *   1. q_norm_w / k_norm_w (may be NULL, together): q <- q / sqrt(mean(q^2) + eps) * q_norm_w over the WHOLE row of heads * dim values, k likewise;
 *   2. the first rot_dims values of every head turn by pos * inv_freq[i] (fp32 product, full-range sine / cosine, both multiplied by rot_mult):
 *      pairs (i, i + rot_dims / 2) or, with interleaved, (2i, 2i + 1); (u, v) -> (u cos - v sin, v cos + u sin); the rest pass unchanged;
 *   3. head_norm: q and k are divided by sqrt(mean over the head's dim values of the square + eps), no weight;
 *   4. v_freq (may be NULL; fp32 [vdim / 2]): all vdim values of every value head turn by pos * v_freq[m], pairs in the same layout;
 *   cache row (slot, position) <- per key head g: [v_g (vdim) | k_g (dim)];   Q[t, h, :] = [0 (vdim) | q_h * scale (dim)].
 * i64h_kattn (vdim > 0) on these computes the attention; i64h_rot_post finishes its output in place:
 *   O[t, h, :] turns by -pos * v_freq[m] (v_freq may be NULL: no turn) and is multiplied by sigmoid(gate[t, h]) (gate may be NULL; row stride ldg). */
typedef struct {
    const float* P;
    int64_t ldp;
    int32_t q_off, k_off, v_off;
    int32_t heads, kv_heads, dim, vdim;
    const float* q_norm_w;
    const float* k_norm_w;
    float eps;
    int32_t rot_dims, interleaved;
    const float* inv_freq;
    float rot_mult;
    int32_t head_norm;
    const float* v_freq;
    float scale;
    const int32_t* positions;
    const int32_t* slot_ids;
    const int32_t* block_table;
    int32_t max_blocks_per_seq, block_size;
    void* cache;
    int32_t cache_dtype;
    float* Q;
    int64_t n;
} i64h_rot_prep_args;
int i64h_rot_prep(const i64h_rot_prep_args* d, void* stream);
typedef struct {
    float* O;            /* fp32 [n, heads, vdim], in place */
    int32_t heads, vdim, interleaved;
    const float* v_freq;
    const int32_t* positions;
    const float* gate;
    int64_t ldg;
    int64_t n;
} i64h_rot_post_args;
int i64h_rot_post(const i64h_rot_post_args* d, void* stream);

/* ---- gated delta rule -------------------------------------------------------------------------------------------------------------------
 * Per sequence and head a (dim x vdim) matrix S in fp32, head a reading the query / key head a / (heads / kv_heads):
 *   S <- g_t S;   u = beta_t (v_t - S^T k_t);   S <- S + k_t u^T;   o_t = S^T q_t       (the read-out sees the token's own write)
 * q_t = X[t, q_off + j * dim : + dim], k_t likewise at k_off, v_t = X[t, v_off + a * vdim : + vdim]; beta_t = G[t, a], g_t = G[t, heads + a].
 * i64h_gdn_gates prepares them: q and k of every query / key head divided by sqrt(sum of squares + unit_eps) in place (unit_eps < 0: left as
 * they are), q times q_scale;  G[t, a] = sigmoid(R[t, b_off + a]),  G[t, heads + a] = exp(-exp(A_log[a]) * softplus(R[t, a_off + a] + dt_bias[a])).
 * state fp32 [slots, heads, vdim, dim] (S transposed; dim <= 256).  All arithmetic fp32, the tokens of a sequence strictly in their order. */
typedef struct {
    float* X;
    int64_t ldx;
    int32_t q_off, k_off, v_off;
    int32_t heads, kv_heads, dim, vdim;
    float* G;            /* fp32 [n, 2 * heads] */
    const float* R;      /* raw projections of beta and of the decay's step (gates only) */
    int64_t ldr;
    int32_t b_off, a_off;
    const float* A_log;
    const float* dt_bias;
    float unit_eps, q_scale;
    const int32_t* seg_start;
    int32_t nseg;
    const int32_t* positions;
    const int32_t* slot_ids;
    float* state;
    float* out;          /* fp32 [n, heads * vdim], row stride ldo */
    int64_t ldo;
    int64_t n;
} i64h_gdn_args;
int i64h_gdn_gates(const i64h_gdn_args* d, void* stream);
int i64h_gdn_scan(const i64h_gdn_args* d, void* stream);

/* ---- router: softmax scores, corrected choice, groups of neighbours, top-k ---------------------------------------------------------------------
 * Per row t of logits (fp32, row stride ld, E entries):  s = softmax(logits[t]);  choice = s + correction (correction may be NULL);
 * with groups > 1 the E entries form `groups` equal groups of neighbours, a group's score is its largest choice and only the entries of
 * the `keep` best groups can be chosen;  idx[t, :] = the `top` entries with the largest choice (ties: the lower index), in that order;
 * wgt[t, k] = s[idx[t, k]] / (sum_k s[idx[t, k]] + 1e-20) * scale.   E <= 1024, top <= 32. */
typedef struct {
    const float* logits;
    int64_t ld;
    int32_t E;
    const float* correction;
    int32_t groups, keep, top;
    float scale;
    int32_t* idx;
    float* wgt;
    int64_t n;
    const float* h;
    int64_t ldh;
    const void* W;
    int32_t K;
} i64h_route_args;
int i64h_route_topk(const i64h_route_args* d, void* stream);

/* ---- mixture of experts: rows per expert, and the weighted sum ----------------------------------------------------------------------------------
 * i64h_moe_plan: from idx int32 [n, top] (entries >= experts are not experts and get no row) the (token, choice) pairs grouped by expert:
 *   group_off int32 [experts + 1] (ascending offsets), pair_token int32 [n * top] (the token of every grouped row, the a_rows of a grouped
 *   Linear), pair_row int32 [n, top] (where the pair's row lies, -1 for a non-expert).  The order of rows inside a group is not fixed;
 *   no result depends on it.  One launch of one workgroup; experts <= 4096.
 * i64h_moe_combine: out[t, :] = sum_k wgt[t, k] * (pair_row[t, k] >= 0 ? Y[pair_row[t, k], :] : h[t, :]) + (shared ? shared[t, :] : 0),
 *   summed in the order k = 0 .. top - 1, the shared row last.  Y fp32 [pairs, W]. */
typedef struct {
    const int32_t* idx;
    int64_t n;
    int32_t top, experts;
    int32_t* group_off;
    int32_t* pair_token;
    int32_t* pair_row;
} i64h_moe_plan_args;
int i64h_moe_plan(const i64h_moe_plan_args* d, void* stream);
typedef struct {
    const float* Y;
    const int32_t* pair_row;
    const float* wgt;
    const float* h;
    const float* shared;
    float* out;
    int64_t n;
    int32_t top, W;
} i64h_moe_combine_args;
int i64h_moe_combine(const i64h_moe_combine_args* d, void* stream);

/* ---- sampling --------------------------------------------------------------------------------------------------------------
 * out[r] = a token drawn from row r of logits fp32 [rows, V]: temperature[r] <= 0 -> the first index of the maximum (greedy);
 * otherwise from softmax(logits / temperature) restricted to the top_k[r] largest (top_k <= 0: all) and then to the smallest
 * set of largest probabilities whose sum reaches top_p[r] (top_p >= 1: all), using the uniform number u[r] in [0, 1). */
int i64h_sample_rows(const float* logits, int64_t* out, int64_t rows, int32_t V, const float* temperature, const int32_t* top_k,
                     const float* top_p, const float* u, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* I64H_DENSE_H */
