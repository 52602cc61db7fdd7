/*
 * zhilight_amd_seq.h -- C ABI of the ragged-batch sequence-mixer kernels (libzhilight_amd_seq.so, zhilight_amd/csrc_seq/).
 *
 * One engine step runs a FLAT list of tokens: portions of prompts and single decoded tokens of several sequences side by side
 * (zls_batch_t).  Every kernel here takes that list, so prefill, chunked prefill, decode and mixed steps are the same launches.
 * Conventions as in zhilight_amd.h: raw device pointers, a hipStream_t as void*, nothing allocates or synchronises, the return value is
 * ZL_OK, a negative ZL_E* code or a positive hipError_t.
 *
 * Number formats.  dtype is ZL_BF16 or ZL_F32 and names the format of weights matrices, of what a kernel hands to a matrix product
 * and of the paged cache.  The residual stream, every projection OUTPUT, norms, softmax, recurrences and all per-sequence state are
 * fp32 in both modes; small parameter vectors (gains, biases, decay rates, sinks) are fp32 arrays (converted once at load).
 */
#ifndef ZHILIGHT_AMD_SEQ_H
#define ZHILIGHT_AMD_SEQ_H

#include "zhilight_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

/* The tokens of one step.  Sequence i owns the flat tokens seq_start[i] .. seq_start[i + 1] - 1; they stand at positions
 * seq_pos0[i], seq_pos0[i] + 1, ...; its recurrent state lives in slot seq_slot[i] of every state array; token position p of it is cached
 * in row p % page_size of page page_table[i * max_pages + p / page_size]. */
typedef struct {
    int32_t n_seq, n_tok;
    int32_t max_pages, page_size;
    int32_t max_count;              /* the longest portion of this step (host side, sizes grids) */
    int32_t reserved;
    const int32_t* seq_start;       /* (n_seq + 1) */
    const int32_t* seq_pos0;        /* (n_seq)     */
    const int32_t* seq_slot;        /* (n_seq)     */
    const int32_t* tok_seq;         /* (n_tok) sequence index of each flat token */
    const int32_t* page_table;      /* (n_seq, max_pages) */
} zls_batch_t;

int zls_version(void);

/* y (m, n) = x (m, k) . w (n, k)^T, fp32 accumulation.  x, w in `dtype`; y fp32 (out_dtype ZL_F32) or `dtype`.  Any m, n, k > 0: rows of
 * up to 8 take a weight-streaming wave-per-column kernel, more an LDS-tiled matrix-core kernel (bf16: v_mfma_f32_16x16x32_bf16; fp32:
 * v_mfma_f32_16x16x4_f32, true fp32 products).  16-byte loads when k, ldx are multiples of 8 (bf16) / 4 (fp32) and the pointers are
 * aligned, element loads otherwise. */
int zls_gemm_nt(const void* x, int64_t ldx, const void* w, void* y, int64_t ldy, int64_t m, int64_t n, int64_t k, int dtype, int out_dtype,
                zl_stream_t s);
/* The same with gathered rows: row r of x is x[x_rows[r]], row c of w is w[w_rows[c]] (device int32 arrays, NULL: in order; ldw: row
 * stride of w).  Always the tiled kernel.  The up-projection of cached rows that lie scattered over pages. */
int zls_gemm_nt_gather(const void* x, int64_t ldx, const int32_t* x_rows, const void* w, int64_t ldw, const int32_t* w_rows, void* y,
                       int64_t ldy, int64_t m, int64_t n, int64_t k, int dtype, int out_dtype, zl_stream_t s);

/* x[t] = table[token[t]] * scale + pos_table[position(t)]  (pos_table NULL: no learned positions).  x fp32 (n_tok, width). */
int zls_embed(const int32_t* tokens, const void* table, const void* pos_table, int64_t vocab, int64_t max_positions, float scale,
              const zls_batch_t* b, float* x, int64_t width, int dtype, zl_stream_t s);

/* Token shift: h[t] = x[t] + (x[t - 1] - x[t]) * mix, where x[t - 1] of a portion's first token is prev[slot] (zeros for a new
 * sequence: the caller clears a slot when it is taken); afterwards prev[slot] = x of the portion's last token.  mix fp32 (width),
 * prev fp32 (slots, width), h (n_tok, width) in `dtype`. */
int zls_token_shift(const float* x, const float* mix, float* prev, const zls_batch_t* b, void* h, int64_t width, int dtype, zl_stream_t s);

/* x[t] += y[t] / sqrt(mean(y[t]^2) + eps) * gain   (ONE gain for all coordinates); x, y fp32 (rows, width).  xt (nullable): the new x
 * once more in `dtype`, what the next matrix product reads. */
int zls_add_scalar_norm(float* x, const float* y, float gain, float eps, int64_t rows, int64_t width, void* xt, int dtype, zl_stream_t s);

/* out[i] = x[rows[i]] / sqrt(mean(x[rows[i]]^2) + eps) * gain, out (n_rows, width) in `dtype` (the rows a projection to the vocabulary
 * is asked for). */
int zls_scalar_norm_rows(const float* x, const int32_t* rows, float gain, float eps, int64_t n_rows, int64_t width, void* out, int dtype,
                         zl_stream_t s);

/* PolyNorm: out = a N(z) + b N(z^2) + c N(z^3) + e, powers element-wise, N(u) = u / sqrt(mean(u^2) + eps) over the row.
 * z fp32 (rows, ff); coef = {a, b, c, e}; out in `dtype`. */
int zls_polynorm(const float* z, const float* coef /* host, 4 */, float eps, int64_t rows, int64_t ff, void* out, int dtype, zl_stream_t s);

/* ---- latent attention --------------------------------------------------------------------------------------------------------- */
/* c = u / sqrt(mean(u^2) + eps) * weight for the `rank` columns u = proj[t][col0 ..] of every token, written to the token's cache row.
 * proj fp32 (n_tok, ld); weight fp32 (rank); cache (pages, page_size, rank) in `dtype`. */
int zls_latent_store(const float* proj, int64_t ld, int64_t col0, const float* weight, float eps, int64_t rank, const zls_batch_t* b,
                     void* cache, int dtype, zl_stream_t s);
/* The same with a rotated key part: the down-projection holds rank + rot numbers from col0; the first rank are normed as above, the last
 * rot (one key part shared by all heads) are turned by the token's position -- pair (2i, 2i + 1) when interleaved, else (i, i + rot / 2),
 * by the angle p * freq[i] (freq fp32 (rot / 2)) -- and stored behind the latent: cache rows hold rank + rot numbers.  The last rot of the
 * qdim coordinates of each of the `heads` query heads (proj[t] from q_col0) are turned the same way in place.  cos and sin are multiplied
 * by rot_gain (1: a plain rotation; frequencies rescaled for longer contexts come with a gain). */
int zls_latent_rope_store(float* proj, int64_t ld, int64_t col0, const float* weight, float eps, int64_t rank, int64_t rot, const float* freq,
                          int interleaved, int64_t q_col0, int64_t heads, int64_t qdim, float rot_gain, const zls_batch_t* b, void* cache,
                          int dtype, zl_stream_t s);

/* Causal attention of every token over its sequence's cached latents c_0 .. c_p, heads sharing the latent:
 *   score_j = scale * (W_uk,h^T q_h) . c_j;  w_j = exp(score_j) / (sum_i exp(score_i) + exp(sink_h));  o_h = W_uv,h (sum_j w_j c_j)
 *   out[t][h] = o_h * sigmoid(gate[t][h])         (sink NULL: no sink term; gate NULL: no gate)
 * q fp32 (n_tok, ldq) from column q_col0, heads x dim; gate fp32 (n_tok, ldg) from column g_col0, one number per head;
 * w_uk (heads * dim, rank), w_uv (heads * vdim, rank) in `dtype`; out (n_tok, heads * vdim) in `dtype`.  fp32 scores, weights and sums. */
/* window > 0: a token at position p attends to the keys p - window < j <= p only (0: every j <= p). */
int zls_latent_attention(const float* q, int64_t ldq, int64_t q_col0, const float* gate, int64_t ldg, int64_t g_col0, const void* w_uk,
                         const void* w_uv, const float* sink, const void* cache, const zls_batch_t* b, float scale, int64_t heads,
                         int64_t dim, int64_t vdim, int64_t rank, void* out, int dtype, int single_only, void* workspace, int64_t n_splits,
                         int no_mfma, int64_t window, zl_stream_t s);
int64_t zls_latent_attention_workspace_bytes(int64_t n_tok, int64_t heads, int64_t rank, int64_t n_splits);
/* The keys of every token are split over n_splits workgroups (the caller picks it so that the launch fills the chip; any value >= 1 is
 * valid) whose partial results go through `workspace`; rank <= 1024.  In bf16 with rank % 8 == 0 and rank <= 512 the split pass runs
 * on the matrix cores unless no_mfma != 0 (then, and otherwise, an fp32 VALU kernel).  single_only != 0: only sequences that bring ONE token are served (their rows of out written); portions are left to
 * zls_latent_attention_prompt.
 *
 * The same attention for PORTIONS (more than one token) on the matrix cores, bf16 only, over keys and values that the caller has
 * up-projected for the step: k (n_ctx, ldk >= heads * dim) and vt = V^T (heads * vdim, ldv) in bf16, where sequence i's context rows
 * 0 .. pos0 + count - 1 stand at rows / columns ctx_start[i] ..; ctx_start[i] is a multiple of 64 (the rows up to the next multiple of 64
 * exist and hold finite numbers), or -1 for a sequence this call leaves out.  dim, vdim <= 256; ldv % 8 == 0. */
/* window as above; ctx_pos0 (int32 (n_seq), nullable: zeros): the position of the first row of a sequence's block in k / vt -- a
 * windowed step need not up-project the context before its oldest visible key. */
int zls_latent_attention_prompt(const float* q, int64_t ldq, int64_t q_col0, const float* gate, int64_t ldg, int64_t g_col0, const void* k,
                                int64_t ldk, const void* vt, int64_t ldv, const float* sink, const int32_t* ctx_start, const zls_batch_t* b,
                                float scale, int64_t heads, int64_t dim, int64_t vdim, void* out, int dtype,
                                int64_t window, const int32_t* ctx_pos0, zl_stream_t s);

/* ---- state-space (Mamba-2) mixer ---------------------------------------------------------------------------------------------- */
/* Causal per-channel convolution + SiLU over the columns col0 .. col0 + channels - 1 of proj: out[t][c] = silu(bias[c] + sum_k
 * w[c][k] * u[t - (taps - 1 - k)][c]); inputs before a portion's first token come from tail[slot] (taps - 1 rows, oldest first; zeros
 * for a new sequence).  zls_conv_tail_update then moves the portion's last taps - 1 inputs into tail[slot]; it must run after
 * zls_conv_silu on the same stream.  proj, out, tail fp32; w fp32 (channels, taps), bias fp32 (channels). */
int zls_conv_silu(const float* proj, int64_t ld, int64_t col0, const float* w, const float* bias, const float* tail, int64_t channels,
                  int64_t taps, const zls_batch_t* b, float* out, zl_stream_t s);
int zls_conv_tail_update(const float* proj, int64_t ld, int64_t col0, float* tail, int64_t channels, int64_t taps, const zls_batch_t* b,
                         zl_stream_t s);
/* The same convolution with its parts chosen: in_bias (nullable, fp32 (channels)) is added to every input u[t][c] before the taps (inputs
 * before a sequence's start stay 0; the tail holds inputs with the bias), bias (nullable) after them, act != 0 applies SiLU.
 * zls_short_conv_tail is its tail update (same in_bias). */
int zls_short_conv(const float* proj, int64_t ld, int64_t col0, const float* w, const float* bias, const float* in_bias, int act,
                   const float* tail, int64_t channels, int64_t taps, const zls_batch_t* b, float* out, zl_stream_t s);
int zls_short_conv_tail(const float* proj, int64_t ld, int64_t col0, const float* in_bias, float* tail, int64_t channels, int64_t taps,
                        const zls_batch_t* b, zl_stream_t s);

/* The recurrence, one workgroup per (sequence, head), tokens in order:
 *   dt = softplus(dt_raw + dt_bias_h);  S <- exp(-exp(a_log_h) dt) S + dt B x^T;  y = S^T C + d_h x
 * xbc fp32 (n_tok, heads * vdim + 2 groups * n_state) = [x | B | C] after the convolution; dt_raw = proj[t][dt_col0 + h] (fp32, ld);
 * state fp32 (slots, heads, n_state, vdim), read at the start and written back at the end; y fp32 (n_tok, heads * vdim).
 * Head h uses group h / (heads / groups).  A workgroup holds up to 1024 / ceil_pow2(n_state / 32) value columns of a head; wider heads
 * are cut into column parts (columns never meet in the recurrence).  vdim <= 1024, n_state <= 2048. */
int zls_ssm_scan(const float* xbc, const float* proj, int64_t ld, int64_t dt_col0, const float* dt_bias, const float* a_log, const float* d,
                 float* state, int64_t heads, int64_t vdim, int64_t n_state, int64_t groups, const zls_batch_t* b, float* y, void* workspace,
                 int64_t seg_len, zl_stream_t s);
/* workspace (nullable) and seg_len > 0: portions longer than seg_len tokens run in segments -- all segments from a zero state in parallel,
 * their start states from a short serial pass, then all segments again from their true start states (the decay is a scalar per head and
 * token, so a segment acts on its start state as S -> prod(decay) S + S_from_zero).  zls_ssm_scan_workspace_bytes sizes the workspace. */
int64_t zls_ssm_scan_workspace_bytes(int64_t n_seq, int64_t max_count, int64_t seg_len, int64_t heads, int64_t vdim, int64_t n_state);

/* out = N_g(y * silu(z)) * weight: the gate first, then every one of `norm_groups` equal parts of the row divided by its own root mean
 * square.  y fp32 (rows, inner); z = proj[t][z_col0 ..] fp32; weight fp32 (inner); out in `dtype`. */
int zls_gated_group_norm(const float* y, const float* proj, int64_t ld, int64_t z_col0, const float* weight, float eps, int64_t rows,
                         int64_t inner, int64_t norm_groups, void* out, int dtype, zl_stream_t s);

/* ---- weighted RMS norm ----------------------------------------------------------------------------------------------------------- */
/* out[i] = x[r] / sqrt(mean(x[r]^2) + eps) * (w + shift), r = rows[i] (rows NULL: r = i); x fp32 (.., width), w fp32 (width), out
 * (n_rows, width) in `dtype`.  shift = 1 serves weights stored around zero, 0 plain weights. */
int zls_rms_norm(const float* x, const int32_t* rows, const float* w, float shift, float eps, int64_t n_rows, int64_t width, void* out,
                 int dtype, zl_stream_t s);
/* x[t] += y[t] in place (fp32 (rows, width)); with w2 (nullable) also h2[t] = the weighted RMS norm of the new x[t] in `dtype`. */
int zls_add_rms_norm(float* x, const float* y, float eps, int64_t rows, int64_t width, const float* w2, float shift, void* h2, int dtype,
                     zl_stream_t s);
/* z[i] <- cap * tanh(z[i] * scale / cap) for n fp32 numbers in place (cap <= 0: z[i] * scale). */
int zls_scale_softcap(float* z, int64_t n, float scale, float cap, zl_stream_t s);

/* ---- layer norm --------------------------------------------------------------------------------------------------------------- */
/* out[i] = (x[r] - mean) / sqrt(var + eps) * w + b with r = rows[i] (rows NULL: r = i), var = mean of the squared deviations; x fp32
 * (.., width), w, b fp32 (width; b nullable), out (n_rows, width) in `dtype`.  Both moments are fp32, the mean taken first. */
int zls_layer_norm(const float* x, const int32_t* rows, const float* w, const float* b, float eps, int64_t n_rows, int64_t width, void* out,
                   int dtype, zl_stream_t s);
/* x[t] += layer_norm(y[t]; w, b) in place (x, y fp32 (rows, width)); with w2 (nullable, then b2 nullable too) also
 * h2[t] = layer_norm(new x[t]; w2, b2) in `dtype`: the input of the next matrix product, from the same launch. */
int zls_add_layer_norm(float* x, const float* y, const float* w, const float* b, float eps, int64_t rows, int64_t width, const float* w2,
                       const float* b2, void* h2, int dtype, zl_stream_t s);

/* ---- softmax attention over a paged key / value cache: rotary positions, unit-RMS queries and keys, turned values, a sliding window,
 *      weights mixed across heads ------------------------------------------------------------------------------------------------- */
/* Per token at position p, in place on the fp32 projection row proj[t] (ld floats):
 *   queries (heads x dim from q_col0) and keys (kv_heads x dim from k_col0): coordinate i < rot_dims / 2 of a head is paired with
 *   i + rot_dims / 2 and the pair (u, v) becomes (u cos a - v sin a, v cos a + u sin a), a = p * qk_freq[i]; the other coordinates stay;
 *   with qk_norm != 0 every head is then divided by sqrt(mean(head^2) + eps);
 *   values (kv_heads x vdim from v_col0): with v_freq (nullable) turned the same way over ALL vdim coordinates, a = p * v_freq[i].
 * Queries are written back to proj; keys go to the token's row of k_cache (pages, page_size, kv_heads * dim), values to the token's
 * column of v_cache, whose pages are transposed: (pages, kv_heads * vdim, page_size); both in `dtype`.  k_cache NULL (then v_cache too): only the queries are served -- a layer that reads
 * another layer's cache.  qk_freq fp32 (rot_dims / 2; rot_dims even, <= dim; 0: no rotation), v_freq fp32 (vdim / 2; vdim even).
 * dim, vdim <= 512.  interleaved != 0: the rotated pairs are the neighbours (2i, 2i + 1) instead of (i, i + rot_dims / 2), pair i turned by
 * p * qk_freq[i] either way.  vmix_src (nullable, fp32 rows of vmix_ld numbers): the values become (1 - vmix_lambda) v + vmix_lambda *
 * vmix_src[t][vmix_col0 ..] (kv_heads * vdim numbers of the same token, e.g. an earlier layer's values) before they are cached.
 * q_norm_w / k_norm_w (nullable, fp32 (dim), shared by the heads; with qk_norm): the normed head is multiplied by the weight. */
int zls_rope_norm_store(float* proj, int64_t ld, int64_t q_col0, int64_t k_col0, int64_t v_col0, int64_t heads, int64_t kv_heads, int64_t dim,
                        int64_t vdim, const float* qk_freq, int64_t rot_dims, const float* v_freq, float eps, int qk_norm, int interleaved,
                        const float* vmix_src, int64_t vmix_ld, int64_t vmix_col0, float vmix_lambda, const float* q_norm_w, const float* k_norm_w,
                        const zls_batch_t* b, void* k_cache, void* v_cache, int dtype, zl_stream_t s);

/* The optional score form of the two attention launches below (NULL: plain scaled scores and a softmax).  For query head g at position p
 * and key j:  s = scale * head_scale[g] * q.k;  s <- softcap * tanh(s / softcap) (softcap > 0);  s += bias[g][min(p - j, bias_rows - 1)];
 * chunk > 0: only keys with j / chunk == p / chunk are visible (chunks counted from position 0; not together with keep_first);
 * sigmoid != 0: the weight of a visible key is sigmoid(s + offset[g]), every key on its own -- nothing is normalised, a split leaves
 * acc = sum_j w_j v_j and ml = (0, 1), and zls_head_mix_gate is called with plain_sum.  All pointers fp32 and nullable. */
typedef struct {
    const float* head_scale;   /* (heads) */
    float softcap;
    const float* bias;         /* (heads, bias_rows) */
    int32_t bias_rows;
    const float* offset;       /* (heads) */
    int32_t chunk;
    int32_t sigmoid;
} zls_score_form_t;

/* Softmax attention of every token over the cached keys j of its sequence with 0 <= p - j < window (window <= 0: all j <= p), and with
 * window > 0 also over the kept first keys j < keep_first (j <= p), at their true positions:
 *   w_g(j) = softmax_j(scale * q_g . k_c(g)(j)),  c(g) = g / (heads / kv_heads)
 *   all_kv == 0:  a[g][:]    = sum_j w_g(j) v_c(g)(j)                      nv = vdim numbers per head
 *   all_kv != 0:  a[g][c][:] = sum_j w_g(j) v_c(j) for EVERY kv head c     nv = kv_heads * vdim
 * The second form is what mixing the heads' weights needs (zls_head_mix_gate): sum_j (sum_g T[h][g] w_g(j)) v_c(h)(j) =
 * sum_g T[h][g] a[g][c(h)].  q fp32 (n_tok, ldq) from q_col0 (as zls_rope_norm_store left it).  Scores, weights and sums are fp32.
 * The pages of a token's window (after the pages that only hold kept first keys) are divided over n_splits workgroups (pages_per_split
 * each; n_splits * pages_per_split must cover the longest such list of the step); split s leaves acc[t][g][s][:] = sum_j e^(s_j - m) v_j,
 * unnormalised, and ml[t][g][s] = (m, sum_j e^(s_j - m)); zls_head_mix_gate merges them.  acc fp32 (n_tok, heads, n_splits, nv), ml fp32
 * (n_tok, heads, n_splits, 2).  single_only != 0: only sequences that bring ONE token are served (portions: zls_window_attention_prompt).
 * The value plane holds a page TRANSPOSED, (kv_heads, vdim, page_size), as zls_rope_norm_store writes it.  nv <= 2048, page_size <= 128
 * and a multiple of 8. */
int zls_window_attention(const float* q, int64_t ldq, int64_t q_col0, const void* k_cache, const void* v_cache, const zls_batch_t* b,
                         float scale, int64_t window, int64_t keep_first, int64_t heads, int64_t kv_heads, int64_t dim, int64_t vdim, int all_kv,
                         float* acc, float* ml, int64_t n_splits, int64_t pages_per_split, int single_only, const zls_score_form_t* form,
                         int dtype, zl_stream_t s);
/* The same attention for query TILES on the matrix cores, bf16 only: tile i = tiles[3 i ..] = (first flat token, rows <= 64, sequence
 * index), consecutive tokens of one sequence.  Writes split 0 of acc for its tokens, unnormalised with ml = (m, sum) like the plain
 * kernel, and ml = (-inf, 0) for the other splits.  page_size 64, dim % 8 == 0, dim <= 256, vdim % 16 == 0. */
int zls_window_attention_prompt(const float* q, int64_t ldq, int64_t q_col0, const void* k_cache, const void* v_cache, const zls_batch_t* b,
                                const int32_t* tiles, int64_t n_tiles, float scale, int64_t window, int64_t keep_first, int64_t heads,
                                int64_t kv_heads, int64_t dim, int64_t vdim, int all_kv, float* acc, float* ml, int64_t n_splits,
                                const zls_score_form_t* form, int dtype, zl_stream_t s);

/* out[t][h][:] = turn_back(sum_g talk[h][g] a[t][g][c(h)][:]) * sigmoid(gate[t][h * vdim + :]), a = the splits of acc merged:
 * a[t][g] = sum_s e^(m_s - M) acc[t][g][s] / (sum_s e^(m_s - M) l_s + e^(sink_g - M)), the last term only with sink (fp32 (heads),
 * nullable: a learned score per head that has no key and no value and is not scaled; M then also covers it).
 * talk fp32 (heads, heads), NULL: no mixing, acc holds vdim numbers per head and split; v_freq (nullable): pair (m, m + vdim / 2) is turned
 * by -p * v_freq[m]; gate fp32 (n_tok, ldg) from g_col0, NULL: no gate; out (n_tok, heads * vdim) in `dtype`.
 * plain_sum != 0: the splits hold sums of finished weights (the sigmoid score form): a[t][g] = sum_s acc[t][g][s], no sink. */
int zls_head_mix_gate(const float* acc, const float* ml, int64_t n_splits, const float* talk, const float* v_freq, const float* gate,
                      int64_t ldg, int64_t g_col0, const float* sink, int plain_sum, const zls_batch_t* b, int64_t heads, int64_t kv_heads,
                      int64_t vdim, void* out, int dtype, zl_stream_t s);

/* ---- linear attention with a scalar decay per head and token ---------------------------------------------------------------------- */
/* S_t = a_t S_{t-1} + b_t k_t v_t^T,  y_t = S_t^T q_t   per head, S fp32 (dim x vdim) carried in state[slot].
 *   q, k (heads x dim) and v (heads x vdim): columns q_col0 / k_col0 / v_col0 of the fp32 rows proj[t] (ld), passed through SiLU first when
 *   act == 1;  a_t = decay_t[t][h] (fp32 (n_tok, heads)) or, with decay_t NULL, the constant decay_h[h];  b_t = gain_t[t][h] or 1.
 *   norm_col != 0: the state has one more column that takes the value 1 for every token, i.e. holds n_t = a_t n_{t-1} + b_t k_t, and y
 *   one more number per head, n_t . q_t.
 * state fp32 (slots, heads, dim, vdim + norm_col); y fp32 (n_tok, heads * (vdim + norm_col)).  Long portions run in segments exactly as
 * zls_ssm_scan's do (same kernel, workspace from zls_ssm_scan_workspace_bytes(n_seq, max_count, seg_len, heads, vdim + norm_col, dim)). */
/* decay_v (nullable; then decay_h and decay_t are NULL): fp32 (n_tok, heads * dim), a decay per KEY CHANNEL and token --
 * S_t = diag(a_t) S_{t-1} + b_t k_t v_t^T (the decay acts on the state's rows). */
int zls_decay_scan(const float* proj, int64_t ld, int64_t q_col0, int64_t k_col0, int64_t v_col0, int act, const float* decay_h,
                   const float* decay_t, const float* gain_t, int norm_col, float* state, int64_t heads, int64_t dim, int64_t vdim,
                   const zls_batch_t* b, float* y, void* workspace, int64_t seg_len, const float* decay_v,
                   zl_stream_t s);

/* Exponential gates with a running maximum (per sequence and head, tokens in order; m carried in m_state[slot][h], 0 for a new sequence):
 *   i = cap tanh((zi + i_bias[h]) / cap),  f = log sigmoid(cap tanh((zf + f_bias[h]) / cap))      (cap <= 0: no cap)
 *   m_t = max(f + m_{t-1}, i);  decay[t][h] = exp(f + m_{t-1} - m_t);  gain[t][h] = exp(i - m_t);  m_out[t][h] = m_t
 * zi / zf = proj[t][i_col0 + h] / proj[t][f_col0 + h] (fp32, ld).  decay, gain, m_out fp32 (n_tok, heads). */
int zls_exp_gates(const float* proj, int64_t ld, int64_t i_col0, int64_t f_col0, const float* i_bias, const float* f_bias, float cap,
                  float* m_state, int64_t heads, const zls_batch_t* b, float* decay, float* gain, float* m_out, zl_stream_t s);

/* The end of a linear-attention mixer: o = y[t][h][0 .. vdim) (row stride of a head: vdim + norm_col);
 *   with m_vals (needs norm_col): o = q_scale * o / (max(|q_scale * y[t][h][vdim]|, exp(-m_vals[t][h])) + den_eps);
 *   every one of `norm_groups` equal parts of the row heads * vdim is divided by sqrt(mean(part^2) + eps), times weight (nullable),
 *   times sigmoid(gate[t][g_col0 + c]) (gate nullable).  out (n_tok, heads * vdim) in `dtype`. */
/* gate_kind 0: the gate is sigmoid(gate); 1: silu(gate).  Without m_vals o is only scaled by q_scale before the norm. */
int zls_linear_attn_finish(const float* y, int64_t norm_col, float q_scale, const float* m_vals, float den_eps, int64_t heads, int64_t vdim,
                           int64_t norm_groups, const float* weight, float eps, const float* gate, int64_t ldg, int64_t g_col0,
                           int64_t n_tok, void* out, int dtype, int gate_kind, zl_stream_t s);
/* alpha[t][c] = sigmoid(sum_j w2[c][j] u[t][j] + bias[c])^(1 / tau) for c < channels: a decay per channel from `low` numbers per token,
 * u[t] = proj[t][u_col0 ..] fp32; w2 (channels, low) in `dtype`, bias fp32 (nullable); sums, the log-sigmoid and alpha are fp32. */
int zls_lowrank_decay(const float* proj, int64_t ld, int64_t u_col0, int64_t low, const void* w2, const float* bias, float tau,
                      int64_t channels, int64_t n_tok, float* alpha, int dtype, zl_stream_t s);

/* ---- mixture of experts over a ragged step ------------------------------------------------------------------------------------------ */
/* Router: s = softmax(logits[t]) over all n_out outputs (score_kind 0) or sigmoid(logits[t][i]) of each (score_kind 1); choice = s +
 * correction (nullable); the outputs form `groups` equal groups of neighbours, a group's score is the sum of its `group_top` largest choice
 * scores (1: its largest), only outputs of the `keep` best groups can be chosen (groups <= 1: all) -- the others count as minus
 * infinity; the `top` largest choice scores are chosen (ties: the lower index).  ids int32 (n_tok, top), weights fp32 (n_tok, top) = s of
 * the chosen (divided by their sum + renorm_eps when renorm != 0), times weight_scale.  n_out <= 1024, n_out % groups == 0.  A token's
 * logits are the first n_out numbers of its row of ld >= n_out numbers. */
int zls_moe_route(const float* logits, int64_t ld, int64_t n_tok, int64_t n_out, const float* correction, int64_t groups, int64_t keep, int64_t top,
                  int renorm, int score_kind, int64_t group_top, float renorm_eps, float weight_scale, int32_t* ids, float* weights,
                  zl_stream_t s);
/* Sort the n_slots = n_tok * top (token, choice) pairs by expert: pairs whose id is >= n_experts (identity outputs) are left out.
 *   sorted_tok[p] = token of the pair at sorted position p;  slot_pos[t * top + k] = p (or -1);
 *   tiles[3 i ..] = (expert, first position, end position) of the i-th run of at most tile_m positions of one expert, expert = -1 for unused
 *   entries up to max_tiles >= n_slots / tile_m + n_experts;  sorted_exp (nullable, n_slots): the expert of sorted position p, -1 for the
 *   positions that no pair takes.  One workgroup. */
int zls_moe_align(const int32_t* ids, int64_t n_slots, int64_t top, int64_t n_experts, int64_t tile_m, int32_t* sorted_tok, int32_t* slot_pos,
                  int32_t* tiles, int64_t max_tiles, int32_t* sorted_exp, zl_stream_t s);
/* y[p] = x[x_rows[p]] . w[expert of p]^T for every sorted position p: w (n_experts, n, k) in `dtype`, x_rows NULL: x[p]; `tiles` from
 * zls_moe_align with the same tile_m (64 or 128: the workgroup's tile).  gated != 0: n = 2 ff rows per expert, stored as blocks of 16 gate rows followed by their 16 up rows
 * (ff % 16 == 0), and y (.., ff) = act(gate, up) in out_dtype with act / act_alpha / act_limit as zls_act_mul's kind / alpha / limit
 * (0: silu(gate) * up).  Otherwise y (.., n).
 * row_expert (nullable; sorted_exp of zls_moe_align) with n_rows = the number of sorted positions: the few-rows form -- a wave per (row,
 * output column) streams the weight row once instead of a 64-row tile per expert; the same results up to the order of the fp32 sums. */
int zls_gemm_nt_grouped(const void* x, int64_t ldx, const int32_t* x_rows, const void* w, const int32_t* tiles, int64_t max_tiles,
                        int64_t tile_m, const int32_t* row_expert, int64_t n_rows, void* y, int64_t ldy, int64_t n, int64_t k, int gated,
                        int dtype, int out_dtype, int act, float act_alpha, float act_limit, zl_stream_t s);
/* out[p][c] = silu(gu[p][c]) * gu[p][ff + c]  for rows 0 .. rows - 1 (gu fp32 (rows, 2 ff)), out in `dtype`. */
int zls_silu_mul(const float* gu, int64_t rows, int64_t ff, void* out, int dtype, zl_stream_t s);
/* out[p][c] = act(g, u) of gu fp32 (rows, 2 ff) in `dtype`: kind 0 silu(g) u; 1 gelu_tanh(g) u (tanh form); 2 g' sigmoid(alpha g') (u' + 1)
 * with g' = min(g, limit), u' = clamp(u, -limit, limit).  block 0: g = gu[p][c], u = gu[p][ff + c]; block > 0 (ff % block == 0): the row
 * holds blocks of `block` gates followed by their `block` ups (the packing of the gated grouped product). */
int zls_act_mul(const float* gu, int64_t rows, int64_t ff, int kind, float alpha, float limit, int64_t block, void* out, int dtype,
                zl_stream_t s);
/* out[t] = sum_k weights[t][k] * (ids[t][k] >= n_experts ? h[t] : y[slot_pos[t * top + k]]), in the order of k; y fp32 (.., width),
 * h (n_tok, width) in `dtype`, out fp32. */
int zls_moe_combine(const float* y, const int32_t* slot_pos, const int32_t* ids, const float* weights, const void* h, int64_t n_tok,
                    int64_t top, int64_t n_experts, int64_t width, float* out, int dtype, zl_stream_t s);

/* ---- a residual kept as several streams ------------------------------------------------------------------------------------------ */
/* The residual of a token is n <= 8 rows x_0 .. x_{n-1} of `width` fp32 numbers; element (t, s, i) of the streams that are READ lies at
 * src[t * src_tok + s * src_stream + i] (src_stream = 0 reads one row as every stream: the start, where all streams equal the embedding).
 * h[r] = N(sum_s read_coef[s] x_s[row r]) with N(u) = u / sqrt(mean(u^2) + eps) * (w + shift), row r = rows[r] (rows NULL: r);
 * read_coef fp32 (n), NULL: all 1 (the sum of the streams); h (n_rows, width) in `dtype`.  The sum runs in the order of the streams. */
int zls_streams_norm(const float* src, int64_t src_tok, int64_t src_stream, int64_t n, const float* read_coef, const int32_t* rows,
                     const float* w, float shift, float eps, int64_t n_rows, int64_t width, void* h, int dtype, zl_stream_t s);
/* A sub-layer's result y fp32 (n_tok, width) enters the streams:  y' = y * sigmoid(gate[t][g_col0 + i] + gate_bias[i]) (gate fp32 (n_tok,
 * ldg), nullable: y' = y; gate_bias nullable);  x_d <- sum_s mix[s][d] x_s + out_coef[d] y' for every stream d at once from the old
 * streams (mix fp32 (n, n) indexed [from][to], out_coef fp32 (n)); written to dst (n_tok, n, width), which may be src.  With read_coef
 * (nullable) also h[t] = N(sum_d read_coef[d] x_d) of the NEW streams in `dtype`: the next sub-layer's input. */
int zls_streams_update(const float* src, int64_t src_tok, int64_t src_stream, float* dst, int64_t n, const float* y, const float* gate,
                       int64_t ldg, int64_t g_col0, const float* gate_bias, const float* mix, const float* out_coef, const float* read_coef,
                       const float* w, float shift, float eps, int64_t n_tok, int64_t width, void* h, int dtype, zl_stream_t s);
/* out[r][c] = act(z[r * ldz + c]) for fp32 z, out (rows, cols) in `dtype`: kind 0 relu(z)^2, 1 gelu_tanh(z), 2 silu(z). */
int zls_unary_act(const float* z, int64_t ldz, int64_t rows, int64_t cols, int kind, void* out, int dtype, zl_stream_t s);

#ifdef __cplusplus
}
#endif
#endif
