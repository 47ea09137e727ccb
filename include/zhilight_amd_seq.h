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

/* Causal attention of every token over its sequence's cached latents c_0 .. c_p, heads sharing the latent:
 *   score_j = scale * (W_uk,h^T q_h) . c_j;  w_j = exp(score_j) / (sum_i exp(score_i) + exp(sink_h));  o_h = W_uv,h (sum_j w_j c_j)
 *   out[t][h] = o_h * sigmoid(gate[t][h])         (sink NULL: no sink term; gate NULL: no gate)
 * q fp32 (n_tok, ldq) from column q_col0, heads x dim; gate fp32 (n_tok, ldg) from column g_col0, one number per head;
 * w_uk (heads * dim, rank), w_uv (heads * vdim, rank) in `dtype`; out (n_tok, heads * vdim) in `dtype`.  fp32 scores, weights and sums. */
int zls_latent_attention(const float* q, int64_t ldq, int64_t q_col0, const float* gate, int64_t ldg, int64_t g_col0, const void* w_uk,
                         const void* w_uv, const float* sink, const void* cache, const zls_batch_t* b, float scale, int64_t heads,
                         int64_t dim, int64_t vdim, int64_t rank, void* out, int dtype, int single_only, void* workspace, int64_t n_splits,
                         int no_mfma, zl_stream_t s);
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
int zls_latent_attention_prompt(const float* q, int64_t ldq, int64_t q_col0, const float* gate, int64_t ldg, int64_t g_col0, const void* k,
                                int64_t ldk, const void* vt, int64_t ldv, const float* sink, const int32_t* ctx_start, const zls_batch_t* b,
                                float scale, int64_t heads, int64_t dim, int64_t vdim, void* out, int dtype, zl_stream_t s);

/* ---- state-space (Mamba-2) mixer ---------------------------------------------------------------------------------------------- */
/* Causal per-channel convolution + SiLU over the columns col0 .. col0 + channels - 1 of proj: out[t][c] = silu(bias[c] + sum_k
 * w[c][k] * u[t - (taps - 1 - k)][c]); inputs before a portion's first token come from tail[slot] (taps - 1 rows, oldest first; zeros
 * for a new sequence).  zls_conv_tail_update then moves the portion's last taps - 1 inputs into tail[slot]; it must run after
 * zls_conv_silu on the same stream.  proj, out, tail fp32; w fp32 (channels, taps), bias fp32 (channels). */
int zls_conv_silu(const float* proj, int64_t ld, int64_t col0, const float* w, const float* bias, const float* tail, int64_t channels,
                  int64_t taps, const zls_batch_t* b, float* out, zl_stream_t s);
int zls_conv_tail_update(const float* proj, int64_t ld, int64_t col0, float* tail, int64_t channels, int64_t taps, const zls_batch_t* b,
                         zl_stream_t s);

/* The recurrence, one workgroup per (sequence, head), tokens in order:
 *   dt = softplus(dt_raw + dt_bias_h);  S <- exp(-exp(a_log_h) dt) S + dt B x^T;  y = S^T C + d_h x
 * xbc fp32 (n_tok, heads * vdim + 2 groups * n_state) = [x | B | C] after the convolution; dt_raw = proj[t][dt_col0 + h] (fp32, ld);
 * state fp32 (slots, heads, n_state, vdim), read at the start and written back at the end; y fp32 (n_tok, heads * vdim).
 * Head h uses group h / (heads / groups).  vdim * ceil_pow2(n_state / 32) <= 1024. */
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

#ifdef __cplusplus
}
#endif
#endif
