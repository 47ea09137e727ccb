// latent_attn.hip -- attention over a PAGED cache of normed low-rank latents, for every token of a ragged step.
//
// Beside csrc/mla_attn.hip (DeepSeek's geometry: 512 + 64 rotated columns, 16-bit, decode rows only, no sink): this one has no rotated
// part, any rank / head sizes, a learned per-head sink in the softmax denominator, a per-head sigmoid output gate, causal portions of
// prompts at any offset, and a 32-bit mode.  Only the latent is cached; keys and values are never materialised:
//     score_j = (W_uk,h^T q_h) . c_j * scale          o_h = W_uv,h . (sum_j w_j c_j)
// k_latent_store   RMS norm (plain weight) of the down-projection -> the token's cache row
// k_latent_attn    one wave per (token, head): the query is folded through W_uk once, then 64 keys at a time -- a lane per key for the
//                  scores (fp32), running maximum / denominator that START at the sink (m = sink, l = 1: the sink counts once, unscaled,
//                  with no value), a lane per latent column for the weighted sum; W_uv and the gate at the end.
#include "seq_common.h"

namespace {

template <int DT>
__global__ __launch_bounds__(256) void k_latent_store(const float* __restrict__ proj, int64_t ld, int col0, const float* __restrict__ weight,
                                                      float eps, int rank, const zls_batch_t b, void* __restrict__ cache) {
    __shared__ float red[16];
    const int t = blockIdx.x;
    const int sq = b.tok_seq[t];
    const int pos = b.seq_pos0[sq] + (t - b.seq_start[sq]);
    const int page = b.page_table[(size_t)sq * b.max_pages + pos / b.page_size];
    const size_t dst = ((size_t)page * b.page_size + pos % b.page_size) * rank;
    const float* u = proj + (size_t)t * ld + col0;
    float ss = 0.f;
    for (int i = threadIdx.x; i < rank; i += 256) ss = fmaf(u[i], u[i], ss);
    ss = zl_block_sum(ss, red);
    const float f = 1.0f / sqrtf(ss / (float)rank + eps);
    for (int i = threadIdx.x; i < rank; i += 256) SeqT<DT>::st(cache, dst + i, u[i] * f * weight[i]);
}

struct AttnP {
    const float* q; const float* gate; const void* w_uk; const void* w_uv; const float* sink; const void* cache; void* out;
    int64_t ldq, ldg;
    int q_col0, g_col0, heads, dim, vdim, rank;
    float scale;
};

// dynamic LDS: qk[rank] | acc[rank] | prob[64] | rowoff[64] (as int)
template <int DT>
__global__ __launch_bounds__(64) void k_latent_attn(const AttnP p, const zls_batch_t b) {
    extern __shared__ float lds[];
    float* qk = lds;
    float* acc = lds + p.rank;
    float* prob = acc + p.rank;
    int* rowoff = reinterpret_cast<int*>(prob + 64);
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const int sq = b.tok_seq[t];
    const int pos = b.seq_pos0[sq] + (t - b.seq_start[sq]);
    const int nkeys = pos + 1;
    const int32_t* pages = b.page_table + (size_t)sq * b.max_pages;
    const float* qh = p.q + (size_t)t * p.ldq + p.q_col0 + (size_t)h * p.dim;

    for (int r = lane; r < p.rank; r += 64) {
        float a = 0.f;
        for (int d = 0; d < p.dim; ++d) a = fmaf(qh[d], SeqT<DT>::ld(p.w_uk, ((size_t)h * p.dim + d) * p.rank + r), a);
        qk[r] = a * p.scale;
        acc[r] = 0.f;
    }
    float m = p.sink ? p.sink[h] : -INFINITY;
    float l = p.sink ? 1.0f : 0.0f;
    __syncthreads();
    for (int j0 = 0; j0 < nkeys; j0 += 64) {
        const int j = j0 + lane;
        const bool valid = j < nkeys;
        float sc = -INFINITY;
        int row = 0;
        if (valid) {
            row = pages[j / b.page_size] * b.page_size + j % b.page_size;
            const size_t base = (size_t)row * p.rank;
            float a = 0.f;
            for (int r = 0; r < p.rank; ++r) a = fmaf(qk[r], SeqT<DT>::ld(p.cache, base + r), a);
            sc = a;
        }
        const float mnew = fmaxf(m, zl_wave_max(sc));               // finite: key j0 is always valid
        const float corr = expf(m - mnew);                          // m = -inf (no sink, first tile): 0
        const float pj = valid ? expf(sc - mnew) : 0.f;
        l = l * corr + zl_wave_sum(pj);
        m = mnew;
        prob[lane] = pj;
        rowoff[lane] = row;
        __syncthreads();
        const int cnt = min(64, nkeys - j0);
        for (int r = lane; r < p.rank; r += 64) {
            float a = acc[r] * corr;
            for (int jj = 0; jj < cnt; ++jj) a = fmaf(prob[jj], SeqT<DT>::ld(p.cache, (size_t)rowoff[jj] * p.rank + r), a);
            acc[r] = a;
        }
        __syncthreads();
    }
    const float g = p.gate ? seq_sigmoid(p.gate[(size_t)t * p.ldg + p.g_col0 + h]) : 1.0f;
    const float inv = g / l;
    for (int d = lane; d < p.vdim; d += 64) {
        const size_t wrow = ((size_t)h * p.vdim + d) * p.rank;
        float a = 0.f;
        for (int r = 0; r < p.rank; ++r) a = fmaf(SeqT<DT>::ld(p.w_uv, wrow + r), acc[r], a);
        SeqT<DT>::st(p.out, ((size_t)t * p.heads + h) * p.vdim + d, a * inv);
    }
}

}  // namespace

extern "C" int zls_latent_store(const float* proj, int64_t ld, int64_t col0, const float* weight, float eps, int64_t rank, const zls_batch_t* b,
                                void* cache, int dtype, zl_stream_t s) {
    ZL_CHECK_ARG(proj && weight && cache && seq_batch_ok(b) && b->page_table && b->page_size > 0 && b->max_pages > 0 && rank > 0, ZL_EINVAL);
    ZL_CHECK_ARG(col0 >= 0 && col0 + rank <= ld, ZL_ESHAPE);
#define CALL(DT) hipLaunchKernelGGL((k_latent_store<DT>), dim3(b->n_tok), dim3(256), 0, (hipStream_t)s, proj, ld, (int)col0, weight, eps, (int)rank, *b, cache);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}

extern "C" int zls_latent_attention(const float* q, int64_t ldq, int64_t q_col0, const float* gate, int64_t ldg, int64_t g_col0, const void* w_uk,
                                    const void* w_uv, const float* sink, const void* cache, const zls_batch_t* b, float scale, int64_t heads,
                                    int64_t dim, int64_t vdim, int64_t rank, void* out, int dtype, zl_stream_t s) {
    ZL_CHECK_ARG(q && w_uk && w_uv && cache && out && seq_batch_ok(b) && b->page_table && b->page_size > 0 && b->max_pages > 0, ZL_EINVAL);
    ZL_CHECK_ARG(heads > 0 && dim > 0 && vdim > 0 && rank > 0 && heads <= 65535, ZL_EINVAL);
    ZL_CHECK_ARG(q_col0 >= 0 && q_col0 + heads * dim <= ldq && (!gate || (g_col0 >= 0 && g_col0 + heads <= ldg)), ZL_ESHAPE);
    const size_t lds = (2 * (size_t)rank + 128) * sizeof(float);
    ZL_CHECK_ARG(lds <= 64 * 1024, ZL_ELIMIT);
    AttnP p;
    p.q = q; p.gate = gate; p.w_uk = w_uk; p.w_uv = w_uv; p.sink = sink; p.cache = cache; p.out = out;
    p.ldq = ldq; p.ldg = ldg; p.q_col0 = (int)q_col0; p.g_col0 = (int)g_col0;
    p.heads = (int)heads; p.dim = (int)dim; p.vdim = (int)vdim; p.rank = (int)rank; p.scale = scale;
#define CALL(DT) hipLaunchKernelGGL((k_latent_attn<DT>), dim3(b->n_tok, (unsigned)heads), dim3(64), lds, (hipStream_t)s, p, *b);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}
