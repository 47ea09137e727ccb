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
    int q_col0, g_col0, heads, dim, vdim, rank, single_only;
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
    if (p.single_only && b.seq_start[sq + 1] - b.seq_start[sq] > 1) return;     // portions go to the prompt kernel (workgroup-uniform)
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

// ---- prompt portions on the matrix cores (bf16 serving) -----------------------------------------------------------------------------
// Keys and values of a portion's whole context are up-projected once per step into dense K (n_ctx, heads * dim) and V^T (heads * vdim,
// n_ctx) (zls_gemm_nt_gather over the cached rows; each sequence's rows start at a multiple of 64).  A workgroup = 64 queries of one
// sequence x one head, a wave = 16 of them.  Per 64-key tile (K and V^T staged in LDS, shared by the four waves):
//   S^T (16 keys x 16 queries) = K_tile . Q^T on v_mfma_f32_16x16x32_bf16 -- a lane then holds 4 consecutive keys of ONE query, which is
//   exactly the B operand of v_mfma_f32_16x16x16_bf16, so the weights never travel through LDS:
//   O^T (vdim x 16 queries) += V^T_tile . P^T, with P = hi + lo (two bf16 halves: the weights keep 16 bits of mantissa).
// Scores, running maximum / denominator (starting at the sink: m = sink, l = 1) and the output sums are fp32, per lane = per query.
typedef __bf16 fa_b8 __attribute__((ext_vector_type(8)));
typedef short fa_s4 __attribute__((ext_vector_type(4)));
typedef float fa_f4 __attribute__((ext_vector_type(4)));

struct FaP {
    const float* q; const float* gate; const uint16_t* k; const uint16_t* vt; const float* sink; const int32_t* ctx_start; uint16_t* out;
    int64_t ldq, ldg, ldk, ldv;
    int q_col0, g_col0, heads, dim, vdim, tiles_per_seq, vec_k;
    float scale;
};

template <int DK, int DV>
__global__ __launch_bounds__(256) void k_latent_fa(const FaP p, const zls_batch_t b) {
    constexpr int KR = DK * 32 + 8, VR = 64 + 8;
    __shared__ __attribute__((aligned(16))) uint16_t Ks[64 * KR];
    __shared__ __attribute__((aligned(16))) uint16_t Vs[DV * 16 * VR];
    const int sq = blockIdx.x / p.tiles_per_seq, tile = blockIdx.x % p.tiles_per_seq, h = blockIdx.y;
    const int first = b.seq_start[sq], count = b.seq_start[sq + 1] - first;
    const int cs = p.ctx_start[sq];
    if (cs < 0 || tile * 64 >= count) return;
    const int pos0 = b.seq_pos0[sq];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nrow = lane & 15, kq = lane >> 4;
    const int qi = tile * 64 + wave * 16 + nrow;
    const bool qvalid = qi < count;
    const int qpos = pos0 + qi;
    const int wave_last = pos0 + min(count, tile * 64 + wave * 16 + 16) - 1;       // the last key any query of this wave sees
    const int block_last = pos0 + min(count, tile * 64 + 64) - 1;

    uint4 qf[DK];
    {
        const float* qr = p.q + (size_t)(first + (qvalid ? qi : 0)) * p.ldq + p.q_col0 + (size_t)h * p.dim;
#pragma unroll
        for (int kk = 0; kk < DK; ++kk) {
            uint32_t w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int d = 32 * kk + 8 * kq + 2 * i;
                const float a = (qvalid && d < p.dim) ? qr[d] : 0.f, c = (qvalid && d + 1 < p.dim) ? qr[d + 1] : 0.f;
                w[i] = ZT<ZL_BF16>::from_f32(a) | (uint32_t)ZT<ZL_BF16>::from_f32(c) << 16;
            }
            qf[kk] = make_uint4(w[0], w[1], w[2], w[3]);
        }
    }
    fa_f4 o[DV];
#pragma unroll
    for (int dt = 0; dt < DV; ++dt) o[dt] = (fa_f4){0.f, 0.f, 0.f, 0.f};
    float m = p.sink ? p.sink[h] : -INFINITY, l = p.sink ? 1.0f : 0.0f;

    for (int j0 = 0; j0 <= block_last; j0 += 64) {
        __syncthreads();
        for (int idx = tid; idx < 64 * DK * 4; idx += 256) {                       // K tile: 64 keys x (DK * 32) columns, zero past dim
            const int key = idx / (DK * 4), d = (idx % (DK * 4)) * 8;
            const uint16_t* src = p.k + (size_t)(cs + j0 + key) * p.ldk + (size_t)h * p.dim + d;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (d + 8 <= p.dim && p.vec_k) v = *reinterpret_cast<const uint4*>(src);
            else if (d < p.dim) {
                uint16_t e[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) e[i] = d + i < p.dim ? src[i] : (uint16_t)0;
                v = make_uint4(e[0] | (uint32_t)e[1] << 16, e[2] | (uint32_t)e[3] << 16, e[4] | (uint32_t)e[5] << 16, e[6] | (uint32_t)e[7] << 16);
            }
            *reinterpret_cast<uint4*>(Ks + key * KR + d) = v;
        }
        for (int idx = tid; idx < DV * 16 * 8; idx += 256) {                       // V^T tile: (DV * 16) rows x 64 keys, zero past vdim
            const int d = idx >> 3, c8 = (idx & 7) * 8;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (d < p.vdim) v = *reinterpret_cast<const uint4*>(p.vt + ((size_t)h * p.vdim + d) * p.ldv + cs + j0 + c8);
            *reinterpret_cast<uint4*>(Vs + d * VR + c8) = v;
        }
        __syncthreads();
        if (j0 > wave_last) continue;                                              // wave-uniform; the barriers above stay in step
        fa_f4 sc[4];
        float mx = -INFINITY;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            sc[c] = (fa_f4){0.f, 0.f, 0.f, 0.f};
            if (j0 + 16 * c <= wave_last) {
#pragma unroll
                for (int kk = 0; kk < DK; ++kk) {
                    const uint4 a = *reinterpret_cast<const uint4*>(Ks + (16 * c + nrow) * KR + 32 * kk + 8 * kq);
                    sc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(fa_b8, a), __builtin_bit_cast(fa_b8, qf[kk]), sc[c], 0, 0, 0);
                }
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int key = j0 + 16 * c + 4 * kq + r;
                const float v = (qvalid && key <= qpos) ? sc[c][r] * p.scale : -INFINITY;
                sc[c][r] = v;
                mx = fmaxf(mx, v);
            }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float mnew = fmaxf(m, mx);
        const bool dead = mnew == -INFINITY;                                       // nothing seen yet and no sink: keep zeros
        const float corr = dead ? 1.0f : expf(m - mnew);
        float ps = 0.f;
        fa_s4 hi[4], lo[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float pv = (dead || sc[c][r] == -INFINITY) ? 0.f : expf(sc[c][r] - mnew);
                ps += pv;
                const uint16_t hb = ZT<ZL_BF16>::from_f32(pv);
                hi[c][r] = (short)hb;
                lo[c][r] = (short)ZT<ZL_BF16>::from_f32(pv - ZT<ZL_BF16>::to_f32(hb));
            }
        }
        ps += __shfl_xor(ps, 16, 64);
        ps += __shfl_xor(ps, 32, 64);
        l = l * corr + ps;
        m = mnew;
#pragma unroll
        for (int dt = 0; dt < DV; ++dt) {
            o[dt] *= corr;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                if (j0 + 16 * c <= wave_last) {
                    const uint2 a2 = *reinterpret_cast<const uint2*>(Vs + (16 * dt + nrow) * VR + 16 * c + 4 * kq);
                    const fa_s4 a = __builtin_bit_cast(fa_s4, a2);
                    o[dt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, hi[c], o[dt], 0, 0, 0);
                    o[dt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, lo[c], o[dt], 0, 0, 0);
                }
            }
        }
    }
    if (!qvalid) return;
    const float g = p.gate ? seq_sigmoid(p.gate[(size_t)(first + qi) * p.ldg + p.g_col0 + h]) : 1.0f;
    const float inv = l > 0.f ? g / l : 0.f;
    uint16_t* orow = p.out + ((size_t)(first + qi) * p.heads + h) * p.vdim;
#pragma unroll
    for (int dt = 0; dt < DV; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int d = 16 * dt + 4 * kq + r;
            if (d < p.vdim) orow[d] = ZT<ZL_BF16>::from_f32(o[dt][r] * inv);
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
                                    int64_t dim, int64_t vdim, int64_t rank, void* out, int dtype, int single_only, zl_stream_t s) {
    ZL_CHECK_ARG(q && w_uk && w_uv && cache && out && seq_batch_ok(b) && b->page_table && b->page_size > 0 && b->max_pages > 0, ZL_EINVAL);
    ZL_CHECK_ARG(heads > 0 && dim > 0 && vdim > 0 && rank > 0 && heads <= 65535, ZL_EINVAL);
    ZL_CHECK_ARG(q_col0 >= 0 && q_col0 + heads * dim <= ldq && (!gate || (g_col0 >= 0 && g_col0 + heads <= ldg)), ZL_ESHAPE);
    const size_t lds = (2 * (size_t)rank + 128) * sizeof(float);
    ZL_CHECK_ARG(lds <= 64 * 1024, ZL_ELIMIT);
    AttnP p;
    p.q = q; p.gate = gate; p.w_uk = w_uk; p.w_uv = w_uv; p.sink = sink; p.cache = cache; p.out = out;
    p.ldq = ldq; p.ldg = ldg; p.q_col0 = (int)q_col0; p.g_col0 = (int)g_col0;
    p.heads = (int)heads; p.dim = (int)dim; p.vdim = (int)vdim; p.rank = (int)rank; p.scale = scale; p.single_only = single_only;
#define CALL(DT) hipLaunchKernelGGL((k_latent_attn<DT>), dim3(b->n_tok, (unsigned)heads), dim3(64), lds, (hipStream_t)s, p, *b);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}

extern "C" int zls_latent_attention_prompt(const float* q, int64_t ldq, int64_t q_col0, const float* gate, int64_t ldg, int64_t g_col0,
                                           const void* k, int64_t ldk, const void* vt, int64_t ldv, const float* sink, const int32_t* ctx_start,
                                           const zls_batch_t* b, float scale, int64_t heads, int64_t dim, int64_t vdim, void* out, int dtype,
                                           zl_stream_t s) {
    ZL_CHECK_ARG(q && k && vt && ctx_start && out && seq_batch_ok(b), ZL_EINVAL);
    ZL_CHECK_ARG(dtype == ZL_BF16, ZL_EDTYPE);
    ZL_CHECK_ARG(heads > 0 && heads <= 65535 && dim > 0 && vdim > 0 && dim <= 256 && vdim <= 256, ZL_ESHAPE);
    ZL_CHECK_ARG(q_col0 >= 0 && q_col0 + heads * dim <= ldq && (!gate || (g_col0 >= 0 && g_col0 + heads <= ldg)), ZL_ESHAPE);
    ZL_CHECK_ARG(ldk >= heads * dim && ldv % 8 == 0 && ((uintptr_t)vt & 15) == 0, ZL_ESHAPE);
    FaP p;
    p.q = q; p.gate = gate; p.k = (const uint16_t*)k; p.vt = (const uint16_t*)vt; p.sink = sink; p.ctx_start = ctx_start; p.out = (uint16_t*)out;
    p.ldq = ldq; p.ldg = ldg; p.ldk = ldk; p.ldv = ldv; p.q_col0 = (int)q_col0; p.g_col0 = (int)g_col0;
    p.heads = (int)heads; p.dim = (int)dim; p.vdim = (int)vdim; p.scale = scale;
    p.tiles_per_seq = (b->max_count + 63) / 64;
    p.vec_k = (dim % 8 == 0 && ldk % 8 == 0 && ((uintptr_t)k & 15) == 0) ? 1 : 0;
    const dim3 grid((unsigned)(b->n_seq * p.tiles_per_seq), (unsigned)heads);
    const int64_t big = dim > vdim ? dim : vdim;
    hipStream_t hs = (hipStream_t)s;
    if (big <= 32) hipLaunchKernelGGL((k_latent_fa<1, 2>), grid, dim3(256), 0, hs, p, *b);
    else if (big <= 64) hipLaunchKernelGGL((k_latent_fa<2, 4>), grid, dim3(256), 0, hs, p, *b);
    else if (big <= 128) hipLaunchKernelGGL((k_latent_fa<4, 8>), grid, dim3(256), 0, hs, p, *b);
    else hipLaunchKernelGGL((k_latent_fa<8, 16>), grid, dim3(256), 0, hs, p, *b);
    return zl_launch_status();
}
