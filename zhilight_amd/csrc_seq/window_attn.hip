// window_attn.hip -- softmax attention over a paged key / value cache for a ragged step: rotary positions on a part of every query and key
// head, unit-RMS queries and keys, values turned by their own position and the sums turned back, a sliding window, weights mixed across
// heads after the softmax, a sigmoid gate per output coordinate.
//
// k_rope_norm_store    a workgroup per token, a wave per head in turn: the head's coordinates in registers, rotated, normed, written back
//                      (queries, fp32, in place) or to the token's row of the paged planes (keys, values; serving format)
// k_window_attention   a workgroup per (token, query head): keys of the window in chunks of kChunk -- a wave per key for the scores
//                      (butterfly over the head size), running maximum and sum over chunks, then a thread per output coordinate for P.V.
//                      With all_kv the weights of a query head are applied to the values of EVERY key / value head: mixing the heads'
//                      weights afterwards is then a small product per token (k_head_mix_gate), sum_g T[h][g] acc[g][c(h)], and no weight
//                      ever has to wait for another head's normaliser.
// k_head_mix_gate      a workgroup per token: the mix over heads, the turn back by the token's own position, the gate
// Positions, angles, scores, weights, sums: fp32.  exp / sin / cos are the accurate library versions.
#include "seq_common.h"

namespace {

constexpr int kMaxE = 8;            // coordinates of a head per lane: dim, vdim <= 64 * kMaxE
constexpr int kChunk = 128;         // keys per pass of k_window_attention
constexpr int kMaxV = 8;            // output coordinates per thread: (all_kv ? kv_heads : 1) * vdim <= 256 * kMaxV

// one head of `size` coordinates in the lanes' registers (coordinate i in lane i % 64, register i / 64): rotate the first n_rot (pairs
// i, i + n_rot / 2) by pos * freq[i], optionally divide by the root mean square; the result stays in v[]
__device__ __forceinline__ void rope_head(float* v, const float* src, int size, int n_rot, const float* __restrict__ freq, float pos, bool norm,
                                          float eps, int lane) {
    const int half = n_rot >> 1;
    float ss = 0.f;
#pragma unroll
    for (int r = 0; r < kMaxE; ++r) {
        const int i = lane + 64 * r;
        float o = 0.f;
        if (i < size) {
            o = src[i];
            if (i < n_rot) {
                const bool lo = i < half;
                const float other = src[lo ? i + half : i - half];
                float sn, cs;
                sincosf(pos * freq[lo ? i : i - half], &sn, &cs);
                o = lo ? o * cs - other * sn : o * cs + other * sn;
            }
            ss = fmaf(o, o, ss);
        }
        v[r] = o;
    }
    if (norm) {
        const float f = 1.0f / sqrtf(zl_wave_sum(ss) / (float)size + eps);
#pragma unroll
        for (int r = 0; r < kMaxE; ++r) v[r] *= f;
    }
}

struct RopeP {
    float* proj; int64_t ld;
    int q_col0, k_col0, v_col0, heads, kv_heads, dim, vdim, rot_dims, qk_norm;
    const float* qk_freq; const float* v_freq;
    float eps;
    void* k_cache; void* v_cache;
};

template <int DT>
__global__ __launch_bounds__(256) void k_rope_norm_store(const RopeP p, const zls_batch_t b) {
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sq = b.tok_seq[t];
    const int posi = b.seq_pos0[sq] + (t - b.seq_start[sq]);
    const float pos = (float)posi;
    float* row = p.proj + (size_t)t * p.ld;
    const size_t crow = (size_t)b.page_table[(size_t)sq * b.max_pages + posi / b.page_size] * b.page_size + posi % b.page_size;
    const int n_kv = p.k_cache ? p.kv_heads : 0;
    float v[kMaxE];
    for (int h = wave; h < p.heads + 2 * n_kv; h += 4) {                 // (a wave owns its heads: no two waves touch the same numbers)
        if (h < p.heads) {
            float* q = row + p.q_col0 + h * p.dim;
            rope_head(v, q, p.dim, p.rot_dims, p.qk_freq, pos, p.qk_norm != 0, p.eps, lane);
#pragma unroll
            for (int r = 0; r < kMaxE; ++r)
                if (lane + 64 * r < p.dim) q[lane + 64 * r] = v[r];
        } else if (h < p.heads + n_kv) {
            const int c = h - p.heads;
            rope_head(v, row + p.k_col0 + c * p.dim, p.dim, p.rot_dims, p.qk_freq, pos, p.qk_norm != 0, p.eps, lane);
#pragma unroll
            for (int r = 0; r < kMaxE; ++r)
                if (lane + 64 * r < p.dim) SeqT<DT>::st(p.k_cache, (crow * p.kv_heads + c) * p.dim + lane + 64 * r, v[r]);
        } else {
            const int c = h - p.heads - n_kv;
            rope_head(v, row + p.v_col0 + c * p.vdim, p.vdim, p.v_freq ? p.vdim : 0, p.v_freq, pos, false, 0.f, lane);
#pragma unroll
            for (int r = 0; r < kMaxE; ++r)
                if (lane + 64 * r < p.vdim) SeqT<DT>::st(p.v_cache, (crow * p.kv_heads + c) * p.vdim + lane + 64 * r, v[r]);
        }
    }
}

struct AttnP {
    const float* q; int64_t ldq; int q_col0;
    const void* k_cache; const void* v_cache;
    float scale; int window, heads, kv_heads, dim, vdim, all_kv;
    float* acc;
};

template <int DT>
__global__ __launch_bounds__(256) void k_window_attention(const AttnP p, const zls_batch_t b) {
    extern __shared__ float lds[];
    __shared__ float red[16];
    __shared__ float sc[kChunk];
    __shared__ int rowi[kChunk];
    float* qs = lds;                                                      // [dim], already times scale
    const int t = blockIdx.x, g = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int sq = b.tok_seq[t];
    const int pos = b.seq_pos0[sq] + (t - b.seq_start[sq]);
    const int lo = p.window > 0 ? max(0, pos - p.window + 1) : 0;
    const int c = g / (p.heads / p.kv_heads);
    const int nv = p.all_kv ? p.kv_heads * p.vdim : p.vdim, voff = p.all_kv ? 0 : c * p.vdim;
    const int32_t* pages = b.page_table + (size_t)sq * b.max_pages;
    for (int i = tid; i < p.dim; i += 256) qs[i] = p.q[(size_t)t * p.ldq + p.q_col0 + g * p.dim + i] * p.scale;
    float A[kMaxV];
#pragma unroll
    for (int r = 0; r < kMaxV; ++r) A[r] = 0.f;
    float m = -INFINITY, l = 0.f;
    __syncthreads();
    for (int j0 = lo; j0 <= pos; j0 += kChunk) {
        const int cn = min(kChunk, pos - j0 + 1);
        for (int jj = wave; jj < cn; jj += 4) {
            const int j = j0 + jj;
            const size_t row = (size_t)pages[j / b.page_size] * b.page_size + j % b.page_size;
            const size_t at = (row * p.kv_heads + c) * p.dim;
            float part = 0.f;
            for (int i = lane; i < p.dim; i += 64) part = fmaf(qs[i], SeqT<DT>::ld(p.k_cache, at + i), part);
            part = zl_wave_sum(part);
            if (lane == 0) { sc[jj] = part; rowi[jj] = (int)row; }
        }
        __syncthreads();
        float cm = -INFINITY;
        for (int jj = tid; jj < cn; jj += 256) cm = fmaxf(cm, sc[jj]);
        const float m_new = fmaxf(m, zl_block_max(cm, red));
        float ps = 0.f;
        for (int jj = tid; jj < cn; jj += 256) { const float e = expf(sc[jj] - m_new); sc[jj] = e; ps += e; }
        const float corr = expf(m - m_new);                               // (first chunk: exp(-inf) = 0 on zero sums)
        l = l * corr + zl_block_sum(ps, red);                             // (its barriers also publish the weights in sc[])
        m = m_new;
#pragma unroll
        for (int r = 0; r < kMaxV; ++r) {
            const int e = tid + 256 * r;
            if (e < nv) {
                float a = A[r] * corr;
                for (int jj = 0; jj < cn; ++jj)
                    a = fmaf(sc[jj], SeqT<DT>::ld(p.v_cache, (size_t)rowi[jj] * p.kv_heads * p.vdim + voff + e), a);
                A[r] = a;
            }
        }
        __syncthreads();                                                  // sc[] / rowi[] are free for the next chunk
    }
    const float inv = 1.0f / l;
    float* out = p.acc + ((size_t)t * p.heads + g) * nv;
#pragma unroll
    for (int r = 0; r < kMaxV; ++r)
        if (tid + 256 * r < nv) out[tid + 256 * r] = A[r] * inv;
}

struct MixP {
    const float* acc; const float* talk; const float* v_freq; const float* gate; int64_t ldg; int g_col0;
    int heads, kv_heads, vdim;
    void* out;
};

template <int DT>
__global__ __launch_bounds__(256) void k_head_mix_gate(const MixP p, const zls_batch_t b) {
    const int t = blockIdx.x;
    const int sq = b.tok_seq[t];
    const float pos = (float)(b.seq_pos0[sq] + (t - b.seq_start[sq]));
    const int per = p.heads / p.kv_heads, half = p.vdim >> 1;
    const int nv = p.talk ? p.kv_heads * p.vdim : p.vdim;                 // a head's stride in acc
    const float* a = p.acc + (size_t)t * p.heads * nv;
    // a thread owns a PAIR (m, m + vdim / 2) of one head (an odd vdim without rotation: the last coordinate alone)
    const int pairs = p.v_freq ? half : (p.vdim + 1) / 2;
    for (int w = threadIdx.x; w < p.heads * pairs; w += 256) {
        const int h = w / pairs, mm = w % pairs;
        const int i0 = mm, i1 = mm + pairs;
        float u = 0.f, v = 0.f;
        if (p.talk) {
            const int c = h / per;
            for (int g = 0; g < p.heads; ++g) {
                const float tw = p.talk[h * p.heads + g];
                const float* ag = a + (size_t)g * nv + c * p.vdim;
                u = fmaf(tw, ag[i0], u);
                if (i1 < p.vdim) v = fmaf(tw, ag[i1], v);
            }
        } else {
            u = a[(size_t)h * nv + i0];
            if (i1 < p.vdim) v = a[(size_t)h * nv + i1];
        }
        if (p.v_freq) {
            float sn, cs;
            sincosf(pos * p.v_freq[mm], &sn, &cs);                        // turned by -pos: (u cs + v sn, v cs - u sn)
            const float u2 = u * cs + v * sn, v2 = v * cs - u * sn;
            u = u2; v = v2;
        }
        const size_t o = (size_t)t * p.heads * p.vdim + (size_t)h * p.vdim;
        if (p.gate) {
            const float* gr = p.gate + (size_t)t * p.ldg + p.g_col0 + h * p.vdim;
            u *= seq_sigmoid(gr[i0]);
            if (i1 < p.vdim) v *= seq_sigmoid(gr[i1]);
        }
        SeqT<DT>::st(p.out, o + i0, u);
        if (i1 < p.vdim) SeqT<DT>::st(p.out, o + i1, v);
    }
}

}  // namespace

extern "C" int zls_rope_norm_store(float* proj, int64_t ld, int64_t q_col0, int64_t k_col0, int64_t v_col0, int64_t heads, int64_t kv_heads,
                                   int64_t dim, int64_t vdim, const float* qk_freq, int64_t rot_dims, const float* v_freq, float eps, int qk_norm,
                                   const zls_batch_t* b, void* k_cache, void* v_cache, int dtype, zl_stream_t s) {
    ZL_CHECK_ARG(proj && seq_batch_ok(b) && b->page_table && b->page_size > 0 && heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0, ZL_EINVAL);
    ZL_CHECK_ARG((k_cache == nullptr) == (v_cache == nullptr), ZL_EINVAL);
    ZL_CHECK_ARG(rot_dims >= 0 && rot_dims <= dim && rot_dims % 2 == 0 && (rot_dims == 0 || qk_freq) && (!v_freq || vdim % 2 == 0), ZL_ESHAPE);
    ZL_CHECK_ARG(dim <= 64 * kMaxE && vdim <= 64 * kMaxE, ZL_ELIMIT);
    ZL_CHECK_ARG(q_col0 >= 0 && q_col0 + heads * dim <= ld, ZL_ESHAPE);
    ZL_CHECK_ARG(!k_cache || (k_col0 >= 0 && k_col0 + kv_heads * dim <= ld && v_col0 >= 0 && v_col0 + kv_heads * vdim <= ld), ZL_ESHAPE);
    RopeP p;
    p.proj = proj; p.ld = ld; p.q_col0 = (int)q_col0; p.k_col0 = (int)k_col0; p.v_col0 = (int)v_col0; p.heads = (int)heads;
    p.kv_heads = (int)kv_heads; p.dim = (int)dim; p.vdim = (int)vdim; p.rot_dims = (int)rot_dims; p.qk_norm = qk_norm; p.qk_freq = qk_freq;
    p.v_freq = v_freq; p.eps = eps; p.k_cache = k_cache; p.v_cache = v_cache;
#define CALL(DT) hipLaunchKernelGGL((k_rope_norm_store<DT>), dim3(b->n_tok), dim3(256), 0, (hipStream_t)s, p, *b);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}

extern "C" int zls_window_attention(const float* q, int64_t ldq, int64_t q_col0, const void* k_cache, const void* v_cache, const zls_batch_t* b,
                                    float scale, int64_t window, int64_t heads, int64_t kv_heads, int64_t dim, int64_t vdim, int all_kv, float* acc,
                                    int dtype, zl_stream_t s) {
    ZL_CHECK_ARG(q && k_cache && v_cache && acc && seq_batch_ok(b) && b->page_table && b->page_size > 0, ZL_EINVAL);
    ZL_CHECK_ARG(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && vdim > 0 && heads <= 65535, ZL_ESHAPE);
    ZL_CHECK_ARG(q_col0 >= 0 && q_col0 + heads * dim <= ldq && window < (1 << 30), ZL_ESHAPE);
    ZL_CHECK_ARG((all_kv ? kv_heads : 1) * vdim <= 256 * kMaxV && dim <= 8192, ZL_ELIMIT);
    AttnP p;
    p.q = q; p.ldq = ldq; p.q_col0 = (int)q_col0; p.k_cache = k_cache; p.v_cache = v_cache; p.scale = scale; p.window = (int)window;
    p.heads = (int)heads; p.kv_heads = (int)kv_heads; p.dim = (int)dim; p.vdim = (int)vdim; p.all_kv = all_kv ? 1 : 0; p.acc = acc;
    const size_t lds = (size_t)dim * sizeof(float);
#define CALL(DT) hipLaunchKernelGGL((k_window_attention<DT>), dim3(b->n_tok, (unsigned)heads), dim3(256), lds, (hipStream_t)s, p, *b);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}

extern "C" int zls_head_mix_gate(const float* acc, const float* talk, const float* v_freq, const float* gate, int64_t ldg, int64_t g_col0,
                                 const zls_batch_t* b, int64_t heads, int64_t kv_heads, int64_t vdim, void* out, int dtype, zl_stream_t s) {
    ZL_CHECK_ARG(acc && out && seq_batch_ok(b) && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && vdim > 0, ZL_EINVAL);
    ZL_CHECK_ARG((!v_freq || vdim % 2 == 0) && (!gate || (g_col0 >= 0 && g_col0 + heads * vdim <= ldg)), ZL_ESHAPE);
    MixP p;
    p.acc = acc; p.talk = talk; p.v_freq = v_freq; p.gate = gate; p.ldg = ldg; p.g_col0 = (int)g_col0; p.heads = (int)heads;
    p.kv_heads = (int)kv_heads; p.vdim = (int)vdim; p.out = out;
#define CALL(DT) hipLaunchKernelGGL((k_head_mix_gate<DT>), dim3(b->n_tok), dim3(256), 0, (hipStream_t)s, p, *b);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}
