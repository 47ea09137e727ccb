// ssm.hip -- the state-space (Mamba-2) mixer's steps over a ragged step: causal short convolution + SiLU with a carried tail, the
// selective recurrence with its fp32 state carried per sequence slot, the gated grouped RMS norm.
//
// k_conv_silu         a thread per (token, channel); taps before the portion come from the slot's tail (oldest row first)
// k_conv_tail_update  after it: a thread per (sequence, channel) shifts the tail by the portion's length (rows in increasing order, each
//                     read before it is overwritten)
// k_ssm_scan          a workgroup per (sequence, head), vdim x NG threads: thread (p, g) keeps S[n][p] for n = g, g + NG, ... in registers
//                     (<= 16), walks the portion's tokens in order; y_p is reduced over g through LDS.  dt, the decay and the state are fp32.
// k_gated_group_norm  y * silu(z), then each of the row's equal parts divided by its own root mean square, times the weight
#include "seq_common.h"

namespace {

__global__ __launch_bounds__(256) void k_conv_silu(const float* __restrict__ proj, int64_t ld, int col0, const float* __restrict__ w,
                                                   const float* __restrict__ bias, const float* __restrict__ tail, int channels, int taps,
                                                   const zls_batch_t b, float* __restrict__ out) {
    const int t = blockIdx.x;
    const int sq = b.tok_seq[t];
    const int first = b.seq_start[sq];
    const int i = t - first;                                           // index inside the portion
    const float* tl = tail + (size_t)b.seq_slot[sq] * (taps - 1) * channels;
    for (int c = blockIdx.y * 256 + threadIdx.x; c < channels; c += gridDim.y * 256) {
        float a = bias ? bias[c] : 0.f;
        for (int k = 0; k < taps; ++k) {
            const int back = taps - 1 - k;                             // the last column is the current token's
            const int src = i - back;
            const float u = src >= 0 ? proj[(size_t)(first + src) * ld + col0 + c]
                                     : tl[(size_t)(taps - 1 + src) * channels + c];     // src = -1 is the newest tail row
            a = fmaf(w[(size_t)c * taps + k], u, a);
        }
        out[(size_t)t * channels + c] = seq_silu(a);
    }
}

__global__ __launch_bounds__(256) void k_conv_tail_update(const float* __restrict__ proj, int64_t ld, int col0, float* __restrict__ tail,
                                                          int channels, int taps, const zls_batch_t b) {
    const int sq = blockIdx.x;
    const int first = b.seq_start[sq], count = b.seq_start[sq + 1] - first;
    float* tl = tail + (size_t)b.seq_slot[sq] * (taps - 1) * channels;
    for (int c = blockIdx.y * 256 + threadIdx.x; c < channels; c += gridDim.y * 256) {
        for (int j = 0; j < taps - 1; ++j) {                           // new row j = input at portion index count - (taps - 1) + j
            const int src = count - (taps - 1) + j;
            tl[(size_t)j * channels + c] = src >= 0 ? proj[(size_t)(first + src) * ld + col0 + c]
                                                    : tl[(size_t)(taps - 1 + src) * channels + c];   // an older row j + count > j
        }
    }
}

struct ScanP {
    const float* xbc; const float* proj; const float* dt_bias; const float* a_log; const float* d; float* state; float* y;
    int64_t ld;
    int dt_col0, heads, vdim, n_state, groups, ng;
};

constexpr int kNPT = 16;

__global__ __launch_bounds__(1024) void k_ssm_scan(const ScanP p, const zls_batch_t b) {
    extern __shared__ float red[];                                     // [ng][vdim]
    const int sq = blockIdx.x, h = blockIdx.y;
    const int P = p.vdim, N = p.n_state, NG = p.ng;
    const int pp = threadIdx.x % P, g = threadIdx.x / P;
    const int grp = h / (p.heads / p.groups);
    const int inner = p.heads * P, chan = inner + 2 * p.groups * N;
    const int first = b.seq_start[sq], count = b.seq_start[sq + 1] - first;
    float* st = p.state + ((size_t)b.seq_slot[sq] * p.heads + h) * N * P;
    float S[kNPT];
#pragma unroll
    for (int i = 0; i < kNPT; ++i) {
        const int n = g + i * NG;
        S[i] = n < N ? st[(size_t)n * P + pp] : 0.f;
    }
    const float rate = expf(p.a_log[h]), bias = p.dt_bias[h], dskip = p.d[h];
    for (int i = 0; i < count; ++i) {
        const size_t t = (size_t)(first + i);
        const float* row = p.xbc + t * chan;
        const float dt = seq_softplus(p.proj[t * p.ld + p.dt_col0 + h] + bias);
        const float decay = expf(-rate * dt);
        const float xv = row[h * P + pp];
        const float* Bv = row + inner + grp * N;
        const float* Cv = Bv + p.groups * N;
        const float dx = dt * xv;
        float part = 0.f;
#pragma unroll
        for (int j = 0; j < kNPT; ++j) {
            const int n = g + j * NG;
            if (n < N) {
                S[j] = fmaf(decay, S[j], Bv[n] * dx);
                part = fmaf(S[j], Cv[n], part);
            }
        }
        red[g * P + pp] = part;
        __syncthreads();
        if (g == 0) {
            float yv = 0.f;
            for (int q = 0; q < NG; ++q) yv += red[q * P + pp];
            p.y[t * inner + h * P + pp] = fmaf(dskip, xv, yv);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < kNPT; ++i) {
        const int n = g + i * NG;
        if (n < N) st[(size_t)n * P + pp] = S[i];
    }
}

template <int DT>
__global__ __launch_bounds__(256) void k_gated_group_norm(const float* __restrict__ y, const float* __restrict__ proj, int64_t ld, int z_col0,
                                                          const float* __restrict__ weight, float eps, int inner, int part,
                                                          void* __restrict__ out) {
    __shared__ float red[16];
    const int t = blockIdx.x, c0 = blockIdx.y * part;
    const float* yr = y + (size_t)t * inner + c0;
    const float* zr = proj + (size_t)t * ld + z_col0 + c0;
    float ss = 0.f;
    for (int i = threadIdx.x; i < part; i += 256) { const float v = yr[i] * seq_silu(zr[i]); ss = fmaf(v, v, ss); }
    ss = zl_block_sum(ss, red);
    const float f = 1.0f / sqrtf(ss / (float)part + eps);
    for (int i = threadIdx.x; i < part; i += 256)
        SeqT<DT>::st(out, (size_t)t * inner + c0 + i, yr[i] * seq_silu(zr[i]) * f * weight[c0 + i]);
}

}  // namespace

extern "C" int zls_conv_silu(const float* proj, int64_t ld, int64_t col0, const float* w, const float* bias, const float* tail, int64_t channels,
                             int64_t taps, const zls_batch_t* b, float* out, zl_stream_t s) {
    ZL_CHECK_ARG(proj && w && out && seq_batch_ok(b) && channels > 0 && taps > 0 && (tail || taps == 1), ZL_EINVAL);
    ZL_CHECK_ARG(col0 >= 0 && col0 + channels <= ld, ZL_ESHAPE);
    const unsigned gy = (unsigned)((channels + 255) / 256 > 64 ? 64 : (channels + 255) / 256);
    hipLaunchKernelGGL(k_conv_silu, dim3(b->n_tok, gy), dim3(256), 0, (hipStream_t)s, proj, ld, (int)col0, w, bias, tail, (int)channels, (int)taps, *b, out);
    return zl_launch_status();
}

extern "C" int zls_conv_tail_update(const float* proj, int64_t ld, int64_t col0, float* tail, int64_t channels, int64_t taps, const zls_batch_t* b,
                                    zl_stream_t s) {
    ZL_CHECK_ARG(proj && seq_batch_ok(b) && channels > 0 && taps > 0, ZL_EINVAL);
    ZL_CHECK_ARG(col0 >= 0 && col0 + channels <= ld, ZL_ESHAPE);
    if (taps == 1) return ZL_OK;
    ZL_CHECK_ARG(tail, ZL_EINVAL);
    const unsigned gy = (unsigned)((channels + 255) / 256 > 64 ? 64 : (channels + 255) / 256);
    hipLaunchKernelGGL(k_conv_tail_update, dim3(b->n_seq, gy), dim3(256), 0, (hipStream_t)s, proj, ld, (int)col0, tail, (int)channels, (int)taps, *b);
    return zl_launch_status();
}

extern "C" int zls_ssm_scan(const float* xbc, const float* proj, int64_t ld, int64_t dt_col0, const float* dt_bias, const float* a_log,
                            const float* d, float* state, int64_t heads, int64_t vdim, int64_t n_state, int64_t groups, const zls_batch_t* b,
                            float* y, zl_stream_t s) {
    ZL_CHECK_ARG(xbc && proj && dt_bias && a_log && d && state && y && seq_batch_ok(b), ZL_EINVAL);
    ZL_CHECK_ARG(heads > 0 && vdim > 0 && n_state > 0 && groups > 0 && heads % groups == 0 && heads <= 65535, ZL_ESHAPE);
    ZL_CHECK_ARG(dt_col0 >= 0 && dt_col0 + heads <= ld && vdim <= 1024, ZL_ESHAPE);
    // NG thread rows: enough that a thread keeps at most kNPT state values, and at least 4 waves when the head is small
    int64_t ng = (n_state + kNPT - 1) / kNPT;
    while (ng * vdim < 256 && ng < n_state) ++ng;
    ZL_CHECK_ARG(ng * vdim <= 1024, ZL_ELIMIT);
    ScanP p;
    p.xbc = xbc; p.proj = proj; p.dt_bias = dt_bias; p.a_log = a_log; p.d = d; p.state = state; p.y = y; p.ld = ld;
    p.dt_col0 = (int)dt_col0; p.heads = (int)heads; p.vdim = (int)vdim; p.n_state = (int)n_state; p.groups = (int)groups; p.ng = (int)ng;
    hipLaunchKernelGGL(k_ssm_scan, dim3(b->n_seq, (unsigned)heads), dim3((unsigned)(ng * vdim)), (size_t)(ng * vdim) * sizeof(float),
                       (hipStream_t)s, p, *b);
    return zl_launch_status();
}

extern "C" int zls_gated_group_norm(const float* y, const float* proj, int64_t ld, int64_t z_col0, const float* weight, float eps, int64_t rows,
                                    int64_t inner, int64_t norm_groups, void* out, int dtype, zl_stream_t s) {
    ZL_CHECK_ARG(y && proj && weight && out && rows > 0 && inner > 0 && norm_groups > 0, ZL_EINVAL);
    ZL_CHECK_ARG(inner % norm_groups == 0 && z_col0 >= 0 && z_col0 + inner <= ld && norm_groups <= 65535, ZL_ESHAPE);
    const int part = (int)(inner / norm_groups);
#define CALL(DT) hipLaunchKernelGGL((k_gated_group_norm<DT>), dim3((unsigned)rows, (unsigned)norm_groups), dim3(256), 0, (hipStream_t)s, y, proj, ld, \
                                    (int)z_col0, weight, eps, (int)inner, part, out);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}
