"""Sequence mixers and feed-forwards for ragged steps: each is a weight container + the kernel sequence of its forward, with every
constant a constructor argument, so that a model description picks and sizes them (tupitar.py does; another design can).

A mixer's forward takes h (n_tok, width) in the serving format and the step's RaggedBatch and returns fp32 (n_tok, width).  What it keeps
between steps it registers with the CacheManager in `bind`: per-token rows as a paged plane, per-sequence state as a slot state.
All per-sequence arithmetic that must not lose bits (norms, softmax, the recurrence, its state) is fp32 inside the kernels in both serving
formats; matrices are in the serving format, small vectors fp32.
"""
import math

import torch

from . import seqops
from ._lib import ZLError


def _mat(get, name, shape, dtype, device):
    t = get(name)
    if tuple(t.shape) != tuple(shape):
        raise ZLError(f"tensor {name}: shape {tuple(t.shape)}, expected {tuple(shape)}")
    return t.to(device=device, dtype=dtype).contiguous()


def _vec(get, name, n, device):
    t = get(name)
    if t.numel() != n:
        raise ZLError(f"tensor {name}: {t.numel()} values, expected {n}")
    return t.to(device=device, dtype=torch.float32).reshape(n).contiguous()


def _rand(gen, shape, std, dtype, device):
    return (torch.randn(shape, generator=gen, device=device, dtype=torch.float32) * std).to(dtype)


class LatentAttention:
    """Causal attention whose keys and values are up-projections of a cached, RMS-normed low-rank latent (no positional rotation); optional
    learned per-head sink in the softmax denominator and per-head sigmoid output gate.
    Tensors under `prefix`: q (heads*dim, width), dkv (rank, width), dkv.norm (rank), uk (heads*dim, rank), uv (heads*vdim, rank),
    sink (heads), g (heads, width), o (width, heads*vdim).  q | dkv | g are fused into one product."""

    def __init__(self, name, width, heads, dim, vdim, rank, scale, eps, sink=True, gate=True):
        self.name, self.width, self.heads, self.dim, self.vdim, self.rank = name, width, heads, dim, vdim, rank
        self.scale, self.eps, self.has_sink, self.has_gate = float(scale), float(eps), sink, gate
        self.cache = None
        self.prompt_kernel = True         # bf16 portions on the matrix-core kernel (False: everything on the latent-space kernel)
        self.decode_mfma = True           # bf16 single tokens: the split pass on the matrix cores (False: the fp32 VALU kernel)

    def load(self, get, prefix, dtype, device):
        H, d, v, r, W = self.heads, self.dim, self.vdim, self.rank, self.width
        parts = [_mat(get, prefix + "q", (H * d, W), dtype, device), _mat(get, prefix + "dkv", (r, W), dtype, device)]
        if self.has_gate:
            parts.append(_mat(get, prefix + "g", (H, W), dtype, device))
        self.w_in = torch.cat(parts, dim=0).contiguous()
        self.dkv_norm = _vec(get, prefix + "dkv.norm", r, device)
        self.w_uk = _mat(get, prefix + "uk", (H * d, r), dtype, device)
        self.w_uv = _mat(get, prefix + "uv", (H * v, r), dtype, device)
        self.sink = _vec(get, prefix + "sink", H, device) if self.has_sink else None
        self.w_o = _mat(get, prefix + "o", (W, H * v), dtype, device)
        return self

    def init_random(self, gen, dtype, device):
        H, d, v, r, W = self.heads, self.dim, self.vdim, self.rank, self.width
        self.w_in = _rand(gen, (H * d + r + (H if self.has_gate else 0), W), W ** -0.5, dtype, device)
        self.dkv_norm = torch.ones(r, device=device)
        self.w_uk = _rand(gen, (H * d, r), r ** -0.5, dtype, device)
        self.w_uv = _rand(gen, (H * v, r), r ** -0.5, dtype, device)
        self.sink = torch.zeros(H, device=device) if self.has_sink else None
        self.w_o = _rand(gen, (W, H * v), (H * v) ** -0.5, dtype, device)
        return self

    def bind(self, cache, dtype):
        self.cache = cache.add_plane(self.name + ".latent", (self.rank,), dtype)

    def weight_bytes(self):
        return sum(t.numel() * t.element_size() for t in (self.w_in, self.w_uk, self.w_uv, self.w_o))

    def forward(self, h, batch):
        H, d, r = self.heads, self.dim, self.rank
        proj = seqops.gemm_nt(h, self.w_in)                                       # fp32 [q | latent | gate]
        seqops.latent_store(proj, H * d, self.dkv_norm, self.eps, r, batch, self.cache)
        gate = proj if self.has_gate else None
        prompt = batch.n_ctx > 0 and self.prompt_kernel and h.dtype == torch.bfloat16 and max(d, self.vdim) <= 256
        a = torch.empty((batch.n_tok, H * self.vdim), dtype=h.dtype, device=h.device)
        if prompt:
            # portions: keys and values of their contexts up-projected once (K = C W_uk^T, V^T = W_uv C^T, gathered from the pages), then
            # the matrix-core kernel; single tokens stay on the latent-space kernel below
            flat = self.cache.view(-1, r)
            k = torch.empty((batch.n_ctx, H * d), dtype=h.dtype, device=h.device)
            vt = torch.empty((H * self.vdim, batch.n_ctx), dtype=h.dtype, device=h.device)
            seqops.gemm_nt_gather(flat, batch.ctx_rows, self.w_uk, None, batch.n_ctx, H * d, k)
            seqops.gemm_nt_gather(self.w_uv, None, flat, batch.ctx_rows, H * self.vdim, batch.n_ctx, vt)
            seqops.latent_attention_prompt(proj, 0, gate, H * d + r, k, vt, self.sink, batch, self.scale, H, d, self.vdim, a)
        if not prompt or batch.n_single:
            seqops.latent_attention(proj, 0, gate, H * d + r, self.w_uk, self.w_uv, self.sink, self.cache, batch, self.scale, H, d, self.vdim,
                                    out=a, single_only=prompt, mfma=self.decode_mfma)
        return seqops.gemm_nt(a, self.w_o)


class Mamba2Mixer:
    """Selective state-space mixer (scalar decay per head, state n_state x vdim per head, B / C shared by the heads of a group), with the
    causal short convolution over x | B | C, the skip term, and the gated grouped RMS norm before the output projection.
    Tensors under `prefix`: in (2*inner + 2*groups*n_state + heads, width) laid out [z | x | B | C | dt], conv (channels, taps), conv.b,
    dt_bias, A_log, D (heads each), norm (inner), o (width, inner)."""

    def __init__(self, name, width, heads, vdim, n_state, groups, taps, norm_groups, eps):
        if heads % groups or (heads * vdim) % norm_groups:
            raise ZLError("mamba2: heads must divide by groups, heads * vdim by norm_groups")
        self.name, self.width, self.heads, self.vdim, self.n_state, self.groups = name, width, heads, vdim, n_state, groups
        self.taps, self.norm_groups, self.eps = taps, norm_groups, float(eps)
        self.inner = heads * vdim
        self.channels = self.inner + 2 * groups * n_state
        self.scan_segment = None          # tokens per segment of a long portion (None: seqops.SCAN_SEGMENT; 0: never in segments)

    def load(self, get, prefix, dtype, device):
        W = self.width
        self.w_in = _mat(get, prefix + "in", (self.inner + self.channels + self.heads, W), dtype, device)
        self.conv_w = _mat(get, prefix + "conv", (self.channels, self.taps), torch.float32, device)
        self.conv_b = _vec(get, prefix + "conv.b", self.channels, device)
        self.dt_bias = _vec(get, prefix + "dt_bias", self.heads, device)
        self.a_log = _vec(get, prefix + "A_log", self.heads, device)
        self.d = _vec(get, prefix + "D", self.heads, device)
        self.norm_w = _vec(get, prefix + "norm", self.inner, device)
        self.w_o = _mat(get, prefix + "o", (W, self.inner), dtype, device)
        return self

    def init_random(self, gen, dtype, device):
        W = self.width
        self.w_in = _rand(gen, (self.inner + self.channels + self.heads, W), W ** -0.5, dtype, device)
        self.conv_w = _rand(gen, (self.channels, self.taps), 0.5, torch.float32, device)
        self.conv_b = torch.zeros(self.channels, device=device)
        self.dt_bias = torch.zeros(self.heads, device=device)
        self.a_log = torch.zeros(self.heads, device=device)
        self.d = torch.ones(self.heads, device=device)
        self.norm_w = torch.ones(self.inner, device=device)
        self.w_o = _rand(gen, (W, self.inner), self.inner ** -0.5, dtype, device)
        return self

    def bind(self, cache, dtype):
        self.tail = cache.add_state(self.name + ".conv", (self.taps - 1, self.channels)) if self.taps > 1 else None
        self.state = cache.add_state(self.name + ".ssm", (self.heads, self.n_state, self.vdim))

    def weight_bytes(self):
        return sum(t.numel() * t.element_size() for t in (self.w_in, self.w_o))

    def forward(self, h, batch):
        proj = seqops.gemm_nt(h, self.w_in)                                       # fp32 [z | x | B | C | dt]
        xbc = seqops.conv_silu(proj, self.inner, self.conv_w, self.conv_b, self.tail, batch)
        y = seqops.ssm_scan(xbc, proj, self.inner + self.channels, self.dt_bias, self.a_log, self.d, self.state, self.heads, self.vdim,
                            self.n_state, self.groups, batch, seg_len=self.scan_segment)
        g = seqops.gated_group_norm(y, proj, 0, self.norm_w, self.eps, self.norm_groups, h.dtype)
        return seqops.gemm_nt(g, self.w_o)


class PolyNormFF:
    """Dense feed-forward down(act(up h)) with the PolyNorm activation: a N(z) + b N(z^2) + c N(z^3) + e, N = division by the row's root
    mean square.  Tensors: up (ff, width), down (width, ff), act (4: a, b, c, e)."""

    def __init__(self, width, ff, eps):
        self.width, self.ff, self.eps = width, ff, float(eps)

    def load(self, get, prefix, dtype, device):
        self.w_up = _mat(get, prefix + "up", (self.ff, self.width), dtype, device)
        self.w_down = _mat(get, prefix + "down", (self.width, self.ff), dtype, device)
        self.coef = [float(v) for v in get(prefix + "act").to(torch.float32).reshape(4)]
        return self

    def init_random(self, gen, dtype, device):
        self.w_up = _rand(gen, (self.ff, self.width), self.width ** -0.5, dtype, device)
        self.w_down = _rand(gen, (self.width, self.ff), self.ff ** -0.5, dtype, device)
        self.coef = [1.0, 0.5, 0.25, 0.0]
        return self

    def weight_bytes(self):
        return sum(t.numel() * t.element_size() for t in (self.w_up, self.w_down))

    def forward(self, h):
        z = seqops.gemm_nt(h, self.w_up)
        return seqops.gemm_nt(seqops.polynorm(z, self.coef, self.eps, h.dtype), self.w_down)
