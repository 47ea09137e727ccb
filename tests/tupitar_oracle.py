"""Plain, slow restatement of the Tupitar design in float64 on the CPU: what the product path (zhilight_amd/seqmix.py, engine.py and the
kernels of csrc_seq/) is held against.  One function per mechanism, whole sequences only, no cache, no batching, nothing shared with the
product code.  Weights are a dict name -> torch tensor with the checkpoint's own tensor names.

Notation: t indexes tokens of one sequence (positions from 0), rms(u) = sqrt(mean(u^2) + eps) over the last axis.
"""
import math

import torch

F64 = torch.float64


def w64(sd, name):
    return sd[name].to(F64)


def unit_rms(u, eps):
    return u / torch.sqrt((u * u).mean(dim=-1, keepdim=True) + eps)


def scalar_norm(u, gain, eps):
    """u / rms(u) * gain with ONE gain for all coordinates."""
    return unit_rms(u, eps) * gain.to(F64).reshape(())


def token_shift(h, mix):
    """h_t + (h_{t-1} - h_t) * mix, with h_{-1} = 0; the previous token's h is taken before the replacement."""
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]], dim=0)
    return h + (prev - h) * mix.to(F64)


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z / (1 + torch.exp(-z))


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30))))


def causal_conv(u, w, b):
    """u (T, C); w (C, taps), the LAST column multiplies the current token; zeros before the start."""
    T, C = u.shape
    taps = w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=F64), u], dim=0)
    out = b.to(F64).expand(T, C).clone()
    for k in range(taps):
        out = out + pad[k:k + T] * w[:, k].to(F64)
    return out


def mamba2_mixer(h, sd, pfx, m, eps):
    """State-space mixer; m = the layer's "mixer" entry of the configuration."""
    H, P, N, G, R = m["heads"], m["vdim"], m["state"], m["groups"], m["norm_groups"]
    inner = H * P
    T = h.shape[0]
    proj = h @ w64(sd, pfx + "in").T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    assert dt.shape[1] == H
    xbc = silu(causal_conv(xbc, sd[pfx + "conv"], sd[pfx + "conv.b"]))
    x = xbc[:, :inner].reshape(T, H, P)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    Cm = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + w64(sd, pfx + "dt_bias"))
    rate = torch.exp(w64(sd, pfx + "A_log"))
    D = w64(sd, pfx + "D")
    S = torch.zeros(H, N, P, dtype=F64)
    y = torch.zeros(T, H, P, dtype=F64)
    per = H // G
    for t in range(T):
        for hd in range(H):
            g = hd // per
            S[hd] = torch.exp(-rate[hd] * dt[t, hd]) * S[hd] + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S[hd].T @ Cm[t, g] + D[hd] * x[t, hd]
    y = y.reshape(T, inner) * silu(z)
    y = unit_rms(y.reshape(T, R, inner // R), eps).reshape(T, inner) * w64(sd, pfx + "norm")
    return y @ w64(sd, pfx + "o").T


def latent_attention_mixer(h, sd, pfx, m, eps):
    """Attention over an RMS-normed low-rank latent, no positions, a per-head sink in the softmax denominator, a per-head sigmoid
    output gate."""
    H, dq, dv, scale = m["heads"], m["dim"], m["vdim"], m["scale"]
    T = h.shape[0]
    q = (h @ w64(sd, pfx + "q").T).reshape(T, H, dq)
    c = unit_rms(h @ w64(sd, pfx + "dkv").T, eps) * w64(sd, pfx + "dkv.norm")
    k = (c @ w64(sd, pfx + "uk").T).reshape(T, H, dq)
    v = (c @ w64(sd, pfx + "uv").T).reshape(T, H, dv)
    gate = torch.sigmoid(h @ w64(sd, pfx + "g").T)             # (T, H)
    sink = w64(sd, pfx + "sink")
    out = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        s = (q[:, hd] @ k[:, hd].T) * scale                     # (T query, T key)
        s = s.masked_fill(torch.ones(T, T, dtype=torch.bool).triu(1), -math.inf)
        mx = torch.maximum(s.max(dim=1, keepdim=True).values, sink[hd])
        e = torch.exp(s - mx)
        den = e.sum(dim=1, keepdim=True) + torch.exp(sink[hd] - mx)
        out[:, hd] = (e / den) @ v[:, hd] * gate[:, hd:hd + 1]
    return out.reshape(T, H * dv) @ w64(sd, pfx + "o").T


def polynorm(z, coef, eps):
    """a N(z) + b N(z^2) + c N(z^3) + e, N = division of the token's vector by its rms."""
    a, b, c, e = coef.to(F64)
    return a * unit_rms(z, eps) + b * unit_rms(z * z, eps) + c * unit_rms(z * z * z, eps) + e


def dense_ff(h, sd, pfx, eps):
    return polynorm(h @ w64(sd, pfx + "up").T, sd[pfx + "act"], eps) @ w64(sd, pfx + "down").T


MIXERS = {"mamba2": mamba2_mixer, "latent_attention": latent_attention_mixer}


def forward(cfg, sd, tokens, return_layers=False):
    """Logits (T, vocab) float64 of one whole sequence; optionally the residual stream after every layer."""
    eps = cfg["norm"]["eps"]
    tok = torch.as_tensor(tokens, dtype=torch.long)
    T = tok.numel()
    x = w64(sd, "embed")[tok] * cfg["embedding"]["scale"] + w64(sd, "pos")[:T]
    layers = []
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = token_shift(x, sd[p + "shift"])
        x = x + scalar_norm(MIXERS[L["type"]](h, sd, p + "mix.", L["mixer"], eps), sd[p + "norm1"], eps)
        if L.get("mlp") is not None:
            assert L["mlp"]["kind"] == "dense"
            x = x + scalar_norm(dense_ff(x, sd, p + "mlp.", eps), sd[p + "norm2"], eps)
        layers.append(x.clone())
    logits = scalar_norm(x, sd["final.norm"], eps) @ w64(sd, "head").T
    return (logits, torch.stack(layers)) if return_layers else logits


def random_weights(cfg, seed=0, dtype=torch.bfloat16):
    """Random checkpoint of a configuration, magnitudes chosen so that every mechanism matters in the logits."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def rn(*shape, s=1.0):
        return (torch.randn(*shape, generator=g) * s).to(dtype)
    sd = {"embed": rn(cfg["vocab"], W, s=1.0 / cfg["embedding"]["scale"]), "pos": rn(cfg["max_positions"], W, s=0.3),
          "final.norm": (1 + 0.1 * torch.randn((), generator=g)).to(dtype), "head": rn(cfg["vocab"], W, s=W ** -0.5)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        sd[p + "norm1"] = (1 + 0.2 * torch.randn((), generator=g)).to(dtype)
        sd[p + "shift"] = torch.rand(W, generator=g).to(dtype)
        if L["type"] == "mamba2":
            inner, gn = m["heads"] * m["vdim"], m["groups"] * m["state"]
            sd[p + "mix.in"] = rn(2 * inner + 2 * gn + m["heads"], W, s=W ** -0.5)
            sd[p + "mix.conv"] = rn(inner + 2 * gn, m["conv"], s=0.5)
            sd[p + "mix.conv.b"] = rn(inner + 2 * gn, s=0.2)
            sd[p + "mix.dt_bias"] = rn(m["heads"], s=1.0)
            sd[p + "mix.A_log"] = (torch.rand(m["heads"], generator=g) * 3 - 3).to(dtype)
            sd[p + "mix.D"] = rn(m["heads"], s=1.0)
            sd[p + "mix.norm"] = (1 + 0.2 * torch.randn(inner, generator=g)).to(dtype)
            sd[p + "mix.o"] = rn(W, inner, s=inner ** -0.5)
        else:
            H, dq, dv, r = m["heads"], m["dim"], m["vdim"], m["kv_rank"]
            sd[p + "mix.q"] = rn(H * dq, W, s=2 * W ** -0.5)
            sd[p + "mix.dkv"] = rn(r, W, s=W ** -0.5)
            sd[p + "mix.dkv.norm"] = (1 + 0.2 * torch.randn(r, generator=g)).to(dtype)
            sd[p + "mix.uk"] = rn(H * dq, r, s=2 * r ** -0.5)
            sd[p + "mix.uv"] = rn(H * dv, r, s=r ** -0.5)
            sd[p + "mix.sink"] = rn(H, s=1.5)
            sd[p + "mix.g"] = rn(H, W, s=W ** -0.5)
            sd[p + "mix.o"] = rn(W, H * dv, s=(H * dv) ** -0.5)
        if L.get("mlp") is not None:
            ff = L["mlp"]["ff"]
            sd[p + "norm2"] = (1 + 0.2 * torch.randn((), generator=g)).to(dtype)
            sd[p + "mlp.up"] = rn(ff, W, s=W ** -0.5)
            sd[p + "mlp.down"] = rn(W, ff, s=ff ** -0.5)
            sd[p + "mlp.act"] = torch.tensor([1.0, 0.5, 0.25, 0.1]).to(dtype) + rn(4, s=0.1)
    return sd


def small_config(order=("latent_attention", "mamba2", "latent_attention"), width=96, vocab=160, seed_sizes=0, no_mlp_at=()):
    """A small configuration of the design with sizes unlike any shipped model (heads != groups, norm_groups > 1, dim != vdim)."""
    layers = []
    for i, t in enumerate(order):
        if t == "mamba2":
            mixer = {"conv": 3 + (i + seed_sizes) % 3, "groups": 2, "heads": 4, "norm_groups": 1 + (i + seed_sizes) % 2 * 3, "state": 24,
                     "vdim": 16}
        else:
            mixer = {"dim": 16, "heads": 3 + (i + seed_sizes) % 3, "kv_rank": 40, "scale": 0.31, "vdim": 24}
        layers.append({"type": t, "mixer": mixer, "mlp": None if i in no_mlp_at else {"ff": 136, "kind": "dense"}})
    return {"architecture": "Tupitar", "embedding": {"scale": 7.5}, "layers": layers, "max_positions": 512, "norm": {"eps": 1e-5},
            "vocab": vocab, "width": width}
