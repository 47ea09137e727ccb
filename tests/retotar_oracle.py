"""Plain, slow restatement of the Retotar design in float64 on the CPU: what the product path (zhilight_amd/retotar.py, mixers.py,
engine.py and the kernels of csrc_seq/) is held against.  One function per mechanism, whole sequences only, no cache, no batching,
nothing shared with the product code.  Weights are a dict name -> torch tensor with the checkpoint's own tensor names; `m` is a layer's
"mixer" entry of the configuration, `f` its "mlp" entry.

Notation: t, s index tokens of one sequence (positions from 0); rms(u) = sqrt(mean(u^2) + eps) over the last axis.
"""
import math

import torch

F64 = torch.float64


def w64(sd, name):
    return sd[name].to(F64)


def unit_rms(u, eps):
    return u / torch.sqrt((u * u).mean(dim=-1, keepdim=True) + eps)


def layer_norm(u, sd, name, eps):
    """(u - mean) / sqrt(var + eps) * w + b, var = mean of squared deviations; the bias is the tensor name + '.b'"""
    mu = u.mean(dim=-1, keepdim=True)
    var = ((u - mu) ** 2).mean(dim=-1, keepdim=True)
    return (u - mu) / torch.sqrt(var + eps) * w64(sd, name) + w64(sd, name + ".b")


def silu(z):
    return z / (1 + torch.exp(-z))


def sigmoid(z):
    return 1 / (1 + torch.exp(-z))


def log_sigmoid(z):
    return -torch.log1p(torch.exp(-z.abs())) + torch.minimum(z, torch.zeros_like(z))


# ---- rotations ---------------------------------------------------------------------------------------------------------------------
def rotate_halves(u, pos, n_rot, base, divide=1.0, sign=1.0):
    """u (T, heads, size): coordinate i < n_rot/2 is paired with i + n_rot/2 and the pair turned by sign * pos * base^(-2i/n_rot) / divide;
    coordinates from n_rot on are left alone."""
    half = n_rot // 2
    i = torch.arange(half, dtype=F64)
    freq = base ** (-2 * i / n_rot) / divide
    ang = sign * pos.to(F64)[:, None] * freq[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = u[..., :half], u[..., half:n_rot]
    out = u.clone()
    out[..., :half] = a * c - b * s
    out[..., half:n_rot] = b * c + a * s
    return out


# ---- softmax attention with a window, mixed heads, turned values -----------------------------------------------------------------------
def attention_kv(h, sd, pfx, m, eps):
    """what the layer caches: keys after rotation and unit-RMS norm, values turned by their own position"""
    T = h.shape[0]
    G, d, v = m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    k = (h @ w64(sd, pfx + "k").T).reshape(T, G, d)
    k = unit_rms(rotate_halves(k, pos, m["rot"]["dims"], m["rot"]["base"], m["rot"]["scaling"]["factor"]), eps)
    val = (h @ w64(sd, pfx + "v").T).reshape(T, G, v)
    val = rotate_halves(val, pos, v, m["rot"]["base"])
    return k, val


def attention_mixer(h, sd, pfx, m, eps, kv=None):
    """kv: (keys, values) of the layer this one borrows them from (None: its own projections)"""
    T = h.shape[0]
    H, G, d, v = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = (h @ w64(sd, pfx + "q").T).reshape(T, H, d)
    q = unit_rms(rotate_halves(q, pos, m["rot"]["dims"], m["rot"]["base"], m["rot"]["scaling"]["factor"]), eps)
    k, val = kv if kv is not None else attention_kv(h, sd, pfx, m, eps)
    per = H // G
    diff = pos[:, None] - pos[None, :]
    visible = (diff >= 0) & (diff < m["mask"]["size"])
    weights = torch.zeros(H, T, T, dtype=F64)
    for hd in range(H):
        sc = (q[:, hd] @ k[:, hd // per].T) * m["scale"]
        sc = sc.masked_fill(~visible, -math.inf)
        weights[hd] = torch.softmax(sc, dim=-1)
    mixed = torch.einsum("hg,gts->hts", w64(sd, pfx + "talk"), weights)
    out = torch.zeros(T, H, v, dtype=F64)
    for hd in range(H):
        out[:, hd] = mixed[hd] @ val[:, hd // per]
    out = rotate_halves(out, pos, v, m["rot"]["base"], sign=-1.0)
    out = out.reshape(T, H * v) * sigmoid(h @ w64(sd, pfx + "g").T)
    return out @ w64(sd, pfx + "o").T


# ---- linear attention with a fixed decay per head ----------------------------------------------------------------------------------------
def lightning_mixer(h, sd, pfx, m, eps):
    T = h.shape[0]
    H, d, v = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w64(sd, pfx + "q").T).reshape(T, H, d)
    k = silu(h @ w64(sd, pfx + "k").T).reshape(T, H, d)
    val = silu(h @ w64(sd, pfx + "v").T).reshape(T, H, v)
    decay = torch.tensor(m["decay"], dtype=F64)
    S = torch.zeros(H, d, v, dtype=F64)
    out = torch.zeros(T, H, v, dtype=F64)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * val[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    out = unit_rms(out.reshape(T, H * v), eps) * w64(sd, pfx + "norm")
    out = out * sigmoid(h @ w64(sd, pfx + "g").T)
    return out @ w64(sd, pfx + "o").T


# ---- matrix memory with exponential gates and a running maximum -------------------------------------------------------------------------
def mlstm_mixer(h, sd, pfx, m, eps):
    T = h.shape[0]
    H, d, v, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ w64(sd, pfx + "q").T).reshape(T, H, d) * d ** -0.5
    k = (h @ w64(sd, pfx + "k").T).reshape(T, H, d)
    val = (h @ w64(sd, pfx + "v").T).reshape(T, H, v)
    gi = cap * torch.tanh((h @ w64(sd, pfx + "i").T + w64(sd, pfx + "i.b")) / cap)
    gf = log_sigmoid(cap * torch.tanh((h @ w64(sd, pfx + "f").T + w64(sd, pfx + "f.b")) / cap))
    S = torch.zeros(H, d, v, dtype=F64)
    n = torch.zeros(H, d, dtype=F64)
    mx = torch.zeros(H, dtype=F64)
    out = torch.zeros(T, H, v, dtype=F64)
    for t in range(T):
        new = torch.maximum(gf[t] + mx, gi[t])
        keep, take = torch.exp(gf[t] + mx - new), torch.exp(gi[t] - new)
        S = keep[:, None, None] * S + take[:, None, None] * k[t][:, :, None] * val[t][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        mx = new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        out[t] = num / den[:, None]
    out = unit_rms(out, eps).reshape(T, H * v) * w64(sd, pfx + "norm")
    out = out * sigmoid(h @ w64(sd, pfx + "g").T)
    return out @ w64(sd, pfx + "o").T


# ---- mixture of experts ----------------------------------------------------------------------------------------------------------------
def moe_route(h, sd, pfx, f):
    """(T, top) chosen outputs of the router (ids past the real experts are identity experts) and their weights"""
    r = f["router"]
    total = r["experts"] + r.get("identity", 0)
    s = torch.softmax(h @ w64(sd, pfx + "router").T, dim=-1)
    choice = s + w64(sd, pfx + "correction")
    groups, keep = r["groups"]["count"], r["groups"]["keep"]
    size = total // groups
    gscore = choice.reshape(-1, groups, size).max(dim=-1).values
    kept = torch.topk(gscore, keep, dim=-1).indices
    allowed = torch.zeros_like(gscore, dtype=torch.bool).scatter_(1, kept, True)
    choice = choice.masked_fill(~allowed[:, :, None].expand(-1, -1, size).reshape(-1, total), -math.inf)
    ids = torch.topk(choice, r["top"], dim=-1).indices
    return ids, torch.gather(s, 1, ids)


def moe_ff(h, sd, pfx, f):
    E = f["router"]["experts"]
    ids, wts = moe_route(h, sd, pfx, f)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(ids[t].tolist(), wts[t]):
            if e >= E:
                out[t] += w * h[t]
            else:
                p = f"{pfx}e{e}."
                a = silu(w64(sd, p + "gate") @ h[t]) * (w64(sd, p + "up") @ h[t])
                out[t] += w * (w64(sd, p + "down") @ a)
    return out


# ---- the model -------------------------------------------------------------------------------------------------------------------------
def forward(cfg, sd, tokens, return_layers=False, bf16_inputs=False):
    """logits (T, vocab) of one whole sequence; with return_layers also the residual stream after every layer.
    bf16_inputs: every sub-layer's input (the norm before it) is rounded to bfloat16, as bf16 serving hands it to the matrix products --
    the reference for sizes at which that rounding alone moves single positions by much (a denominator near its floor)."""
    eps = cfg["norm"]["eps"]

    def pre(u, name):
        h = layer_norm(u, sd, name, eps)
        return h.to(torch.bfloat16).to(F64) if bf16_inputs else h
    x = w64(sd, "embed")[torch.as_tensor(tokens, dtype=torch.long)] * cfg["embedding"]["scale"]
    kv, layers = {}, []
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        h = pre(x, p + "norm1")
        if l["type"] == "attention":
            if m.get("kv_from") is None:
                kv[i] = attention_kv(h, sd, p + "mix.", m, eps)
                y = attention_mixer(h, sd, p + "mix.", m, eps, kv[i])
            else:
                y = attention_mixer(h, sd, p + "mix.", m, eps, kv[m["kv_from"]])
        elif l["type"] == "lightning":
            y = lightning_mixer(h, sd, p + "mix.", m, eps)
        elif l["type"] == "mlstm":
            y = mlstm_mixer(h, sd, p + "mix.", m, eps)
        else:
            raise ValueError(l["type"])
        x = x + layer_norm(y, sd, p + "norm1b", eps)
        if l.get("mlp") is not None:
            y = moe_ff(pre(x, p + "norm2"), sd, p + "mlp.", l["mlp"])
            x = x + layer_norm(y, sd, p + "norm2b", eps)
        layers.append(x.clone())
    logits = pre(x, "final.norm") @ w64(sd, "head").T
    return (logits, layers) if return_layers else logits


# ---- small configurations and random weights for the tests --------------------------------------------------------------------------------
SIZES = [
    # attention: 2 query heads per kv head, a third of the head rotated; experts in 4 groups of 2 with 2 identity outputs
    dict(att=dict(heads=4, kv_heads=2, dim=24, vdim=16, scale=0.7, mask={"size": 20}, rot={"dims": 8, "base": 10000.0, "scaling": {"factor": 4.0}}),
         lin=dict(heads=3, dim=16, vdim=24, decay=[0.5, 0.9, 0.995]),
         mls=dict(heads=2, dim=40, vdim=12, gate_cap=10.0),
         moe=dict(ff=48, experts=6, identity=2, groups=4, keep=2, top=3)),
    # one kv head per query head, the whole head rotated, no scaling, a window of 5; one group, no identity, one expert per token, an ff that
    # is no multiple of 16
    dict(att=dict(heads=3, kv_heads=3, dim=10, vdim=22, scale=0.3, mask={"size": 5}, rot={"dims": 10, "base": 100.0, "scaling": {"factor": 1.0}}),
         lin=dict(heads=1, dim=8, vdim=8, decay=[0.97]),
         mls=dict(heads=5, dim=6, vdim=20, gate_cap=4.0),
         moe=dict(ff=40, experts=5, identity=0, groups=1, keep=1, top=1)),
    # heads wider than a wave, one kv head for all, a window longer than the prompts; many experts, more identity outputs
    dict(att=dict(heads=6, kv_heads=1, dim=72, vdim=80, scale=0.12, mask={"size": 4096}, rot={"dims": 36, "base": 500000.0, "scaling": {"factor": 1.5}}),
         lin=dict(heads=2, dim=100, vdim=130, decay=[0.8, 0.999]),
         mls=dict(heads=2, dim=72, vdim=36, gate_cap=30.0),
         moe=dict(ff=32, experts=13, identity=3, groups=2, keep=1, top=4)),
    # as many kv heads as query heads and wide values: more output coordinates (kv_heads * vdim = 640) than one pass of a kernel holds
    dict(att=dict(heads=8, kv_heads=8, dim=16, vdim=80, scale=0.4, mask={"size": 150}, rot={"dims": 4, "base": 30.0, "scaling": {"factor": 1.0}}),
         lin=dict(heads=2, dim=24, vdim=8, decay=[0.6, 0.9]),
         mls=dict(heads=1, dim=16, vdim=16, gate_cap=8.0),
         moe=dict(ff=16, experts=4, identity=4, groups=2, keep=2, top=2)),
]
_KIND = {"attention": "att", "shared": "att", "lightning": "lin", "mlstm": "mls"}


def small_config(order=("lightning", "mlstm", "attention", "shared"), width=72, vocab=97, sizes=0, no_mlp_at=()):
    """order: mixer types; "shared" = an attention layer on the keys and values of the nearest earlier attention layer with its own"""
    z = SIZES[sizes]
    layers, lender = [], None
    for i, t in enumerate(order):
        m = {k: (dict(v) if isinstance(v, dict) else v) for k, v in z[_KIND[t]].items()}
        if t == "shared":
            m["kv_from"] = lender
        elif t == "attention":
            lender = i
        f = z["moe"]
        mlp = None if i in no_mlp_at else {"kind": "moe", "expert": {"ff": f["ff"]}, "router": {
            "experts": f["experts"], "identity": f["identity"], "top": f["top"], "groups": {"count": f["groups"], "keep": f["keep"]}}}
        layers.append({"type": "attention" if t == "shared" else t, "mixer": m, "mlp": mlp})
    return {"architecture": "Retotar", "embedding": {"scale": 0.7}, "layers": layers, "norm": {"eps": 1e-5}, "vocab": vocab, "width": width}


def random_weights(cfg, seed=0, fixed_choice=False):
    """every tensor the configuration asks for, bf16-representable values (so that both serving formats start from the same numbers).
    fixed_choice: the routers' correction terms lie more than 1 apart, so that they alone order the choice scores (probabilities lie in
    [0, 1]) and no choice is a close call; the weights of the chosen outputs still follow the probabilities."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    sd = {}

    def mat(name, rows, cols, std=None):
        sd[name] = (torch.randn(rows, cols, generator=g) * (std if std is not None else cols ** -0.5)).to(torch.bfloat16)

    def norm(name, n):
        sd[name] = (1.0 + 0.2 * torch.randn(n, generator=g)).to(torch.bfloat16)
        sd[name + ".b"] = (0.1 * torch.randn(n, generator=g)).to(torch.bfloat16)

    mat("embed", cfg["vocab"], W, 1.5)
    mat("head", cfg["vocab"], W)
    norm("final.norm", W)
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        norm(p + "norm1", W)
        norm(p + "norm1b", W)
        H, d, v = m["heads"], m["dim"], m["vdim"]
        mat(p + "mix.q", H * d, W)
        mat(p + "mix.g", H * v, W)
        mat(p + "mix.o", W, H * v)
        if l["type"] == "attention":
            if m.get("kv_from") is None:
                mat(p + "mix.k", m["kv_heads"] * d, W)
                mat(p + "mix.v", m["kv_heads"] * v, W)
            sd[p + "mix.talk"] = (torch.eye(H) * 0.8 + 0.3 * torch.randn(H, H, generator=g)).to(torch.bfloat16)
        else:
            mat(p + "mix.k", H * d, W)
            mat(p + "mix.v", H * v, W)
            sd[p + "mix.norm"] = (1.0 + 0.2 * torch.randn(H * v, generator=g)).to(torch.bfloat16)
            if l["type"] == "mlstm":
                # keys lean towards the queries, so that the normaliser n . q seldom passes through zero: there the output is a quotient of
                # two small numbers, and any rounding of the input moves it by much (the floor of the denominator has its own test)
                sd[p + "mix.k"] = (0.8 * sd[p + "mix.q"].float() + 0.6 * sd[p + "mix.k"].float()).to(torch.bfloat16)
                mat(p + "mix.i", H, W, 0.4)
                mat(p + "mix.f", H, W, 0.4)
                sd[p + "mix.i.b"] = (0.5 * torch.randn(H, generator=g)).to(torch.bfloat16)
                sd[p + "mix.f.b"] = (2.0 + torch.randn(H, generator=g)).to(torch.bfloat16)
        f = l.get("mlp")
        if f is not None:
            norm(p + "norm2", W)
            norm(p + "norm2b", W)
            r = f["router"]
            total = r["experts"] + r.get("identity", 0)
            mat(p + "mlp.router", total, W, 2.0 * W ** -0.5)
            sd[p + "mlp.correction"] = (0.3 * torch.randn(total, generator=g) - 0.5).to(torch.bfloat16)      # choice scores go negative
            if fixed_choice:
                sd[p + "mlp.correction"] = (-1.5 * torch.randperm(total, generator=g).double()).to(torch.bfloat16)
            for e in range(r["experts"]):
                mat(f"{p}mlp.e{e}.gate", f["expert"]["ff"], W)
                mat(f"{p}mlp.e{e}.up", f["expert"]["ff"], W)
                mat(f"{p}mlp.e{e}.down", W, f["expert"]["ff"])
    return sd
