"""Retotar: a decoder-only model whose layers each pick one sequence mixer -- windowed softmax attention (optionally on another layer's keys
and values), linear attention with a fixed decay per head, or an mLSTM matrix memory -- and an optional mixture-of-experts feed-forward,
described layer by layer in config.json.

Shape of a layer (x is the fp32 residual stream; LN = layer norm with weight and bias, before AND after every sub-layer):
    x = x + LN1b(mixer(LN1(x)))
    x = x + LN2b(ff(LN2(x)))            when the layer has a feed-forward
Embedding: table[token] * scale, no learned positions.  Output: LN, then the vocabulary projection.

Configuration keys: vocab, width, embedding.scale, norm.eps, layers[i] = {type, mixer, mlp}:
    type "attention"   mixer: heads, kv_heads, dim, vdim, scale, mask.size, rot.{dims, base, scaling.factor}, kv_from (optional layer index)
    type "lightning"   mixer: heads, dim, vdim, decay (one per head)
    type "mlstm"       mixer: heads, dim, vdim, gate_cap
    mlp (or null)      kind "moe", expert.ff, router.{experts, top, identity, groups.{count, keep}}
Tensors: embed, head, final.norm(.b), l<i>.norm1 / norm1b / norm2 / norm2b (.b), l<i>.mix.*, l<i>.mlp.* (see the mixer classes).

The model runs RAGGED steps exactly as Tupitar does: every launch covers all tokens of a step; keys and values live in paged planes of the
engine's CacheManager, recurrent states in its slot states.  A post-norm launch also writes the next sub-layer's pre-norm output, so a layer
is: product, mixer kernels, product, add+norm, [router product, route, align, two grouped products, combine, add+norm].
"""
from dataclasses import dataclass, field
from typing import List, Optional

import torch

from . import seqops
from ._lib import ZLError
from .mixers import DecayLinearAttention, MLSTMMixer, RoutedExpertsFF, WindowAttention, _vec
from .registry import register_model

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
           torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


@dataclass
class RetotarLayerConfig:
    type: str
    mixer: dict
    mlp: Optional[dict]


@dataclass
class RetotarConfig:
    vocab: int
    width: int
    embedding_scale: float
    eps: float
    max_positions: int
    layers: List[RetotarLayerConfig] = field(default_factory=list)

    @classmethod
    def from_dict(cls, cfg):
        try:
            layers = [RetotarLayerConfig(l["type"], dict(l["mixer"]), None if l.get("mlp") is None else dict(l["mlp"])) for l in cfg["layers"]]
            c = cls(int(cfg["vocab"]), int(cfg["width"]), float(cfg["embedding"]["scale"]), float(cfg["norm"]["eps"]),
                    int(cfg.get("max_positions", 1 << 24)), layers)       # (positions are fp32 numbers: exact up to 2^24)
        except KeyError as e:
            raise ZLError(f"Retotar config: missing key {e}")
        for i, l in enumerate(c.layers):
            if l.type not in MIXER_BUILDERS:
                raise ZLError(f"Retotar config: layer {i}: unknown mixer type {l.type!r}")
            if l.mlp is not None and l.mlp.get("kind", "moe") != "moe":
                raise ZLError(f"Retotar config: layer {i}: unknown feed-forward kind {l.mlp.get('kind')!r}")
            src = l.mixer.get("kv_from")
            if src is not None and not (l.type == "attention" and 0 <= int(src) < i and c.layers[int(src)].type == "attention"
                                        and c.layers[int(src)].mixer.get("kv_from") is None):
                raise ZLError(f"Retotar config: layer {i}: kv_from must name an earlier attention layer with projections of its own")
        return c


def _attention(name, width, m, eps, layers):
    rot = m.get("rot") or {}
    src = m.get("kv_from")
    return WindowAttention(name, width, int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), float(m["scale"]),
                           int((m.get("mask") or {}).get("size", 0)), int(rot.get("dims", 0)), float(rot.get("base", 10000.0)),
                           float((rot.get("scaling") or {}).get("factor", 1.0)), eps, qk_norm=True, rotate_values=True, talk=True, gate=True,
                           kv_source=None if src is None else layers[int(src)].mixer)


def _lightning(name, width, m, eps, layers):
    return DecayLinearAttention(name, width, int(m["heads"]), int(m["dim"]), int(m["vdim"]), list(m["decay"]), eps, act="silu")


def _mlstm(name, width, m, eps, layers):
    return MLSTMMixer(name, width, int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["gate_cap"]), eps)


MIXER_BUILDERS = {"attention": _attention, "lightning": _lightning, "mlstm": _mlstm}


def _experts(width, f):
    r = f["router"]
    g = r.get("groups") or {}
    return RoutedExpertsFF(width, int(f["expert"]["ff"]), int(r["experts"]), int(r["top"]), identity=int(r.get("identity", 0)),
                           groups=int(g.get("count", 1)), keep=int(g.get("keep", g.get("count", 1))), correction=True, renorm=False)


class LayerNormParams:
    """weight and bias (tensor `name` and `name`.b), fp32"""

    def __init__(self, width):
        self.width, self.w, self.b = width, None, None

    def load(self, get, name, device):
        self.w, self.b = _vec(get, name, self.width, device), _vec(get, name + ".b", self.width, device)
        return self

    def init_random(self, gen, device):
        self.w = 1.0 + 0.1 * torch.randn(self.width, generator=gen, device=device)
        self.b = 0.1 * torch.randn(self.width, generator=gen, device=device)
        return self


class RetotarLayer:
    def __init__(self, idx, cfg: RetotarConfig, lc: RetotarLayerConfig, layers):
        self.idx, self.name, self.width, self.eps = idx, f"l{idx}", cfg.width, cfg.eps
        self.mixer = MIXER_BUILDERS[lc.type](self.name + ".mix", cfg.width, lc.mixer, cfg.eps, layers)
        self.ff = _experts(cfg.width, lc.mlp) if lc.mlp is not None else None
        self.norm1, self.norm1b = LayerNormParams(cfg.width), LayerNormParams(cfg.width)
        self.norm2, self.norm2b = (LayerNormParams(cfg.width), LayerNormParams(cfg.width)) if self.ff is not None else (None, None)

    def load(self, get, dtype, device):
        p = self.name + "."
        self.norm1.load(get, p + "norm1", device)
        self.norm1b.load(get, p + "norm1b", device)
        self.mixer.load(get, p + "mix.", dtype, device)
        if self.ff is not None:
            self.norm2.load(get, p + "norm2", device)
            self.norm2b.load(get, p + "norm2b", device)
            self.ff.load(get, p + "mlp.", dtype, device)

    def init_random(self, gen, dtype, device):
        for n in (self.norm1, self.norm1b, self.norm2, self.norm2b):
            if n is not None:
                n.init_random(gen, device)
        self.mixer.init_random(gen, dtype, device)
        if self.ff is not None:
            self.ff.init_random(gen, dtype, device)

    def bind(self, cache, dtype):
        self.mixer.bind(cache, dtype)

    def forward(self, x, h, batch, dtype, next_norm):
        """h = LN1(x) in the serving format; returns the next layer's LN1 of the new x (None without next_norm)"""
        y = self.mixer.forward(h, batch)
        after = self.norm2 if self.ff is not None else next_norm
        h = seqops.add_layer_norm(x, y, self.norm1b.w, self.norm1b.b, self.eps, after.w if after else None, after.b if after else None, dtype)
        if self.ff is not None:
            y = self.ff.forward(h)
            h = seqops.add_layer_norm(x, y, self.norm2b.w, self.norm2b.b, self.eps, next_norm.w if next_norm else None,
                                      next_norm.b if next_norm else None, dtype)
        return h

    def weight_bytes(self):
        return self.mixer.weight_bytes() + (self.ff.weight_bytes() if self.ff is not None else 0)


@register_model("Retotar")
class RetotarModel:
    ragged = True                    # the engine drives it with RaggedBatch steps and a CacheManager

    def __init__(self, cfg: RetotarConfig, dtype="bfloat16", device="cuda:0"):
        if dtype not in _DTYPES:
            raise ZLError(f"Retotar serves in bfloat16 or float32, not {dtype}")
        self.cfg, self.dtype, self.device = cfg, _DTYPES[dtype], torch.device(device)
        self.layers = []
        for i, lc in enumerate(cfg.layers):
            self.layers.append(RetotarLayer(i, cfg, lc, self.layers))
        self.final_norm = LayerNormParams(cfg.width)
        self.embed = self.head = None
        self.page_size = 64

    @classmethod
    def from_config(cls, cfg: dict, dtype="bfloat16", device="cuda:0"):
        return cls(RetotarConfig.from_dict(cfg), dtype, device)

    @property
    def vocab_size(self):
        return self.cfg.vocab

    @property
    def max_positions(self):
        return self.cfg.max_positions

    def load_weights(self, ckpt):
        c, dev, dt = self.cfg, self.device, self.dtype

        def get(name):
            return ckpt[name]
        for name in ("embed", "head"):
            t = get(name)
            if tuple(t.shape) != (c.vocab, c.width):
                raise ZLError(f"tensor {name}: shape {tuple(t.shape)}, expected {(c.vocab, c.width)}")
            setattr(self, name, t.to(device=dev, dtype=dt).contiguous())
        self.final_norm.load(get, "final.norm", dev)
        for layer in self.layers:
            layer.load(get, dt, dev)
        return self

    def init_random(self, seed=0):
        c, dev, dt = self.cfg, self.device, self.dtype
        gen = torch.Generator(device=dev).manual_seed(seed)
        self.embed = (torch.randn(c.vocab, c.width, generator=gen, device=dev) / max(c.embedding_scale, 1e-6)).to(dt)
        self.head = (torch.randn(c.vocab, c.width, generator=gen, device=dev) * c.width ** -0.5).to(dt)
        self.final_norm.init_random(gen, dev)
        for layer in self.layers:
            layer.init_random(gen, dt, dev)
        return self

    def bind_cache(self, cache):
        """register every layer's per-token planes and per-sequence states with the engine's cache manager"""
        if cache.page_size != self.page_size:
            raise ZLError("cache page size mismatch")
        for layer in self.layers:
            layer.bind(cache, self.dtype)
        return cache

    def _run(self, tokens, batch, keep=None):
        c = self.cfg
        x = seqops.embed(tokens, self.embed, None, c.embedding_scale, batch)
        if not self.layers:
            return x
        h = seqops.layer_norm(x, self.layers[0].norm1.w, self.layers[0].norm1.b, c.eps, self.dtype)
        for i, layer in enumerate(self.layers):
            nxt = self.layers[i + 1].norm1 if i + 1 < len(self.layers) else None
            h = layer.forward(x, h, batch, self.dtype, nxt)
            if keep is not None:
                keep.append(x.clone())
        return x

    def forward(self, tokens, batch, want_rows):
        """tokens: int32 device (n_tok) in the batch's flat order; want_rows: int32 device, flat token indices whose logits are wanted
        (None or empty: the step only advances caches and states).  Returns fp32 logits (len(want_rows), vocab) or None."""
        x = self._run(tokens, batch)
        if want_rows is None or want_rows.numel() == 0:
            return None
        hn = seqops.layer_norm(x, self.final_norm.w, self.final_norm.b, self.cfg.eps, self.dtype, rows=want_rows)
        return seqops.gemm_nt(hn, self.head)

    def forward_layers(self, tokens, batch):
        """the residual stream after every layer (debugging and tests): list of fp32 (n_tok, width) copies"""
        out = []
        self._run(tokens, batch, keep=out)
        return out

    def weight_bytes(self):
        return sum(l.weight_bytes() for l in self.layers) + sum(t.numel() * t.element_size() for t in (self.embed, self.head))
