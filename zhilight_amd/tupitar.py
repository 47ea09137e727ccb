"""Tupitar: a decoder-only model whose layers each pick one sequence mixer -- latent attention or a Mamba-2 state-space mixer -- and an
optional PolyNorm feed-forward, described layer by layer in config.json.

Shape of a layer (x is the fp32 residual stream; there is no norm BEFORE a sub-layer, a scalar-gain RMS norm AFTER it):
    h = shift(x)                        token shift: x_t + (x_{t-1} - x_t) * mix, the previous row carried per sequence
    x = x + g1 * mixer(h) / rms(mixer(h))
    x = x + g2 * ff(x) / rms(ff(x))     when the layer has a feed-forward
Embedding: table[token] * scale + learned position row.  Output: scalar-gain RMS norm, then the vocabulary projection.

The model runs RAGGED steps (seqops.RaggedBatch): every launch covers all tokens of the step, so whole prompts, portions of prompts,
single decoded tokens and mixtures are one code path; what a sequence carries between steps lives in the engine's CacheManager (latents in
paged planes; token-shift rows, convolution tails and recurrent states in slot states).
"""
from dataclasses import dataclass, field
from typing import List, Optional

import torch

from . import seqops
from ._lib import ZLError
from .mixers import LatentAttention, Mamba2Mixer, PolyNormFF
from .registry import register_model

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
           torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


@dataclass
class TupitarLayerConfig:
    type: str
    mixer: dict
    mlp: Optional[dict]


@dataclass
class TupitarConfig:
    vocab: int
    width: int
    max_positions: int
    embedding_scale: float
    eps: float
    layers: List[TupitarLayerConfig] = field(default_factory=list)

    @classmethod
    def from_dict(cls, cfg):
        try:
            layers = [TupitarLayerConfig(l["type"], dict(l["mixer"]), None if l.get("mlp") is None else dict(l["mlp"])) for l in cfg["layers"]]
            c = cls(int(cfg["vocab"]), int(cfg["width"]), int(cfg["max_positions"]), float(cfg["embedding"]["scale"]),
                    float(cfg["norm"]["eps"]), layers)
        except KeyError as e:
            raise ZLError(f"Tupitar config: missing key {e}")
        for i, l in enumerate(c.layers):
            if l.type not in MIXER_BUILDERS:
                raise ZLError(f"Tupitar config: layer {i}: unknown mixer type {l.type!r}")
            if l.mlp is not None and l.mlp.get("kind") != "dense":
                raise ZLError(f"Tupitar config: layer {i}: unknown feed-forward kind {l.mlp.get('kind')!r}")
        return c


def _latent_attention(name, width, m, eps):
    return LatentAttention(name, width, int(m["heads"]), int(m["dim"]), int(m["vdim"]), int(m["kv_rank"]), float(m["scale"]), eps,
                           sink=True, gate=True)


def _mamba2(name, width, m, eps):
    return Mamba2Mixer(name, width, int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m["groups"]), int(m["conv"]),
                       int(m["norm_groups"]), eps)


MIXER_BUILDERS = {"latent_attention": _latent_attention, "mamba2": _mamba2}


class TupitarLayer:
    def __init__(self, idx, cfg: TupitarConfig, lc: TupitarLayerConfig):
        self.idx, self.name, self.width, self.eps = idx, f"l{idx}", cfg.width, cfg.eps
        self.mixer = MIXER_BUILDERS[lc.type](self.name + ".mix", cfg.width, lc.mixer, cfg.eps)
        self.ff = PolyNormFF(cfg.width, int(lc.mlp["ff"]), cfg.eps) if lc.mlp is not None else None
        self.gain1 = self.gain2 = 1.0
        self.shift = self.prev = None

    def load(self, get, dtype, device):
        p = self.name + "."
        self.shift = get(p + "shift").to(device=device, dtype=torch.float32).reshape(self.width).contiguous()
        self.gain1 = float(get(p + "norm1").to(torch.float32).reshape(()))
        self.mixer.load(get, p + "mix.", dtype, device)
        if self.ff is not None:
            self.gain2 = float(get(p + "norm2").to(torch.float32).reshape(()))
            self.ff.load(get, p + "mlp.", dtype, device)

    def init_random(self, gen, dtype, device):
        self.shift = torch.rand(self.width, generator=gen, device=device, dtype=torch.float32)
        self.mixer.init_random(gen, dtype, device)
        if self.ff is not None:
            self.ff.init_random(gen, dtype, device)

    def bind(self, cache, dtype):
        self.prev = cache.add_state(self.name + ".shift", (self.width,))
        self.mixer.bind(cache, dtype)

    def forward(self, x, batch, dtype):
        h = seqops.token_shift(x, self.shift, self.prev, batch, dtype)
        y = self.mixer.forward(h, batch)
        xt = seqops.add_scalar_norm(x, y, self.gain1, self.eps, out_dtype=dtype if self.ff is not None else None)
        if self.ff is not None:
            seqops.add_scalar_norm(x, self.ff.forward(xt), self.gain2, self.eps)
        return x

    def weight_bytes(self):
        return self.mixer.weight_bytes() + (self.ff.weight_bytes() if self.ff is not None else 0)


@register_model("Tupitar")
class TupitarModel:
    ragged = True                    # the engine drives it with RaggedBatch steps and a CacheManager

    def __init__(self, cfg: TupitarConfig, dtype="bfloat16", device="cuda:0"):
        if dtype not in _DTYPES:
            raise ZLError(f"Tupitar serves in bfloat16 or float32, not {dtype}")
        self.cfg, self.dtype, self.device = cfg, _DTYPES[dtype], torch.device(device)
        self.layers = [TupitarLayer(i, cfg, lc) for i, lc in enumerate(cfg.layers)]
        self.embed = self.pos = self.head = None
        self.final_gain = 1.0
        self.page_size = 64

    @classmethod
    def from_config(cls, cfg: dict, dtype="bfloat16", device="cuda:0"):
        return cls(TupitarConfig.from_dict(cfg), dtype, device)

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
        for name, shape in (("embed", (c.vocab, c.width)), ("pos", (c.max_positions, c.width)), ("head", (c.vocab, c.width))):
            t = get(name)
            if tuple(t.shape) != shape:
                raise ZLError(f"tensor {name}: shape {tuple(t.shape)}, expected {shape}")
            setattr(self, name, t.to(device=dev, dtype=dt).contiguous())
        self.final_gain = float(get("final.norm").to(torch.float32).reshape(()))
        for layer in self.layers:
            layer.load(get, dt, dev)
        return self

    def init_random(self, seed=0):
        c, dev, dt = self.cfg, self.device, self.dtype
        gen = torch.Generator(device=dev).manual_seed(seed)
        self.embed = (torch.randn(c.vocab, c.width, generator=gen, device=dev) / max(c.embedding_scale, 1e-6)).to(dt)
        self.pos = (torch.randn(c.max_positions, c.width, generator=gen, device=dev) * 0.1).to(dt)
        self.head = (torch.randn(c.vocab, c.width, generator=gen, device=dev) * c.width ** -0.5).to(dt)
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

    def forward(self, tokens, batch, want_rows):
        """tokens: int32 device (n_tok) in the batch's flat order; want_rows: int32 device, flat token indices whose logits are wanted
        (None or empty: the step only advances caches and states).  Returns fp32 logits (len(want_rows), vocab) or None."""
        c = self.cfg
        x = seqops.embed(tokens, self.embed, self.pos, c.embedding_scale, batch)
        for layer in self.layers:
            layer.forward(x, batch, self.dtype)
        if want_rows is None or want_rows.numel() == 0:
            return None
        hn = seqops.scalar_norm_rows(x, want_rows, self.final_gain, c.eps, self.dtype)
        return seqops.gemm_nt(hn, self.head)

    def forward_layers(self, tokens, batch):
        """the residual stream after every layer (debugging and tests): list of fp32 (n_tok, width) copies"""
        x = seqops.embed(tokens, self.embed, self.pos, self.cfg.embedding_scale, batch)
        out = []
        for layer in self.layers:
            layer.forward(x, batch, self.dtype)
            out.append(x.clone())
        return out

    def weight_bytes(self):
        return sum(l.weight_bytes() for l in self.layers) + sum(t.numel() * t.element_size() for t in (self.embed, self.pos, self.head))
