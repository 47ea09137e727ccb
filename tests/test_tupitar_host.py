"""Host-side pieces of the ragged-step engine that need no GPU: the checkpoint reader, the registry and configuration, the cache manager's
pages and slots, and the oracle's own consistency (its mechanisms against direct per-token definitions)."""
import json
import math
import struct

import numpy as np
import pytest
import torch

import tupitar_oracle as O


def test_safetensors_reader_roundtrip(tmp_path):
    from zhilight_amd.checkpoint import load_dir
    a = torch.randn(3, 5).to(torch.bfloat16)
    b = torch.arange(7, dtype=torch.int32)
    c = torch.tensor(1.25, dtype=torch.bfloat16)
    blobs, header, off = [], {}, 0
    for name, t, code in (("a.w", a, "BF16"), ("b", b, "I32"), ("c", c, "BF16")):
        raw = t.contiguous().view(torch.uint8).numpy().tobytes() if t.dim() else t.reshape(1).view(torch.uint8).numpy().tobytes()
        header[name] = {"dtype": code, "shape": list(t.shape), "data_offsets": [off, off + len(raw)]}
        off += len(raw)
        blobs.append(raw)
    hj = json.dumps(header).encode()
    (tmp_path / "model.safetensors").write_bytes(struct.pack("<Q", len(hj)) + hj + b"".join(blobs))
    ck = load_dir(str(tmp_path))
    assert torch.equal(ck["a.w"], a) and torch.equal(ck["b"], b) and ck["c"].shape == () and float(ck["c"]) == 1.25
    with pytest.raises(KeyError):
        ck["nope"]


def test_registry_picks_the_class_by_config():
    from zhilight_amd import registry
    from zhilight_amd._lib import ZLError
    from zhilight_amd.llama import LLaMA
    from zhilight_amd.tupitar import TupitarConfig, TupitarModel
    assert registry.model_class(O.small_config()) is TupitarModel
    assert registry.model_class({"architectures": ["LlamaForCausalLM"], "model_type": "llama"}) is LLaMA
    with pytest.raises(ZLError):
        registry.model_class({"architecture": "unheard-of"})
    cfg = O.small_config(no_mlp_at=(1,))
    c = TupitarConfig.from_dict(cfg)
    assert c.layers[1].mlp is None and c.layers[0].mlp["ff"] == 136 and c.eps == 1e-5
    cfg["layers"][0]["type"] = "something else"
    with pytest.raises(ZLError):
        TupitarConfig.from_dict(cfg)


def test_cache_manager_pages_and_slots():
    from zhilight_amd._lib import ZLError
    from zhilight_amd.cache import CacheManager
    cm = CacheManager(max_tokens=5 * 64, max_seqs=2, device="cpu")
    st = cm.add_state("s", (3,))
    plane = cm.add_plane("p", (4,), torch.float32)
    assert plane.shape == (5, 64, 4)
    assert cm.admit("a") == 0 and cm.admit("b") == 1
    with pytest.raises(ZLError):
        cm.admit("c")
    assert cm.extend("a", 65) == (0, 0, [0, 1])
    assert cm.extend("b", 64)[2] == [2]
    assert cm.extend("b", 1) == (64, 1, [2, 3])
    assert cm.extend("a", 63)[2] == [0, 1] and cm.length("a") == 128
    assert cm.can_extend("a", 64) and not cm.can_extend("a", 65)
    with pytest.raises(ZLError):
        cm.extend("a", 65)
    st[0] = 5.0
    cm.release("a")
    assert cm.free_pages == [0, 1, 4] and cm.free_slots == [0]
    assert cm.admit("c") == 0 and float(st[0].abs().max()) == 0.0           # a slot is cleared when it is taken again
    assert cm.extend("c", 130)[2] == [0, 1, 4]


def test_oracle_recurrence_matches_a_direct_sum():
    """the state-space mixer's y_t against the unrolled sum  y_t = sum_{s<=t} (prod_{s<r<=t} a_r) dt_s (C_t . B_s) x_s + D x_t  for one head"""
    cfg = O.small_config(("mamba2",))
    m = cfg["layers"][0]["mixer"]
    sd = O.random_weights(cfg, 1)
    T, W = 12, cfg["width"]
    h = torch.randn(T, W, generator=torch.Generator().manual_seed(2)).double()
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    proj = h @ sd["l0.mix.in"].double().T
    xbc = O.silu(O.causal_conv(proj[:, inner:2 * inner + 2 * G * N], sd["l0.mix.conv"], sd["l0.mix.conv.b"]))
    dt = O.softplus(proj[:, 2 * inner + 2 * G * N:] + sd["l0.mix.dt_bias"].double())
    a = torch.exp(-torch.exp(sd["l0.mix.A_log"].double()) * dt)
    hd, g = 3, 3 // (H // G)
    x = xbc[:, hd * P:(hd + 1) * P]
    B = xbc[:, inner + g * N: inner + (g + 1) * N]
    C = xbc[:, inner + G * N + g * N: inner + G * N + (g + 1) * N]
    y = torch.zeros(T, P, dtype=torch.float64)
    for t in range(T):
        for s in range(t + 1):
            y[t] += torch.prod(a[s + 1:t + 1, hd]) * dt[s, hd] * (C[t] @ B[s]) * x[s]
        y[t] += sd["l0.mix.D"].double()[hd] * x[t]
    z = proj[:, :inner]
    full = O.mamba2_mixer(h, sd, "l0.mix.", m, 1e-5)
    # undo the output side for the one head is not possible after the norm: compare through a mixer whose other heads are silenced instead
    gated = torch.zeros(T, inner, dtype=torch.float64)
    gated[:, hd * P:(hd + 1) * P] = y * O.silu(z[:, hd * P:(hd + 1) * P])
    sd2 = dict(sd)
    w_in = sd["l0.mix.in"].clone().float()
    keep = torch.zeros(inner, dtype=torch.bool)
    keep[hd * P:(hd + 1) * P] = True
    w_in[:inner][~keep] = 0.0                                               # z = 0 -> silu(z) = 0: the other heads vanish before the norm
    sd2["l0.mix.in"] = w_in
    R = m["norm_groups"]
    want = (O.unit_rms(gated.reshape(T, R, inner // R), 1e-5).reshape(T, inner) * sd["l0.mix.norm"].double()) @ sd["l0.mix.o"].double().T
    got = O.mamba2_mixer(h, sd2, "l0.mix.", m, 1e-5)
    assert torch.allclose(got, want, rtol=1e-9, atol=1e-11)
    assert full.shape == got.shape


def test_oracle_attention_first_token_and_sink():
    cfg = O.small_config(("latent_attention",))
    m = cfg["layers"][0]["mixer"]
    sd = O.random_weights(cfg, 3)
    h = torch.randn(4, cfg["width"], generator=torch.Generator().manual_seed(4)).double()
    out = O.latent_attention_mixer(h, sd, "l0.mix.", m, 1e-5)
    # token 0 sees one key: weight e^s / (e^s + e^sink) on v_0, per head
    H, dq, dv = m["heads"], m["dim"], m["vdim"]
    q = (sd["l0.mix.q"].double() @ h[0]).reshape(H, dq)
    c = O.unit_rms(sd["l0.mix.dkv"].double() @ h[0], 1e-5) * sd["l0.mix.dkv.norm"].double()
    k = (sd["l0.mix.uk"].double() @ c).reshape(H, dq)
    v = (sd["l0.mix.uv"].double() @ c).reshape(H, dv)
    s = (q * k).sum(-1) * m["scale"]
    wgt = torch.exp(s) / (torch.exp(s) + torch.exp(sd["l0.mix.sink"].double()))
    gate = torch.sigmoid(sd["l0.mix.g"].double() @ h[0])
    want = sd["l0.mix.o"].double() @ (v * (wgt * gate)[:, None]).reshape(-1)
    assert torch.allclose(out[0], want, rtol=1e-10, atol=1e-12)
    # causality: a later token does not change earlier outputs
    h2 = h.clone()
    h2[3] += 1.0
    assert torch.equal(O.latent_attention_mixer(h2, sd, "l0.mix.", m, 1e-5)[:3], out[:3])


def test_scheduler_cuts_prompts_and_respects_budgets():
    """the scheduler alone, with a model stub that needs no device: token budget per step, arrival order, at most max_seqs live requests,
    decode tokens first"""
    from zhilight_amd.cache import CacheManager
    from zhilight_amd.engine import Engine, SamplingParams

    class Stub:
        ragged, page_size, max_positions, device, vocab_size = True, 64, 10_000, torch.device("cpu"), 11

        def bind_cache(self, cache):
            return cache
    eng = Engine(Stub(), max_tokens=6 * 64, max_seqs=2, max_step_tokens=100)
    steps = []

    def fake_run(entries):
        steps.append([(e.rid, len(e.tokens), list(e.want)) for e in entries])
        for e in entries:
            if e.rid not in eng.cache.seqs:
                eng.cache.admit(e.rid)
            eng.cache.extend(e.rid, len(e.tokens))
        n = sum(len(e.want) for e in entries)
        return torch.zeros(n, 11) if n else None
    eng.run_step = fake_run
    eng.sample = lambda logits, reqs: [1] * len(reqs)
    for i, n in enumerate((150, 30, 20)):
        eng.add_request(f"r{i}", list(range(n)), SamplingParams(max_new_tokens=3))
    while eng.has_work():
        eng.step()
    assert steps[0] == [("r0", 100, [])]
    assert steps[1] == [("r0", 50, [49]), ("r1", 30, [29])]                  # the rest of r0, then r1 within the budget; r2 must wait
    assert steps[2][0] == ("r0", 1, [0]) and steps[2][1] == ("r1", 1, [0])   # decodes first
    assert all(len({e[0] for e in s}) <= 2 for s in steps)
    assert all(sum(e[1] for e in s) <= 100 for s in steps)
    assert {r.rid: len(r.output) for r in eng.finished.values()} == {"r0": 3, "r1": 3, "r2": 3}
    assert not eng.cache.seqs and len(eng.cache.free_pages) == 6


def test_seq_header_and_loader_name_the_same_entry_points():
    import os
    import re
    from zhilight_amd import seqops
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = open(os.path.join(root, "include", "zhilight_amd_seq.h")).read()
    declared = set(re.findall(r"\b(zls_[a-z0-9_]+)\s*\(", text))
    assert declared == set(seqops.SYMBOLS)
    if os.path.exists(seqops.SO_PATH):
        lib = seqops.lib()
        assert all(hasattr(lib, n) for n in declared)
