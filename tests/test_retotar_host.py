"""Host-side pieces of Retotar that need no GPU: configuration reader and registry, how layers share a cache, the packing of the expert
weights, and the restatement's own consistency (its mechanisms against direct per-token definitions)."""
import math

import pytest
import torch

import retotar_oracle as O

EPS = 1e-5


def test_registry_and_configuration():
    from zhilight_amd import registry
    from zhilight_amd._lib import ZLError
    from zhilight_amd.retotar import RetotarConfig, RetotarModel
    cfg = O.small_config(no_mlp_at=(1,))
    assert registry.model_class(cfg) is RetotarModel and "retotar" in registry.registered()
    c = RetotarConfig.from_dict(cfg)
    assert c.layers[1].mlp is None and c.layers[3].mixer["kv_from"] == 2 and c.eps == 1e-5 and c.embedding_scale == 0.7
    for breakage in (lambda d: d["layers"][0].update(type="something else"),
                     lambda d: d["layers"][3]["mixer"].update(kv_from=3),          # itself
                     lambda d: d["layers"][3]["mixer"].update(kv_from=1),          # not an attention layer
                     lambda d: d["layers"][2]["mlp"].update(kind="dense"),
                     lambda d: d.pop("vocab")):
        bad = O.small_config()
        breakage(bad)
        with pytest.raises(ZLError):
            RetotarConfig.from_dict(bad)


def test_model_layout_from_the_configuration():
    """built on the CPU without weights: which mixers exist, who lends its cache to whom, what the cache manager is asked for"""
    from zhilight_amd.cache import CacheManager
    from zhilight_amd.mixers import DecayLinearAttention, MLSTMMixer, WindowAttention
    from zhilight_amd.retotar import RetotarModel
    cfg = O.small_config(("attention", "lightning", "shared", "mlstm", "shared"), no_mlp_at=(4,))
    model = RetotarModel.from_config(cfg, dtype="float32", device="cpu")
    kinds = [type(l.mixer) for l in model.layers]
    assert kinds == [WindowAttention, DecayLinearAttention, WindowAttention, MLSTMMixer, WindowAttention]
    assert model.layers[2].mixer.kv_source is model.layers[0].mixer and model.layers[4].mixer.kv_source is model.layers[0].mixer
    assert model.layers[4].ff is None and model.layers[4].norm2 is None and model.layers[0].ff.identity == 2
    cache = model.bind_cache(CacheManager(256, 3, "cpu"))
    m = cfg["layers"][0]["mixer"]
    assert sorted(cache.planes) == ["l0.mix.k", "l0.mix.v"]
    assert cache.planes["l0.mix.k"].shape == (4, 64, m["kv_heads"] * m["dim"]) and model.layers[4].mixer.v_cache is cache.planes["l0.mix.v"]
    lin, mls = cfg["layers"][1]["mixer"], cfg["layers"][3]["mixer"]
    assert cache.states["l1.mix.S"].shape == (3, lin["heads"], lin["dim"], lin["vdim"])
    assert cache.states["l3.mix.S"].shape == (3, mls["heads"], mls["dim"], mls["vdim"] + 1) and cache.states["l3.mix.m"].shape == (3, mls["heads"])


def test_rotary_table_and_gate_up_packing():
    from zhilight_amd.mixers import RoutedExpertsFF, rotary_frequencies
    f = rotary_frequencies(8, 100.0, 4.0)
    assert f.dtype == torch.float32 and torch.allclose(f.double(), torch.tensor([1.0, 100 ** -0.25, 0.1, 100 ** -0.75], dtype=torch.float64) / 4, rtol=1e-7)
    ff = RoutedExpertsFF(8, 32, 3, 1)
    gate, up = torch.arange(32.0)[:, None].expand(32, 8), -torch.arange(32.0)[:, None].expand(32, 8)
    packed = ff._pack_gate_up(gate, up)
    assert packed[:16, 0].tolist() == list(range(16)) and packed[16:32, 0].tolist() == [-float(i) for i in range(16)]
    assert packed[32:48, 0].tolist() == list(range(16, 32))
    assert not RoutedExpertsFF(8, 40, 3, 1).fused_act


def test_restatement_attention_against_a_per_token_definition():
    cfg = O.small_config(("attention",), sizes=0)
    m = cfg["layers"][0]["mixer"]
    sd = O.random_weights(cfg, 1)
    T = 40
    h = torch.randn(T, cfg["width"], dtype=torch.float64, generator=torch.Generator().manual_seed(2))
    ref = O.attention_mixer(h, sd, "l0.mix.", m, EPS)
    H, G, d, v, n_rot = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["rot"]["dims"]

    def turn(vec, p, n, divide=1.0, sign=1.0):
        out = vec.clone()
        for i in range(n // 2):
            a = sign * p * m["rot"]["base"] ** (-2 * i / n) / divide
            out[i] = vec[i] * math.cos(a) - vec[i + n // 2] * math.sin(a)
            out[i + n // 2] = vec[i + n // 2] * math.cos(a) + vec[i] * math.sin(a)
        return out
    Wq, Wk, Wv, Wg, Wo, talk = (sd["l0.mix." + n].double() for n in ("q", "k", "v", "g", "o", "talk"))
    fac = m["rot"]["scaling"]["factor"]
    t = T - 1
    keys = {}
    for j in range(T):
        for c in range(G):
            kk = turn((Wk @ h[j])[c * d:(c + 1) * d], j, n_rot, fac)
            keys[j, c] = (kk / math.sqrt(float((kk * kk).mean()) + EPS), turn((Wv @ h[j])[c * v:(c + 1) * v], j, v))
    vis = [j for j in range(T) if 0 <= t - j < m["mask"]["size"]]
    w = torch.zeros(H, T, dtype=torch.float64)
    for hd in range(H):
        q = turn((Wq @ h[t])[hd * d:(hd + 1) * d], t, n_rot, fac)
        q = q / math.sqrt(float((q * q).mean()) + EPS)
        sc = torch.tensor([float(q @ keys[j, hd // (H // G)][0]) * m["scale"] for j in vis], dtype=torch.float64)
        w[hd, vis] = torch.softmax(sc, 0)
    mixed = talk @ w
    out = torch.cat([turn(sum(mixed[hd, j] * keys[j, hd // (H // G)][1] for j in vis), t, v, sign=-1.0) for hd in range(H)])
    out = Wo @ (out / (1 + torch.exp(-(Wg @ h[t]))))
    assert torch.allclose(out, ref[t], rtol=1e-9, atol=1e-10)


def test_restatement_recurrences_in_closed_form():
    """lightning: o_t = sum_s decay^(t-s) (q_t . k_s) v_s; mLSTM without the running maximum (plain exponentials are safe at these sizes)"""
    cfg = O.small_config(("lightning", "mlstm"), sizes=0)
    sd = O.random_weights(cfg, 3)
    T = 30
    h = torch.randn(T, cfg["width"], dtype=torch.float64, generator=torch.Generator().manual_seed(4))
    m = cfg["layers"][0]["mixer"]
    H, d, v = m["heads"], m["dim"], m["vdim"]
    q, k, val = (O.silu(h @ sd["l0.mix." + n].double().T).reshape(T, H, -1) for n in ("q", "k", "v"))
    out = torch.zeros(T, H, v, dtype=torch.float64)
    for t in range(T):
        for s in range(t + 1):
            for hd in range(H):
                out[t, hd] += m["decay"][hd] ** (t - s) * float(q[t, hd] @ k[s, hd]) * val[s, hd]
    out = O.unit_rms(out.reshape(T, H * v), EPS) * sd["l0.mix.norm"].double() * O.sigmoid(h @ sd["l0.mix.g"].double().T)
    assert torch.allclose(out @ sd["l0.mix.o"].double().T, O.lightning_mixer(h, sd, "l0.mix.", m, EPS), rtol=1e-9, atol=1e-10)

    m = cfg["layers"][1]["mixer"]
    H, d, v, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    p = "l1.mix."
    q = (h @ sd[p + "q"].double().T).reshape(T, H, d) / math.sqrt(d)
    k, val = (h @ sd[p + "k"].double().T).reshape(T, H, d), (h @ sd[p + "v"].double().T).reshape(T, H, v)
    gi = cap * torch.tanh((h @ sd[p + "i"].double().T + sd[p + "i.b"].double()) / cap)
    gf = torch.log(O.sigmoid(cap * torch.tanh((h @ sd[p + "f"].double().T + sd[p + "f.b"].double()) / cap)))
    out = torch.zeros(T, H, v, dtype=torch.float64)
    for hd in range(H):
        mx = 0.0
        for t in range(T):
            mx = max(float(gf[t, hd]) + mx, float(gi[t, hd]))
            # unnormalised memory: sum_s exp(i_s + sum_{r in (s, t]} f_r) k_s v_s^T; the running maximum only rescales it by exp(-m_t)
            wts = torch.tensor([math.exp(float(gi[s, hd]) + float(gf[s + 1:t + 1, hd].sum()) - mx) for s in range(t + 1)], dtype=torch.float64)
            num = ((wts * (k[:t + 1, hd] @ q[t, hd]))[:, None] * val[:t + 1, hd]).sum(0)
            den = max(abs(float((wts * (k[:t + 1, hd] @ q[t, hd])).sum())), math.exp(-mx)) + 1e-6
            out[t, hd] = num / den
    out = O.unit_rms(out, EPS).reshape(T, H * v) * sd[p + "norm"].double() * O.sigmoid(h @ sd[p + "g"].double().T)
    assert torch.allclose(out @ sd[p + "o"].double().T, O.mlstm_mixer(h, sd, p, m, EPS), rtol=1e-8, atol=1e-9)


def test_restatement_router_by_hand():
    """8 outputs in 4 groups of 2, 2 groups kept, 3 picks; all choice scores negative"""
    f = {"router": {"experts": 6, "identity": 2, "top": 3, "groups": {"count": 4, "keep": 2}}}
    W = 8
    sd = {"p.router": torch.eye(8) * 1.0, "p.correction": torch.tensor([-0.9, -0.2, -0.5, -0.6, -0.3, -0.95, -0.25, -0.9])}
    h = torch.zeros(1, W, dtype=torch.float64)
    h[0, 3] = 2.0                                               # output 3 gets most of the probability
    s = torch.softmax(h @ sd["p.router"].double().T, -1)[0]
    choice = s + sd["p.correction"].double()
    gs = [max(float(choice[2 * g]), float(choice[2 * g + 1])) for g in range(4)]
    kept = sorted(range(4), key=lambda g: -gs[g])[:2]
    cand = sorted((i for i in range(8) if i // 2 in kept), key=lambda i: -float(choice[i]))[:3]
    ids, wts = O.moe_route(h, sd, "p.", f)
    assert ids[0].tolist() == cand and torch.allclose(wts[0], s[cand]) and float(choice.max()) < 0.0
