"""Tupitar on the GPU against the plain float64 restatement in tests/tupitar_oracle.py: every mechanism alone, then the model through the
engine's step function -- whole prompts, token-by-token decoding, portions down to two tokens, mixed batches, reused pages and slots, far
keys and page borders, odd sizes, greedy generation through the scheduler.  Small random configurations made here; nothing is read from disk.
fp32 serving is held to rounding of fp32 sums, bf16 serving to bf16 rounding of the matrix-product inputs."""
import math

import numpy as np
import pytest
import torch

import tupitar_oracle as O

pytestmark = pytest.mark.gpu

F32_TOL, BF16_TOL = 3e-5, 4e-2


def rel(got, ref):
    got, ref = got.double().cpu(), ref.double().cpu()
    return float((got - ref).pow(2).mean().sqrt() / ref.pow(2).mean().sqrt().clamp_min(1e-30))


def tol(dtype):
    return F32_TOL if dtype == torch.float32 else BF16_TOL


def make(cfg, sd, dtype, dev, max_tokens=2048, max_seqs=4, max_step_tokens=512):
    from zhilight_amd.engine import Engine
    from zhilight_amd.registry import model_class
    model = model_class(cfg).from_config(cfg, dtype=dtype, device=dev).load_weights(sd)
    return Engine(model, max_tokens=max_tokens, max_seqs=max_seqs, max_step_tokens=max_step_tokens)


def run_portions(eng, rid, tokens, portions, release=True):
    """feed `tokens` of one request in the given portion sizes, wanting every position; returns (T, vocab) logits"""
    from zhilight_amd.engine import Entry
    out, at = [], 0
    for n in portions:
        out.append(eng.run_step([Entry(rid, tokens[at:at + n], list(range(n)))]))
        at += n
    assert at == len(tokens)
    if release:
        eng.release(rid)
    return torch.cat(out, dim=0)


def tokens_of(cfg, n, seed):
    return np.random.default_rng(seed).integers(0, cfg["vocab"], n).tolist()


# ------------------------------------------------------------------------------------------------------------------------------------
# mechanisms alone
# ------------------------------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,n,k", [(1, 70, 96), (3, 129, 100), (8, 64, 90), (9, 200, 96), (5, 70, 96), (16, 33, 320), (12, 129, 1000), (4, 17, 8),
                                   (70, 65, 33), (130, 582, 320), (257, 48, 1024), (300, 260, 264)])
def test_gemm_any_shape(dev, dtype, m, n, k):
    from zhilight_amd import seqops
    g = torch.Generator().manual_seed(m * 1000 + n + k)
    x = torch.randn(m, k, generator=g).to(dtype)
    w = torch.randn(n, k, generator=g).to(dtype)
    got = seqops.gemm_nt(x.to(dev), w.to(dev))
    assert got.dtype == torch.float32
    ref = x.double() @ w.double().T
    assert rel(got, ref) < (2e-6 if dtype == torch.float32 else 1e-6)      # inputs are exact in both formats: only the fp32 sums differ


def one_seq_batch(n, dev, pos0=0, slot=0, page_size=64, pages=None):
    from zhilight_amd import seqops
    pages = pages if pages is not None else list(range((pos0 + n + page_size - 1) // page_size))
    return seqops.RaggedBatch([(n, pos0, slot, pages)], page_size, dev)


def test_token_shift_carries_the_previous_row(dev):
    from zhilight_amd import seqops
    g = torch.Generator().manual_seed(1)
    x = torch.randn(11, 50, generator=g)
    mix = torch.rand(50, generator=g)
    ref = O.token_shift(x.double(), mix)
    prev = torch.zeros(3, 50, device=dev)
    prev[0] = 7.0                                                   # another slot's row must not leak in
    got = []
    for lo, hi in ((0, 1), (1, 3), (3, 4), (4, 11)):                # first token alone, two tokens, a decoded token, a longer portion
        got.append(seqops.token_shift(x[lo:hi].to(dev).contiguous(), mix.to(dev), prev, one_seq_batch(hi - lo, dev, lo, slot=2), torch.float32))
    assert rel(torch.cat(got), ref) < 1e-6
    assert torch.equal(prev[2].cpu(), x[10]) and float(prev[0].min()) == 7.0


def test_norms_and_polynorm(dev):
    from zhilight_amd import seqops
    g = torch.Generator().manual_seed(2)
    x, y = torch.randn(5, 77, generator=g), torch.randn(5, 77, generator=g) * 3
    ref = x.double() + O.scalar_norm(y.double(), torch.tensor(1.7), 1e-5)
    xd = x.to(dev)
    xt = seqops.add_scalar_norm(xd, y.to(dev), 1.7, 1e-5, out_dtype=torch.bfloat16)
    assert rel(xd, ref) < 1e-6 and rel(xt, ref) < 4e-3
    rows = torch.tensor([4, 0, 4], dtype=torch.int32, device=dev)
    got = seqops.scalar_norm_rows(xd, rows, 0.6, 1e-5, torch.float32)
    assert rel(got, O.scalar_norm(ref[[4, 0, 4]], torch.tensor(0.6), 1e-5)) < 1e-6
    z = torch.randn(6, 136, generator=g) * 2
    coef = torch.tensor([0.9, -0.4, 0.3, 0.2])
    assert rel(seqops.polynorm(z.to(dev), coef.tolist(), 1e-5, torch.float32), O.polynorm(z.double(), coef, 1e-5)) < 1e-6


def mixer_sd(cfg, i, seed):
    sd = O.random_weights(cfg, seed)
    p = f"l{i}.mix."
    return {k[len(p):]: v for k, v in sd.items() if k.startswith(p)}, sd


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("portions", [[150], [2, 61, 1, 1, 64, 21], [63, 2, 85], [1] * 40 + [3] + [1] * 70])
@pytest.mark.parametrize("kernels", ["matrix cores", "plain"])
def test_latent_attention_alone(dev, dtype, portions, kernels):
    from zhilight_amd.cache import CacheManager
    from zhilight_amd.mixers import LatentAttention
    cfg = O.small_config(("latent_attention",))
    m = cfg["layers"][0]["mixer"]
    sub, _ = mixer_sd(cfg, 0, 3)
    W, T = cfg["width"], sum(portions)
    h = torch.randn(T, W, generator=torch.Generator().manual_seed(4)).to(dtype)
    ref = O.latent_attention_mixer(h.double(), {"x." + k: v for k, v in sub.items()}, "x.", m, 1e-5)
    cache = CacheManager(256, 2, dev)
    mix = LatentAttention("a", W, m["heads"], m["dim"], m["vdim"], m["kv_rank"], m["scale"], 1e-5).load(lambda n: sub[n], "", dtype, dev)
    mix.bind(cache, dtype)
    mix.prompt_kernel = mix.decode_mfma = kernels == "matrix cores"     # (bf16 only; fp32 serving has the one plain kernel)
    cache.admit("s")
    got, at = [], 0
    for n in portions:
        pos0, slot, pages = cache.extend("s", n)
        got.append(mix.forward(h[at:at + n].to(dev).contiguous(), one_seq_batch(n, dev, pos0, slot, pages=list(pages))))
        at += n
    assert rel(torch.cat(got), ref) < tol(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("portions", [[90], [1, 1, 2, 3, 40, 1, 42], [2] * 10 + [70]])
@pytest.mark.parametrize("variant", [0, 1, 2])
@pytest.mark.parametrize("segment", [0, 7, 16])
def test_mamba2_alone(dev, dtype, portions, variant, segment):
    from zhilight_amd.cache import CacheManager
    from zhilight_amd.mixers import Mamba2Mixer
    cfg = O.small_config(("mamba2",), seed_sizes=variant)
    m = cfg["layers"][0]["mixer"]
    if variant == 2:                                                # groups == heads, one norm group, a state size that divides nothing
        m.update(groups=4, norm_groups=1, state=21, conv=2)
    sub, _ = mixer_sd(cfg, 0, 5 + variant)
    W, T = cfg["width"], sum(portions)
    h = torch.randn(T, W, generator=torch.Generator().manual_seed(6)).to(dtype)
    ref = O.mamba2_mixer(h.double(), {"x." + k: v for k, v in sub.items()}, "x.", m, 1e-5)
    cache = CacheManager(256, 3, dev)
    mix = Mamba2Mixer("m", W, m["heads"], m["vdim"], m["state"], m["groups"], m["conv"], m["norm_groups"], 1e-5).load(lambda n: sub[n], "", dtype, dev)
    mix.bind(cache, dtype)
    mix.scan_segment = segment                                      # long portions in segments of 7 / 16 tokens (0: one pass)
    cache.admit("other")
    cache.admit("s")                                                # slot 1: slot 0's state stays zero and must stay untouched
    got, at = [], 0
    for n in portions:
        pos0, slot, pages = cache.extend("s", n)
        got.append(mix.forward(h[at:at + n].to(dev).contiguous(), one_seq_batch(n, dev, pos0, slot, pages=list(pages))))
        at += n
    assert rel(torch.cat(got), ref) < tol(dtype)
    assert float(mix.state[0].abs().max()) == 0.0 and float(mix.state[1].abs().max()) > 0.0


def _aim_query(sd, pfx, m, h, i_star, j_star, eps, strength):
    """rewrite row i_star of h so that, for every head, its query points exactly at key j_star: that score stands out by `strength`"""
    H, d = m["heads"], m["dim"]
    hd = h.double()
    c = O.unit_rms(hd[j_star] @ sd[pfx + "dkv"].double().T, eps) * sd[pfx + "dkv.norm"].double()
    k = sd[pfx + "uk"].double() @ c                                                      # (H * d)
    k = k.reshape(H, d)
    target = (k / (k.pow(2).sum(-1, keepdim=True) * m["scale"]) * strength).reshape(-1)   # q.k*scale = strength per head
    h[i_star] = (torch.linalg.pinv(sd[pfx + "q"].double()) @ target).to(h.dtype)
    return h


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("j_star", [0, 1, 63, 64, 65, 127, 128, 200])
def test_latent_attention_finds_one_far_key(dev, dtype, j_star):
    """one query (in a prompt portion, and decoded alone) whose whole weight lies on ONE key far back, at and around page borders: a key that
    is dropped, shifted by one or read from a wrong page changes the output completely"""
    from zhilight_amd.cache import CacheManager
    from zhilight_amd.mixers import LatentAttention
    cfg = O.small_config(("latent_attention",))
    m = cfg["layers"][0]["mixer"]
    sub, _ = mixer_sd(cfg, 0, 7)
    sub["sink"] = torch.full_like(sub["sink"], 2.0)
    sd = {"x." + k: v for k, v in sub.items()}
    W, T = cfg["width"], 260
    h = torch.randn(T, W, generator=torch.Generator().manual_seed(8)) * 0.3
    for i_star in (230, 259):
        h = _aim_query(sd, "x.", m, h, i_star, j_star, 1e-5, 25.0)
    h = h.to(dtype)
    ref = O.latent_attention_mixer(h.double(), sd, "x.", m, 1e-5)
    # the far key carries (nearly) all of the weight in the oracle: the test would notice its loss
    without = h.double().clone()
    without[j_star] = 0.0
    assert rel(O.latent_attention_mixer(without, sd, "x.", m, 1e-5)[[230, 259]], ref[[230, 259]]) > 0.15
    cache = CacheManager(320, 2, dev)
    cache.free_pages = [3, 0, 4, 1, 2]                              # pages out of order
    mix = LatentAttention("a", W, m["heads"], m["dim"], m["vdim"], m["kv_rank"], m["scale"], 1e-5).load(lambda n: sub[n], "", dtype, dev)
    mix.bind(cache, dtype)
    cache.admit("s")
    got, at = [], 0
    for n in [129, 110] + [1] * 21:                                 # 230 inside a portion, 259 decoded alone
        pos0, slot, pages = cache.extend("s", n)
        got.append(mix.forward(h[at:at + n].to(dev).contiguous(), one_seq_batch(n, dev, pos0, slot, pages=list(pages))))
        at += n
    got = torch.cat(got)
    assert rel(got[[230, 259]], ref[[230, 259]]) < tol(dtype)
    assert rel(got, ref) < tol(dtype)


def test_sink_counts_once_and_has_no_value(dev):
    """a large sink takes most of the weight away; the first token (one key) shows it best: out = v_0 * e^s / (e^s + e^sink)"""
    from zhilight_amd.cache import CacheManager
    from zhilight_amd.mixers import LatentAttention
    cfg = O.small_config(("latent_attention",))
    m = cfg["layers"][0]["mixer"]
    sub, _ = mixer_sd(cfg, 0, 9)
    outs = []
    for sink in (-30.0, 3.0):
        sub["sink"] = torch.full_like(sub["sink"], sink)
        h = torch.randn(5, cfg["width"], generator=torch.Generator().manual_seed(10))
        ref = O.latent_attention_mixer(h.double(), {"x." + k: v for k, v in sub.items()}, "x.", m, 1e-5)
        cache = CacheManager(64, 1, dev)
        mix = LatentAttention("a", cfg["width"], m["heads"], m["dim"], m["vdim"], m["kv_rank"], m["scale"], 1e-5).load(lambda n: sub[n], "", torch.float32, dev)
        mix.bind(cache, torch.float32)
        cache.admit("s")
        pos0, slot, pages = cache.extend("s", 5)
        got = mix.forward(h.to(dev), one_seq_batch(5, dev, pos0, slot, pages=list(pages)))
        assert rel(got, ref) < F32_TOL
        outs.append(got)
    assert rel(outs[1], outs[0]) > 0.3


# ------------------------------------------------------------------------------------------------------------------------------------
# the model through the engine
# ------------------------------------------------------------------------------------------------------------------------------------
CONFIGS = {
    "mixed_order": dict(order=("latent_attention", "mamba2", "latent_attention")),
    "mamba_first": dict(order=("mamba2", "latent_attention", "mamba2", "mamba2"), width=100, seed_sizes=1, no_mlp_at=(1,)),
    "odd_width": dict(order=("latent_attention", "mamba2"), width=90, vocab=131, seed_sizes=2, no_mlp_at=(0, 1)),
}


@pytest.fixture(scope="module", params=sorted(CONFIGS))
def case(request):
    cfg = O.small_config(**CONFIGS[request.param])
    if request.param == "odd_width":
        cfg["layers"][0]["mixer"].update(heads=1, dim=24, vdim=8, kv_rank=33)
        cfg["layers"][1]["mixer"].update(heads=6, groups=3, vdim=8, state=20, norm_groups=2, conv=5)
    sd = O.random_weights(cfg, seed=11)
    toks = tokens_of(cfg, 200, 12)
    return cfg, sd, toks, O.forward(cfg, sd, toks)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_whole_prompt(dev, case, dtype):
    cfg, sd, toks, ref = case
    eng = make(cfg, sd, dtype, dev)
    assert rel(run_portions(eng, "a", toks, [len(toks)]), ref) < tol(dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_prefill_then_token_by_token(dev, case, dtype):
    cfg, sd, toks, ref = case
    eng = make(cfg, sd, dtype, dev)
    got = run_portions(eng, "a", toks, [40] + [1] * 160)            # long decoding: 160 single tokens, across page borders
    assert rel(got, ref) < tol(dtype)
    assert rel(got[-20:], ref[-20:]) < tol(dtype)
    got1 = run_portions(eng, "b", toks[:70], [1] * 70)              # from the very first token
    assert rel(got1, ref[:70]) < tol(dtype)


@pytest.mark.parametrize("portions", [[2] * 100, [3, 2, 59, 1, 64, 7, 64], [64, 64, 64, 8], [199, 1], [1, 199]])
def test_portions_do_not_change_fp32_logits(dev, case, portions):
    cfg, sd, toks, ref = case
    eng = make(cfg, sd, torch.float32, dev)
    assert rel(run_portions(eng, "a", toks, portions), ref) < F32_TOL


def test_portions_bf16(dev, case):
    cfg, sd, toks, ref = case
    eng = make(cfg, sd, torch.bfloat16, dev)
    assert rel(run_portions(eng, "a", toks, [5, 2, 60, 3, 130]), ref) < BF16_TOL


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_unequal_batch_equals_each_alone_and_reuses_pages_and_slots(dev, case, dtype):
    """four requests of unequal length in mixed steps (portions beside single tokens, one request pausing), in a pool that holds them only
    because finished requests give pages and slots back; every request's logits equal what it gets alone in a fresh engine"""
    from zhilight_amd.engine import Entry
    cfg, sd, toks, ref = case
    lens = {"a": 200, "b": 37, "c": 130, "d": 66, "e": 90}
    seqs = {k: tokens_of(cfg, n, 20 + i) if k != "a" else toks for i, (k, n) in enumerate(lens.items())}
    alone = {}
    for k, t in seqs.items():
        alone[k] = run_portions(make(cfg, sd, dtype, dev), k, t, [len(t)])
    assert rel(alone["a"], ref) < tol(dtype)
    eng = make(cfg, sd, dtype, dev, max_tokens=9 * 64, max_seqs=4)  # 12 pages in all; at most 8 at a time
    for layer in eng.model.layers:                                  # state-space layers: portions above 24 tokens in segments,
        if hasattr(layer.mixer, "scan_segment"):                    # beside shorter portions and single tokens in the same step
            layer.mixer.scan_segment = 24
    plan = [
        [("a", 50), ("b", 30), ("c", 2)],
        [("a", 1), ("b", 7), ("c", 100)],                           # b ends here
        [("a", 60), ("c", 1), ("d", 3)],                            # d takes b's slot
        [("a", 1), ("d", 63)],                                      # c pauses
        [("a", 80), ("c", 27)],                                     # c ends
        [("a", 8), ("e", 64)],                                      # a ends; e takes a freed slot and freed pages
        [("e", 26)],
    ]
    at = {k: 0 for k in seqs}
    got = {k: [] for k in seqs}
    slots = {}
    for step in plan:
        entries = [Entry(k, seqs[k][at[k]:at[k] + n], list(range(n))) for k, n in step]
        lg = eng.run_step(entries)
        row = 0
        for k, n in step:
            slots[k] = eng.cache.seqs[k]["slot"]
            got[k].append(lg[row:row + n])
            row += n
            at[k] += n
            if at[k] == len(seqs[k]):
                eng.release(k)
    assert slots["d"] == slots["b"] and slots["e"] in (slots["b"], slots["c"])           # slots of finished requests, taken again
    assert not eng.cache.seqs and len(eng.cache.free_pages) == 9 and len(eng.cache.free_slots) == 4
    for k in seqs:
        g = torch.cat(got[k])
        assert at[k] == len(seqs[k])
        assert rel(g, alone[k]) < (1e-5 if dtype == torch.float32 else 2e-2), k


def test_reused_pages_give_the_same_bits(dev, case):
    cfg, sd, toks, _ = case
    eng = make(cfg, sd, torch.bfloat16, dev, max_tokens=256, max_seqs=1)
    first = run_portions(eng, "x", toks[:150], [150])
    run_portions(eng, "y", tokens_of(cfg, 250, 30), [250])           # dirties every page and the only slot
    again = run_portions(eng, "z", toks[:150], [150])
    assert torch.equal(first, again)


def test_greedy_generation_through_the_scheduler(dev, case):
    """Engine.generate: several prompts of unequal length under a small step budget (prompts are cut into portions, decodes ride along);
    every generated token is the oracle's greedy choice for that request's own history"""
    from zhilight_amd.engine import SamplingParams
    cfg, sd, toks, _ = case
    prompts = [toks[:70], toks[100:103], toks[50:51], tokens_of(cfg, 45, 31), tokens_of(cfg, 9, 32), tokens_of(cfg, 130, 33)]
    eng = make(cfg, sd, torch.float32, dev, max_tokens=8 * 64, max_seqs=3, max_step_tokens=48)
    outs = eng.generate(prompts, SamplingParams(max_new_tokens=12))
    assert not eng.cache.seqs and len(eng.cache.free_pages) == 8
    for p, o in zip(prompts, outs):
        assert len(o) == 12
        full = O.forward(cfg, sd, p + o)
        for i, t in enumerate(o):
            row = full[len(p) - 1 + i]
            assert float(row.max() - row[t]) <= 1e-4 * float(row.abs().max()), (len(p), i)


def test_seeded_sampling_is_reproducible_and_respects_top_k(dev, case):
    from zhilight_amd.engine import SamplingParams
    cfg, sd, toks, _ = case
    runs = []
    for _ in range(2):
        eng = make(cfg, sd, torch.float32, dev)
        runs.append(eng.generate([toks[:20], toks[30:45]], SamplingParams(max_new_tokens=8, temperature=0.8, top_k=5, top_p=0.9, seed=3)))
    assert runs[0] == runs[1]
    p, o = toks[:20], runs[0][0]
    full = O.forward(cfg, sd, p + o)
    for i, t in enumerate(o):
        row = full[len(p) - 1 + i]
        assert t in torch.topk(row, 6).indices.tolist()


MEDIUM = {
    "a": dict(width=256, vocab=300, att=dict(dim=64, heads=6, kv_rank=160, scale=0.125, vdim=48),
              ssm=dict(conv=4, groups=2, heads=8, norm_groups=2, state=128, vdim=64), ff=520, order="asa"),
    "b": dict(width=384, vocab=520, att=dict(dim=128, heads=20, kv_rank=512, scale=0.09, vdim=128),
              ssm=dict(conv=2, groups=3, heads=6, norm_groups=1, state=64, vdim=32), ff=1000, order="sas"),
    "c": dict(width=200, vocab=210, att=dict(dim=40, heads=5, kv_rank=72, scale=0.2, vdim=72),
              ssm=dict(conv=3, groups=1, heads=3, norm_groups=3, state=48, vdim=20), ff=264, order="aas"),
}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("name", sorted(MEDIUM))
def test_medium_sizes_whole_chunked_and_decoded(dev, name, dtype):
    """sizes that take the other instantiations of the kernels (head sizes 40 .. 128, ranks 72 .. 512, more than 16 heads, state-space heads of
    20 .. 64 columns with 48 .. 128 states): a whole prompt, portions with single tokens between them, and a batch of two"""
    from zhilight_amd.engine import Entry
    z = MEDIUM[name]
    layers = [{"type": "latent_attention" if ch == "a" else "mamba2", "mixer": dict(z["att"] if ch == "a" else z["ssm"]),
               "mlp": None if i == 1 and name == "b" else {"ff": z["ff"], "kind": "dense"}} for i, ch in enumerate(z["order"])]
    cfg = {"architecture": "Tupitar", "embedding": {"scale": 11.0}, "layers": layers, "max_positions": 400, "norm": {"eps": 1e-6},
           "vocab": z["vocab"], "width": z["width"]}
    sd = O.random_weights(cfg, seed=41)
    toks, other = tokens_of(cfg, 150, 42), tokens_of(cfg, 70, 43)
    ref, ref_other = O.forward(cfg, sd, toks), O.forward(cfg, sd, other)
    eng = make(cfg, sd, dtype, dev, max_tokens=512)
    assert rel(run_portions(eng, "w", toks, [150]), ref) < tol(dtype)
    assert rel(run_portions(eng, "c", toks, [37, 1, 1, 30, 2, 65, 1, 13]), ref) < tol(dtype)
    got = {"x": [], "y": []}
    at = {"x": 0, "y": 0}
    seqs = {"x": toks, "y": other}
    for step in ([("x", 100), ("y", 3)], [("x", 1), ("y", 66)], [("x", 49), ("y", 1)]):
        lg = eng.run_step([Entry(k, seqs[k][at[k]:at[k] + n], list(range(n))) for k, n in step])
        row = 0
        for k, n in step:
            got[k].append(lg[row:row + n])
            row += n
            at[k] += n
    assert rel(torch.cat(got["x"]), ref) < tol(dtype) and rel(torch.cat(got["y"]), ref_other) < tol(dtype)
