"""Host-side pieces of Gaparax that need no GPU: configuration reader and registry, what the model asks of the cache manager, the
distance-bias table and the rescaled rotary frequencies, rows attached to an input projection, and the restatement's own consistency
(its mechanisms against direct per-token definitions and closed forms)."""
import math

import pytest
import torch

import gaparax_oracle as O

EPS = 1e-5
F64 = torch.float64


def small_config():
    att = {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 8, "scale": 0.25, "softcap": 12.0, "bias_max": 30, "mask": {"size": 20}}
    lat = {"heads": 2, "dim": 8, "rot_dim": 4, "vdim": 8, "kv_rank": 12, "scale": 0.3,
           "rot": {"base": 50.0, "dims": 4, "scaling": {"factor": 4.0, "original": 16, "fast": 4.0, "slow": 1.0}}}
    moe = {"kind": "moe", "expert": {"ff": 16}, "router": {"experts": 6, "top": 2, "scale": 2.0, "groups": {"count": 3, "keep": 2}}}
    return {"architecture": "Gaparax", "vocab": 50, "width": 32, "streams": 2, "norm": {"eps": EPS},
            "layers": [{"type": "attention", "mixer": dict(att), "mlp": {"kind": "dense", "ff": 48}},
                       {"type": "latent_attention", "mixer": lat, "mlp": moe},
                       {"type": "attention", "mixer": dict(att, kv_heads=4), "mlp": None}]}


def test_registry_and_configuration():
    from zhilight_amd import registry
    from zhilight_amd._lib import ZLError
    from zhilight_amd.gaparax import GaparaxConfig, GaparaxModel
    cfg = small_config()
    assert registry.model_class(cfg) is GaparaxModel and "gaparax" in registry.registered()
    c = GaparaxConfig.from_dict(cfg)
    assert c.layers[2].mlp is None and c.eps == EPS and c.streams == 2 and len(c.layers) == 3 and (c.vocab, c.width) == (50, 32)
    for breakage in (lambda d: d["layers"][0].update(type="something else"),
                     lambda d: d["layers"][1]["mlp"].update(kind="sparse"),
                     lambda d: d.pop("norm"),
                     lambda d: d.pop("streams"),
                     lambda d: d.update(streams=9),
                     lambda d: d.pop("vocab")):
        bad = small_config()
        breakage(bad)
        with pytest.raises(ZLError):
            GaparaxConfig.from_dict(bad)
    bad = small_config()
    bad["layers"][1]["mixer"]["rot"]["dims"] = 2                  # the rotated part is rotated as a whole
    with pytest.raises(ZLError):
        GaparaxModel.from_config(bad, dtype="float32", device="cpu")


def test_model_layout_from_the_configuration():
    """built on the CPU without weights: which mixers and feed-forwards exist, with which constants, and what the cache manager is asked for"""
    from zhilight_amd.cache import CacheManager
    from zhilight_amd.gaparax import GaparaxModel
    from zhilight_amd.mixers import LatentAttention, PlainFF, RoutedExpertsFF, WindowAttention
    model = GaparaxModel.from_config(small_config(), dtype="float32", device="cpu")
    assert [type(l.mixer) for l in model.layers] == [WindowAttention, LatentAttention, WindowAttention]
    assert [type(l.ff) for l in model.layers] == [PlainFF, RoutedExpertsFF, type(None)]
    a = model.layers[0].mixer
    assert a.sigmoid and a.chunk == 20 and a.window == 0 and a.qk_norm and a.norm_weight and a.has_head_scale and a.has_gate and not a.has_sink
    assert (a.softcap, a.rel_far, a.rot_dims, a.heads, a.kv_heads, model.layers[2].mixer.kv_heads) == (12.0, 30, 0, 4, 2, 4)
    la = model.layers[1].mixer
    assert la.has_sink and not la.has_gate and la.window == 0 and la.rot_layout == "half" and la.rot_scaling["factor"] == 4.0
    ff = model.layers[1].ff
    assert (ff.score, ff.group_top, ff.act, ff.renorm, ff.has_correction, ff.groups, ff.keep, ff.top, ff.weight_scale) == \
        ("softmax", 1, "silu", False, False, 3, 2, 2, 2.0)
    assert model.layers[0].ff.act == "relu2" and model.layers[2].port2 is None and model.layers[0].port2.n == 2
    cache = model.bind_cache(CacheManager(256, 3, "cpu"))
    assert sorted(cache.planes) == ["l0.mix.k", "l0.mix.v", "l1.mix.latent", "l2.mix.k", "l2.mix.v"] and not cache.states
    assert cache.planes["l1.mix.latent"].shape == (4, 64, 12 + 4)           # only the latent and the shared rotated key part are cached
    assert cache.planes["l0.mix.k"].shape == (4, 64, 2 * 16) and cache.planes["l2.mix.v"].shape == (4, 64, 4 * 8)


def test_side_rows_ride_in_the_input_projection():
    from zhilight_amd._lib import ZLError
    from zhilight_amd.mixers import PlainFF
    ff = PlainFF(8, 12)
    ff.w_up, ff.w_down = torch.zeros(12, 8), torch.zeros(8, 12)
    ff.attach_side(torch.ones(5, 8))
    assert ff.side_col0 == 12 and ff.w_up.shape == (17, 8) and bool((ff.w_up[12:] == 1).all())
    with pytest.raises(ZLError):
        ff.attach_side(torch.ones(5, 7))


def test_distance_bias_table_against_the_bucket_definition():
    from zhilight_amd._lib import ZLError
    from zhilight_amd.mixers import distance_bias_table
    rows, far = 12, 150
    table = torch.arange(rows * 2, dtype=torch.float32).reshape(rows, 2)
    got = distance_bias_table(table, far, 0, "cpu")
    half = rows // 2
    for n in range(far + 1):
        row = n if n < half else min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))
        assert got[0, n] == table[row, 0] and got[1, n] == table[row, 1]
        assert row == O.distance_bucket(n, rows, far)
    assert O.distance_bucket(5, rows, far) == 5 and O.distance_bucket(6, rows, far) == 6 and O.distance_bucket(far, rows, far) == rows - 1
    assert [O.distance_bucket(n, rows, far) for n in (10, 11, 149, 10 ** 6)] == [6, 7, 11, 11]
    assert distance_bias_table(table, far, 70, "cpu").shape == (2, 70)       # no query looks further than its chunk
    with pytest.raises(ZLError):
        distance_bias_table(table, 6, 0, "cpu")                             # the logarithmic half needs a largest distance beyond the exact half
    bias = O.distance_bias(5, table.double(), far)
    assert bias.shape == (2, 5, 5) and float(bias[1, 4, 1]) == float(table[3, 1]) and float(bias[0, 1, 3]) == 0.0


def test_rescaled_frequencies():
    from zhilight_amd.mixers import scaled_frequencies
    dims, base = 24, 15000.0
    sc = {"factor": 5.0, "original": 512, "fast": 24.0, "slow": 1.5}
    f, gain = O.scaled_frequencies(dims, base, sc)
    plain, one = O.scaled_frequencies(dims, base, None)
    assert one == 1.0 and torch.allclose(plain, torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64))
    assert abs(gain - (0.1 * math.log(5.0) + 1.0)) < 1e-15
    # a pair that turns more than `fast` times over the original context keeps its frequency, one that turns less than `slow` times is divided
    turns = plain * 512 / (2 * math.pi)
    for i in range(dims // 2):
        if turns[i] > 24.0 * 1.7:
            assert f[i] == plain[i]
        if turns[i] < 1.5 / 1.7:
            assert abs(float(f[i] / plain[i]) - 1.0 / 5.0) < 1e-12
        assert plain[i] / 5.0 - 1e-18 <= f[i] <= plain[i] + 1e-18
    assert bool((f[1:] < f[:-1]).all())
    got, g2 = scaled_frequencies(dims, base, sc)
    assert float(((got.double() - f) / f).abs().max()) < 1e-7 and abs(g2 - gain) < 1e-15
    # lo = hi: the ramp's width falls back to 0.001 -- a step
    f2, _ = O.scaled_frequencies(8, 100.0, {"factor": 2.0, "original": 64, "fast": 1.0, "slow": 1.0})
    assert bool(((f2 == O.scaled_frequencies(8, 100.0, None)[0]) | (f2 == O.scaled_frequencies(8, 100.0, None)[0] / 2.0)).all())


def test_rotation_of_half_pairs_with_a_gain():
    T, H, size, dims = 5, 2, 10, 6
    x = torch.randn(T, H, size, generator=torch.Generator().manual_seed(2), dtype=F64)
    pos = torch.tensor([0, 1, 2, 40, 1000])
    freq = torch.tensor([1.0, 0.3, 0.01], dtype=F64)
    got = O.rotate_half(x, pos, dims, freq, 1.25)
    for t in range(T):
        for i in range(dims // 2):
            a = float(pos[t]) * float(freq[i])
            u, v = x[t, :, i], x[t, :, i + dims // 2]
            assert torch.allclose(got[t, :, i], 1.25 * (u * math.cos(a) - v * math.sin(a)), atol=1e-12)
            assert torch.allclose(got[t, :, i + dims // 2], 1.25 * (v * math.cos(a) + u * math.sin(a)), atol=1e-12)
    assert torch.equal(got[..., dims:], x[..., dims:]) and torch.allclose(got[0, :, :dims], 1.25 * x[0, :, :dims])
    # scores depend on the distance only
    q, k = torch.randn(1, 1, dims, dtype=F64), torch.randn(1, 1, dims, dtype=F64)
    s = [float((O.rotate_half(q, torch.tensor([p + 7]), dims, freq, 1.25) * O.rotate_half(k, torch.tensor([p]), dims, freq, 1.25)).sum()) for p in (0, 3, 90)]
    assert abs(s[0] - s[1]) < 1e-9 and abs(s[0] - s[2]) < 1e-9


def test_chunks_sink_and_sigmoid_weights():
    vis = O.chunk_visible(10, 4)
    assert vis[9].tolist() == [False] * 8 + [True, True] and vis[7].tolist() == [False] * 4 + [True] * 4 + [False] * 2
    assert vis[4].tolist() == [False] * 4 + [True] + [False] * 5 and vis[3].tolist() == [True] * 4 + [False] * 6
    assert O.chunk_visible(4, 0).tolist() == torch.tril(torch.ones(4, 4, dtype=torch.bool)).tolist()
    w = O.sink_softmax(torch.zeros(1, 1, dtype=F64), torch.ones(1, 1, dtype=torch.bool), torch.tensor(math.log(3.0), dtype=F64))
    assert abs(float(w) - 0.25) < 1e-15                                       # one key of score 0 beside a sink of weight 3
    # sigmoid weights: two visible keys of score 0 with offset 0 weigh one half EACH (nothing is normalised); the cap bounds a score
    q, k, v = torch.zeros(2, 1, 2, dtype=F64), torch.zeros(2, 1, 2, dtype=F64), torch.ones(2, 1, 3, dtype=F64)
    out = O.sigmoid_attention(q, k, v, 1.0, torch.ones(1, dtype=F64), 0.0, None, O.chunk_visible(2, 0), torch.zeros(1, dtype=F64))
    assert torch.allclose(out[:, 0, 0], torch.tensor([0.5, 1.0], dtype=F64))
    q2, k2 = torch.full((1, 1, 1), 100.0, dtype=F64), torch.full((1, 1, 1), 100.0, dtype=F64)
    capped = O.sigmoid_attention(q2, k2, torch.ones(1, 1, 1, dtype=F64), 1.0, torch.ones(1, dtype=F64), 2.0, None, O.chunk_visible(1, 0), torch.tensor([-2.0], dtype=F64))
    assert abs(float(capped) - 0.5) < 1e-9                                    # the score 10000 is capped at 2, the offset takes it to 0


def test_router_against_brute_force():
    r = {"experts": 6, "top": 2, "scale": 1.75, "groups": {"count": 3, "keep": 2}}
    g = torch.Generator().manual_seed(6)
    sd = {"router": torch.randn(6, 8, generator=g, dtype=F64)}
    h = torch.randn(30, 8, generator=g, dtype=F64)
    margins = []
    ids, wts = O.route(h, sd, "", r, margins)
    s = torch.softmax(h @ sd["router"].T, -1)
    for t in range(30):
        groups = sorted(range(3), key=lambda i: -max(s[t, 2 * i], s[t, 2 * i + 1]))[:2]
        allowed = [2 * i + j for i in groups for j in (0, 1)]
        best = sorted(allowed, key=lambda i: -s[t, i])[:2]
        assert ids[t].tolist() == best
        assert torch.allclose(wts[t], 1.75 * s[t, best])
    assert float(wts.sum(-1).max()) > 1.0 and len(margins) == 1 and margins[0] > 0


def test_streams_reduce_to_a_plain_residual():
    """one stream with read coefficient 1, mixing 1 and write factor 1 is x + gate * sublayer(norm(x))"""
    cfg = small_config()
    cfg["streams"] = 1
    cfg["layers"] = cfg["layers"][:1]
    sd = O.random_weights(cfg, 4)
    for q in (1, 2):
        for n in ("in", "out", "mix"):
            sd[f"l0.hc{q}.{n}"] = torch.ones_like(sd[f"l0.hc{q}.{n}"])
    toks = [3, 9, 1, 40, 7]
    layers = []
    O.model(toks, sd, cfg, layers)
    x = sd["embed"].double()[toks]
    h = O.rms_norm(x, sd["l0.norm1"].double(), EPS)
    x = x + O.sigmoid_attention_mixer(h, sd, "l0.mix.", cfg["layers"][0]["mixer"], EPS) * torch.sigmoid(h @ sd["l0.rg1"].double().T + sd["l0.rg1.b"].double())
    h = O.rms_norm(x, sd["l0.norm2"].double(), EPS)
    x = x + O.dense_ff(h, sd, "l0.mlp.") * torch.sigmoid(h @ sd["l0.rg2"].double().T + sd["l0.rg2.b"].double())
    assert torch.allclose(layers[0], x, atol=1e-10)


def test_model_restatement_is_causal():
    cfg = small_config()
    sd = O.random_weights(cfg, 7)
    toks = torch.randint(0, 50, (40,), generator=torch.Generator().manual_seed(8)).tolist()
    layers = []
    full = O.model(toks, sd, cfg, layers)
    part = O.model(toks[:25], sd, cfg)
    assert torch.allclose(full[:25], part, atol=1e-9) and len(layers) == 3 and layers[0].shape == (40, 32)
    fixed = O.random_weights(cfg, 7, fixed_choice=True)
    margins = []
    O.model(toks, fixed, cfg, None, margins)
    assert min(margins) > 0.1
