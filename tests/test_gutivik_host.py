"""Host-side pieces of Gutivik that need no GPU: configuration reader and registry, what the model asks of the cache manager, which layer
lends its values to which, the widened up-projections of the latent attention, and the restatement's own consistency (its mechanisms
against direct per-token definitions and closed forms)."""
import math

import pytest
import torch

import gutivik_oracle as O

EPS = 1e-5
F64 = torch.float64


def small_config():
    att = {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 8, "conv": 3, "rot": {"dims": 8, "base": 100.0}, "mask": {"size": 20, "keep_first": 2},
           "scale": 0.25, "v_mix": True}
    lat = {"heads": 2, "dim": 8, "rot_dim": 4, "vdim": 8, "kv_rank": 12, "mask": {"size": 9}, "rot": {"base": 50.0, "dims": 4}, "scale": 0.3}
    gla = {"heads": 2, "dim": 8, "vdim": 4, "tau": 4.0}
    moe = {"kind": "moe", "expert": {"ff": 16, "limit": 1.0}, "router": {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 2}}}
    return {"architecture": "Gutivik", "vocab": 50, "width": 32, "norm": {"eps": EPS}, "logit_scale": 0.5, "logit_softcap": 10.0,
            "layers": [{"type": "attention", "mixer": dict(att), "mlp": {"kind": "dense", "ff": 48}},
                       {"type": "latent_attention", "mixer": lat, "mlp": moe},
                       {"type": "gla", "mixer": gla, "mlp": None},
                       {"type": "attention", "mixer": dict(att, v_mix=False), "mlp": None},
                       {"type": "attention", "mixer": dict(att), "mlp": dict(moe)}]}


def test_registry_and_configuration():
    from zhilight_amd import registry
    from zhilight_amd._lib import ZLError
    from zhilight_amd.gutivik import GutivikConfig, GutivikModel
    cfg = small_config()
    assert registry.model_class(cfg) is GutivikModel and "gutivik" in registry.registered()
    c = GutivikConfig.from_dict(cfg)
    assert c.layers[2].mlp is None and c.eps == EPS and c.logit_scale == 0.5 and c.logit_softcap == 10.0 and len(c.layers) == 5
    plain = dict(cfg)
    plain.pop("logit_scale"), plain.pop("logit_softcap")
    assert GutivikConfig.from_dict(plain).logit_scale == 1.0 and GutivikConfig.from_dict(plain).logit_softcap == 0.0
    for breakage in (lambda d: d["layers"][0].update(type="something else"),
                     lambda d: d["layers"][1]["mlp"].update(kind="sparse"),
                     lambda d: d.pop("norm"),
                     lambda d: d.pop("vocab")):
        bad = small_config()
        breakage(bad)
        with pytest.raises(ZLError):
            GutivikConfig.from_dict(bad)


def test_model_layout_from_the_configuration():
    """built on the CPU without weights: which mixers exist, who lends its values to whom, what the cache manager is asked for"""
    from zhilight_amd.cache import CacheManager
    from zhilight_amd.gutivik import GutivikModel
    from zhilight_amd.mixers import GatedFF, GatedLinearAttention, LatentAttention, RoutedExpertsFF, WindowAttention
    cfg = small_config()
    model = GutivikModel.from_config(cfg, dtype="float32", device="cpu")
    assert [type(l.mixer) for l in model.layers] == [WindowAttention, LatentAttention, GatedLinearAttention, WindowAttention, WindowAttention]
    assert [type(l.ff) for l in model.layers] == [GatedFF, RoutedExpertsFF, type(None), type(None), RoutedExpertsFF]
    a0, a3, a4 = model.layers[0].mixer, model.layers[3].mixer, model.layers[4].mixer
    assert a0.v_mix and a0.v_mix_source is None                  # the first blending layer lends, the later ones borrow from IT
    assert not a3.v_mix and a3.v_mix_source is None
    assert a4.v_mix and a4.v_mix_source is a0
    assert a0.interleaved and a0.has_sink and a0.has_bias and a0.taps == 3 and a0.keep_first == 2 and a0.window == 20 and not a0.qk_norm
    ff = model.layers[1].ff
    assert (ff.score, ff.group_top, ff.act, ff.renorm, ff.groups, ff.keep, ff.top, ff.limit) == ("sigmoid", 2, "swish_clamp", True, 3, 2, 2, 1.0)
    cache = model.bind_cache(CacheManager(256, 3, "cpu"))
    assert sorted(cache.planes) == ["l0.mix.k", "l0.mix.v", "l1.mix.latent", "l3.mix.k", "l3.mix.v", "l4.mix.k", "l4.mix.v"]
    assert cache.planes["l1.mix.latent"].shape == (4, 64, 12 + 4)           # only the latent and the shared rotated key part are cached
    assert cache.planes["l0.mix.k"].shape == (4, 64, 2 * 16) and cache.planes["l0.mix.v"].shape == (4, 64, 2 * 8)
    assert cache.states["l0.mix.conv"].shape == (3, 2, 4 * 16 + 2 * 16 + 2 * 8)    # the last taps - 1 projected rows of q | k | v
    assert cache.states["l2.mix.S"].shape == (3, 2, 8, 4) and cache.states["l2.mix.S"].dtype == torch.float32


def test_widened_up_projections_reproduce_keys_and_values():
    from zhilight_amd.mixers import LatentAttention
    H, d, r, v, R = 3, 6, 4, 5, 10
    g = torch.Generator().manual_seed(1)
    mix = LatentAttention("m", 16, H, d, v, R, 0.3, EPS, sink=False, gate=False, rot_dim=r, rot_base=100.0, window=7)
    uk, uv = torch.randn(H * d, R, generator=g, dtype=F64), torch.randn(H * v, R, generator=g, dtype=F64)
    k2, v2 = mix._widen(uk, uv)
    row = torch.randn(9, R + r, generator=g, dtype=F64)                     # cached rows [latent | rotated key part]
    keys = (row @ k2.T).reshape(9, H, d + r)
    assert torch.equal(keys[..., :d], (row[:, :R] @ uk.T).reshape(9, H, d))
    assert torch.equal(keys[..., d:], row[:, None, R:].expand(9, H, r))
    assert torch.equal(row @ v2.T, row[:, :R] @ uv.T)
    assert (mix.qdim, mix.row) == (d + r, R + r)


def test_rotation_of_neighbouring_pairs():
    T, H, size, dims, base = 5, 2, 10, 6, 50.0
    x = torch.randn(T, H, size, generator=torch.Generator().manual_seed(2), dtype=F64)
    pos = torch.tensor([0, 1, 2, 40, 1000])
    got = O.rotate_pairs(x, pos, dims, base)
    for t in range(T):
        for i in range(dims // 2):
            a = float(pos[t]) * base ** (-2.0 * i / dims)
            u, v = x[t, :, 2 * i], x[t, :, 2 * i + 1]
            assert torch.allclose(got[t, :, 2 * i], u * math.cos(a) - v * math.sin(a), atol=1e-12)
            assert torch.allclose(got[t, :, 2 * i + 1], v * math.cos(a) + u * math.sin(a), atol=1e-12)
    assert torch.equal(got[..., dims:], x[..., dims:]) and torch.equal(got[0], x[0])
    # scores depend on the distance only
    q, k = torch.randn(1, 1, dims, dtype=F64), torch.randn(1, 1, dims, dtype=F64)
    s = [float((O.rotate_pairs(q, torch.tensor([p + 7]), dims, base) * O.rotate_pairs(k, torch.tensor([p]), dims, base)).sum()) for p in (0, 3, 90)]
    assert abs(s[0] - s[1]) < 1e-9 and abs(s[0] - s[2]) < 1e-9


def test_short_convolution_against_conv1d():
    g = torch.Generator().manual_seed(3)
    u, w = torch.randn(12, 5, generator=g, dtype=F64), torch.randn(5, 4, generator=g, dtype=F64)
    ref = torch.nn.functional.conv1d(torch.nn.functional.pad(u.T[None], (3, 0)), w[:, None, :], groups=5)[0].T
    assert torch.allclose(O.short_conv(u, w), ref, atol=1e-12)
    assert torch.allclose(O.short_conv(u, w)[0], w[:, 3] * u[0])              # the last tap is the current token's


def test_visibility_and_sink():
    vis = O.visible(10, 3, 2)
    assert vis[9].tolist() == [True, True, False, False, False, False, False, True, True, True]
    assert vis[2].tolist() == [True, True, True] + [False] * 7 and vis[0].tolist() == [True] + [False] * 9
    assert O.visible(4, 0, 0).tolist() == torch.tril(torch.ones(4, 4, dtype=torch.bool)).tolist()
    q, k, v = torch.zeros(1, 1, 2, dtype=F64), torch.zeros(1, 1, 2, dtype=F64), torch.ones(1, 1, 3, dtype=F64)
    out = O.softmax_attention(q, k, v, 1.0, torch.ones(1, 1, dtype=torch.bool), torch.tensor([math.log(3.0)], dtype=F64))
    assert torch.allclose(out, torch.full((1, 1, 3), 0.25, dtype=F64))        # one key of score 0 beside a sink of weight 3


def test_gated_linear_attention_closed_form():
    """W_a2 = 0: alpha is the same number for every channel and token, so o_t = sum_s alpha^(t-s) (q_t . k_s) v_s"""
    cfg = small_config()
    m = cfg["layers"][2]["mixer"]
    sd = {k[len("l2.mix."):]: v.double() for k, v in O.random_weights(cfg, 4).items() if k.startswith("l2.mix.")}
    sd["a2"] = torch.zeros_like(sd["a2"])
    sd["a2.b"] = torch.full_like(sd["a2.b"], 1.5)
    sd["norm"] = torch.ones_like(sd["norm"])
    h = torch.randn(7, 32, generator=torch.Generator().manual_seed(5), dtype=F64)
    H, d, e = m["heads"], m["dim"], m["vdim"]
    alpha = (1.0 / (1.0 + math.exp(-1.5))) ** (1.0 / m["tau"])
    q, k, v = (h @ sd["q"].T).reshape(7, H, d) * d ** -0.5, (h @ sd["k"].T).reshape(7, H, d), (h @ sd["v"].T).reshape(7, H, e)
    o = torch.zeros(7, H, e, dtype=F64)
    for t in range(7):
        for s in range(t + 1):
            o[t] += alpha ** (t - s) * (q[t] * k[s]).sum(-1, keepdim=True) * v[s]
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + EPS)
    g = h @ sd["g"].T
    ref = (o.reshape(7, -1) * g * torch.sigmoid(g)) @ sd["o"].T
    assert torch.allclose(O.gla_mixer(h, sd, "", m, EPS), ref, atol=1e-10)


def test_router_against_brute_force():
    f = {"router": {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 2}}, "expert": {"ff": 4, "limit": 1.0}}
    g = torch.Generator().manual_seed(6)
    sd = {"router": torch.randn(6, 8, generator=g, dtype=F64), "correction": torch.randn(6, generator=g, dtype=F64) - 1.0}
    h = torch.randn(30, 8, generator=g, dtype=F64)
    ids, wts = O.route(h, sd, "", f)
    s = torch.sigmoid(h @ sd["router"].T)
    c = s + sd["correction"]
    for t in range(30):
        groups = sorted(range(3), key=lambda i: -(c[t, 2 * i] + c[t, 2 * i + 1]))[:2]        # groups of two: the sum of both
        allowed = [2 * i + j for i in groups for j in (0, 1)]
        best = sorted(allowed, key=lambda i: -c[t, i])[:2]
        assert ids[t].tolist() == best
        assert torch.allclose(wts[t], s[t, best] / s[t, best].sum())
    assert abs(float(wts.sum(-1).mean()) - 1.0) < 1e-12


def test_model_restatement_is_causal_and_capped():
    cfg = small_config()
    sd = O.random_weights(cfg, 7)
    toks = torch.randint(0, 50, (40,), generator=torch.Generator().manual_seed(8)).tolist()
    full, streams = O.model(cfg, sd, toks)
    part, _ = O.model(cfg, sd, toks[:25])
    assert torch.allclose(full[:25], part, atol=1e-9) and len(streams) == 5 and streams[0].shape == (40, 32)
    assert float(full.abs().max()) < 10.0
