"""Gutivik on the GPU against the plain float64 restatement in tests/gutivik_oracle.py: every mechanism alone, then the model through the
engine's step function -- whole prompts, token-by-token decoding, portions down to two tokens, mixed batches, reused pages and slots, keys
far back, at page borders and just inside / outside every window and the kept first tokens, odd sizes, greedy generation through the
scheduler.  Small random configurations made here; nothing is read from disk.

fp32 serving is held to rounding of fp32 sums everywhere, bf16 serving to bf16 rounding of the matrix-product inputs.  Through a whole
model in bf16 a router sees a rounded input, and with random weights some of its choices are closer calls than that rounding; the bf16
MODEL tests therefore use correction terms that fix the order of the choice scores (the weights still follow the scores); the choice itself
is tested in fp32 through the same models and on the router alone."""
import math

import numpy as np
import pytest
import torch

import gutivik_oracle as O

pytestmark = pytest.mark.gpu

F32_TOL, BF16_TOL = 3e-5, 4e-2
EPS = 1e-5
F64 = torch.float64


def rel(got, ref):
    got, ref = got.double().cpu(), ref.double().cpu()
    return float((got - ref).pow(2).mean().sqrt() / ref.pow(2).mean().sqrt().clamp_min(1e-30))


def rel_rows(got, ref):
    got, ref = got.double().cpu(), ref.double().cpu()
    return (got - ref).pow(2).mean(-1).sqrt() / ref.pow(2).mean().sqrt().clamp_min(1e-30)


def tol(dtype):
    return F32_TOL if dtype == torch.float32 else BF16_TOL


def assert_close(got, ref, dtype, what=""):
    """all positions together within the tolerance, and no single position more than four times off"""
    e = rel_rows(got, ref)
    assert rel(got, ref) < tol(dtype) and float(e.max()) < 4 * tol(dtype), (what, rel(got, ref), float(e.max()), int(e.argmax()))


def bf(t):
    return t.to(torch.bfloat16).to(F64)


# ------------------------------------------------------------------------------------------------------------------------------------
# configurations
# ------------------------------------------------------------------------------------------------------------------------------------
def attention_cfg(heads=4, kv_heads=2, dim=40, vdim=32, conv=3, rot=16, base=10000.0, size=70, keep=3, scale=0.2, v_mix=True):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv,
                                           "rot": {"dims": rot, "base": base}, "mask": {"size": size, "keep_first": keep}, "scale": scale,
                                           "v_mix": v_mix}, "mlp": None}


def latent_cfg(heads=4, dim=24, rot=16, vdim=16, rank=48, size=50, base=5000.0, scale=0.18):
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": vdim, "kv_rank": rank,
                                                  "mask": {"size": size}, "rot": {"base": base, "dims": rot}, "scale": scale}, "mlp": None}


def gla_cfg(heads=2, dim=40, vdim=24, tau=8.0):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}, "mlp": None}


def dense(ff=144):
    return {"kind": "dense", "ff": ff}


def moe(ff=48, limit=1.0, experts=12, count=3, keep=2, top=2):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": {"experts": experts, "top": top, "groups": {"count": count, "keep": keep}}}


def with_mlp(layer, mlp):
    layer = dict(layer)
    layer["mlp"] = mlp
    return layer


def model_cfg(layers, width=96, vocab=160, scale=0.5, cap=20.0):
    return {"architecture": "Gutivik", "vocab": vocab, "width": width, "norm": {"eps": EPS}, "logit_scale": scale, "logit_softcap": cap,
            "layers": layers}


def cfg_a():
    """every mixer and both feed-forwards; the second attention layer blends the first one's values and keeps more first tokens than a page"""
    return model_cfg([with_mlp(attention_cfg(), dense()), with_mlp(latent_cfg(), moe()), gla_cfg(),
                      with_mlp(attention_cfg(dim=32, conv=2, rot=32, size=33, keep=70, scale=0.25), moe(ff=40, experts=8, count=4, keep=2, top=3)),
                      with_mlp(latent_cfg(heads=2, dim=16, rot=8, vdim=24, rank=40, size=130), dense(100))])


def cfg_odd():
    """sizes no matrix-core kernel takes, and values that a particular model may make equal or 1: heads = kv heads, one kv head, one tap,
    no convolution, rotated part = the whole head, window 1, no kept tokens, one group, one pick, an ff that is no multiple of 16"""
    return model_cfg([with_mlp(attention_cfg(heads=3, kv_heads=3, dim=20, vdim=12, conv=1, rot=20, size=1, keep=0, v_mix=False), moe(ff=20, experts=5, count=1, keep=1, top=1)),
                      with_mlp(latent_cfg(heads=3, dim=10, rot=4, vdim=7, rank=21, size=9), dense(50)),
                      with_mlp(gla_cfg(heads=1, dim=70, vdim=9, tau=1.0), moe(ff=32, experts=6, count=6, keep=4, top=3)),
                      attention_cfg(heads=4, kv_heads=1, dim=16, vdim=16, conv=0, rot=4, size=0, keep=0, v_mix=True),
                      attention_cfg(heads=2, kv_heads=1, dim=24, vdim=16, conv=4, rot=0, size=300, keep=2, v_mix=True)],
                     width=72, vocab=90, scale=1.0, cap=0.0)


def make(cfg, sd, dtype, dev, max_tokens=2048, max_seqs=4, max_step_tokens=512):
    from zhilight_amd.engine import Engine
    from zhilight_amd.registry import model_class
    model = model_class(cfg).from_config(cfg, dtype=dtype, device=dev).load_weights(sd)
    return Engine(model, max_tokens=max_tokens, max_seqs=max_seqs, max_step_tokens=max_step_tokens)


def run_portions(eng, rid, tokens, portions, release=True):
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


def new_cache(dev, max_tokens=1024, slots=3):
    from zhilight_amd.cache import CacheManager
    return CacheManager(max_tokens, slots, dev)


def feed(mixer, cache, h, portions, dev, sid="s"):
    """h through a mixer in portions; returns all outputs"""
    from zhilight_amd import seqops
    out, at = [], 0
    for n in portions:
        pos0, slot, pages = cache.extend(sid, n)
        b = seqops.RaggedBatch([(n, pos0, slot, list(pages))], cache.page_size, dev)
        out.append(mixer.forward(h[at:at + n].to(dev).contiguous(), b))
        at += n
    assert at == h.shape[0]
    return torch.cat(out)


def sub(sd, prefix):
    return {k[len(prefix):]: v for k, v in sd.items() if k.startswith(prefix)}


# ------------------------------------------------------------------------------------------------------------------------------------
# mechanisms alone
# ------------------------------------------------------------------------------------------------------------------------------------
def test_rms_norm_alone_and_fused_with_the_residual_sum(dev):
    from zhilight_amd import seqops
    g = torch.Generator().manual_seed(2)
    W = 77
    x, y = torch.randn(6, W, generator=g) + 3.0, torch.randn(6, W, generator=g) * 4 - 1.0
    w1, w2 = 0.3 * torch.randn(W, generator=g), 1.0 + 0.3 * torch.randn(W, generator=g)
    xd = x.to(dev)
    assert rel(seqops.rms_norm(xd, w1.to(dev), EPS, torch.float32, around_zero=True), O.rms_norm(x.double(), w1.double(), EPS, True)) < 1e-6
    assert rel(seqops.rms_norm(xd, w2.to(dev), EPS, torch.float32), O.rms_norm(x.double(), w2.double(), EPS, False)) < 1e-6
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=dev)
    assert rel(seqops.rms_norm(xd, w1.to(dev), EPS, torch.float32, rows=rows, around_zero=True), O.rms_norm(x.double(), w1.double(), EPS, True)[[5, 0, 5]]) < 1e-6
    new = x.double() + y.double()
    h2 = seqops.add_rms_norm(xd, y.to(dev), EPS, w1.to(dev), torch.bfloat16, around_zero=True)
    assert rel(xd, new) < 1e-7 and rel(h2, O.rms_norm(new, w1.double(), EPS, True)) < 4e-3
    assert seqops.add_rms_norm(xd, y.to(dev), EPS) is None and rel(xd, new + y.double()) < 1e-7
    # a tiny row: eps inside the root decides
    z = torch.full((1, W), 1e-4)
    assert rel(seqops.rms_norm(z.to(dev), w2.to(dev), 1e-2, torch.float32), O.rms_norm(z.double(), w2.double(), 1e-2, False)) < 1e-6


def test_scaled_and_capped_logits(dev):
    from zhilight_amd import seqops
    z = torch.linspace(-300, 300, 1001)
    assert rel(seqops.scale_softcap(z.clone().to(dev), 0.4, 25.0), 25.0 * torch.tanh(z.double() * 0.4 / 25.0)) < 1e-6
    assert rel(seqops.scale_softcap(z.clone().to(dev), 0.5, 0.0), z.double() * 0.5) < 1e-7


def test_gated_activations(dev):
    from zhilight_amd import seqops
    g = torch.Generator().manual_seed(3)
    gu = (torch.randn(5, 2 * 48, generator=g) * 3).to(dev)
    a, u = gu.double().cpu()[:, :48], gu.double().cpu()[:, 48:]
    assert rel(seqops.act_mul(gu, torch.float32, kind="gelu_tanh"), O.gelu_tanh(a) * u) < 1e-6
    lim = 1.3
    ref = torch.clamp(a, max=lim) * torch.sigmoid(1.702 * torch.clamp(a, max=lim)) * (torch.clamp(u, -lim, lim) + 1.0)
    assert rel(seqops.act_mul(gu, torch.float32, kind="swish_clamp", alpha=1.702, limit=lim), ref) < 1e-6
    assert rel(seqops.act_mul(gu, torch.float32, kind="silu"), a * torch.sigmoid(a) * u) < 1e-6
    # the packed layout: blocks of 16 gates followed by their 16 ups
    packed = torch.stack([gu[:, :48].reshape(5, 3, 16), gu[:, 48:].reshape(5, 3, 16)], dim=2).reshape(5, 96).contiguous()
    assert rel(seqops.act_mul(packed, torch.float32, kind="swish_clamp", alpha=1.702, limit=lim, block=16), ref) < 1e-6


@pytest.mark.parametrize("taps", [1, 2, 4])
def test_short_convolution_with_input_bias_in_portions(dev, taps):
    from zhilight_amd import seqops
    g = torch.Generator().manual_seed(taps)
    C, T = 300, 41
    u, w, b = torch.randn(T, C + 7, generator=g), torch.randn(C, taps, generator=g), torch.randn(C, generator=g)
    ref = O.short_conv(u[:, 3:3 + C].double() + b.double(), w.double())
    cache = new_cache(dev)
    tail = cache.add_state("t", (taps - 1, C)) if taps > 1 else None
    for attempt in range(2):                                   # the second sequence takes the slot the first one left: zeros again
        cache.admit("s")
        out, at = [], 0
        for n in (1, 1, 2, 5, 1, 3, 28):
            pos0, slot, pages = cache.extend("s", n)
            bt = seqops.RaggedBatch([(n, pos0, slot, list(pages))], 64, dev)
            out.append(seqops.short_conv(u[at:at + n].to(dev).contiguous(), 3, w.to(dev), b.to(dev), tail, bt))
            at += n
        assert rel(torch.cat(out), ref) < 1e-6, attempt
        cache.release("s")


def attention_kernels(q, k, v, window, keep, sink, scale, dtype, dev, portions, mfma=True, n_splits=None, shuffle_pages=False):
    """[q | k | v] rows through the cache-writing kernel (no rotation), the attention kernels and the merge, in portions"""
    from zhilight_amd import seqops
    T, H, d = q.shape
    G, e = k.shape[1], v.shape[2]
    cache = new_cache(dev, max_tokens=64 * ((T + 63) // 64 + 3))
    if shuffle_pages:
        cache.free_pages = cache.free_pages[::-1]
    kp, vp = cache.add_plane("k", (G * d,), dtype), cache.add_plane("v", (G * e,), dtype)
    cache.admit("s")
    rows = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], dim=1).float()
    out, at = [], 0
    for n in portions:
        pos0, slot, pages = cache.extend("s", n)
        b = seqops.RaggedBatch([(n, pos0, slot, list(pages))], 64, dev)
        proj = rows[at:at + n].to(dev).contiguous()
        seqops.rope_norm_store(proj, 0, H * d, H * d + G * d, H, G, d, e, None, 0, None, EPS, False, b, kp, vp)
        acc, ml, ns = seqops.window_attention(proj, 0, kp, vp, b, scale, window, H, G, d, e, all_kv=False, mfma=mfma, n_splits=n_splits,
                                              keep_first=keep)
        out.append(seqops.head_mix_gate(acc, ml, ns, None, None, None, 0, b, H, G, e, torch.float32, sink=None if sink is None else sink.to(dev)))
        at += n
    assert at == T
    return torch.cat(out).reshape(T, H, e)


def aimed(T, H, G, d, e, pairs, seed):
    """random queries, keys, values (bf16-representable); for every (query i, key j) of `pairs` the key j points along query i's first
    head of every group and carries a large value: the score stands out, so a mask that is one position off changes the output visibly"""
    g = torch.Generator().manual_seed(seed)
    q, k, v = bf(torch.randn(T, H, d, generator=g)), bf(torch.randn(T, G, d, generator=g)), bf(torch.randn(T, G, e, generator=g))
    for i, j in pairs:
        for c in range(G):
            qh = q[i, c * (H // G)]
            k[j, c] = bf(5.0 * qh / qh.norm() * math.sqrt(d) / 2)
            v[j, c] = bf(20.0 * torch.randn(e, generator=g))
    return q, k, v


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window,keep", [(1, 0), (2, 5), (33, 3), (64, 64), (65, 70), (100, 1)])
def test_attention_window_edges_kept_first_keys_and_sink(dev, dtype, window, keep):
    """queries aimed at the last key the window still holds, the first one it has dropped, the last kept first key and the first one that
    is not kept -- inside a portion and decoded alone -- against the float64 softmax over the visibility matrix"""
    T, H, G, d, e = 330, 4, 2, 24, 16
    portions = [150, 1, 1, 1, 60, 2, 1, 1, 64, 1, 1, 47]                      # queries 150-152, 215-216, 281-282 are single tokens
    singles = [150, 151, 215, 281, 282]
    inside = [100, 149, 160, 212, 230, 329]
    pairs = []
    for n, i in enumerate(singles + inside):
        j = [i - window + 1, i - window, keep - 1, keep][n % 4]
        if 0 <= j <= i:
            pairs.append((i, j))
    q, k, v = aimed(T, H, G, d, e, pairs, window)
    sink = torch.tensor([0.5, -1.0, 3.0, 0.0])
    scale = 0.3
    ref = O.softmax_attention(q, k, v, scale, O.visible(T, window, keep), sink.double())
    no_mask = O.softmax_attention(q, k, v, scale, O.visible(T, window + 1, keep + 1), sink.double())
    assert rel(no_mask, ref) > 0.05                                             # the aimed keys do show
    for mfma, splits in ((True, None), (False, None), (False, 3)):
        got = attention_kernels(q, k, v, window, keep, sink, scale, dtype, dev, portions, mfma=mfma, n_splits=splits, shuffle_pages=splits == 3)
        assert_close(got.reshape(T, -1), ref.reshape(T, -1), dtype, (window, keep, mfma, splits))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_one_far_key_across_pages_without_window(dev, dtype):
    T, H, G, d, e = 300, 2, 1, 32, 32
    for j in (0, 1, 63, 64, 65, 127, 128, 200):
        q, k, v = aimed(T, H, G, d, e, [(290, j), (299, j)], j)
        ref = O.softmax_attention(q, k, v, 0.25, O.visible(T, 0, 0), None)
        got = attention_kernels(q, k, v, 0, 0, None, 0.25, dtype, dev, [296, 1, 1, 1, 1], shuffle_pages=True)
        assert_close(got.reshape(T, -1), ref.reshape(T, -1), dtype, j)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("d,e", [(8, 16), (72, 48), (160, 16), (256, 128)])
def test_attention_head_sizes(dev, dtype, d, e):
    """the other instantiations of the matrix-core kernel (32-coordinate steps of the head size) and long heads in the plain kernel"""
    T, H, G = 200, 4, 2
    q, k, v = aimed(T, H, G, d, e, [(150, 101), (199, 100), (120, 2), (190, 3)], d)
    sink = torch.tensor([0.0, 1.0, -2.0, 0.5])
    ref = O.softmax_attention(q, k, v, d ** -0.5, O.visible(T, 50, 3), sink.double())
    got = attention_kernels(q, k, v, 50, 3, sink, d ** -0.5, dtype, dev, [130, 1, 1, 68])
    assert_close(got.reshape(T, -1), ref.reshape(T, -1), dtype, (d, e))


def build_mixer(layer, sd, prefix, width, dtype, dev, cache, source=None):
    from zhilight_amd import gutivik
    class L:                                                                    # what a builder looks at in the earlier layers
        def __init__(self, mixer):
            self.mixer = mixer
    mix = gutivik.MIXER_BUILDERS[layer["type"]]("m" + prefix, width, layer["mixer"], EPS, [L(source)] if source is not None else [])
    mix.load(lambda n: sd[n], prefix, dtype, dev)
    mix.bind(cache, dtype)
    return mix


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_mixer_with_convolution_rotation_and_blended_values(dev, dtype):
    W, T = 96, 200
    first, second = attention_cfg(), attention_cfg(dim=32, conv=2, rot=32, size=33, keep=70, scale=0.25)
    cfg = model_cfg([first, second])
    sd = O.random_weights(cfg, 5)
    g = torch.Generator().manual_seed(6)
    h = bf(torch.randn(T, W, generator=g))
    ref1, v1 = O.attention_mixer(h, sd, "l0.mix.", first["mixer"], EPS, None)
    ref2, _ = O.attention_mixer(h, sd, "l1.mix.", second["mixer"], EPS, v1)
    alone2, _ = O.attention_mixer(h, sd, "l1.mix.", second["mixer"], EPS, None)
    assert rel(alone2, ref2) > 0.05                                             # the blend shows
    from zhilight_amd import seqops
    for portions in ([T], [1] * 6 + [2, 3, 61, 64, 1, 1, 62]):
        cache = new_cache(dev)
        m1 = build_mixer(first, sd, "l0.mix.", W, dtype, dev, cache)
        m2 = build_mixer(second, sd, "l1.mix.", W, dtype, dev, cache, source=m1)
        assert m2.v_mix_source is m1
        cache.admit("s")
        o1, o2, at = [], [], 0
        for n in portions:
            pos0, slot, pages = cache.extend("s", n)
            b = seqops.RaggedBatch([(n, pos0, slot, list(pages))], 64, dev)
            hd = h[at:at + n].to(dev).to(dtype).contiguous()
            o1.append(m1.forward(hd, b))
            o2.append(m2.forward(hd, b))
            at += n
        assert_close(torch.cat(o1), ref1, dtype, ("first", len(portions)))
        assert_close(torch.cat(o2), ref2, dtype, ("second", len(portions)))


def latent_rows(layer, sd, p, T, pairs, seed):
    """mixer inputs h = [q | down-projection] for identity input matrices; for (i, j) in pairs query i's plain parts point along the
    up-projected key of token j, which carries a large latent"""
    m = layer["mixer"]
    H, d, r, R = m["heads"], m["dim"], m["rot_dim"], m["kv_rank"]
    g = torch.Generator().manual_seed(seed)
    h = bf(torch.randn(T, H * (d + r) + R + r, generator=g))
    q0 = H * (d + r)
    for i, j in pairs:
        c = O.rms_norm(h[j, q0:q0 + R], sd[p + "dkv.norm"].double(), EPS, False)
        kj = (c @ sd[p + "uk"].double().T).reshape(H, d)
        for hh in range(H):
            h[i, hh * (d + r):hh * (d + r) + d] = bf(4.0 * kj[hh] / kj[hh].norm() * math.sqrt(d))
            h[i, hh * (d + r) + d:(hh + 1) * (d + r)] = 0.0
    return h


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [1, 2, 40, 64, 65, 130, 0])
def test_latent_attention_rotated_part_and_window_edges(dev, dtype, window):
    layer = latent_cfg(heads=4, dim=24, rot=16, vdim=16, rank=48, size=window)
    m = layer["mixer"]
    H, d, r, R = m["heads"], m["dim"], m["rot_dim"], m["kv_rank"]
    W = H * (d + r) + R + r
    cfg = model_cfg([layer], width=W)
    sd = O.random_weights(cfg, 7)
    eye = torch.eye(W)
    sd["l0.mix.q"], sd["l0.mix.dkv"] = eye[:H * (d + r)].to(torch.bfloat16), eye[H * (d + r):].to(torch.bfloat16)
    T = 300
    portions = [140, 1, 1, 1, 70, 2, 1, 1, 83]
    singles, inside = [140, 141, 142, 214, 215], [90, 139, 150, 212, 230, 299]
    w = window if window > 0 else 250
    pairs = [(i, j) for n, i in enumerate(singles + inside) for j in [[i - w + 1, i - w][n % 2]] if 0 <= j < i]
    h = latent_rows(layer, sd, "l0.mix.", T, pairs, window)
    ref = O.latent_attention_mixer(h, sd, "l0.mix.", m, EPS)
    wrong = dict(m, mask={"size": w + 1})
    assert rel(O.latent_attention_mixer(h, sd, "l0.mix.", wrong, EPS), ref) > 0.02 or window == 0
    for prompt_kernel, mfma in ((True, True), (False, False)):
        cache = new_cache(dev)
        mix = build_mixer(layer, sd, "l0.mix.", W, dtype, dev, cache)
        mix.prompt_kernel, mix.decode_mfma = prompt_kernel, mfma
        cache.admit("s")
        got = feed(mix, cache, h.to(dtype), portions, dev)
        assert_close(got, ref, dtype, (window, prompt_kernel))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,dim,rot,vdim,rank", [(3, 64, 64, 48, 512), (2, 128, 64, 128, 64), (2, 200, 32, 72, 40), (1, 16, 8, 20, 24),
                                                     (2, 24, 8, 40, 32), (2, 100, 20, 128, 48), (2, 200, 40, 200, 48)])
def test_latent_attention_head_and_latent_sizes(dev, dtype, heads, dim, rot, vdim, rank):
    """every instantiation of the prompt kernel (key and value sizes apart) and of the single-token kernels, up to a cached row of
    512 + 64 numbers"""
    layer = latent_cfg(heads=heads, dim=dim, rot=rot, vdim=vdim, rank=rank, size=90, scale=(dim + rot) ** -0.5)
    W, T = 128, 200
    cfg = model_cfg([layer], width=W)
    sd = O.random_weights(cfg, 9)
    h = bf(torch.randn(T, W, generator=torch.Generator().manual_seed(10)))
    ref = O.latent_attention_mixer(h, sd, "l0.mix.", layer["mixer"], EPS)
    cache = new_cache(dev)
    mix = build_mixer(layer, sd, "l0.mix.", W, dtype, dev, cache)
    cache.admit("s")
    assert_close(feed(mix, cache, h.to(dtype), [120] + [1] * 20 + [60], dev), ref, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,dim,vdim,tau", [(2, 40, 24, 8.0), (1, 70, 9, 1.0), (3, 16, 64, 12.0), (2, 128, 128, 4.0), (2, 8, 16, 2.0), (1, 256, 96, 4.0)])
def test_gated_linear_attention_in_portions_and_segments(dev, dtype, heads, dim, vdim, tau):
    layer = gla_cfg(heads, dim, vdim, tau)
    W, T = 80, 150
    cfg = model_cfg([layer], width=W)
    sd = O.random_weights(cfg, 11)
    g = torch.Generator().manual_seed(12)
    h = bf(torch.randn(T, W, generator=g))
    ref = O.gla_mixer(h, sd, "l0.mix.", layer["mixer"], EPS)
    for portions, seg in (([T], 0), ([T], 16), ([1, 1, 2, 3, 40, 1, 64, 38], None), ([70, 80], 32)):
        cache = new_cache(dev)
        mix = build_mixer(layer, sd, "l0.mix.", W, dtype, dev, cache)
        mix.scan_segment = seg
        cache.admit("other")                                                   # a neighbour slot that must stay untouched
        cache.admit("s")
        mix.state[0].fill_(7.0)
        got = feed(mix, cache, h.to(dtype), portions, dev)
        assert_close(got, ref, dtype, (portions[:2], seg))
        assert bool((mix.state[0] == 7.0).all())


def test_decay_from_the_low_rank_pair_stays_in_fp32(dev):
    """sigmoid(z)^(1/tau) for large |z|: the logarithm must not be taken of a rounded sigmoid"""
    from zhilight_amd import seqops
    z = torch.tensor([[-60.0, -20.0, -1.0, 0.0, 1.0, 20.0, 60.0, 90.0]])
    w2 = torch.eye(8)
    for tau in (1.0, 16.0):
        got = seqops.lowrank_decay(z.to(dev), 0, w2.to(dev), torch.zeros(8, device=dev), tau)
        ref = torch.exp(torch.nn.functional.logsigmoid(z.double()) / tau)
        assert float(((got.cpu().double() - ref).abs() / ref).max()) < 1e-5


@pytest.mark.parametrize("experts,count,keep,top", [(12, 3, 2, 2), (16, 4, 1, 3), (8, 4, 2, 3), (6, 6, 4, 3), (5, 1, 1, 1), (9, 3, 3, 4)])
def test_router_choice_against_the_restatement(dev, experts, count, keep, top):
    from zhilight_amd import seqops
    f = moe(experts=experts, count=count, keep=keep, top=top)
    W, T = 64, 200
    g = torch.Generator().manual_seed(experts)
    h = bf(torch.randn(T, W, generator=g))
    sd = {"router": bf(torch.randn(experts, W, generator=g) * 0.3), "correction": bf(torch.randn(experts, generator=g) * 2.0 - 1.5)}
    ids_ref, w_ref = O.route(h, sd, "", f)
    logits = (h @ sd["router"].T).float().to(dev)
    ids, wts = seqops.moe_route(logits, sd["correction"].float().to(dev), count, keep, top, True, score="sigmoid", group_top=2, renorm_eps=1e-20)
    assert (ids.cpu().long() == ids_ref).all()                                  # (negative choice scores: a dropped group is minus infinity, not 0)
    assert rel(wts, w_ref) < 1e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("ff,T", [(48, 1), (48, 7), (48, 300), (20, 5), (20, 130)])
def test_experts_on_both_product_kernels(dev, dtype, ff, T):
    from zhilight_amd import gutivik
    f = moe(ff=ff, limit=0.8, experts=6, count=2, keep=1, top=2)
    W = 64
    cfg = model_cfg([with_mlp(gla_cfg(), f)], width=W)
    sd = O.random_weights(cfg, 13, fixed_choice=True)
    g = torch.Generator().manual_seed(14)
    h = bf(torch.randn(T, W, generator=g))
    ref = O.experts_ff(h, sd, "l0.mlp.", f)
    mix = gutivik.FF_BUILDERS["moe"](W, f).load(lambda n: sd[n], "l0.mlp.", dtype, dev)
    assert_close(mix.forward(h.to(dev).to(dtype).contiguous()), ref, dtype, (ff, T))
    # the clamps bite in these weights
    unclamped = dict(f, expert={"ff": ff, "limit": 1e9})
    assert rel(O.experts_ff(h, sd, "l0.mlp.", unclamped), ref) > 0.05


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_dense_feed_forward(dev, dtype):
    from zhilight_amd import gutivik
    W, T, f = 72, 33, dense(100)
    cfg = model_cfg([with_mlp(gla_cfg(), f)], width=W)
    sd = O.random_weights(cfg, 15)
    h = bf(torch.randn(T, W, generator=torch.Generator().manual_seed(16)))
    mix = gutivik.FF_BUILDERS["dense"](W, f).load(lambda n: sd[n], "l0.mlp.", dtype, dev)
    assert_close(mix.forward(h.to(dev).to(dtype).contiguous()), O.dense_ff(h, sd, "l0.mlp."), dtype)


# ------------------------------------------------------------------------------------------------------------------------------------
# the model through the engine
# ------------------------------------------------------------------------------------------------------------------------------------
@pytest.fixture(scope="module")
def model_a():
    cfg = cfg_a()
    sd = O.random_weights(cfg, 21, fixed_choice=True)
    toks = tokens_of(cfg, 230, 22)
    logits, streams = O.model(cfg, sd, toks)
    return cfg, sd, toks, logits, streams


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_whole_prompt_and_every_layer(dev, dtype, model_a):
    from zhilight_amd import seqops
    cfg, sd, toks, logits, streams = model_a
    eng = make(cfg, sd, dtype, dev)
    assert_close(run_portions(eng, "w", toks, [len(toks)]), logits, dtype)
    eng.cache.admit("L")
    pos0, slot, pages = eng.cache.extend("L", len(toks))
    b = seqops.RaggedBatch([(len(toks), pos0, slot, list(pages))], 64, dev)
    for i, (got, ref) in enumerate(zip(eng.model.forward_layers(torch.tensor(toks, dtype=torch.int32, device=dev), b), streams)):
        assert_close(got, ref, dtype, f"layer {i}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_token_by_token_from_the_first_token_and_after_a_prompt(dev, dtype, model_a):
    cfg, sd, toks, logits, _ = model_a
    eng = make(cfg, sd, dtype, dev)
    assert_close(run_portions(eng, "d0", toks[:100], [1] * 100), logits[:100], dtype, "from the first token")
    assert_close(run_portions(eng, "d1", toks, [50] + [1] * 180), logits, dtype, "long decoding")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_portions_of_many_sizes(dev, dtype, model_a):
    cfg, sd, toks, logits, _ = model_a
    eng = make(cfg, sd, dtype, dev)
    for portions in ([2] * 20 + [3, 5, 1, 60, 64, 1, 2, 54], [63, 1, 64, 65, 37], [128, 2, 100]):
        assert_close(run_portions(eng, "p", toks, portions), logits, dtype, portions[:3])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mixed_batches_with_reused_pages_and_slots(dev, dtype):
    """five unequal requests in mixed steps (portions beside single tokens) in a pool that only holds them because pages and slots come
    back; each request's logits equal its logits alone"""
    from zhilight_amd.engine import Entry
    cfg = cfg_a()
    sd = O.random_weights(cfg, 23, fixed_choice=True)
    lens = [150, 97, 201, 64, 33]
    reqs = {f"r{i}": tokens_of(cfg, n, 30 + i) for i, n in enumerate(lens)}
    refs = {k: O.model(cfg, sd, v)[0] for k, v in reqs.items()}
    eng = make(cfg, sd, dtype, dev, max_tokens=64 * 8, max_seqs=3)
    got = {k: [] for k in reqs}
    at = {k: 0 for k in reqs}
    waiting, live = list(reqs), []
    rng = np.random.default_rng(5)
    pages = lambda k: (len(reqs[k]) + 63) // 64
    while waiting or live:
        while waiting and len(live) < 3 and sum(pages(k) for k in live) + pages(waiting[0]) <= 8:
            live.append(waiting.pop(0))
        entries = []
        for k in live:
            left = len(reqs[k]) - at[k]
            n = min(left, int(rng.choice([1, 1, 2, 7, 40, 64])))
            entries.append(Entry(k, reqs[k][at[k]:at[k] + n], list(range(n))))
        out = eng.run_step(entries)
        row = 0
        for e in entries:
            got[e.rid].append(out[row:row + len(e.tokens)])
            row += len(e.tokens)
            at[e.rid] += len(e.tokens)
            if at[e.rid] == len(reqs[e.rid]):
                eng.release(e.rid)
                live.remove(e.rid)
    for k in reqs:
        assert_close(torch.cat(got[k]), refs[k], dtype, k)
    assert len(eng.cache.free_pages) == 8 and len(eng.cache.free_slots) == 3


def test_same_bits_after_pages_and_slots_were_used_by_others(dev):
    cfg = cfg_a()
    sd = O.random_weights(cfg, 24, fixed_choice=True)
    eng = make(cfg, sd, torch.bfloat16, dev, max_tokens=64 * 4, max_seqs=2)
    a, b = tokens_of(cfg, 130, 1), tokens_of(cfg, 120, 2)
    first = run_portions(eng, "a", a, [100, 1, 29])
    run_portions(eng, "b", b, [120], release=False)
    eng.release("b")
    again = run_portions(eng, "a2", a, [100, 1, 29])
    assert torch.equal(first, again)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_odd_sizes_whole_in_portions_and_decoded(dev, dtype):
    cfg = cfg_odd()
    sd = O.random_weights(cfg, 25, fixed_choice=True)
    toks = tokens_of(cfg, 140, 26)
    logits, _ = O.model(cfg, sd, toks)
    eng = make(cfg, sd, dtype, dev)
    assert_close(run_portions(eng, "w", toks, [140]), logits, dtype, "whole")
    assert_close(run_portions(eng, "p", toks, [2, 2, 1, 60, 5, 1, 1, 68]), logits, dtype, "portions")
    assert_close(run_portions(eng, "d", toks[:70], [1] * 70), logits[:70], dtype, "decoded")


def test_router_choices_through_the_model_in_fp32(dev):
    """ordinary correction terms (close calls allowed): fp32 serving follows the restatement's choices"""
    cfg = cfg_a()
    sd = O.random_weights(cfg, 27)
    toks = tokens_of(cfg, 120, 28)
    logits, _ = O.model(cfg, sd, toks)
    eng = make(cfg, sd, torch.float32, dev)
    assert_close(run_portions(eng, "w", toks, [50, 1, 1, 68]), logits, torch.float32)


def test_medium_configuration_other_kernel_instantiations(dev):
    """head sizes up to 128, a latent of 256 + 64, 16 heads on 4 kv heads, 32 experts in 8 groups, a portion long enough for scan segments"""
    cfg = model_cfg([with_mlp(attention_cfg(heads=16, kv_heads=4, dim=128, vdim=64, conv=4, rot=64, size=200, keep=6, scale=0.09), dense(512)),
                     with_mlp(latent_cfg(heads=8, dim=64, rot=64, vdim=64, rank=256, size=100, scale=0.09), moe(ff=64, limit=2.0, experts=32, count=8, keep=3, top=4)),
                     with_mlp(gla_cfg(heads=4, dim=64, vdim=128, tau=12.0), moe(ff=64, limit=2.0, experts=32, count=8, keep=3, top=4)),
                     attention_cfg(heads=16, kv_heads=4, dim=128, vdim=64, conv=4, rot=64, size=200, keep=6, scale=0.09)],
                    width=256, vocab=300)
    sd = O.random_weights(cfg, 29, fixed_choice=True)
    toks = tokens_of(cfg, 420, 30)
    logits, _ = O.model(cfg, sd, toks)
    for dtype in (torch.float32, torch.bfloat16):
        eng = make(cfg, sd, dtype, dev)
        assert_close(run_portions(eng, "w", toks, [300, 1, 1, 118]), logits, dtype, "medium")


def test_greedy_generation_through_the_scheduler(dev):
    """Engine.generate under a small step budget (prompts cut into portions, decode tokens beside them) gives what feeding the restatement
    its own arg-max gives"""
    from zhilight_amd.engine import SamplingParams
    cfg = cfg_a()
    sd = O.random_weights(cfg, 31, fixed_choice=True)
    prompts = [tokens_of(cfg, n, 40 + n) for n in (40, 9, 75)]
    eng = make(cfg, sd, torch.float32, dev, max_tokens=64 * 10, max_seqs=2, max_step_tokens=48)
    outs = eng.generate(prompts, SamplingParams(max_new_tokens=4))
    for p, out in zip(prompts, outs):
        seq = list(p)
        for tok in out:
            logits, _ = O.model(cfg, sd, seq)
            top2 = torch.topk(logits[-1], 2).values
            if float(top2[0] - top2[1]) > 1e-3:                                 # (a tie within rounding may go either way)
                assert int(torch.argmax(logits[-1])) == tok
            seq.append(tok)
