"""Gaparax on the GPU against the plain float64 restatement in tests/gaparax_oracle.py: every mechanism alone, then the model through the
engine's step function -- whole prompts, token-by-token decoding, portions down to two tokens, mixed batches, reused pages and slots, keys
far back, at page borders and just inside / outside every chunk, odd sizes, greedy generation through the scheduler.  Small random
configurations made here; nothing is read from disk.

fp32 serving is held to rounding of fp32 sums everywhere, bf16 serving to bf16 rounding of the matrix-product inputs.  Through a whole
model in bf16 a router sees a rounded input, and with random weights some of its choices are closer calls than that rounding; the bf16
MODEL tests therefore use routers whose order of logits is fixed with wide gaps (gaparax_oracle.random_weights, fixed_choice; the gaps
are asserted); the choice itself is tested in fp32 through the same models and on the router alone."""
import math

import numpy as np
import pytest
import torch

import gaparax_oracle as O

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
SCALING = {"factor": 6.0, "original": 48, "fast": 12.0, "slow": 2.0}


def attention_cfg(heads=4, kv_heads=2, dim=40, vdim=32, scale=0.2, cap=25.0, far=60, size=70):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "softcap": cap,
                                           "bias_max": far, "mask": {"size": size}}, "mlp": None}


def latent_cfg(heads=4, dim=24, rot=16, vdim=16, rank=48, base=300.0, scale=0.18, scaling=SCALING):
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": vdim, "kv_rank": rank, "scale": scale,
                                                  "rot": {"base": base, "dims": rot, "scaling": scaling}}, "mlp": None}


def dense(ff=144):
    return {"kind": "dense", "ff": ff}


def moe(ff=48, experts=12, count=3, keep=2, top=2, scale=1.7):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "scale": scale, "groups": {"count": count, "keep": keep}}}


def with_mlp(layer, mlp):
    layer = dict(layer)
    layer["mlp"] = mlp
    return layer


def model_cfg(layers, width=96, vocab=160, streams=3):
    return {"architecture": "Gaparax", "vocab": vocab, "width": width, "streams": streams, "norm": {"eps": EPS}, "layers": layers}


def cfg_a():
    """both mixers and both feed-forwards; chunks of 70 and 33 positions (neither a multiple nor a divisor of a page), 4 heads on 2"""
    return model_cfg([with_mlp(attention_cfg(), dense()), with_mlp(latent_cfg(), moe()),
                      with_mlp(attention_cfg(dim=32, vdim=16, size=33, far=20, cap=4.0, scale=0.3), moe(ff=40, experts=8, count=4, keep=2, top=3)),
                      latent_cfg(heads=2, dim=16, rot=8, vdim=24, rank=40),
                      with_mlp(attention_cfg(heads=2, kv_heads=1, size=128), dense(100))])


def cfg_odd():
    """sizes no matrix-core kernel takes, and values that a particular model may make equal or 1: one stream, heads = kv heads, one kv
    head, chunks of 1 position and longer than any prompt, no cap, a bias table that ends inside the chunk, no frequency scaling,
    a rotated part as long as the plain one, one group, one pick, a router scale of 1, an ff that is no multiple of 16"""
    return model_cfg([with_mlp(attention_cfg(heads=3, kv_heads=3, dim=20, vdim=12, size=1, cap=0.0, far=9), moe(ff=20, experts=5, count=1, keep=1, top=1, scale=1.0)),
                      with_mlp(latent_cfg(heads=3, dim=10, rot=10, vdim=7, rank=21, scaling=None), dense(50)),
                      with_mlp(attention_cfg(heads=4, kv_heads=1, dim=16, vdim=16, size=1000, far=30), moe(ff=32, experts=6, count=6, keep=4, top=3)),
                      attention_cfg(heads=2, kv_heads=1, dim=24, vdim=16, size=64, far=500),
                      latent_cfg(heads=1, dim=8, rot=4, vdim=20, rank=12, scaling={"factor": 2.0, "original": 16, "fast": 4.0, "slow": 1.0})],
                     width=72, vocab=90, streams=1)


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


def oracle_model(cfg, sd, toks, fixed=True):
    """(logits, the sum of the streams after every layer); with fixed-choice weights no router choice may be a close call"""
    layers, margins = [], []
    logits = O.model(toks, sd, cfg, layers, margins)
    assert not fixed or not margins or min(margins) > 0.1, margins
    return logits, layers


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


def build_mixer(layer, sd, prefix, width, dtype, dev, cache):
    from zhilight_amd import gaparax
    mix = gaparax.MIXER_BUILDERS[layer["type"]]("m" + prefix, width, layer["mixer"], EPS)
    mix.load(lambda n: sd[n], prefix, dtype, dev)
    mix.bind(cache, dtype)
    return mix


# ------------------------------------------------------------------------------------------------------------------------------------
# mechanisms alone
# ------------------------------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("n", [1, 2, 3, 8])
def test_residual_streams_read_update_and_fused_next_read(dev, n):
    from zhilight_amd import seqops
    g = torch.Generator().manual_seed(n)
    T, W = 7, 77
    xs = torch.randn(T, n, W, generator=g) * 2 + 0.5
    y, gate = torch.randn(T, W, generator=g) * 3, torch.randn(T, W + 5, generator=g) * 2
    gb, mix, out = torch.randn(W, generator=g), torch.eye(n) + 0.4 * torch.randn(n, n, generator=g), torch.randn(n, generator=g)
    rd, w = torch.randn(n, generator=g), 1.0 + 0.3 * torch.randn(W, generator=g)
    X = xs.double()
    # reading: the normed weighted sum, all rows and gathered rows, and the plain sum of the streams
    ref_h = O.rms_norm(torch.einsum("s,tsw->tw", rd.double(), X), w.double(), EPS)
    assert rel(seqops.streams_norm(xs.to(dev), n, rd.to(dev), w.to(dev), EPS, torch.float32), ref_h) < 1e-6
    rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=dev)
    assert rel(seqops.streams_norm(xs.to(dev), n, None, w.to(dev), EPS, torch.float32, rows=rows), O.rms_norm(X.sum(1), w.double(), EPS)[[5, 0, 5]]) < 1e-6
    # updating in place with a gated result, and the next read in the same launch
    yg = y.double() * torch.sigmoid(gate.double()[:, 3:3 + W] + gb.double())
    new = torch.einsum("sd,tsw->tdw", mix.double(), X) + out.double()[None, :, None] * yg[:, None, :]
    xd = xs.to(dev)
    h2 = seqops.streams_update(xd, xd, n, y.to(dev), mix.to(dev), out.to(dev), gate=gate.to(dev), g_col0=3, gate_bias=gb.to(dev),
                               next_coef=rd.to(dev), next_weight=w.to(dev), eps=EPS, dtype=torch.bfloat16)
    assert rel(xd, new) < 1e-6 and rel(h2, O.rms_norm(torch.einsum("s,tsw->tw", rd.double(), new), w.double(), EPS)) < 4e-3
    # no gate, nothing read afterwards
    xd = xs.to(dev)
    assert seqops.streams_update(xd, xd, n, y.to(dev), mix.to(dev), out.to(dev)) is None
    assert rel(xd, torch.einsum("sd,tsw->tdw", mix.double(), X) + out.double()[None, :, None] * y.double()[:, None, :]) < 1e-6
    # the start: one row read as n equal streams, written to the streams
    x0 = xs[:, 0].contiguous()
    dst = torch.full((T, n, W), 9.0, device=dev)
    seqops.streams_update(x0.to(dev), dst, n, y.to(dev), mix.to(dev), out.to(dev))
    X0 = x0.double()[:, None, :].expand(T, n, W)
    assert rel(dst, torch.einsum("sd,tsw->tdw", mix.double(), X0) + out.double()[None, :, None] * y.double()[:, None, :]) < 1e-6
    assert rel(seqops.streams_norm(x0.to(dev), n, rd.to(dev), w.to(dev), EPS, torch.float32), O.rms_norm(rd.double().sum() * x0.double(), w.double(), EPS)) < 1e-6
    # a tiny row: eps inside the root decides
    z = torch.full((1, n, W), 1e-4)
    assert rel(seqops.streams_norm(z.to(dev), n, None, w.to(dev), 1e-2, torch.float32), O.rms_norm(z.double().sum(1), w.double(), 1e-2)) < 1e-6


def test_unary_activations(dev):
    from zhilight_amd import seqops
    z = (torch.randn(5, 60, generator=torch.Generator().manual_seed(3)) * 3).to(dev)
    a = z.double().cpu()
    assert rel(seqops.unary_act(z, torch.float32, "relu2"), torch.relu(a) ** 2) < 1e-6
    assert rel(seqops.unary_act(z, torch.float32, "gelu_tanh"), O.gelu_tanh(a)) < 1e-6
    assert rel(seqops.unary_act(z, torch.float32, "silu"), a * torch.sigmoid(a)) < 1e-6
    assert rel(seqops.unary_act(z, torch.float32, "relu2", cols=41), torch.relu(a[:, :41]) ** 2) < 1e-6          # (the leading columns of wider rows)


def test_distance_bias_table_and_rescaled_frequencies_follow_the_restatement():
    from zhilight_amd import mixers
    for rows, far in ((18, 200), (12, 40), (14, 9), (2, 5), (32, 128), (16, 128)):
        table = torch.arange(rows * 3, dtype=torch.float32).reshape(rows, 3)
        got = mixers.distance_bias_table(table, far, 0, "cpu")
        assert got.shape == (3, far + 1)
        for n in range(far + 1):
            assert got[1, n] == table[O.distance_bucket(n, rows, far), 1], (rows, far, n)
        assert O.distance_bucket(10 * far, rows, far) == rows - 1                       # (everything from `far` on: the last row)
        assert mixers.distance_bias_table(table, far, 7, "cpu").shape == (3, min(7, far + 1))
    for dims, base, sc in ((24, 30000.0, {"factor": 5.0, "original": 512, "fast": 24.0, "slow": 1.5}), (8, 100.0, SCALING), (64, 1e6, None),
                           (4, 50.0, {"factor": 2.0, "original": 16, "fast": 4.0, "slow": 1.0}), (32, 1e4, {"factor": 40.0, "original": 4096, "fast": 1.0, "slow": 0.5})):
        f, gain = mixers.scaled_frequencies(dims, base, sc)
        rf, rgain = O.scaled_frequencies(dims, base, sc)
        assert float(((f.double() - rf) / rf).abs().max()) < 1e-7 and abs(gain - rgain) < 1e-12


def attention_kernels(q, k, v, wq, wk, form_args, scale, dtype, dev, portions, mfma=True, n_splits=None, shuffle_pages=False):
    """[q | k | v] rows through the cache-writing kernel (weighted norms, no rotation), the attention kernels in the sigmoid score form and
    the sum over the splits, in portions"""
    from zhilight_amd import seqops
    T, H, d = q.shape
    G, e = k.shape[1], v.shape[2]
    cache = new_cache(dev, max_tokens=64 * ((T + 63) // 64 + 3))
    if shuffle_pages:
        cache.free_pages = cache.free_pages[::-1]
    kp, vp = cache.add_plane("k", (G * d,), dtype), cache.add_plane("v", (G * e,), dtype)
    cache.admit("s")
    rows = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], dim=1).float()
    form = seqops.score_form(H, **{n: (t.float().to(dev).contiguous() if torch.is_tensor(t) else t) for n, t in form_args.items()})
    out, at = [], 0
    for n in portions:
        pos0, slot, pages = cache.extend("s", n)
        b = seqops.RaggedBatch([(n, pos0, slot, list(pages))], 64, dev)
        proj = rows[at:at + n].to(dev).contiguous()
        seqops.rope_norm_store(proj, 0, H * d, H * d + G * d, H, G, d, e, None, 0, None, EPS, True, b, kp, vp, q_norm_w=wq.float().to(dev),
                               k_norm_w=wk.float().to(dev))
        acc, ml, ns = seqops.window_attention(proj, 0, kp, vp, b, scale, 0, H, G, d, e, all_kv=False, mfma=mfma, n_splits=n_splits, form=form)
        out.append(seqops.head_mix_gate(acc, ml, ns, None, None, None, 0, b, H, G, e, torch.float32, plain_sum=bool(form_args.get("sigmoid"))))
        at += n
    assert at == T
    return torch.cat(out).reshape(T, H, e)


def aimed(T, H, G, d, e, pairs, seed):
    """random queries, keys, values (bf16-representable); for every (query i, key j) of `pairs` the key j points along query i's first
    head of every group and carries a large value: its score stands out, so a mask that is one position off changes the output visibly"""
    g = torch.Generator().manual_seed(seed)
    q, k, v = bf(torch.randn(T, H, d, generator=g)), bf(torch.randn(T, G, d, generator=g)), bf(torch.randn(T, G, e, generator=g))
    for i, j in pairs:
        for c in range(G):
            k[j, c] = q[i, c * (H // G)]
            v[j, c] = bf(20.0 * torch.randn(e, generator=g))
    return q, k, v


def sigmoid_reference(q, k, v, wq, wk, scale, temp, cap, table, far, chunk, offset):
    T = q.shape[0]
    bias = O.distance_bias(T, table, far) if table is not None else None
    return O.sigmoid_attention(O.rms_norm(q, wq, EPS), O.rms_norm(k, wk, EPS), v, scale, temp, cap, bias, O.chunk_visible(T, chunk), offset)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("chunk", [1, 2, 33, 64, 65, 80, 100])
def test_sigmoid_attention_chunk_edges(dev, dtype, chunk):
    """queries aimed at the first key of their chunk and at the last key of the chunk before -- inside a portion and decoded alone --
    against the float64 sigmoid weights over the chunk's visibility matrix; low offsets keep every other key's weight small"""
    T, H, G, d, e = 330, 4, 2, 24, 16
    portions = [150, 1, 1, 1, 60, 2, 1, 1, 64, 1, 1, 47]                      # queries 150-152, 215-216, 281-282 are single tokens
    singles, inside = [150, 151, 215, 281, 282], [100, 149, 160, 199, 212, 230, 329]
    pairs = []
    for n, i in enumerate(singles + inside):
        start = i // chunk * chunk
        j = start if n % 2 == 0 else start - 1
        if 0 <= j <= i:
            pairs.append((i, j))
    q, k, v = aimed(T, H, G, d, e, pairs, chunk)
    g = torch.Generator().manual_seed(chunk + 1)
    wq, wk = bf(1.0 + 0.2 * torch.randn(d, generator=g)), bf(1.0 + 0.2 * torch.randn(d, generator=g))
    temp, offset = bf(torch.tensor([1.5, 1.2, 1.8, 1.4])), bf(torch.tensor([-6.0, -5.0, -7.0, -5.5]))
    table, far = bf(0.5 * torch.randn(10, H, generator=g)), 50
    scale, cap = 0.3, 30.0
    ref = sigmoid_reference(q, k, v, wq, wk, scale, temp, cap, table, far, chunk, offset)
    other = sigmoid_reference(q, k, v, wq, wk, scale, temp, cap, table, far, chunk + 1, offset)
    assert rel(other, ref) > 0.05                                               # the aimed keys do show
    from zhilight_amd import mixers
    bias = mixers.distance_bias_table(table.float(), far, chunk, "cpu")
    args = dict(head_scale=temp, softcap=cap, bias=bias, offset=offset, chunk=chunk, sigmoid=True)
    for mfma, splits in ((True, None), (False, None), (False, 3)):
        got = attention_kernels(q, k, v, wq, wk, args, scale, dtype, dev, portions, mfma=mfma, n_splits=splits, shuffle_pages=splits == 3)
        assert_close(got.reshape(T, -1), ref.reshape(T, -1), dtype, (chunk, mfma, splits))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_sigmoid_attention_bias_rows_cap_and_head_factor_show(dev, dtype):
    """a bias table with large, distinct rows (every bucket edge moves the weights), scores beyond the cap, unequal factors per head; a
    table that ends before the chunk does (distances beyond it take the last row); no chunks at all; a table of more distances than the
    matrix-core kernel keeps in LDS"""
    from zhilight_amd import mixers
    T, H, G, d, e = 200, 4, 1, 32, 16
    g = torch.Generator().manual_seed(5)
    q, k, v = bf(torch.randn(T, H, d, generator=g)), bf(torch.randn(T, G, d, generator=g)), bf(torch.randn(T, G, e, generator=g))
    wq, wk = bf(1.0 + 0.3 * torch.randn(d, generator=g)), bf(1.0 + 0.3 * torch.randn(d, generator=g))
    temp, offset = bf(torch.tensor([0.5, 3.0, 1.0, 6.0])), bf(torch.tensor([-2.0, -3.0, -1.0, -4.0]))
    for rows, far, chunk, cap in ((16, 40, 150, 2.0), (6, 20, 0, 3.0), (12, 300, 90, 0.0), (10, 3000, 0, 3.0)):
        table = bf(torch.linspace(-3.0, 3.0, rows)[:, None] * torch.tensor([1.0, -1.0, 0.5, 2.0])[None, :])
        ref = sigmoid_reference(q, k, v, wq, wk, 0.25, temp, cap, table, far, chunk, offset)
        assert far > 1000 or rel(sigmoid_reference(q, k, v, wq, wk, 0.25, temp, cap, table, 2 * far, chunk, offset), ref) > 0.02   # the buckets show
        assert rel(sigmoid_reference(q, k, v, wq, wk, 0.25, temp, 0.0 if cap else 1.0, table, far, chunk, offset), ref) > 0.02   # the cap shows
        assert rel(sigmoid_reference(q, k, v, wq, wk, 0.25, torch.ones(H, dtype=F64), cap, table, far, chunk, offset), ref) > 0.02
        bias = mixers.distance_bias_table(table.float(), far, chunk, "cpu")
        args = dict(head_scale=temp, softcap=cap, bias=bias, offset=offset, chunk=chunk, sigmoid=True)
        for mfma in (True, False):
            got = attention_kernels(q, k, v, wq, wk, args, 0.25, dtype, dev, [120, 1, 1, 1, 77], mfma=mfma, shuffle_pages=True)
            assert_close(got.reshape(T, -1), ref.reshape(T, -1), dtype, (rows, far, chunk, mfma))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_score_form_with_a_softmax(dev, dtype):
    """the same score form (factor per head, cap, distance bias, chunks) under a softmax instead of sigmoids: the splits are merged with
    their maxima and sums"""
    from zhilight_amd import mixers
    T, H, G, d, e, cap, scale = 200, 4, 2, 24, 16, 3.0, 0.3
    g = torch.Generator().manual_seed(11)
    q, k, v = bf(torch.randn(T, H, d, generator=g)), bf(torch.randn(T, G, d, generator=g)), bf(torch.randn(T, G, e, generator=g))
    wq, wk = bf(1.0 + 0.2 * torch.randn(d, generator=g)), bf(1.0 + 0.2 * torch.randn(d, generator=g))
    temp, table = bf(torch.tensor([0.5, 2.0, 1.0, 4.0])), bf(torch.randn(10, H, generator=g))
    qn, kn = O.rms_norm(q, wq, EPS), O.rms_norm(k, wk, EPS)
    for chunk, far in ((70, 40), (0, 2500)):                                    # (the second table is longer than the kernel's LDS row)
        bias, vis = O.distance_bias(T, table, far), O.chunk_visible(T, chunk)
        ref = torch.zeros(T, H, e, dtype=F64)
        for a in range(H):
            sc = cap * torch.tanh((qn[:, a] @ kn[:, a // 2].T) * scale * temp[a] / cap) + bias[a]
            ref[:, a] = torch.softmax(sc.masked_fill(~vis, -math.inf), -1) @ v[:, a // 2]
        args = dict(head_scale=temp, softcap=cap, bias=mixers.distance_bias_table(table.float(), far, chunk, "cpu"), chunk=chunk)
        for mfma, splits in ((True, None), (False, 2)):
            got = attention_kernels(q, k, v, wq, wk, args, scale, dtype, dev, [130, 1, 1, 68], mfma=mfma, n_splits=splits)
            assert_close(got.reshape(T, -1), ref.reshape(T, -1), dtype, (chunk, mfma))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d,e", [(4, 2, 8, 16), (3, 3, 72, 48), (2, 1, 160, 16), (4, 1, 256, 128), (2, 2, 20, 12)])
def test_sigmoid_attention_head_sizes_and_groups(dev, dtype, H, G, d, e):
    """the other instantiations of the matrix-core kernel (32-coordinate steps of the head size), long heads in the plain kernel, sizes
    only the plain kernel takes, heads = kv heads and one kv head"""
    from zhilight_amd import mixers
    T, chunk = 200, 80
    q, k, v = aimed(T, H, G, d, e, [(150, 80), (199, 159), (120, 79), (190, 160)], d)
    g = torch.Generator().manual_seed(d)
    wq, wk = bf(1.0 + 0.2 * torch.randn(d, generator=g)), bf(1.0 + 0.2 * torch.randn(d, generator=g))
    temp, offset = bf(1.0 + 0.3 * torch.rand(H, generator=g)), bf(-5.0 - torch.rand(H, generator=g))
    table = bf(0.5 * torch.randn(8, H, generator=g))
    scale = 8.0 / d
    ref = sigmoid_reference(q, k, v, wq, wk, scale, temp, 20.0, table, 30, chunk, offset)
    args = dict(head_scale=temp, softcap=20.0, bias=mixers.distance_bias_table(table.float(), 30, chunk, "cpu"), offset=offset, chunk=chunk, sigmoid=True)
    got = attention_kernels(q, k, v, wq, wk, args, scale, dtype, dev, [130, 1, 1, 68])
    assert_close(got.reshape(T, -1), ref.reshape(T, -1), dtype, (d, e))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_mixer_in_portions(dev, dtype):
    W, T = 96, 200
    for layer in (attention_cfg(), attention_cfg(heads=2, kv_heads=1, dim=32, vdim=16, size=33, far=20, cap=4.0, scale=0.3)):
        cfg = model_cfg([layer])
        sd = O.random_weights(cfg, 5)
        h = bf(torch.randn(T, W, generator=torch.Generator().manual_seed(6)))
        ref = O.sigmoid_attention_mixer(h, sd, "l0.mix.", layer["mixer"], EPS)
        ungated = dict(sd)
        ungated["l0.mix.g"] = torch.zeros_like(sd["l0.mix.g"])
        assert rel(O.sigmoid_attention_mixer(h, ungated, "l0.mix.", layer["mixer"], EPS), ref) > 0.05     # the gate shows
        for portions in ([T], [1] * 6 + [2, 3, 61, 64, 1, 1, 62]):
            cache = new_cache(dev)
            mix = build_mixer(layer, sd, "l0.mix.", W, dtype, dev, cache)
            cache.admit("s")
            assert_close(feed(mix, cache, h.to(dtype), portions, dev), ref, dtype, portions[:2])


def latent_rows(layer, sd, p, T, pairs, seed):
    """mixer inputs h = [q | down-projection] for identity input matrices; for (i, j) in pairs query i's plain parts point along the
    up-projected key of token j, which gets large values through a large latent direction"""
    m = layer["mixer"]
    H, d, r, R = m["heads"], m["dim"], m["rot_dim"], m["kv_rank"]
    g = torch.Generator().manual_seed(seed)
    h = bf(torch.randn(T, H * (d + r) + R + r, generator=g))
    q0 = H * (d + r)
    for i, j in pairs:
        c = O.rms_norm(h[j, q0:q0 + R], sd[p + "dkv.norm"].double(), EPS)
        kj = (c @ sd[p + "uk"].double().T).reshape(H, d)
        for a in range(H):
            h[i, a * (d + r):a * (d + r) + d] = bf(4.0 * kj[a] / kj[a].norm() * math.sqrt(d))
            h[i, a * (d + r) + d:(a + 1) * (d + r)] = 0.0
    return h


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_latent_attention_one_far_key_across_pages_with_sink(dev, dtype):
    """one key far back, at page borders and at the very start, found by queries inside a portion and decoded alone; rescaled rotary
    frequencies in the half layout, a sink per head; both kernel families"""
    layer = latent_cfg(heads=4, dim=24, rot=16, vdim=16, rank=48)
    m = layer["mixer"]
    H, d, r, R = m["heads"], m["dim"], m["rot_dim"], m["kv_rank"]
    W = H * (d + r) + R + r
    cfg = model_cfg([layer], width=W)
    sd = O.random_weights(cfg, 7)
    eye = torch.eye(W)
    sd["l0.mix.q"], sd["l0.mix.dkv"] = eye[:H * (d + r)].to(torch.bfloat16), eye[H * (d + r):].to(torch.bfloat16)
    sd["l0.mix.sink"] = torch.tensor([2.0, -1.0, 0.0, 4.0]).to(torch.bfloat16)
    T = 300
    for j in (0, 1, 63, 64, 65, 127, 128, 200):
        h = latent_rows(layer, sd, "l0.mix.", T, [(290, j), (297, j), (299, j)], j)
        ref = O.latent_attention_mixer(h, sd, "l0.mix.", m, EPS)
        hidden = h.clone()
        hidden[j] = h[j + 1]
        assert rel(O.latent_attention_mixer(hidden, sd, "l0.mix.", m, EPS)[[290, 297, 299]], ref[[290, 297, 299]]) > 0.05      # the far key shows
        for prompt_kernel, mfma in ((True, True), (False, False)):
            cache = new_cache(dev)
            cache.free_pages = cache.free_pages[::-1]
            mix = build_mixer(layer, sd, "l0.mix.", W, dtype, dev, cache)
            mix.prompt_kernel, mix.decode_mfma = prompt_kernel, mfma
            cache.admit("s")
            assert_close(feed(mix, cache, h.to(dtype), [296, 1, 1, 1, 1], dev), ref, dtype, (j, prompt_kernel))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_latent_attention_sink_rotation_layout_and_scaling_show(dev, dtype):
    layer = latent_cfg()
    W, T = 96, 180
    cfg = model_cfg([layer])
    sd = O.random_weights(cfg, 8)
    h = bf(torch.randn(T, W, generator=torch.Generator().manual_seed(9)))
    m = layer["mixer"]
    ref = O.latent_attention_mixer(h, sd, "l0.mix.", m, EPS)
    no_sink = dict(sd)
    no_sink["l0.mix.sink"] = torch.full_like(sd["l0.mix.sink"], -30.0)
    assert rel(O.latent_attention_mixer(h, no_sink, "l0.mix.", m, EPS), ref) > 0.05
    unscaled = dict(m, rot=dict(m["rot"], scaling=None))
    assert rel(O.latent_attention_mixer(h, sd, "l0.mix.", unscaled, EPS), ref) > 0.02
    for portions in ([T], [1] * 5 + [2, 60, 1, 64, 48], [100] + [1] * 80):
        cache = new_cache(dev)
        mix = build_mixer(layer, sd, "l0.mix.", W, dtype, dev, cache)
        cache.admit("s")
        assert_close(feed(mix, cache, h.to(dtype), portions, dev), ref, dtype, portions[:2])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,dim,rot,vdim,rank", [(3, 64, 64, 48, 512), (2, 128, 64, 128, 64), (1, 16, 8, 20, 24), (2, 100, 20, 128, 48)])
def test_latent_attention_head_and_latent_sizes(dev, dtype, heads, dim, rot, vdim, rank):
    layer = latent_cfg(heads=heads, dim=dim, rot=rot, vdim=vdim, rank=rank, scale=(dim + rot) ** -0.5,
                       scaling={"factor": 7.0, "original": 64, "fast": 16.0, "slow": 1.0})
    W, T = 128, 200
    cfg = model_cfg([layer], width=W)
    sd = O.random_weights(cfg, 9)
    h = bf(torch.randn(T, W, generator=torch.Generator().manual_seed(10)))
    ref = O.latent_attention_mixer(h, sd, "l0.mix.", layer["mixer"], EPS)
    cache = new_cache(dev)
    mix = build_mixer(layer, sd, "l0.mix.", W, dtype, dev, cache)
    cache.admit("s")
    assert_close(feed(mix, cache, h.to(dtype), [120] + [1] * 20 + [60], dev), ref, dtype)


@pytest.mark.parametrize("experts,count,keep,top,scale", [(12, 2, 1, 3, 2.2), (12, 3, 2, 2, 1.0), (16, 4, 1, 3, 0.5), (8, 4, 2, 3, 3.0), (6, 6, 4, 3, 1.5),
                                                         (5, 1, 1, 1, 1.0), (9, 3, 3, 4, 2.0), (8, 8, 3, 3, 1.0)])
def test_router_choice_against_the_restatement(dev, experts, count, keep, top, scale):
    from zhilight_amd import seqops
    r = moe(experts=experts, count=count, keep=keep, top=top, scale=scale)["router"]
    W, T = 64, 200
    g = torch.Generator().manual_seed(experts + count)
    h = bf(torch.randn(T, W, generator=g))
    sd = {"router": bf(torch.randn(experts, W, generator=g) * 0.3)}
    ids_ref, w_ref = O.route(h, sd, "", r)
    logits = (h @ sd["router"].T).float().to(dev)
    ids, wts = seqops.moe_route(logits, None, count, keep, top, False, score="softmax", group_top=1, weight_scale=scale)
    assert (ids.cpu().long() == ids_ref).all()
    assert rel(wts, w_ref) < 1e-6                                               # (the scores themselves times the scale: not renormalised)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("ff,T", [(48, 1), (48, 7), (48, 300), (20, 5), (20, 130)])
def test_experts_on_both_product_kernels(dev, dtype, ff, T):
    from zhilight_amd import gaparax
    f = moe(ff=ff, experts=6, count=2, keep=1, top=2, scale=1.9)
    W = 64
    cfg = model_cfg([with_mlp(latent_cfg(), f)], width=W)
    sd = O.random_weights(cfg, 13)
    g = torch.Generator().manual_seed(14)
    h = bf(torch.randn(T, W, generator=g))
    sd["l0.mlp.router"] = bf(torch.randn(6, W, generator=g) * 0.5).to(torch.bfloat16)
    margins = []
    O.route(h, sd, "l0.mlp.", f["router"], margins)
    assert margins[0] > 1e-4                                                    # (exact inputs: only a tie within fp32 sums could differ)
    ref = O.experts_ff(h, sd, "l0.mlp.", f)
    ff_ = gaparax.FF_BUILDERS["moe"](W, f).load(lambda n: sd[n], "l0.mlp.", dtype, dev)
    assert_close(ff_.forward(h.to(dev).to(dtype).contiguous()), ref, dtype, (ff, T))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_dense_feed_forward_with_side_rows(dev, dtype):
    """down(relu(up h)^2); rows attached to the up projection come back as fp32 columns behind it and leave the result alone"""
    from zhilight_amd import gaparax
    W, T, f = 72, 33, dense(100)
    cfg = model_cfg([with_mlp(latent_cfg(), f)], width=W)
    sd = O.random_weights(cfg, 15)
    h = bf(torch.randn(T, W, generator=torch.Generator().manual_seed(16)))
    ff_ = gaparax.FF_BUILDERS["dense"](W, f).load(lambda n: sd[n], "l0.mlp.", dtype, dev)
    side = bf(torch.randn(W, W, generator=torch.Generator().manual_seed(17)) * W ** -0.5)
    ff_.attach_side(side.to(dev).to(dtype))
    assert_close(ff_.forward(h.to(dev).to(dtype).contiguous()), O.dense_ff(h, sd, "l0.mlp."), dtype)
    z, c0 = ff_.side
    assert c0 == 100 and rel(z[:, c0:c0 + W], h @ side.T) < 1e-5


# ------------------------------------------------------------------------------------------------------------------------------------
# the model through the engine
# ------------------------------------------------------------------------------------------------------------------------------------
@pytest.fixture(scope="module")
def model_a():
    cfg = cfg_a()
    sd = O.random_weights(cfg, 21, fixed_choice=True)
    toks = tokens_of(cfg, 230, 22)
    logits, layers = oracle_model(cfg, sd, toks)
    return cfg, sd, toks, logits, layers


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_whole_prompt_and_every_layer(dev, dtype, model_a):
    from zhilight_amd import seqops
    cfg, sd, toks, logits, layers = model_a
    eng = make(cfg, sd, dtype, dev)
    assert_close(run_portions(eng, "w", toks, [len(toks)]), logits, dtype)
    eng.cache.admit("L")
    pos0, slot, pages = eng.cache.extend("L", len(toks))
    b = seqops.RaggedBatch([(len(toks), pos0, slot, list(pages))], 64, dev)
    for i, (got, ref) in enumerate(zip(eng.model.forward_layers(torch.tensor(toks, dtype=torch.int32, device=dev), b), layers)):
        assert_close(got, ref, dtype, f"layer {i}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_token_by_token_from_the_first_token_and_after_a_prompt(dev, dtype, model_a):
    cfg, sd, toks, logits, _ = model_a
    eng = make(cfg, sd, dtype, dev)
    assert_close(run_portions(eng, "d0", toks[:100], [1] * 100), logits[:100], dtype, "from the first token")
    assert_close(run_portions(eng, "d1", toks, [50] + [1] * 180), logits, dtype, "long decoding across chunk and page borders")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_portions_of_many_sizes(dev, dtype, model_a):
    cfg, sd, toks, logits, _ = model_a
    eng = make(cfg, sd, dtype, dev)
    for portions in ([2] * 20 + [3, 5, 1, 60, 64, 1, 2, 54], [63, 1, 64, 65, 37], [128, 2, 100], [69, 2, 31, 2, 126]):
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
    refs = {k: oracle_model(cfg, sd, v)[0] for k, v in reqs.items()}
    eng = make(cfg, sd, dtype, dev, max_tokens=64 * 8, max_seqs=3)
    got = {k: [] for k in reqs}
    at = {k: 0 for k in reqs}
    waiting, live = list(reqs), []
    rng = np.random.default_rng(5)

    def pages(k):
        return (len(reqs[k]) + 63) // 64
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


def test_same_bits_after_pages_were_used_by_others(dev):
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
    logits, _ = oracle_model(cfg, sd, toks)
    eng = make(cfg, sd, dtype, dev)
    assert_close(run_portions(eng, "w", toks, [140]), logits, dtype, "whole")
    assert_close(run_portions(eng, "p", toks, [2, 2, 1, 60, 5, 1, 1, 68]), logits, dtype, "portions")
    assert_close(run_portions(eng, "d", toks[:70], [1] * 70), logits[:70], dtype, "decoded")


def test_router_choices_through_the_model_in_fp32(dev):
    """ordinary routers (close calls allowed): fp32 serving follows the restatement's choices"""
    cfg = cfg_a()
    sd = O.random_weights(cfg, 27)
    toks = tokens_of(cfg, 120, 28)
    logits, _ = oracle_model(cfg, sd, toks, fixed=False)
    eng = make(cfg, sd, torch.float32, dev)
    assert_close(run_portions(eng, "w", toks, [50, 1, 1, 68]), logits, torch.float32)


def test_medium_configuration_other_kernel_instantiations(dev):
    """head sizes up to 128, 16 heads on 4 kv heads, a latent of 256 + 64, 32 experts in 8 groups, four streams"""
    cfg = model_cfg([with_mlp(attention_cfg(heads=16, kv_heads=4, dim=128, vdim=64, size=200, far=120, scale=0.09), dense(512)),
                     with_mlp(latent_cfg(heads=8, dim=64, rot=64, vdim=64, rank=256, scale=0.09, base=10000.0,
                                         scaling={"factor": 10.0, "original": 128, "fast": 24.0, "slow": 2.0}),
                              moe(ff=64, experts=32, count=8, keep=3, top=4)),
                     with_mlp(attention_cfg(heads=8, kv_heads=8, dim=64, vdim=128, size=112, far=300, scale=0.12), moe(ff=64, experts=32, count=8, keep=3, top=4))],
                    width=256, vocab=300, streams=4)
    sd = O.random_weights(cfg, 29, fixed_choice=True)
    toks = tokens_of(cfg, 420, 30)
    logits, _ = oracle_model(cfg, sd, toks)
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
            logits = O.model(seq, sd, cfg)
            top2 = torch.topk(logits[-1], 2).values
            if float(top2[0] - top2[1]) > 1e-3:                                 # (a tie within rounding may go either way)
                assert int(torch.argmax(logits[-1])) == tok
            seq.append(tok)


def test_trace_replayer_on_a_model_folder(dev, tmp_path, capsys):
    """a folder with config.json and model.safetensors through the registry's loader and the trace replayer: two requests in mixed steps
    (a portion beside single tokens), one leaves and its pages are taken again; the written logits are the restatement's"""
    import io
    import json
    from safetensors.torch import save_file
    from zhilight_amd import trace
    cfg = cfg_a()
    sd = O.random_weights(cfg, 33, fixed_choice=True)
    folder, out = tmp_path / "model", tmp_path / "out"
    folder.mkdir()
    (folder / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in sd.items()}, str(folder / "model.safetensors"))
    a, b, c = tokens_of(cfg, 90, 1), tokens_of(cfg, 70, 2), tokens_of(cfg, 100, 3)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:60], "want": [0, 59]}, {"id": "b", "tokens": b[:2], "want": [1]}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[2:70], "want": [67]}, {"id": "a", "tokens": a[60:61], "want": [0]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[61:90], "want": []}], "end": []},
             {"step": 3, "entries": [{"id": "c", "tokens": c, "want": [99]}, {"id": "a", "tokens": [a[0]], "want": [0]}], "end": ["a", "c"]}]
    stream = io.StringIO("".join(json.dumps(s) + "\n" for s in steps))
    assert trace.replay(str(folder), "float32", str(out), max_tokens=256, max_seqs=2, stream=stream, device=str(dev)) == 0
    assert [l for l in capsys.readouterr().out.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2", "done 3"]
    la, lb, lc = O.model(a + [a[0]], sd, cfg), O.model(b, sd, cfg), O.model(c, sd, cfg)
    want = {0: torch.stack([la[0], la[59], lb[1]]), 1: torch.stack([lb[69], la[60]]), 3: torch.stack([lc[99], la[90]])}
    assert not (out / "2.f32").exists()
    for n, ref in want.items():
        got = torch.from_numpy(np.fromfile(str(out / f"{n}.f32"), dtype="<f4").reshape(ref.shape[0], cfg["vocab"]))
        assert_close(got, ref, torch.float32, f"step {n}")
