"""A plain float64 restatement of the Gutivik design, one function per mechanism, whole sequences at a time, no cache and no batching.

It shares no code with zhilight_amd: the product path (gutivik.py, mixers.py, the kernels) is held against it.  `weights` is a mapping
name -> tensor with the names of the checkpoint ("l<i>.mix.q", "l<i>.mlp.e<j>.gate", ...); `cfg` is the dictionary of config.json.

Notation: T tokens at positions 0 .. T-1, h (T, width) a sub-layer's input, matrices stored (out, in).
"""
import math

import torch

F64 = torch.float64


def _w(weights, name):
    return weights[name].to(F64)


def rms_norm(x, w, eps, around_zero):
    """x / sqrt(mean(x^2) + eps) * (w, or 1 + w when the weight is stored around zero)"""
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y * ((1.0 + w) if around_zero else w)


def rotate_pairs(x, pos, dims, base):
    """x (T, heads, size): coordinates (2i, 2i+1), i < dims/2, turned by the angle pos * base^(-2i/dims); the rest unchanged"""
    out = x.clone()
    i = torch.arange(dims // 2, dtype=F64)
    ang = pos.to(F64)[:, None] * torch.pow(torch.tensor(float(base), dtype=F64), -2.0 * i / dims)[None, :]      # (T, dims/2)
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def short_conv(u, w):
    """u (T, C), w (C, taps): y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the start"""
    T, C = u.shape
    taps = w.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def visible(T, window, keep_first):
    """(T, T) bool: query i sees key j <= i with i - j < window, or j < keep_first (window 0: every j <= i)"""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    near = (i - j < window) if window > 0 else torch.ones(T, T, dtype=torch.bool)
    return (j <= i) & (near | (j < keep_first))


def softmax_attention(q, k, v, scale, mask, sink=None):
    """q (T, H, d), k (T, G, d), v (T, G, e); head h reads kv head h // (H / G); sink (H) adds exp(sink_h) to the denominator only"""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~mask, -math.inf)
        m = s.max(-1, keepdim=True).values
        if sink is not None:
            m = torch.maximum(m, sink[h].expand_as(m))
        e = torch.exp(s - m)
        den = e.sum(-1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(sink[h] - m)
        out[:, h] = (e / den) @ v[:, g]
    return out


def attention_mixer(h, weights, p, m, eps, v_first):
    """grouped attention with biases, a short convolution after the projections, rotated pairs, a window that keeps the first tokens, a
    sink, and values mixed with the first such layer's; returns (output, this layer's values before mixing)"""
    T = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    parts = {}
    for n in ("q", "k", "v"):
        u = h @ _w(weights, p + n).T + _w(weights, p + n + ".b")
        if m.get("conv"):
            u = short_conv(u, _w(weights, p + n + ".conv"))
        parts[n] = u
    q, k, v = parts["q"].reshape(T, H, d), parts["k"].reshape(T, G, d), parts["v"].reshape(T, G, e)
    rot = m.get("rot")
    if rot:
        q, k = rotate_pairs(q, pos, rot["dims"], rot["base"]), rotate_pairs(k, pos, rot["dims"], rot["base"])
    own_v = v
    if m.get("v_mix") and v_first is not None:
        lam = _w(weights, p + "vmix").reshape(())
        v = (1.0 - lam) * v + lam * v_first
    mask = m.get("mask") or {}
    vis = visible(T, mask.get("size", 0), mask.get("keep_first", 0))
    sink = _w(weights, p + "sink") if (p + "sink") in weights else None
    o = softmax_attention(q, k, v, m["scale"], vis, sink)
    return o.reshape(T, H * e) @ _w(weights, p + "o").T, own_v


def latent_attention_mixer(h, weights, p, m, eps):
    """keys and values from a normed low-rank latent, plus one rotated key part shared by all heads; sliding window; plain softmax"""
    T = h.shape[0]
    H, d, r, e, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    q = (h @ _w(weights, p + "q").T).reshape(T, H, d + r)
    down = h @ _w(weights, p + "dkv").T
    c = rms_norm(down[:, :R], _w(weights, p + "dkv.norm"), eps, False)
    k_rot = down[:, R:].reshape(T, 1, r)
    base = m["rot"]["base"]
    q_rot = rotate_pairs(q[..., d:].contiguous(), pos, r, base)
    k_rot = rotate_pairs(k_rot, pos, r, base)
    k_plain = (c @ _w(weights, p + "uk").T).reshape(T, H, d)
    v = (c @ _w(weights, p + "uv").T).reshape(T, H, e)
    qf = torch.cat([q[..., :d], q_rot], -1)
    kf = torch.cat([k_plain, k_rot.expand(T, H, r)], -1)
    vis = visible(T, (m.get("mask") or {}).get("size", 0), 0)
    o = softmax_attention(qf, kf, v, m["scale"], vis, None)
    return o.reshape(T, H * e) @ _w(weights, p + "o").T


def gla_mixer(h, weights, p, m, eps):
    """gated linear attention: a decay per key channel, S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, token by token"""
    T = h.shape[0]
    H, d, e, tau = m["heads"], m["dim"], m["vdim"], float(m["tau"])
    q = (h @ _w(weights, p + "q").T).reshape(T, H, d) * d ** -0.5
    k = (h @ _w(weights, p + "k").T).reshape(T, H, d)
    v = (h @ _w(weights, p + "v").T).reshape(T, H, e)
    z = (h @ _w(weights, p + "a1").T) @ _w(weights, p + "a2").T + _w(weights, p + "a2.b")
    alpha = torch.exp(torch.nn.functional.logsigmoid(z) / tau).reshape(T, H, d)
    S = torch.zeros(H, d, e, dtype=F64)
    o = torch.zeros(T, H, e, dtype=F64)
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hde,hd->he", S, q[t])
    o = rms_norm(o, _w(weights, p + "norm"), eps, False)
    g = h @ _w(weights, p + "g").T
    return (o.reshape(T, H * e) * (g * torch.sigmoid(g))) @ _w(weights, p + "o").T


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def dense_ff(h, weights, p):
    return (gelu_tanh(h @ _w(weights, p + "gate").T) * (h @ _w(weights, p + "up").T)) @ _w(weights, p + "down").T


def route(h, weights, p, f):
    """(ids (T, top), weights (T, top)): sigmoid scores; choice by score + correction inside the best `keep` groups (a group's score: the
    sum of its two largest choice scores); weights = the picks' plain scores over their sum"""
    r = f["router"]
    E, top = r["experts"], r["top"]
    g = r.get("groups") or {}
    n_groups, keep = g.get("count", 1), g.get("keep", g.get("count", 1))
    s = torch.sigmoid(h @ _w(weights, p + "router").T)
    choice = s + _w(weights, p + "correction")
    T = h.shape[0]
    ids = torch.zeros(T, top, dtype=torch.long)
    wts = torch.zeros(T, top, dtype=F64)
    size = E // n_groups
    for t in range(T):
        ch = choice[t].clone()
        if n_groups > 1:
            gs = torch.stack([ch[i * size:(i + 1) * size].topk(min(2, size)).values.sum() for i in range(n_groups)])
            kept = set(torch.argsort(-gs, stable=True)[:keep].tolist())
            for i in range(n_groups):
                if i not in kept:
                    ch[i * size:(i + 1) * size] = -math.inf
        pick = torch.argsort(-ch, stable=True)[:top]
        ids[t] = pick
        wts[t] = s[t, pick] / (s[t, pick].sum() + 1e-20)
    return ids, wts


def expert(h, weights, p, limit):
    g = torch.clamp(h @ _w(weights, p + "gate").T, max=limit)
    u = torch.clamp(h @ _w(weights, p + "up").T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ _w(weights, p + "down").T


def experts_ff(h, weights, p, f):
    ids, wts = route(h, weights, p, f)
    out = torch.zeros(h.shape[0], weights[p + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        for j in range(ids.shape[1]):
            out[t] += wts[t, j] * expert(h[t:t + 1], weights, f"{p}e{int(ids[t, j])}.", float(f["expert"]["limit"]))[0]
    return out


def model(cfg, weights, tokens, round_to=None):
    """(logits (T, vocab), [residual stream after every layer]).  round_to: a dtype every sub-layer input is rounded to (shows what a
    16-bit product path may cost); None: none"""
    eps = float(cfg["norm"]["eps"])
    x = _w(weights, "embed")[torch.as_tensor(tokens, dtype=torch.long)]
    rnd = (lambda t: t.to(round_to).to(F64)) if round_to is not None else (lambda t: t)
    v_first, streams = None, []
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = rnd(rms_norm(x, _w(weights, p + "norm1"), eps, True))
        if layer["type"] == "attention":
            y, own_v = attention_mixer(h, weights, p + "mix.", m, eps, v_first)
            if m.get("v_mix") and v_first is None:
                v_first = own_v
        elif layer["type"] == "latent_attention":
            y = latent_attention_mixer(h, weights, p + "mix.", m, eps)
        elif layer["type"] == "gla":
            y = gla_mixer(h, weights, p + "mix.", m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + y
        f = layer.get("mlp")
        if f is not None:
            h = rnd(rms_norm(x, _w(weights, p + "norm2"), eps, True))
            x = x + (dense_ff(h, weights, p + "mlp.") if f["kind"] == "dense" else experts_ff(h, weights, p + "mlp.", f))
        streams.append(x.clone())
    hn = rnd(rms_norm(x, _w(weights, "final.norm"), eps, True))
    logits = (hn @ _w(weights, "head").T) * float(cfg.get("logit_scale", 1.0))
    cap = float(cfg.get("logit_softcap", 0.0) or 0.0)
    if cap > 0:
        logits = cap * torch.tanh(logits / cap)
    return logits, streams


def random_weights(cfg, seed=0, fixed_choice=False, low=8):
    """every tensor the configuration asks for, bf16-representable values (both serving formats start from the same numbers).
    fixed_choice: the routers' correction terms are distinct powers of two times 1.25 -- more than 1 apart, and the sums of any two are
    distinct as well -- so that they alone order the choice scores AND the groups' scores (sigmoid scores lie in (0, 1)): no choice is
    a close call under a rounded router input; the weights of the chosen experts still follow the scores."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    sd = {}

    def mat(name, rows, cols, std=None):
        sd[name] = (torch.randn(rows, cols, generator=g) * (std if std is not None else cols ** -0.5)).to(torch.bfloat16)

    def vec(name, n, std=0.2, mean=0.0):
        sd[name] = (mean + std * torch.randn(n, generator=g)).to(torch.bfloat16)

    mat("embed", cfg["vocab"], W, 1.5)
    mat("head", cfg["vocab"], W)
    vec("final.norm", W)
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        vec(p + "norm1", W)
        H, d, v = m["heads"], m["dim"], m["vdim"]
        if l["type"] == "attention":
            G = m["kv_heads"]
            for n, rows in (("q", H * d), ("k", G * d), ("v", G * v)):
                mat(p + "mix." + n, rows, W)
                vec(p + "mix." + n + ".b", rows, 0.3)
                if m.get("conv"):
                    sd[p + "mix." + n + ".conv"] = (torch.randn(rows, m["conv"], generator=g) * 0.6).to(torch.bfloat16)
            sd[p + "mix.vmix"] = torch.tensor(0.3 + 0.1 * i).to(torch.bfloat16)
            vec(p + "mix.sink", H, 1.0)
            mat(p + "mix.o", W, H * v)
        elif l["type"] == "latent_attention":
            r, R = m["rot_dim"], m["kv_rank"]
            mat(p + "mix.q", H * (d + r), W)
            mat(p + "mix.dkv", R + r, W)
            vec(p + "mix.dkv.norm", R, 0.2, 1.0)
            mat(p + "mix.uk", H * d, R)
            mat(p + "mix.uv", H * v, R)
            mat(p + "mix.o", W, H * v)
        else:
            for n, rows in (("q", H * d), ("k", H * d), ("v", H * v), ("g", H * v), ("a1", low)):
                mat(p + "mix." + n, rows, W)
            mat(p + "mix.a2", H * d, low, 1.0)
            vec(p + "mix.a2.b", H * d, 1.0, 2.0)
            vec(p + "mix.norm", v, 0.2, 1.0)
            mat(p + "mix.o", W, H * v)
        f = l.get("mlp")
        if f is None:
            continue
        vec(p + "norm2", W)
        if f["kind"] == "dense":
            mat(p + "mlp.gate", f["ff"], W)
            mat(p + "mlp.up", f["ff"], W)
            mat(p + "mlp.down", W, f["ff"])
        else:
            E, ff = f["router"]["experts"], f["expert"]["ff"]
            mat(p + "mlp.router", E, W)
            if fixed_choice:
                sd[p + "mlp.correction"] = (1.25 * 2.0 ** torch.randperm(E, generator=g).double()).to(torch.bfloat16)
            else:
                vec(p + "mlp.correction", E, 0.3)
            for e in range(E):
                mat(f"{p}mlp.e{e}.gate", ff, W, 2.0 * W ** -0.5)           # (wide enough that the clamps bite)
                mat(f"{p}mlp.e{e}.up", ff, W, 2.0 * W ** -0.5)
                mat(f"{p}mlp.e{e}.down", W, ff)
    return sd
