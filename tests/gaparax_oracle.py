"""A plain float64 restatement of the Gaparax design, one function per mechanism, whole sequences at a time, no cache and no batching.

It shares no code with zhilight_amd: the product path (gaparax.py, mixers.py, the kernels) is held against it.  `weights` is a mapping
name -> tensor with the names of the checkpoint ("l<i>.mix.q", "l<i>.mlp.e<j>.gate", "l<i>.hc1.mix", ...); `cfg` is the dictionary of
config.json.

Notation: T tokens at positions 0 .. T-1, h (T, width) a sub-layer's input, matrices stored (out, in), S residual streams.
"""
import math

import torch

F64 = torch.float64


def _w(weights, name):
    return weights[name].to(F64)


def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * w over the last axis"""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


# ---- distance bias ---------------------------------------------------------------------------------------------------------------------
def distance_bucket(n, rows, far):
    """the table row of the distance n >= 0: the first rows // 2 distances have a row each, the rest share the remaining rows on a
    logarithmic scale that reaches the last row at the distance `far`"""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def distance_bias(T, table, far):
    """(H, T, T): table[bucket(i - j), h] for j <= i, 0 elsewhere; table (rows, H)"""
    rows, H = table.shape
    out = torch.zeros(H, T, T, dtype=F64)
    for i in range(T):
        for j in range(i + 1):
            out[:, i, j] = table[distance_bucket(i - j, rows, far)]
    return out


def chunk_visible(T, size):
    """(T, T) bool: query i sees key j <= i of its own chunk, chunks of `size` positions counted from position 0 (size 0: every j <= i)"""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    same = (i // size == j // size) if size > 0 else torch.ones(T, T, dtype=torch.bool)
    return (j <= i) & same


# ---- sigmoid attention -----------------------------------------------------------------------------------------------------------------
def sigmoid_attention(q, k, v, scale, temp, cap, bias, vis, offset):
    """q (T, H, d), k (T, G, d), v (T, G, e); head a reads kv head a // (H / G); score = q.k * scale * temp[a], capped by cap * tanh(. / cap)
    when cap > 0, plus bias[a] (T, T); the weight of a visible key is sigmoid(score + offset[a]), every key on its own"""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * scale * temp[a]
        if cap > 0:
            s = cap * torch.tanh(s / cap)
        if bias is not None:
            s = s + bias[a]
        w = torch.where(vis, torch.sigmoid(s + offset[a]), torch.zeros((), dtype=F64))
        out[:, a] = w @ v[:, g]
    return out


def sigmoid_attention_mixer(h, weights, p, m, eps):
    """grouped attention whose weights are sigmoids, not a softmax: q and k normed per head, score scaled, multiplied by a number per head,
    capped by tanh, a distance bias added, then sigmoid(score + offset_h) for every visible key of the query's chunk; the heads' sums are
    gated by sigmoid(W_g h) before the output projection"""
    T = h.shape[0]
    H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_norm((h @ _w(weights, p + "q").T).reshape(T, H, d), _w(weights, p + "q.norm"), eps)
    k = rms_norm((h @ _w(weights, p + "k").T).reshape(T, G, d), _w(weights, p + "k.norm"), eps)
    v = (h @ _w(weights, p + "v").T).reshape(T, G, e)
    temp, offset, cap = _w(weights, p + "temp"), _w(weights, p + "pb"), float(m.get("softcap") or 0.0)
    bias = distance_bias(T, _w(weights, p + "rel"), m["bias_max"])
    vis = chunk_visible(T, int((m.get("mask") or {}).get("size", 0)))
    out = sigmoid_attention(q, k, v, m["scale"], temp, cap, bias, vis, offset)
    gate = torch.sigmoid(h @ _w(weights, p + "g").T)
    return (out.reshape(T, H * e) * gate) @ _w(weights, p + "o").T


# ---- rotation with rescaled frequencies ---------------------------------------------------------------------------------------------------
def scaled_frequencies(dims, base, scaling):
    """(frequencies (dims / 2), magnitude): base^(-2i/dims), and with `scaling` {factor, original, fast, slow} a blend per pair between the
    frequency and frequency / factor -- pairs that turn more than `fast` times over `original` positions keep theirs, pairs that turn less
    than `slow` times are divided, a linear ramp over the pair index between -- and cos / sin scaled by 0.1 ln(factor) + 1"""
    i = torch.arange(dims // 2, dtype=F64)
    f = torch.pow(torch.tensor(float(base), dtype=F64), -2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])

    def pair_index(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(pair_index(float(scaling["fast"]))), 0)
    hi = min(math.ceil(pair_index(float(scaling["slow"]))), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_half(x, pos, dims, freq, magnitude):
    """x (T, heads, size): coordinate i < dims/2 pairs with i + dims/2, the pair turned by pos * freq[i], cos and sin times magnitude"""
    out = x.clone()
    ang = pos.to(F64)[:, None] * freq[None, :]
    c, s = (torch.cos(ang) * magnitude)[:, None, :], (torch.sin(ang) * magnitude)[:, None, :]
    u, v = x[..., :dims // 2], x[..., dims // 2:dims]
    out[..., :dims // 2] = u * c - v * s
    out[..., dims // 2:dims] = v * c + u * s
    return out


def sink_softmax(s, vis, sink):
    """softmax over the visible keys whose denominator also holds exp(sink); s (T, T)"""
    s = s.masked_fill(~vis, -math.inf)
    m = torch.maximum(s.max(-1, keepdim=True).values, sink.expand(s.shape[0], 1))
    e = torch.exp(s - m)
    return e / (e.sum(-1, keepdim=True) + torch.exp(sink - m))


def latent_attention_mixer(h, weights, p, m, eps):
    """keys and values from a normed low-rank latent, plus one rotated key part shared by all heads; causal; softmax with a sink"""
    T = h.shape[0]
    H, d, r, e, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    q = (h @ _w(weights, p + "q").T).reshape(T, H, d + r)
    down = h @ _w(weights, p + "dkv").T
    c = rms_norm(down[:, :R], _w(weights, p + "dkv.norm"), eps)
    rot = m["rot"]
    freq, mag = scaled_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
    q_rot = rotate_half(q[..., d:].contiguous(), pos, rot["dims"], freq, mag)
    k_rot = rotate_half(down[:, R:].reshape(T, 1, r), pos, rot["dims"], freq, mag)
    k_plain = (c @ _w(weights, p + "uk").T).reshape(T, H, d)
    v = (c @ _w(weights, p + "uv").T).reshape(T, H, e)
    vis = chunk_visible(T, 0)
    sink = _w(weights, p + "sink")
    out = torch.zeros(T, H, e, dtype=F64)
    for a in range(H):
        s = (q[:, a, :d] @ k_plain[:, a].T + q_rot[:, a] @ k_rot[:, 0].T) * m["scale"]
        out[:, a] = sink_softmax(s, vis, sink[a]) @ v[:, a]
    return out.reshape(T, H * e) @ _w(weights, p + "o").T


# ---- feed-forwards ---------------------------------------------------------------------------------------------------------------------
def dense_ff(h, weights, p):
    """down(relu(up h)^2)"""
    z = torch.relu(h @ _w(weights, p + "up").T)
    return (z * z) @ _w(weights, p + "down").T


def route(h, weights, p, r, margins=None):
    """(ids (T, top), weights (T, top)): softmax over all experts; only experts of the `keep` groups with the largest best member count;
    the `top` largest scores, weighted by score * router.scale.  margins (a list): receives the smallest difference of logits that decided
    a choice -- between the last kept and the first dropped group, and between the last chosen and the first unchosen allowed expert"""
    z = h @ _w(weights, p + "router").T
    s = torch.softmax(z, -1)
    T, E = s.shape
    g = r.get("groups") or {}
    count = int(g.get("count", 1))
    keep = int(g.get("keep", count))
    per = E // count
    best = s.reshape(T, count, per).max(-1).values
    kept = torch.zeros(T, count, dtype=torch.bool)
    kept.scatter_(1, best.topk(keep, dim=-1).indices, True)
    allowed = kept[:, :, None].expand(T, count, per).reshape(T, E)
    ids = s.masked_fill(~allowed, -1.0).topk(int(r["top"]), dim=-1).indices
    if margins is not None:
        gz = z.reshape(T, count, per).max(-1).values.sort(-1, descending=True).values
        az = z.masked_fill(~allowed, -math.inf).sort(-1, descending=True).values
        top = int(r["top"])
        gaps = []
        if keep < count:
            gaps.append(gz[:, keep - 1] - gz[:, keep])
        if top < keep * per:
            gaps.append(az[:, top - 1] - az[:, top])
        if gaps:
            margins.append(float(torch.stack(gaps).min()))
    return ids, s.gather(1, ids) * float(r.get("scale", 1.0))


def experts_ff(h, weights, p, f, margins=None):
    """sum over the chosen experts of weight * down(silu(gate h) * (up h))"""
    ids, wts = route(h, weights, p, f["router"], margins)
    out = torch.zeros(h.shape[0], _w(weights, p + "e0.down").shape[0], dtype=F64)
    for t in range(h.shape[0]):
        for c in range(ids.shape[1]):
            e = p + "e%d." % int(ids[t, c])
            a = h[t] @ _w(weights, e + "gate").T
            out[t] += wts[t, c] * ((a * torch.sigmoid(a) * (h[t] @ _w(weights, e + "up").T)) @ _w(weights, e + "down").T)
    return out


# ---- layers ----------------------------------------------------------------------------------------------------------------------------
MIXERS = {"attention": sigmoid_attention_mixer, "latent_attention": latent_attention_mixer}


def sublayer(xs, weights, p, q, fn, eps):
    """one sub-layer over S residual streams xs (S, T, width): read a weighted sum of the streams, norm it, run fn, gate the result by
    sigmoid(W h + b) of the normed input, then mix the streams and add the result to each with its own factor"""
    u = torch.einsum("s,stw->tw", _w(weights, f"{p}hc{q}.in"), xs)
    h = rms_norm(u, _w(weights, f"{p}norm{q}"), eps)
    y = fn(h)
    y = y * torch.sigmoid(h @ _w(weights, f"{p}rg{q}").T + _w(weights, f"{p}rg{q}.b"))
    mixed = torch.einsum("su,stw->utw", _w(weights, f"{p}hc{q}.mix"), xs)          # (the matrix is indexed [from, to])
    return mixed + _w(weights, f"{p}hc{q}.out")[:, None, None] * y[None]


def model(tokens, weights, cfg, keep_layers=None, margins=None):
    """logits (T, vocab) of one sequence; keep_layers: a list that receives the sum of the streams after every layer; margins: see route"""
    eps = float(cfg["norm"]["eps"])
    x = _w(weights, "embed")[torch.as_tensor(tokens, dtype=torch.long)]
    xs = x[None].repeat(int(cfg["streams"]), 1, 1)
    for i, l in enumerate(cfg["layers"]):
        p = f"l{i}."
        xs = sublayer(xs, weights, p, 1, lambda h: MIXERS[l["type"]](h, weights, p + "mix.", l["mixer"], eps), eps)
        f = l.get("mlp")
        if f is not None:
            fn = (lambda h: dense_ff(h, weights, p + "mlp.")) if f["kind"] == "dense" else (lambda h: experts_ff(h, weights, p + "mlp.", f, margins))
            xs = sublayer(xs, weights, p, 2, fn, eps)
        if keep_layers is not None:
            keep_layers.append(xs.sum(0))
    return rms_norm(xs.sum(0), _w(weights, "final.norm"), eps) @ _w(weights, "head").T


# ---- test weights ------------------------------------------------------------------------------------------------------------------------
def random_weights(cfg, seed=0, rel_rows=12, fixed_choice=False):
    """every tensor the configuration asks for, bf16-representable values (both serving formats start from the same numbers).
    fixed_choice: the routers read ONE reserved coordinate of the residual only -- coordinate 0 of the embedding holds a number whose sign
    and size the token decides, and no sub-layer writes to it -- with evenly spaced multiples per expert, so that the order of the logits
    is one fixed order or its reverse, with wide gaps: no choice is a close call under a rounded router input, while the chosen experts'
    weights still follow the softmax of logits that vary with the token."""
    g = torch.Generator().manual_seed(seed)
    W, S = cfg["width"], cfg["streams"]
    sd = {}

    def mat(name, rows, cols, std=None):
        sd[name] = (torch.randn(rows, cols, generator=g) * (std if std is not None else cols ** -0.5)).to(torch.bfloat16)

    def vec(name, n, std=0.2, mean=0.0):
        sd[name] = (mean + std * torch.randn(n, generator=g)).to(torch.bfloat16)

    mat("embed", cfg["vocab"], W, 1.5)
    if fixed_choice:
        size = 2.0 + 2.0 * torch.rand(cfg["vocab"], generator=g)
        sd["embed"][:, 0] = torch.where(torch.arange(cfg["vocab"]) % 3 == 0, -size, size).to(torch.bfloat16)
    mat("head", cfg["vocab"], W)
    vec("final.norm", W, 0.2, 1.0)
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        H, d, v = m["heads"], m["dim"], m["vdim"]
        if l["type"] == "attention":
            G = m["kv_heads"]
            for n, rows in (("q", H * d), ("k", G * d), ("v", G * v), ("g", H * v)):
                mat(p + "mix." + n, rows, W)
            vec(p + "mix.q.norm", d, 0.3, 1.0)
            vec(p + "mix.k.norm", d, 0.3, 1.0)
            vec(p + "mix.temp", H, 0.4, 1.5)
            vec(p + "mix.pb", H, 0.7, -1.5)
            sd[p + "mix.rel"] = (torch.randn(rel_rows + 2 * (i % 2), H, generator=g) * 1.2).to(torch.bfloat16)
            mat(p + "mix.o", W, H * v)
        else:
            r, R = m["rot_dim"], m["kv_rank"]
            mat(p + "mix.q", H * (d + r), W)
            mat(p + "mix.dkv", R + r, W)
            vec(p + "mix.dkv.norm", R, 0.2, 1.0)
            mat(p + "mix.uk", H * d, R)
            mat(p + "mix.uv", H * v, R)
            vec(p + "mix.sink", H, 1.0)
            mat(p + "mix.o", W, H * v)
        f = l.get("mlp")
        for q in (1, 2) if f is not None else (1,):
            vec(f"{p}norm{q}", W, 0.2, 1.0)
            vec(f"{p}hc{q}.in", S, 0.3, 1.0 / S)
            vec(f"{p}hc{q}.out", S, 0.3, 0.8)
            sd[f"{p}hc{q}.mix"] = (torch.eye(S) + 0.25 * torch.randn(S, S, generator=g)).to(torch.bfloat16)
            mat(f"{p}rg{q}", W, W)
            vec(f"{p}rg{q}.b", W, 0.5, 0.5)
        if f is None:
            continue
        if f["kind"] == "dense":
            mat(p + "mlp.up", f["ff"], W)
            mat(p + "mlp.down", W, f["ff"])
        else:
            E, ff = f["router"]["experts"], f["expert"]["ff"]
            mat(p + "mlp.router", E, W, 2.0 * W ** -0.5)
            for e in range(E):
                mat(f"{p}mlp.e{e}.gate", ff, W)
                mat(f"{p}mlp.e{e}.up", ff, W)
                mat(f"{p}mlp.e{e}.down", W, ff)
            if fixed_choice:
                r = torch.zeros(E, W)
                r[:, 0] = 0.8 * torch.randperm(E, generator=g).double() - 0.4 * E
                sd[p + "mlp.router"] = r.to(torch.bfloat16)
    if fixed_choice:
        for name, t in sd.items():
            if name.endswith((".mix.o", ".mlp.down")) or (".mlp.e" in name and name.endswith(".down")):
                t[:1] = 0.0
    return sd
