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
    out = torch.zeros(T, H, e, dtype=F64)
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * m["scale"] * temp[a]
        if cap > 0:
            s = cap * torch.tanh(s / cap)
        s = s + bias[a]
        w = torch.where(vis, torch.sigmoid(s + offset[a]), torch.zeros((), dtype=F64))
        out[:, a] = w @ v[:, g]
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


def route(h, weights, p, r):
    """(ids (T, top), weights (T, top)): softmax over all experts; only experts of the `keep` groups with the largest best member count;
    the `top` largest scores, weighted by score * router.scale"""
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
    return ids, s.gather(1, ids) * float(r.get("scale", 1.0))


def experts_ff(h, weights, p, f):
    """sum over the chosen experts of weight * down(silu(gate h) * (up h))"""
    ids, wts = route(h, weights, p, f["router"])
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


def model(tokens, weights, cfg, keep_layers=None):
    """logits (T, vocab) of one sequence; keep_layers: a list that receives the sum of the streams after every layer"""
    eps = float(cfg["norm"]["eps"])
    x = _w(weights, "embed")[torch.as_tensor(tokens, dtype=torch.long)]
    xs = x[None].repeat(int(cfg["streams"]), 1, 1)
    for i, l in enumerate(cfg["layers"]):
        p = f"l{i}."
        xs = sublayer(xs, weights, p, 1, lambda h: MIXERS[l["type"]](h, weights, p + "mix.", l["mixer"], eps), eps)
        f = l.get("mlp")
        if f is not None:
            fn = (lambda h: dense_ff(h, weights, p + "mlp.")) if f["kind"] == "dense" else (lambda h: experts_ff(h, weights, p + "mlp.", f))
            xs = sublayer(xs, weights, p, 2, fn, eps)
        if keep_layers is not None:
            keep_layers.append(xs.sum(0))
    return rms_norm(xs.sum(0), _w(weights, "final.norm"), eps) @ _w(weights, "head").T
