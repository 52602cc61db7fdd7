"""Gaparax: a decoder-only model whose residual is kept as SEVERAL streams, whose sub-layers' results pass a sigmoid gate before they enter
the streams, and whose layers each pick one sequence mixer -- grouped attention with sigmoid weights inside chunks of positions, normed
queries and keys, a factor per head, capped scores and a learned bias by distance; latent attention with a rotated key part whose
frequencies are rescaled, and a sink -- and a dense or mixture-of-experts feed-forward, described layer by layer in config.json.

Shape of a layer (x_0 .. x_{S-1} are the fp32 streams of a token, all equal to the embedding at the start; N = RMS norm with a plain
weight, u / sqrt(mean(u^2) + eps) * w).  For sub-layer q (1: the mixer, 2: the feed-forward, when the layer has one):
    h   = N_q(sum_s in_q[s] x_s)
    y   = sublayer(h) * sigmoid(W_rg,q h + b_rg,q)
    x_d = sum_s mix_q[s][d] x_s + out_q[d] y           for every stream d at once, from the old streams
Embedding: table[token].  Output: N of the sum of the streams, then the vocabulary projection.

Configuration keys: vocab, width, streams, norm.eps, layers[i] = {type, mixer, mlp}:
    type "attention"         mixer: heads, kv_heads, dim, vdim, scale, softcap, bias_max, mask.size
    type "latent_attention"  mixer: heads, dim, rot_dim, vdim, kv_rank, scale, rot.{dims, base, scaling.{factor, original, fast, slow}}
    mlp (or null)            kind "dense": ff;  kind "moe": expert.ff, router.{experts, top, scale, groups.{count, keep}}
Tensors: embed, head, final.norm, l<i>.norm1 / norm2, l<i>.hc1 / hc2 .in / .out / .mix, l<i>.rg1 / rg2 (+ .b), l<i>.mix.*, l<i>.mlp.* (see
the mixer classes in mixers.py).

The model runs RAGGED steps like the other models of the engine: every launch covers all tokens of a step; cached rows live in paged
planes of the engine's CacheManager.  The gate's projection rides in the sub-layer's own first product (the mixers' input projection,
the dense feed-forward's up projection, the experts' router), and one launch between two products writes the streams AND the next
sub-layer's normed input, so a layer is: product, mixer kernels, product, streams update, feed-forward launches, streams update.
"""
from dataclasses import dataclass, field
from typing import List, Optional

import torch

from . import seqops
from ._lib import ZLError
from .mixers import LatentAttention, PlainFF, RoutedExpertsFF, WindowAttention, _mat, _rand, _vec
from .registry import register_model

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
           torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}

MAX_STREAMS = 8              # what the stream kernels hold in registers per element


@dataclass
class GaparaxLayerConfig:
    type: str
    mixer: dict
    mlp: Optional[dict]


@dataclass
class GaparaxConfig:
    vocab: int
    width: int
    streams: int
    eps: float
    max_positions: int
    layers: List[GaparaxLayerConfig] = field(default_factory=list)

    @classmethod
    def from_dict(cls, cfg):
        try:
            layers = [GaparaxLayerConfig(l["type"], dict(l["mixer"]), None if l.get("mlp") is None else dict(l["mlp"])) for l in cfg["layers"]]
            c = cls(int(cfg["vocab"]), int(cfg["width"]), int(cfg["streams"]), float(cfg["norm"]["eps"]),
                    int(cfg.get("max_positions", 1 << 24)), layers)                       # (positions are fp32: exact to 2^24)
        except KeyError as e:
            raise ZLError(f"Gaparax config: missing key {e}")
        if not 1 <= c.streams <= MAX_STREAMS:
            raise ZLError(f"Gaparax config: streams must be 1 .. {MAX_STREAMS}")
        for i, l in enumerate(c.layers):
            if l.type not in MIXER_BUILDERS:
                raise ZLError(f"Gaparax config: layer {i}: unknown mixer type {l.type!r}")
            if l.mlp is not None and l.mlp.get("kind") not in FF_BUILDERS:
                raise ZLError(f"Gaparax config: layer {i}: unknown feed-forward kind {l.mlp.get('kind')!r}")
        return c


def _attention(name, width, m, eps):
    mask = m.get("mask") or {}
    return WindowAttention(name, width, int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]), int(m["vdim"]), float(m["scale"]), 0, 0, 10000.0, 1.0,
                           eps, qk_norm=True, rotate_values=False, talk=False, gate=True, norm_weight=True, head_scale=True,
                           softcap=float(m.get("softcap") or 0.0), rel_far=int(m["bias_max"]), chunk=int(mask.get("size", 0)), weights="sigmoid")


def _latent(name, width, m, eps):
    rot = m.get("rot") or {}
    rot_dim = int(m.get("rot_dim", 0))
    if rot_dim and int(rot.get("dims", rot_dim)) != rot_dim:
        raise ZLError("Gaparax config: the rotated part of a latent attention layer is rotated as a whole (rot.dims = rot_dim)")
    return LatentAttention(name, width, int(m["heads"]), int(m["dim"]), int(m["vdim"]), int(m["kv_rank"]), float(m["scale"]), eps, sink=True,
                           gate=False, rot_dim=rot_dim, rot_base=float(rot.get("base", 10000.0)), window=0, rot_layout="half",
                           rot_scaling=rot.get("scaling"))


MIXER_BUILDERS = {"attention": _attention, "latent_attention": _latent}


def _dense(width, f):
    return PlainFF(width, int(f["ff"]), act="relu2")


def _experts(width, f):
    r = f["router"]
    g = r.get("groups") or {}
    return RoutedExpertsFF(width, int(f["expert"]["ff"]), int(r["experts"]), int(r["top"]), identity=0, groups=int(g.get("count", 1)),
                           keep=int(g.get("keep", g.get("count", 1))), correction=False, renorm=False, score="softmax", group_top=1, act="silu",
                           weight_scale=float(r.get("scale", 1.0)))


FF_BUILDERS = {"dense": _dense, "moe": _experts}


class StreamPort:
    """How ONE sub-layer meets the streams: the coefficients of the sum it reads, the norm of that sum, the gate of its result, the matrix
    that mixes the streams and the factors with which its result enters them.  Tensors: <layer>.norm<q>, .hc<q>.in / .out (streams),
    .hc<q>.mix (streams, streams) indexed [from][to], .rg<q> (width, width), .rg<q>.b (width)."""

    def __init__(self, prefix, q, streams, width):
        self.prefix, self.q, self.n, self.width = prefix, q, streams, width
        self.read = self.out = self.mix = self.norm = self.gate_w = self.gate_b = None

    def load(self, get, dtype, device):
        p, q, n, W = self.prefix, self.q, self.n, self.width
        self.norm = _vec(get, f"{p}norm{q}", W, device)
        self.read, self.out = _vec(get, f"{p}hc{q}.in", n, device), _vec(get, f"{p}hc{q}.out", n, device)
        self.mix = _mat(get, f"{p}hc{q}.mix", (n, n), torch.float32, device)
        self.gate_w, self.gate_b = _mat(get, f"{p}rg{q}", (W, W), dtype, device), _vec(get, f"{p}rg{q}.b", W, device)

    def init_random(self, gen, dtype, device):
        n, W = self.n, self.width
        self.norm = 1.0 + 0.1 * torch.randn(W, generator=gen, device=device)
        self.read = 1.0 / n + 0.1 * torch.randn(n, generator=gen, device=device)
        self.out = 1.0 + 0.1 * torch.randn(n, generator=gen, device=device)
        self.mix = torch.eye(n, device=device) + 0.1 * torch.randn(n, n, generator=gen, device=device)
        self.gate_w, self.gate_b = _rand(gen, (W, W), W ** -0.5, dtype, device), torch.zeros(W, device=device)

    def attach(self, sub):
        """the gate's projection joins the sub-layer's input product when it has one to join"""
        self.fused = hasattr(sub, "attach_side")
        if self.fused:
            sub.attach_side(self.gate_w)
            self.gate_w = None                         # (the rows live in the sub-layer's matrix now)

    def gate_of(self, sub, h):
        """(fp32 tensor, first column) of W_rg h"""
        if self.fused:
            return sub.side
        return seqops.gemm_nt(h, self.gate_w), 0


class GaparaxLayer:
    def __init__(self, idx, cfg: GaparaxConfig, lc: GaparaxLayerConfig):
        self.idx, self.name, self.width, self.eps, self.n = idx, f"l{idx}", cfg.width, cfg.eps, cfg.streams
        self.mixer = MIXER_BUILDERS[lc.type](self.name + ".mix", cfg.width, lc.mixer, cfg.eps)
        self.ff = FF_BUILDERS[lc.mlp["kind"]](cfg.width, lc.mlp) if lc.mlp is not None else None
        self.port1 = StreamPort(self.name + ".", 1, cfg.streams, cfg.width)
        self.port2 = StreamPort(self.name + ".", 2, cfg.streams, cfg.width) if self.ff is not None else None

    def load(self, get, dtype, device):
        self.mixer.load(get, self.name + ".mix.", dtype, device)
        self.port1.load(get, dtype, device)
        self.port1.attach(self.mixer)
        if self.ff is not None:
            self.ff.load(get, self.name + ".mlp.", dtype, device)
            self.port2.load(get, dtype, device)
            self.port2.attach(self.ff)

    def init_random(self, gen, dtype, device):
        self.mixer.init_random(gen, dtype, device)
        self.port1.init_random(gen, dtype, device)
        self.port1.attach(self.mixer)
        if self.ff is not None:
            self.ff.init_random(gen, dtype, device)
            self.port2.init_random(gen, dtype, device)
            self.port2.attach(self.ff)

    def first_port(self):
        return self.port1

    def forward(self, src, xs, h, batch, dtype, next_port):
        """src: the streams that are read (xs itself, or the embedding rows before the first update); h = this layer's first normed input
        in the serving format; returns the next layer's (None without next_port)"""
        y = self.mixer.forward(h, batch)
        g, g0 = self.port1.gate_of(self.mixer, h)
        nxt = self.port2 if self.ff is not None else next_port
        h = self._update(self.port1, src, xs, y, g, g0, nxt, dtype)
        if self.ff is not None:
            y = self.ff.forward(h)
            g, g0 = self.port2.gate_of(self.ff, h)
            h = self._update(self.port2, xs, xs, y, g, g0, next_port, dtype)
        return h

    def _update(self, port, src, xs, y, g, g0, nxt, dtype):
        return seqops.streams_update(src, xs, self.n, y, port.mix, port.out, gate=g, g_col0=g0, gate_bias=port.gate_b,
                                     next_coef=nxt.read if nxt is not None else None, next_weight=nxt.norm if nxt is not None else None,
                                     eps=self.eps, dtype=dtype)

    def weight_bytes(self):
        ports = sum(p.gate_w.numel() * p.gate_w.element_size() for p in (self.port1, self.port2) if p is not None and not p.fused)
        return self.mixer.weight_bytes() + (self.ff.weight_bytes() if self.ff is not None else 0) + ports


@register_model("Gaparax")
class GaparaxModel:
    ragged = True                    # the engine drives it with RaggedBatch steps and a CacheManager

    def __init__(self, cfg: GaparaxConfig, dtype="bfloat16", device="cuda:0"):
        if dtype not in _DTYPES:
            raise ZLError(f"Gaparax serves in bfloat16 or float32, not {dtype}")
        self.cfg, self.dtype, self.device = cfg, _DTYPES[dtype], torch.device(device)
        self.layers = [GaparaxLayer(i, cfg, lc) for i, lc in enumerate(cfg.layers)]
        self.final_norm = self.embed = self.head = None
        self.page_size = 64

    @classmethod
    def from_config(cls, cfg: dict, dtype="bfloat16", device="cuda:0"):
        return cls(GaparaxConfig.from_dict(cfg), dtype, device)

    @property
    def vocab_size(self):
        return self.cfg.vocab

    @property
    def max_positions(self):
        return self.cfg.max_positions

    def load_weights(self, ckpt):
        c, dev, dt = self.cfg, self.device, self.dtype

        def get(name):
            return ckpt[name]
        for name in ("embed", "head"):
            t = get(name)
            if tuple(t.shape) != (c.vocab, c.width):
                raise ZLError(f"tensor {name}: shape {tuple(t.shape)}, expected {(c.vocab, c.width)}")
            setattr(self, name, t.to(device=dev, dtype=dt).contiguous())
        self.final_norm = _vec(get, "final.norm", c.width, dev)
        for layer in self.layers:
            layer.load(get, dt, dev)
        return self

    def init_random(self, seed=0):
        c, dev, dt = self.cfg, self.device, self.dtype
        gen = torch.Generator(device=dev).manual_seed(seed)
        self.embed = torch.randn(c.vocab, c.width, generator=gen, device=dev).to(dt)
        self.head = (torch.randn(c.vocab, c.width, generator=gen, device=dev) * c.width ** -0.5).to(dt)
        self.final_norm = 1.0 + 0.1 * torch.randn(c.width, generator=gen, device=dev)
        for layer in self.layers:
            layer.init_random(gen, dt, dev)
        return self

    def bind_cache(self, cache):
        """register every layer's per-token planes with the engine's cache manager"""
        if cache.page_size != self.page_size:
            raise ZLError("cache page size mismatch")
        for layer in self.layers:
            layer.mixer.bind(cache, self.dtype)
        return cache

    def _run(self, tokens, batch, keep=None):
        """returns (streams, n): fp32 (n_tok, n, width) -- or the embedding rows (n_tok, width) read as n equal streams without layers"""
        c = self.cfg
        x = seqops.embed(tokens, self.embed, None, 1.0, batch)
        if not self.layers:
            return x
        xs = torch.empty((batch.n_tok, c.streams, c.width), dtype=torch.float32, device=x.device)
        port = self.layers[0].first_port()
        h = seqops.streams_norm(x, c.streams, port.read, port.norm, c.eps, self.dtype)          # (all streams still equal the embedding)
        src = x
        for i, layer in enumerate(self.layers):
            nxt = self.layers[i + 1].first_port() if i + 1 < len(self.layers) else None
            h = layer.forward(src, xs, h, batch, self.dtype, nxt)
            src = xs
            if keep is not None:
                keep.append(xs.sum(1))
        return xs

    def forward(self, tokens, batch, want_rows):
        """tokens: int32 device (n_tok) in the batch's flat order; want_rows: int32 device, flat token indices whose logits are wanted
        (None or empty: the step only advances the caches).  Returns fp32 logits (len(want_rows), vocab) or None."""
        xs = self._run(tokens, batch)
        if want_rows is None or want_rows.numel() == 0:
            return None
        hn = seqops.streams_norm(xs, self.cfg.streams, None, self.final_norm, self.cfg.eps, self.dtype, rows=want_rows)
        return seqops.gemm_nt(hn, self.head)

    def forward_layers(self, tokens, batch):
        """the sum of the streams after every layer (debugging and tests): list of fp32 (n_tok, width)"""
        out = []
        self._run(tokens, batch, keep=out)
        return out

    def weight_bytes(self):
        return sum(l.weight_bytes() for l in self.layers) + sum(t.numel() * t.element_size() for t in (self.embed, self.head))
