"""Gutivik: a decoder-only model whose layers each pick one sequence mixer -- grouped softmax attention with a short convolution, a window
that keeps the first tokens, a sink and blended values; latent attention with a rotated key part and a window; gated linear attention
with a decay per key channel -- and a dense or mixture-of-experts feed-forward, described layer by layer in config.json.

Shape of a layer (x is the fp32 residual stream; N = RMS norm with a weight stored around zero, x / sqrt(mean(x^2) + eps) * (1 + w)):
    x = x + mixer(N1(x))
    x = x + ff(N2(x))                    when the layer has a feed-forward
Embedding: table[token].  Output: N, the vocabulary projection times logit_scale, then cap * tanh(. / cap) when logit_softcap is set.

Configuration keys: vocab, width, norm.eps, logit_scale, logit_softcap, layers[i] = {type, mixer, mlp}:
    type "attention"         mixer: heads, kv_heads, dim, vdim, scale, conv (taps), rot.{dims, base}, mask.{size, keep_first}, v_mix
    type "latent_attention"  mixer: heads, dim, rot_dim, vdim, kv_rank, scale, rot.base, mask.size
    type "gla"               mixer: heads, dim, vdim, tau
    mlp (or null)            kind "dense": ff;  kind "moe": expert.{ff, limit}, router.{experts, top, groups.{count, keep}}
Tensors: embed, head, final.norm, l<i>.norm1 / norm2, l<i>.mix.*, l<i>.mlp.* (see the mixer classes in mixers.py).

The model runs RAGGED steps like the other models of the engine: every launch covers all tokens of a step; cached rows live in paged
planes of the engine's CacheManager, recurrent states and convolution tails in its slot states.  A residual launch also writes the next
sub-layer's normed input, so a layer is: product, mixer kernels, product, add+norm, feed-forward launches, add+norm.
"""
from dataclasses import dataclass, field
from typing import List, Optional

import torch

from . import seqops
from ._lib import ZLError
from .mixers import GatedFF, GatedLinearAttention, LatentAttention, RoutedExpertsFF, WindowAttention, _vec
from .registry import register_model

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
           torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}

SWISH_ALPHA = 1.702          # the experts' activation: g sigmoid(1.702 g) (u + 1)
RENORM_EPS = 1e-20           # joins the sum of the chosen experts' scores
GROUP_TOP = 2                # a group of experts scores by the sum of its two best choice scores


@dataclass
class GutivikLayerConfig:
    type: str
    mixer: dict
    mlp: Optional[dict]


@dataclass
class GutivikConfig:
    vocab: int
    width: int
    eps: float
    logit_scale: float
    logit_softcap: float
    max_positions: int
    layers: List[GutivikLayerConfig] = field(default_factory=list)

    @classmethod
    def from_dict(cls, cfg):
        try:
            layers = [GutivikLayerConfig(l["type"], dict(l["mixer"]), None if l.get("mlp") is None else dict(l["mlp"])) for l in cfg["layers"]]
            c = cls(int(cfg["vocab"]), int(cfg["width"]), float(cfg["norm"]["eps"]), float(cfg.get("logit_scale", 1.0)),
                    float(cfg.get("logit_softcap") or 0.0), int(cfg.get("max_positions", 1 << 24)), layers)   # (positions are fp32: exact to 2^24)
        except KeyError as e:
            raise ZLError(f"Gutivik config: missing key {e}")
        for i, l in enumerate(c.layers):
            if l.type not in MIXER_BUILDERS:
                raise ZLError(f"Gutivik config: layer {i}: unknown mixer type {l.type!r}")
            if l.mlp is not None and l.mlp.get("kind") not in FF_BUILDERS:
                raise ZLError(f"Gutivik config: layer {i}: unknown feed-forward kind {l.mlp.get('kind')!r}")
        return c


def _attention(name, width, m, eps, layers):
    rot, mask = m.get("rot") or {}, m.get("mask") or {}
    first = None                                       # the first layer that blends values lends its own to the later ones
    if m.get("v_mix"):
        first = next((l.mixer for l in layers if isinstance(l.mixer, WindowAttention) and l.mixer.v_mix), None)
    return WindowAttention(name, width, int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), float(m["scale"]),
                           int(mask.get("size", 0)), int(rot.get("dims", 0)), float(rot.get("base", 10000.0)), 1.0, eps, qk_norm=False,
                           rotate_values=False, talk=False, gate=False, rope_interleaved=True, bias=True, conv_taps=int(m.get("conv", 0)),
                           keep_first=int(mask.get("keep_first", 0)), sink=True, v_mix=bool(m.get("v_mix")), v_mix_source=first)


def _latent(name, width, m, eps, layers):
    rot, mask = m.get("rot") or {}, m.get("mask") or {}
    return LatentAttention(name, width, int(m["heads"]), int(m["dim"]), int(m["vdim"]), int(m["kv_rank"]), float(m["scale"]), eps, sink=False,
                           gate=False, rot_dim=int(m.get("rot_dim", 0)), rot_base=float(rot.get("base", 10000.0)), window=int(mask.get("size", 0)))


def _gla(name, width, m, eps, layers):
    return GatedLinearAttention(name, width, int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["tau"]), eps)


MIXER_BUILDERS = {"attention": _attention, "latent_attention": _latent, "gla": _gla}


def _dense(width, f):
    return GatedFF(width, int(f["ff"]), act="gelu_tanh")


def _experts(width, f):
    r = f["router"]
    g = r.get("groups") or {}
    return RoutedExpertsFF(width, int(f["expert"]["ff"]), int(r["experts"]), int(r["top"]), identity=0, groups=int(g.get("count", 1)),
                           keep=int(g.get("keep", g.get("count", 1))), correction=True, renorm=True, score="sigmoid", group_top=GROUP_TOP,
                           renorm_eps=RENORM_EPS, act="swish_clamp", act_alpha=SWISH_ALPHA, limit=float(f["expert"]["limit"]))


FF_BUILDERS = {"dense": _dense, "moe": _experts}


class GutivikLayer:
    def __init__(self, idx, cfg: GutivikConfig, lc: GutivikLayerConfig, layers):
        self.idx, self.name, self.width, self.eps = idx, f"l{idx}", cfg.width, cfg.eps
        self.mixer = MIXER_BUILDERS[lc.type](self.name + ".mix", cfg.width, lc.mixer, cfg.eps, layers)
        self.ff = FF_BUILDERS[lc.mlp["kind"]](cfg.width, lc.mlp) if lc.mlp is not None else None
        self.norm1 = self.norm2 = None                 # fp32 (width), stored around zero

    def load(self, get, dtype, device):
        p = self.name + "."
        self.norm1 = _vec(get, p + "norm1", self.width, device)
        self.mixer.load(get, p + "mix.", dtype, device)
        if self.ff is not None:
            self.norm2 = _vec(get, p + "norm2", self.width, device)
            self.ff.load(get, p + "mlp.", dtype, device)

    def init_random(self, gen, dtype, device):
        self.norm1 = 0.1 * torch.randn(self.width, generator=gen, device=device)
        self.mixer.init_random(gen, dtype, device)
        if self.ff is not None:
            self.norm2 = 0.1 * torch.randn(self.width, generator=gen, device=device)
            self.ff.init_random(gen, dtype, device)

    def forward(self, x, h, batch, dtype, next_norm):
        """h = N1(x) in the serving format; returns the next layer's N1 of the new x (None without next_norm)"""
        y = self.mixer.forward(h, batch)
        h = seqops.add_rms_norm(x, y, self.eps, self.norm2 if self.ff is not None else next_norm, dtype, around_zero=True)
        if self.ff is not None:
            h = seqops.add_rms_norm(x, self.ff.forward(h), self.eps, next_norm, dtype, around_zero=True)
        return h

    def weight_bytes(self):
        return self.mixer.weight_bytes() + (self.ff.weight_bytes() if self.ff is not None else 0)


@register_model("Gutivik")
class GutivikModel:
    ragged = True                    # the engine drives it with RaggedBatch steps and a CacheManager

    def __init__(self, cfg: GutivikConfig, dtype="bfloat16", device="cuda:0"):
        if dtype not in _DTYPES:
            raise ZLError(f"Gutivik serves in bfloat16 or float32, not {dtype}")
        self.cfg, self.dtype, self.device = cfg, _DTYPES[dtype], torch.device(device)
        self.layers = []
        for i, lc in enumerate(cfg.layers):
            self.layers.append(GutivikLayer(i, cfg, lc, self.layers))
        self.final_norm = self.embed = self.head = None
        self.page_size = 64

    @classmethod
    def from_config(cls, cfg: dict, dtype="bfloat16", device="cuda:0"):
        return cls(GutivikConfig.from_dict(cfg), dtype, device)

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
        self.final_norm = 0.1 * torch.randn(c.width, generator=gen, device=dev)
        for layer in self.layers:
            layer.init_random(gen, dt, dev)
        return self

    def bind_cache(self, cache):
        """register every layer's per-token planes and per-sequence states with the engine's cache manager"""
        if cache.page_size != self.page_size:
            raise ZLError("cache page size mismatch")
        for layer in self.layers:
            layer.mixer.bind(cache, self.dtype)
        return cache

    def _run(self, tokens, batch, keep=None):
        c = self.cfg
        x = seqops.embed(tokens, self.embed, None, 1.0, batch)
        if not self.layers:
            return x
        h = seqops.rms_norm(x, self.layers[0].norm1, c.eps, self.dtype, around_zero=True)
        for i, layer in enumerate(self.layers):
            nxt = self.layers[i + 1].norm1 if i + 1 < len(self.layers) else None
            h = layer.forward(x, h, batch, self.dtype, nxt)
            if keep is not None:
                keep.append(x.clone())
        return x

    def forward(self, tokens, batch, want_rows):
        """tokens: int32 device (n_tok) in the batch's flat order; want_rows: int32 device, flat token indices whose logits are wanted
        (None or empty: the step only advances caches and states).  Returns fp32 logits (len(want_rows), vocab) or None."""
        x = self._run(tokens, batch)
        if want_rows is None or want_rows.numel() == 0:
            return None
        hn = seqops.rms_norm(x, self.final_norm, self.cfg.eps, self.dtype, rows=want_rows, around_zero=True)
        logits = seqops.gemm_nt(hn, self.head)
        if self.cfg.logit_scale != 1.0 or self.cfg.logit_softcap > 0:
            seqops.scale_softcap(logits, self.cfg.logit_scale, self.cfg.logit_softcap)
        return logits

    def forward_layers(self, tokens, batch):
        """the residual stream after every layer (debugging and tests): list of fp32 (n_tok, width) copies"""
        out = []
        self._run(tokens, batch, keep=out)
        return out

    def weight_bytes(self):
        return sum(l.weight_bytes() for l in self.layers) + sum(t.numel() * t.element_size() for t in (self.embed, self.head))
