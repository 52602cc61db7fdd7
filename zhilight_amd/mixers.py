"""Sequence mixers and feed-forwards for ragged steps: each is a weight container + the kernel sequence of its forward, with every
constant a constructor argument, so that a model description picks and sizes them (tupitar.py and retotar.py do; another design can).

A mixer's forward takes h (n_tok, width) in the serving format and the step's RaggedBatch and returns fp32 (n_tok, width).  What it keeps
between steps it registers with the CacheManager in `bind`: per-token rows as a paged plane, per-sequence state as a slot state.
All per-sequence arithmetic that must not lose bits (norms, softmax, the recurrence, its state) is fp32 inside the kernels in both serving
formats; matrices are in the serving format, small vectors fp32.
"""
import math

import torch

from . import seqops
from ._lib import ZLError


def _mat(get, name, shape, dtype, device):
    t = get(name)
    if tuple(t.shape) != tuple(shape):
        raise ZLError(f"tensor {name}: shape {tuple(t.shape)}, expected {tuple(shape)}")
    return t.to(device=device, dtype=dtype).contiguous()


def _vec(get, name, n, device):
    t = get(name)
    if t.numel() != n:
        raise ZLError(f"tensor {name}: {t.numel()} values, expected {n}")
    return t.to(device=device, dtype=torch.float32).reshape(n).contiguous()


def _rand(gen, shape, std, dtype, device):
    return (torch.randn(shape, generator=gen, device=device, dtype=torch.float32) * std).to(dtype)


class SideRows:
    """Mixers and feed-forwards whose first step is ONE product over their input can carry more rows in it for their caller: a layer that
    needs another projection of the same input (a gate of the sub-layer's result, say) attaches its matrix after load / init_random and
    finds the fp32 outputs in `side` = (tensor, first column) after forward -- one launch and one pass over the input less."""
    side = None
    side_col0 = None
    _side_matrix = "w_in"

    def attach_side(self, w):
        m = getattr(self, self._side_matrix)
        if w.shape[1] != m.shape[1] or w.dtype != m.dtype:
            raise ZLError("side rows must have the input projection's width and format")
        self.side_col0 = m.shape[0]
        setattr(self, self._side_matrix, torch.cat([m, w], dim=0).contiguous())


class LatentAttention(SideRows):
    """Causal attention whose keys and values are up-projections of a cached, RMS-normed low-rank latent; optional learned per-head sink in
    the softmax denominator, per-head sigmoid output gate, sliding window (`window` > 0: position p sees p - window < j <= p), and a
    ROTATED part: with rot_dim > 0 every query head has rot_dim more coordinates behind its `dim` unrotated ones, the down-projection
    rot_dim more rows behind the latent -- one key part shared by all heads -- and both are turned by the position (neighbouring pairs
    (2i, 2i + 1), angle p * rot_base^(-2i / rot_dim)); score = (q_plain . k_plain + q_rot . k_rot) * scale.  The cached row is [latent |
    rotated key part]; the up-projections are widened on the host (identity columns in uk, zeros in uv), so the kernels see one latent of
    rank + rot_dim numbers and heads of dim + rot_dim.  rot_layout "half" pairs coordinate i with i + rot_dim / 2 instead of its
    neighbour; rot_scaling {factor, original, fast, slow} rescales the frequencies for contexts longer than `original` (scaled_frequencies).
    Tensors under `prefix`: q (heads*(dim+rot_dim), width), dkv (rank+rot_dim, width), dkv.norm (rank), uk (heads*dim, rank), uv (heads*vdim,
    rank), sink (heads), g (heads, width), o (width, heads*vdim).  q | dkv | g are fused into one product."""

    def __init__(self, name, width, heads, dim, vdim, rank, scale, eps, sink=True, gate=True, rot_dim=0, rot_base=10000.0, window=0,
                 rot_layout="pairs", rot_scaling=None):
        if rot_dim % 2 or rot_dim < 0 or window < 0 or rot_layout not in ("pairs", "half"):
            raise ZLError("latent attention: the rotated part is even, the window not negative, the layout pairs or half")
        self.rot_layout, self.rot_scaling, self.rot_gain = rot_layout, (dict(rot_scaling) if rot_scaling else None), 1.0
        self.name, self.width, self.heads, self.dim, self.vdim, self.rank = name, width, heads, dim, vdim, rank
        self.scale, self.eps, self.has_sink, self.has_gate = float(scale), float(eps), sink, gate
        self.rot, self.rot_base, self.window = int(rot_dim), float(rot_base), int(window)
        self.qdim, self.row = dim + self.rot, rank + self.rot      # a query head's size; a cached row's size
        self.cache = None
        self.prompt_kernel = True         # bf16 portions on the matrix-core kernel (False: everything on the latent-space kernel)
        self.decode_mfma = True           # bf16 single tokens: the split pass on the matrix cores (False: the fp32 VALU kernel)

    def _widen(self, uk, uv):
        """the up-projections over the cached row [latent | rotated key part]: a head's keys are [W_uk,h c | k_rot] (identity columns pass
        the shared part through, exactly: 1.0 times a number, summed with zeros), its values ignore the part (zero columns)"""
        H, d, v, r, t = self.heads, self.dim, self.vdim, self.rank, self.rot
        if t == 0:
            return uk.contiguous(), uv.contiguous()
        k2 = torch.zeros((H, d + t, r + t), dtype=uk.dtype, device=uk.device)
        k2[:, :d, :r] = uk.reshape(H, d, r)
        k2[:, d:, r:] = torch.eye(t, dtype=uk.dtype, device=uk.device)
        v2 = torch.zeros((H * v, r + t), dtype=uv.dtype, device=uv.device)
        v2[:, :r] = uv
        return k2.reshape(H * (d + t), r + t).contiguous(), v2.contiguous()

    def load(self, get, prefix, dtype, device):
        H, d, v, r, W = self.heads, self.dim, self.vdim, self.rank, self.width
        parts = [_mat(get, prefix + "q", (H * self.qdim, W), dtype, device), _mat(get, prefix + "dkv", (self.row, W), dtype, device)]
        if self.has_gate:
            parts.append(_mat(get, prefix + "g", (H, W), dtype, device))
        self.w_in = torch.cat(parts, dim=0).contiguous()
        self.dkv_norm = _vec(get, prefix + "dkv.norm", r, device)
        self.w_uk, self.w_uv = self._widen(_mat(get, prefix + "uk", (H * d, r), dtype, device), _mat(get, prefix + "uv", (H * v, r), dtype, device))
        self.sink = _vec(get, prefix + "sink", H, device) if self.has_sink else None
        self.w_o = _mat(get, prefix + "o", (W, H * v), dtype, device)
        self._tables(device)
        return self

    def _tables(self, device):
        self.freq = None
        if self.rot:
            self.freq, self.rot_gain = scaled_frequencies(self.rot, self.rot_base, self.rot_scaling, device)

    def init_random(self, gen, dtype, device):
        H, d, v, r, W = self.heads, self.dim, self.vdim, self.rank, self.width
        self.w_in = _rand(gen, (H * self.qdim + self.row + (H if self.has_gate else 0), W), W ** -0.5, dtype, device)
        self.dkv_norm = torch.ones(r, device=device)
        self.w_uk, self.w_uv = self._widen(_rand(gen, (H * d, r), r ** -0.5, dtype, device), _rand(gen, (H * v, r), r ** -0.5, dtype, device))
        self.sink = torch.zeros(H, device=device) if self.has_sink else None
        self.w_o = _rand(gen, (W, H * v), (H * v) ** -0.5, dtype, device)
        self._tables(device)
        return self

    def bind(self, cache, dtype):
        self.cache = cache.add_plane(self.name + ".latent", (self.row,), dtype)

    def weight_bytes(self):
        return sum(t.numel() * t.element_size() for t in (self.w_in, self.w_uk, self.w_uv, self.w_o))

    def forward(self, h, batch):
        H, d, r = self.heads, self.qdim, self.row                                # (sizes as the kernels see them: with the rotated part)
        proj = seqops.gemm_nt(h, self.w_in)                                       # fp32 [q | latent, rotated key part | gate]
        self.side = (proj, self.side_col0)
        seqops.latent_store(proj, H * d, self.dkv_norm, self.eps, self.rank, batch, self.cache, rot=self.rot, freq=self.freq,
                            interleaved=self.rot_layout == "pairs", q_col0=0, heads=H, qdim=d, rot_gain=self.rot_gain)
        gate = proj if self.has_gate else None
        prompt = batch.n_ctx > 0 and self.prompt_kernel and h.dtype == torch.bfloat16 and max(d, self.vdim) <= 256
        a = torch.empty((batch.n_tok, H * self.vdim), dtype=h.dtype, device=h.device)
        if prompt:
            # portions: keys and values of their contexts (as far back as the window reaches) up-projected once (K = C W_uk^T, V^T = W_uv C^T,
            # gathered from the pages), then the matrix-core kernel; single tokens stay on the latent-space kernel below
            _, _, ctx_rows, n_ctx = batch.context(self.window)
            flat = self.cache.view(-1, r)
            k = torch.empty((n_ctx, H * d), dtype=h.dtype, device=h.device)
            vt = torch.empty((H * self.vdim, n_ctx), dtype=h.dtype, device=h.device)
            seqops.gemm_nt_gather(flat, ctx_rows, self.w_uk, None, n_ctx, H * d, k)
            seqops.gemm_nt_gather(self.w_uv, None, flat, ctx_rows, H * self.vdim, n_ctx, vt)
            seqops.latent_attention_prompt(proj, 0, gate, H * d + r, k, vt, self.sink, batch, self.scale, H, d, self.vdim, a, window=self.window)
        if not prompt or batch.n_single:
            seqops.latent_attention(proj, 0, gate, H * d + r, self.w_uk, self.w_uv, self.sink, self.cache, batch, self.scale, H, d, self.vdim,
                                    out=a, single_only=prompt, mfma=self.decode_mfma, window=self.window)
        return seqops.gemm_nt(a, self.w_o)


class Mamba2Mixer:
    """Selective state-space mixer (scalar decay per head, state n_state x vdim per head, B / C shared by the heads of a group), with the
    causal short convolution over x | B | C, the skip term, and the gated grouped RMS norm before the output projection.
    Tensors under `prefix`: in (2*inner + 2*groups*n_state + heads, width) laid out [z | x | B | C | dt], conv (channels, taps), conv.b,
    dt_bias, A_log, D (heads each), norm (inner), o (width, inner)."""

    def __init__(self, name, width, heads, vdim, n_state, groups, taps, norm_groups, eps):
        if heads % groups or (heads * vdim) % norm_groups:
            raise ZLError("mamba2: heads must divide by groups, heads * vdim by norm_groups")
        self.name, self.width, self.heads, self.vdim, self.n_state, self.groups = name, width, heads, vdim, n_state, groups
        self.taps, self.norm_groups, self.eps = taps, norm_groups, float(eps)
        self.inner = heads * vdim
        self.channels = self.inner + 2 * groups * n_state
        self.scan_segment = None          # tokens per segment of a long portion (None: seqops.SCAN_SEGMENT; 0: never in segments)

    def load(self, get, prefix, dtype, device):
        W = self.width
        self.w_in = _mat(get, prefix + "in", (self.inner + self.channels + self.heads, W), dtype, device)
        self.conv_w = _mat(get, prefix + "conv", (self.channels, self.taps), torch.float32, device)
        self.conv_b = _vec(get, prefix + "conv.b", self.channels, device)
        self.dt_bias = _vec(get, prefix + "dt_bias", self.heads, device)
        self.a_log = _vec(get, prefix + "A_log", self.heads, device)
        self.d = _vec(get, prefix + "D", self.heads, device)
        self.norm_w = _vec(get, prefix + "norm", self.inner, device)
        self.w_o = _mat(get, prefix + "o", (W, self.inner), dtype, device)
        return self

    def init_random(self, gen, dtype, device):
        W = self.width
        self.w_in = _rand(gen, (self.inner + self.channels + self.heads, W), W ** -0.5, dtype, device)
        self.conv_w = _rand(gen, (self.channels, self.taps), 0.5, torch.float32, device)
        self.conv_b = torch.zeros(self.channels, device=device)
        self.dt_bias = torch.zeros(self.heads, device=device)
        self.a_log = torch.zeros(self.heads, device=device)
        self.d = torch.ones(self.heads, device=device)
        self.norm_w = torch.ones(self.inner, device=device)
        self.w_o = _rand(gen, (W, self.inner), self.inner ** -0.5, dtype, device)
        return self

    def bind(self, cache, dtype):
        self.tail = cache.add_state(self.name + ".conv", (self.taps - 1, self.channels)) if self.taps > 1 else None
        self.state = cache.add_state(self.name + ".ssm", (self.heads, self.n_state, self.vdim))

    def weight_bytes(self):
        return sum(t.numel() * t.element_size() for t in (self.w_in, self.w_o))

    def forward(self, h, batch):
        proj = seqops.gemm_nt(h, self.w_in)                                       # fp32 [z | x | B | C | dt]
        xbc = seqops.conv_silu(proj, self.inner, self.conv_w, self.conv_b, self.tail, batch)
        y = seqops.ssm_scan(xbc, proj, self.inner + self.channels, self.dt_bias, self.a_log, self.d, self.state, self.heads, self.vdim,
                            self.n_state, self.groups, batch, seg_len=self.scan_segment)
        g = seqops.gated_group_norm(y, proj, 0, self.norm_w, self.eps, self.norm_groups, h.dtype)
        return seqops.gemm_nt(g, self.w_o)


class PolyNormFF:
    """Dense feed-forward down(act(up h)) with the PolyNorm activation: a N(z) + b N(z^2) + c N(z^3) + e, N = division by the row's root
    mean square.  Tensors: up (ff, width), down (width, ff), act (4: a, b, c, e)."""

    def __init__(self, width, ff, eps):
        self.width, self.ff, self.eps = width, ff, float(eps)

    def load(self, get, prefix, dtype, device):
        self.w_up = _mat(get, prefix + "up", (self.ff, self.width), dtype, device)
        self.w_down = _mat(get, prefix + "down", (self.width, self.ff), dtype, device)
        self.coef = [float(v) for v in get(prefix + "act").to(torch.float32).reshape(4)]
        return self

    def init_random(self, gen, dtype, device):
        self.w_up = _rand(gen, (self.ff, self.width), self.width ** -0.5, dtype, device)
        self.w_down = _rand(gen, (self.width, self.ff), self.ff ** -0.5, dtype, device)
        self.coef = [1.0, 0.5, 0.25, 0.0]
        return self

    def weight_bytes(self):
        return sum(t.numel() * t.element_size() for t in (self.w_up, self.w_down))

    def forward(self, h):
        z = seqops.gemm_nt(h, self.w_up)
        return seqops.gemm_nt(seqops.polynorm(z, self.coef, self.eps, h.dtype), self.w_down)


def rotary_frequencies(n_rot, base, divide=1.0, device="cpu"):
    """base^(-2i / n_rot) / divide for the n_rot / 2 pairs, worked out in float64 and rounded once to fp32"""
    i = torch.arange(n_rot // 2, dtype=torch.float64)
    return (torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / n_rot) / float(divide)).to(torch.float32).to(device)


def scaled_frequencies(n_rot, base, scaling=None, device="cpu"):
    """(frequencies fp32 (n_rot / 2), gain) of a rotation whose frequencies are rescaled for contexts longer than the `original` one
    (scaling = {factor, original, fast, slow}; None: the plain frequencies and gain 1).  A pair that turns more than `fast` times over
    `original` positions keeps its frequency f_i = base^(-2i / n_rot), one that turns less than `slow` times gets f_i / factor, and
    between the two pair indices lo = floor(index(fast)), hi = ceil(index(slow)) -- index(t) = n_rot ln(original / (2 pi t)) / (2 ln base),
    clamped to the head -- the two are blended linearly in i.  cos and sin are multiplied by the gain 0.1 ln(factor) + 1.  Worked out in
    float64, rounded once."""
    if not scaling:
        return rotary_frequencies(n_rot, base, 1.0, device), 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def index(turns):
        return n_rot * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(index(float(scaling["fast"]))), 0)
    hi = min(math.ceil(index(float(scaling["slow"]))), n_rot - 1)
    i = torch.arange(n_rot // 2, dtype=torch.float64)
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / n_rot)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return (f / factor * ramp + f * (1.0 - ramp)).to(torch.float32).to(device), 0.1 * math.log(factor) + 1.0


def distance_bias_table(rel, far, longest, device):
    """The bias of every distance 0 .. L - 1 from a table `rel` (rows, heads) of bucketed distances: the first rows // 2 distances have a
    row each, larger ones share the other rows on a logarithmic scale that reaches the last row at the distance `far`
    (row = half + floor(ln(n / half) / ln(far / half) * (rows - half)), at most rows - 1).  Returns fp32 (heads, L), L = far + 1 -- every
    distance from `far` on has the last row, the kernels clamp -- or `longest` when no query ever looks that far."""
    rows, heads = rel.shape
    half = rows // 2
    if half < 1 or far <= half:
        raise ZLError("distance bias: the table needs two rows or more and a largest distance beyond its exact half")
    L = int(far) + 1 if longest <= 0 else min(int(far) + 1, int(longest))
    n = torch.arange(L, dtype=torch.float64)
    big = half + torch.floor(torch.log(torch.clamp(n, min=1.0) / half) / math.log(far / half) * (rows - half)).to(torch.int64)
    row = torch.where(n < half, n.to(torch.int64), torch.clamp(big, max=rows - 1))
    return rel.to(torch.float32)[row.to(rel.device)].t().contiguous().to(device)


class WindowAttention(SideRows):
    """Softmax attention with grouped key / value heads over a paged cache: rotary positions on the first `rot_dims` coordinates of every
    query and key head (pairs i, i + rot_dims / 2; every frequency divided by `rot_scaling`), queries and keys divided by their root mean
    square afterwards (qk_norm), a sliding window of `window` positions (0: none), optionally
      * values turned by their own position over all vdim coordinates before they are cached and the heads' sums turned back by the query's
        position (rotate_values; frequencies from the same base, never scaled),
      * the heads' softmax weights mixed by a (heads, heads) matrix after the softmax (tensor `talk`),
      * a sigmoid gate per output coordinate computed from the mixer's input (tensor `g`),
      * keys and values borrowed from another layer's cache (kv_source: that layer's WindowAttention; then no k / v tensors),
      * rotated pairs that are neighbours (2i, 2i + 1) instead of (i, i + rot_dims / 2) (rope_interleaved),
      * biases on q, k, v (bias; tensors q.b, k.b, v.b) and a short causal convolution over time on every channel of q, k, v right after the
        projection (conv_taps > 0; tensors q.conv, k.conv, v.conv (channels, taps); the last taps - 1 projected rows are slot state),
      * the sequence's first keep_first keys visible behind the window, at their true positions,
      * a learned sink per head in the softmax denominator (tensor `sink`; no key, no value, not scaled),
      * values blended with ANOTHER such layer's values of the same token before they are cached, v <- (1 - lam) v + lam v_other with lam
        the scalar tensor `vmix` (v_mix_source: that layer's WindowAttention, which ran earlier in the same step),
      * a weight on the query / key norm shared by the heads (norm_weight; tensors q.norm, k.norm (dim)), a factor on the scores per head
        (head_scale; tensor `temp`), scores capped by softcap * tanh(. / softcap), a learned bias by the distance between query and key
        added after the cap (rel_far > 0; tensor `rel` (rows, heads), see distance_bias_table),
      * queries that only see the keys of their own chunk of `chunk` positions, chunks counted from position 0 of the sequence,
      * weights that are no softmax: weights="sigmoid" gives every visible key sigmoid(score + offset_h) (tensor `pb` (heads)), not
        normalised over the keys.
    Tensors under `prefix`: q (heads*dim, width), k (kv_heads*dim, width), v (kv_heads*vdim, width), talk (heads, heads), g (heads*vdim, width),
    o (width, heads*vdim).  q | k | v | g are one product."""

    def __init__(self, name, width, heads, kv_heads, dim, vdim, scale, window, rot_dims, rot_base, rot_scaling, eps, qk_norm=True,
                 rotate_values=True, talk=True, gate=True, kv_source=None, rope_interleaved=False, bias=False, conv_taps=0, keep_first=0,
                 sink=False, v_mix=False, v_mix_source=None, norm_weight=False, head_scale=False, softcap=0.0, rel_far=0, chunk=0,
                 weights="softmax"):
        if weights not in ("softmax", "sigmoid") or (weights == "sigmoid" and (sink or talk)) or (chunk and keep_first) or chunk < 0:
            raise ZLError("attention: sigmoid weights have no sink and no mixing; chunks keep no first keys")
        if norm_weight and not qk_norm:
            raise ZLError("attention: a norm weight needs the query / key norm")
        self.norm_weight, self.has_head_scale, self.softcap, self.rel_far, self.chunk = bool(norm_weight), bool(head_scale), float(softcap or 0.0), \
            int(rel_far or 0), int(chunk or 0)
        self.sigmoid = weights == "sigmoid"
        self.q_norm_w = self.k_norm_w = self.temp = self.rel = self.offset = self.form = None
        if heads % kv_heads or rot_dims % 2 or rot_dims > dim or (rotate_values and vdim % 2):
            raise ZLError("attention: heads must divide by kv_heads, rotated sizes must be even and fit the head")
        if kv_source is not None and (kv_source.kv_heads, kv_source.dim, kv_source.vdim) != (kv_heads, dim, vdim):
            raise ZLError("attention: a borrowed cache must have this layer's key / value shape")
        if kv_source is not None and (bias or conv_taps or v_mix):
            raise ZLError("attention: a layer that borrows keys and values has no key / value projections to bias, convolve or blend")
        if v_mix_source is not None and (v_mix_source.kv_heads * v_mix_source.vdim != kv_heads * vdim):
            raise ZLError("attention: blended values must have this layer's value shape")
        self.interleaved, self.has_bias, self.taps, self.keep_first = bool(rope_interleaved), bool(bias), int(conv_taps), int(keep_first)
        self.has_sink, self.v_mix, self.v_mix_source = bool(sink), bool(v_mix), v_mix_source
        self.sink = self.in_bias = self.conv_w = self.tail = self.last_values = None
        self.vmix_lambda = 0.0
        self.name, self.width, self.heads, self.kv_heads, self.dim, self.vdim = name, width, heads, kv_heads, dim, vdim
        self.scale, self.window, self.rot_dims, self.rot_base, self.rot_scaling = float(scale), int(window), rot_dims, float(rot_base), float(rot_scaling)
        self.eps, self.qk_norm, self.rotate_values, self.has_talk, self.has_gate = float(eps), qk_norm, rotate_values, talk, gate
        self.kv_source = kv_source
        self.k_cache = self.v_cache = None
        self.prompt_kernel = True         # bf16 portions on the matrix-core kernel (False: everything on the plain kernel)
        self.n_splits = None              # workgroups per (token, head) of the plain kernel (None: enough to fill the chip)

    def _cols(self):
        H, G, d, v = self.heads, self.kv_heads, self.dim, self.vdim
        own = self.kv_source is None
        kq, vq = H * d, H * d + (G * d if own else 0)
        g0 = vq + (G * v if own else 0)
        return kq, vq, g0, g0 + (H * v if self.has_gate else 0)

    def _tables(self, device):
        self.qk_freq = rotary_frequencies(self.rot_dims, self.rot_base, self.rot_scaling, device) if self.rot_dims else None
        self.v_freq = rotary_frequencies(self.vdim, self.rot_base, 1.0, device) if self.rotate_values else None
        self.form = None
        if self.has_head_scale or self.softcap > 0 or self.rel is not None or self.chunk or self.sigmoid:
            self.form = seqops.score_form(self.heads, self.temp, self.softcap, self.rel, self.offset, self.chunk, self.sigmoid)

    def _load_form(self, get, prefix, device):
        d, H = self.dim, self.heads
        if self.norm_weight:
            self.q_norm_w, self.k_norm_w = _vec(get, prefix + "q.norm", d, device), _vec(get, prefix + "k.norm", d, device)
        if self.has_head_scale:
            self.temp = _vec(get, prefix + "temp", H, device)
        if self.rel_far:
            rel = get(prefix + "rel")
            if rel.dim() != 2 or rel.shape[1] != H:
                raise ZLError(f"tensor {prefix}rel: shape {tuple(rel.shape)}, expected (rows, {H})")
            longest = min(x for x in (self.chunk, self.window) if x > 0) if (self.chunk or self.window) else 0
            self.rel = distance_bias_table(rel, self.rel_far, longest, device)
        if self.sigmoid:
            self.offset = _vec(get, prefix + "pb", H, device)

    def load(self, get, prefix, dtype, device):
        H, G, d, v, W = self.heads, self.kv_heads, self.dim, self.vdim, self.width
        parts = [_mat(get, prefix + "q", (H * d, W), dtype, device)]
        if self.kv_source is None:
            parts += [_mat(get, prefix + "k", (G * d, W), dtype, device), _mat(get, prefix + "v", (G * v, W), dtype, device)]
        if self.has_gate:
            parts.append(_mat(get, prefix + "g", (H * v, W), dtype, device))
        self.w_in = torch.cat(parts, dim=0).contiguous()
        self.talk = _mat(get, prefix + "talk", (H, H), torch.float32, device) if self.has_talk else None
        self.w_o = _mat(get, prefix + "o", (W, H * v), dtype, device)
        names = ("q", "k", "v") if self.kv_source is None else ("q",)
        sizes = {"q": H * d, "k": G * d, "v": G * v}
        if self.has_bias:
            self.in_bias = torch.cat([_vec(get, prefix + n + ".b", sizes[n], device) for n in names]).contiguous()
        if self.taps:
            self.conv_w = torch.cat([_mat(get, prefix + n + ".conv", (sizes[n], self.taps), torch.float32, device) for n in names]).contiguous()
        elif self.has_bias:
            self.conv_w = torch.ones((sum(sizes[n] for n in names), 1), device=device)       # (one tap of weight 1: the bias alone)
        self.sink = _vec(get, prefix + "sink", H, device) if self.has_sink else None
        if self.v_mix:
            self.vmix_lambda = float(_vec(get, prefix + "vmix", 1, device)[0])
        self._load_form(get, prefix, device)
        self._tables(device)
        return self

    def init_random(self, gen, dtype, device):
        H, v, W = self.heads, self.vdim, self.width
        self.w_in = _rand(gen, (self._cols()[3], W), W ** -0.5, dtype, device)
        self.talk = (torch.eye(H, device=device) + 0.1 * torch.randn(H, H, generator=gen, device=device)) if self.has_talk else None
        self.w_o = _rand(gen, (W, H * v), (H * v) ** -0.5, dtype, device)
        C = self._cols()[2]
        if self.has_bias:
            self.in_bias = 0.1 * torch.randn(C, generator=gen, device=device)
        if self.taps:
            self.conv_w = torch.randn(C, self.taps, generator=gen, device=device) * self.taps ** -0.5
        elif self.has_bias:
            self.conv_w = torch.ones((C, 1), device=device)
        self.sink = torch.zeros(H, device=device) if self.has_sink else None
        self.vmix_lambda = 0.5 if self.v_mix else 0.0
        d = self.dim
        if self.norm_weight:
            self.q_norm_w, self.k_norm_w = 1.0 + 0.1 * torch.randn(d, generator=gen, device=device), 1.0 + 0.1 * torch.randn(d, generator=gen, device=device)
        if self.has_head_scale:
            self.temp = 1.0 + 0.1 * torch.randn(H, generator=gen, device=device)
        if self.rel_far:
            longest = min(x for x in (self.chunk, self.window) if x > 0) if (self.chunk or self.window) else 0
            self.rel = distance_bias_table(0.5 * torch.randn(32, H, generator=gen, device=device), max(self.rel_far, 17), longest, device)
        if self.sigmoid:
            self.offset = -2.0 + 0.1 * torch.randn(H, generator=gen, device=device)
        self._tables(device)
        return self

    def bind(self, cache, dtype):
        if self.kv_source is not None:                      # (the lender is an earlier layer: it is bound already)
            self.k_cache, self.v_cache = self.kv_source.k_cache, self.kv_source.v_cache
            return
        self.k_cache = cache.add_plane(self.name + ".k", (self.kv_heads * self.dim,), dtype)
        self.v_cache = cache.add_plane(self.name + ".v", (self.kv_heads * self.vdim,), dtype)      # (the kernels keep a page transposed)
        if self.taps > 1:
            self.tail = cache.add_state(self.name + ".conv", (self.taps - 1, self._cols()[2]))

    def weight_bytes(self):
        return sum(t.numel() * t.element_size() for t in (self.w_in, self.w_o))

    def forward(self, h, batch):
        H, G, d, v = self.heads, self.kv_heads, self.dim, self.vdim
        k0, v0, g0, _ = self._cols()
        own = self.kv_source is None
        proj = seqops.gemm_nt(h, self.w_in)                                       # fp32 [q | k | v | gate]
        self.side = (proj, self.side_col0)
        # biases and the short convolution give a second buffer [q | k | v] (the gate stays in proj); otherwise q is rotated inside proj
        qkv = seqops.short_conv(proj, 0, self.conv_w, self.in_bias, self.tail, batch) if self.conv_w is not None else proj
        blend = None
        if self.v_mix and self.v_mix_source is not None:
            src, col = self.v_mix_source.last_values
            blend = (src, col, self.vmix_lambda)
        self.last_values = (qkv, v0) if self.v_mix else None                      # (this step's values before blending, for a later layer)
        seqops.rope_norm_store(qkv, 0, k0, v0, H, G, d, v, self.qk_freq, self.rot_dims, self.v_freq, self.eps, self.qk_norm, batch,
                               self.k_cache if own else None, self.v_cache if own else None, interleaved=self.interleaved, vmix=blend,
                               q_norm_w=self.q_norm_w, k_norm_w=self.k_norm_w)
        acc, ml, n_splits = seqops.window_attention(qkv, 0, self.k_cache, self.v_cache, batch, self.scale, self.window, H, G, d, v,
                                                    all_kv=self.has_talk, mfma=self.prompt_kernel, n_splits=self.n_splits,
                                                    keep_first=self.keep_first, form=self.form)
        a = seqops.head_mix_gate(acc, ml, n_splits, self.talk, self.v_freq, proj if self.has_gate else None, g0, batch, H, G, v, h.dtype,
                                 sink=self.sink, plain_sum=self.sigmoid)
        return seqops.gemm_nt(a, self.w_o)


class DecayLinearAttention:
    """Linear attention with a fixed decay per head: q, k, v = act(projections); S_t = decay_h S_{t-1} + k_t v_t^T, o_t = S_t^T q_t per head,
    the state fp32 per sequence; then the RMS norm over all heads together with a weight, the sigmoid gate, the output projection.
    Tensors under `prefix`: q, k (heads*dim, width), v, g (heads*vdim, width), norm (heads*vdim), o (width, heads*vdim)."""

    def __init__(self, name, width, heads, dim, vdim, decay, eps, act="silu", norm_groups=1):
        if len(decay) != heads:
            raise ZLError("linear attention: one decay per head")
        self.name, self.width, self.heads, self.dim, self.vdim = name, width, heads, dim, vdim
        self.decay_values, self.eps, self.act, self.norm_groups = [float(x) for x in decay], float(eps), act, norm_groups
        self.scan_segment = None

    def load(self, get, prefix, dtype, device):
        H, d, v, W = self.heads, self.dim, self.vdim, self.width
        self.w_in = torch.cat([_mat(get, prefix + "q", (H * d, W), dtype, device), _mat(get, prefix + "k", (H * d, W), dtype, device),
                               _mat(get, prefix + "v", (H * v, W), dtype, device), _mat(get, prefix + "g", (H * v, W), dtype, device)], dim=0).contiguous()
        self.norm_w = _vec(get, prefix + "norm", H * v, device)
        self.w_o = _mat(get, prefix + "o", (W, H * v), dtype, device)
        self.decay = torch.tensor(self.decay_values, dtype=torch.float64).to(torch.float32).to(device)
        return self

    def init_random(self, gen, dtype, device):
        H, d, v, W = self.heads, self.dim, self.vdim, self.width
        self.w_in = _rand(gen, (2 * H * d + 2 * H * v, W), W ** -0.5, dtype, device)
        self.norm_w = torch.ones(H * v, device=device)
        self.w_o = _rand(gen, (W, H * v), (H * v) ** -0.5, dtype, device)
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=device)
        return self

    def bind(self, cache, dtype):
        self.state = cache.add_state(self.name + ".S", (self.heads, self.dim, self.vdim))

    def weight_bytes(self):
        return sum(t.numel() * t.element_size() for t in (self.w_in, self.w_o))

    def forward(self, h, batch):
        H, d, v = self.heads, self.dim, self.vdim
        proj = seqops.gemm_nt(h, self.w_in)                                       # fp32 [q | k | v | gate]
        y = seqops.decay_scan(proj, 0, H * d, 2 * H * d, self.act == "silu", self.decay, None, None, False, self.state, H, d, v, batch,
                              seg_len=self.scan_segment)
        a = seqops.linear_attn_finish(y, False, 1.0, None, 0.0, H, v, self.norm_groups, self.norm_w, self.eps, proj, 2 * H * d + H * v, h.dtype)
        return seqops.gemm_nt(a, self.w_o)


class GatedLinearAttention:
    """Linear attention with a learned decay per KEY CHANNEL and token: q = W_q h * dim^-1/2, k = W_k h, v = W_v h;
        alpha = sigmoid(W_a2 (W_a1 h) + b)^(1 / tau)   (heads x dim, from a low-rank pair of projections)
        S_t = diag(alpha_t) S_{t-1} + k_t v_t^T,  o_t = S_t^T q_t   per head, S fp32 per sequence, from zero
    then each head's o divided by its root mean square over vdim, times a weight shared by the heads, times silu(W_g h), and the output
    projection.  The logarithm of the decay, the decay and the recurrence are fp32; the scale dim^-1/2 is applied to o (the recurrence is
    linear in q).  Tensors under `prefix`: q, k (heads*dim, width), v, g (heads*vdim, width), a1 (low, width), a2 (heads*dim, low), a2.b
    (heads*dim), norm (vdim), o (width, heads*vdim).  q | k | v | g | a1 are one product."""

    def __init__(self, name, width, heads, dim, vdim, tau, eps):
        if tau <= 0:
            raise ZLError("gated linear attention: tau > 0")
        self.name, self.width, self.heads, self.dim, self.vdim = name, width, heads, dim, vdim
        self.tau, self.eps = float(tau), float(eps)
        self.scan_segment = None

    def load(self, get, prefix, dtype, device):
        H, d, v, W = self.heads, self.dim, self.vdim, self.width
        a1 = get(prefix + "a1")
        self.low = int(a1.shape[0])
        self.w_in = torch.cat([_mat(get, prefix + "q", (H * d, W), dtype, device), _mat(get, prefix + "k", (H * d, W), dtype, device),
                               _mat(get, prefix + "v", (H * v, W), dtype, device), _mat(get, prefix + "g", (H * v, W), dtype, device),
                               _mat(get, prefix + "a1", (self.low, W), dtype, device)], dim=0).contiguous()
        self.w_a2 = _mat(get, prefix + "a2", (H * d, self.low), dtype, device)
        self.a2_bias = _vec(get, prefix + "a2.b", H * d, device)
        self.norm_w = _vec(get, prefix + "norm", v, device).repeat(H).contiguous()
        self.w_o = _mat(get, prefix + "o", (W, H * v), dtype, device)
        return self

    def init_random(self, gen, dtype, device, low=16):
        H, d, v, W = self.heads, self.dim, self.vdim, self.width
        self.low = low
        self.w_in = _rand(gen, (2 * H * d + 2 * H * v + low, W), W ** -0.5, dtype, device)
        self.w_a2 = _rand(gen, (H * d, low), low ** -0.5, dtype, device)
        self.a2_bias = torch.full((H * d,), 2.0, device=device)
        self.norm_w = torch.ones(H * v, device=device)
        self.w_o = _rand(gen, (W, H * v), (H * v) ** -0.5, dtype, device)
        return self

    def bind(self, cache, dtype):
        self.state = cache.add_state(self.name + ".S", (self.heads, self.dim, self.vdim))

    def weight_bytes(self):
        return sum(t.numel() * t.element_size() for t in (self.w_in, self.w_a2, self.w_o))

    def forward(self, h, batch):
        H, d, v = self.heads, self.dim, self.vdim
        proj = seqops.gemm_nt(h, self.w_in)                                       # fp32 [q | k | v | gate | low-rank decay input]
        g0 = 2 * H * d + H * v
        alpha = seqops.lowrank_decay(proj, g0 + H * v, self.w_a2, self.a2_bias, self.tau)
        y = seqops.decay_scan(proj, 0, H * d, 2 * H * d, False, None, None, None, False, self.state, H, d, v, batch, seg_len=self.scan_segment,
                              decay_v=alpha)
        a = seqops.linear_attn_finish(y, False, d ** -0.5, None, 0.0, H, v, H, self.norm_w, self.eps, proj, g0, h.dtype, gate_act="silu")
        return seqops.gemm_nt(a, self.w_o)


class PlainFF(SideRows):
    """Dense feed-forward down(act(up h)) without biases and without a gate; act: "relu2" (the square of relu), "gelu_tanh" or "silu".
    Tensors under `prefix`: up (ff, width), down (width, ff)."""
    _side_matrix = "w_up"

    def __init__(self, width, ff, act="relu2"):
        if act not in seqops.UNARY_ACTS:
            raise ZLError(f"feed-forward: unknown activation {act!r}")
        self.width, self.ff, self.act = width, ff, act

    def load(self, get, prefix, dtype, device):
        self.w_up = _mat(get, prefix + "up", (self.ff, self.width), dtype, device)
        self.w_down = _mat(get, prefix + "down", (self.width, self.ff), dtype, device)
        return self

    def init_random(self, gen, dtype, device):
        self.w_up = _rand(gen, (self.ff, self.width), self.width ** -0.5, dtype, device)
        self.w_down = _rand(gen, (self.width, self.ff), self.ff ** -0.5, dtype, device)
        return self

    def weight_bytes(self):
        return sum(t.numel() * t.element_size() for t in (self.w_up, self.w_down))

    def forward(self, h):
        z = seqops.gemm_nt(h, self.w_up)                                          # fp32 [up | side rows]
        self.side = (z, self.side_col0)
        return seqops.gemm_nt(seqops.unary_act(z, h.dtype, kind=self.act, cols=self.ff), self.w_down)


class GatedFF:
    """Dense gated feed-forward down(act(gate h) * (up h)) without biases; act: "gelu_tanh" (the tanh form) or "silu".
    Tensors under `prefix`: gate, up (ff, width), down (width, ff).  gate | up are one product."""

    def __init__(self, width, ff, act="gelu_tanh"):
        if act not in ("gelu_tanh", "silu"):
            raise ZLError(f"feed-forward: unknown activation {act!r}")
        self.width, self.ff, self.act = width, ff, act

    def load(self, get, prefix, dtype, device):
        self.w_gu = torch.cat([_mat(get, prefix + "gate", (self.ff, self.width), dtype, device),
                               _mat(get, prefix + "up", (self.ff, self.width), dtype, device)], dim=0).contiguous()
        self.w_down = _mat(get, prefix + "down", (self.width, self.ff), dtype, device)
        return self

    def init_random(self, gen, dtype, device):
        self.w_gu = _rand(gen, (2 * self.ff, self.width), self.width ** -0.5, dtype, device)
        self.w_down = _rand(gen, (self.width, self.ff), self.ff ** -0.5, dtype, device)
        return self

    def weight_bytes(self):
        return sum(t.numel() * t.element_size() for t in (self.w_gu, self.w_down))

    def forward(self, h):
        return seqops.gemm_nt(seqops.act_mul(seqops.gemm_nt(h, self.w_gu), h.dtype, kind=self.act), self.w_down)


class MLSTMMixer:
    """Matrix memory with exponential gates (mLSTM): per head a log input gate i and a log forget gate f = log sigmoid(.), both capped by
    cap * tanh(. / cap), a running maximum m (from 0) that keeps the exponentials in range:
        m_t = max(f + m_{t-1}, i);  S_t = e^{f + m_{t-1} - m_t} S_{t-1} + e^{i - m_t} k v^T;  n_t the same with k alone
        o = S_t^T q / (max(|n_t . q|, e^{-m_t}) + 1e-6),  q scaled by dim^-1/2
    then each head divided by its root mean square, a weight over all heads, the sigmoid gate, the output projection.  S, n, m are fp32 per
    sequence; n rides in the scan as one more value column that is 1 for every token.
    Tensors under `prefix`: q, k (heads*dim, width), v, g (heads*vdim, width), i, f (heads, width), i.b, f.b (heads), norm (heads*vdim),
    o (width, heads*vdim)."""

    def __init__(self, name, width, heads, dim, vdim, gate_cap, eps, den_eps=1e-6):
        self.name, self.width, self.heads, self.dim, self.vdim = name, width, heads, dim, vdim
        self.cap, self.eps, self.den_eps = float(gate_cap), float(eps), float(den_eps)
        self.scan_segment = None

    def load(self, get, prefix, dtype, device):
        H, d, v, W = self.heads, self.dim, self.vdim, self.width
        self.w_in = torch.cat([_mat(get, prefix + "q", (H * d, W), dtype, device), _mat(get, prefix + "k", (H * d, W), dtype, device),
                               _mat(get, prefix + "v", (H * v, W), dtype, device), _mat(get, prefix + "g", (H * v, W), dtype, device),
                               _mat(get, prefix + "i", (H, W), dtype, device), _mat(get, prefix + "f", (H, W), dtype, device)], dim=0).contiguous()
        self.i_bias, self.f_bias = _vec(get, prefix + "i.b", H, device), _vec(get, prefix + "f.b", H, device)
        self.norm_w = _vec(get, prefix + "norm", H * v, device)
        self.w_o = _mat(get, prefix + "o", (W, H * v), dtype, device)
        return self

    def init_random(self, gen, dtype, device):
        H, d, v, W = self.heads, self.dim, self.vdim, self.width
        self.w_in = _rand(gen, (2 * H * d + 2 * H * v + 2 * H, W), W ** -0.5, dtype, device)
        self.i_bias = torch.zeros(H, device=device)
        self.f_bias = torch.full((H,), 3.0, device=device)
        self.norm_w = torch.ones(H * v, device=device)
        self.w_o = _rand(gen, (W, H * v), (H * v) ** -0.5, dtype, device)
        return self

    def bind(self, cache, dtype):
        self.state = cache.add_state(self.name + ".S", (self.heads, self.dim, self.vdim + 1))
        self.m_state = cache.add_state(self.name + ".m", (self.heads,))

    def weight_bytes(self):
        return sum(t.numel() * t.element_size() for t in (self.w_in, self.w_o))

    def forward(self, h, batch):
        H, d, v = self.heads, self.dim, self.vdim
        proj = seqops.gemm_nt(h, self.w_in)                                       # fp32 [q | k | v | gate | i | f]
        g0 = 2 * H * d + H * v
        decay, gain, m = seqops.exp_gates(proj, g0 + H * v, g0 + H * v + H, self.i_bias, self.f_bias, self.cap, self.m_state, H, batch)
        y = seqops.decay_scan(proj, 0, H * d, 2 * H * d, False, None, decay, gain, True, self.state, H, d, v, batch, seg_len=self.scan_segment)
        a = seqops.linear_attn_finish(y, True, d ** -0.5, m, self.den_eps, H, v, H, self.norm_w, self.eps, proj, g0, h.dtype)
        return seqops.gemm_nt(a, self.w_o)


class RoutedExpertsFF(SideRows):
    """Mixture of gated feed-forward experts, down(silu(gate h) * (up h)), without biases.  The router gives one logit per expert and per
    IDENTITY output (the last `identity` of its outputs: their "expert" returns h itself); probabilities = softmax over all outputs; an
    output is chosen by probability + `correction`, within the `keep` best of `groups` equal groups of neighbouring outputs (a group scores
    by its best member); the `top` chosen outputs are weighted by their plain probabilities (renormalised only if `renorm`), times
    `weight_scale`.
    Tensors under `prefix`: router (experts + identity, width), correction (experts + identity), e<j>.gate / e<j>.up (ff, width),
    e<j>.down (width, ff).  Gate and up rows of all experts are stacked in blocks of 16 (16 gate rows, their 16 up rows), so that the grouped
    product's epilogue finishes the activation."""
    _side_matrix = "w_router"

    def __init__(self, width, ff, experts, top, identity=0, groups=1, keep=1, correction=True, renorm=False, score="softmax", group_top=1,
                 renorm_eps=0.0, act="silu", act_alpha=1.0, limit=0.0, weight_scale=1.0):
        """score: "softmax" over all outputs or "sigmoid" of each logit; group_top: a group scores by the sum of its group_top best choice
        scores; act: "silu" -- silu(gate) up --, or "swish_clamp" -- g sigmoid(act_alpha g) (u + 1) with g = min(gate, limit),
        u = clamp(up, -limit, limit)"""
        if score not in ("softmax", "sigmoid") or act not in ("silu", "swish_clamp") or group_top < 1:
            raise ZLError("experts: unknown score function or activation")
        self.score, self.group_top, self.renorm_eps, self.act, self.act_alpha, self.limit = score, int(group_top), float(renorm_eps), act, \
            float(act_alpha), float(limit)
        self.weight_scale = float(weight_scale)
        total = experts + identity
        if groups < 1 or total % groups or not 1 <= keep <= groups or top > keep * (total // groups):
            raise ZLError("experts: groups must divide the router outputs, and the kept groups must hold `top` outputs")
        self.width, self.ff, self.experts, self.top, self.identity = width, ff, experts, top, identity
        self.groups, self.keep, self.has_correction, self.renorm = groups, keep, correction, renorm
        self.packed = ff % 16 == 0                       # gate / up rows in blocks of 16: what the gated epilogue reads
        self.fused_act = self.packed                     # (the grouped product's epilogue finishes the activation)
        self.few_rows = seqops.MOE_FEW_ROWS
        self.tile_m = None                # rows per expert tile of the grouped products (None: by the experts' average share)

    def _pack_gate_up(self, gate, up):
        if not self.packed:
            return torch.cat([gate, up], dim=0)
        f, w = gate.shape
        return torch.stack([gate.reshape(f // 16, 16, w), up.reshape(f // 16, 16, w)], dim=1).reshape(2 * f, w)

    def load(self, get, prefix, dtype, device):
        E, f, W = self.experts, self.ff, self.width
        self.w_router = _mat(get, prefix + "router", (E + self.identity, W), dtype, device)
        self.correction = _vec(get, prefix + "correction", E + self.identity, device) if self.has_correction else None
        self.w_gu = torch.empty((E, 2 * f, W), dtype=dtype, device=device)
        self.w_down = torch.empty((E, W, f), dtype=dtype, device=device)
        for e in range(E):
            p = f"{prefix}e{e}."
            self.w_gu[e] = self._pack_gate_up(_mat(get, p + "gate", (f, W), dtype, device), _mat(get, p + "up", (f, W), dtype, device))
            self.w_down[e] = _mat(get, p + "down", (W, f), dtype, device)
        return self

    def init_random(self, gen, dtype, device):
        E, f, W = self.experts, self.ff, self.width
        self.w_router = _rand(gen, (E + self.identity, W), W ** -0.5, dtype, device)
        self.correction = torch.zeros(E + self.identity, device=device) if self.has_correction else None
        self.w_gu = _rand(gen, (E, 2 * f, W), W ** -0.5, dtype, device)
        self.w_down = _rand(gen, (E, W, f), f ** -0.5, dtype, device)
        return self

    def weight_bytes(self):
        return sum(t.numel() * t.element_size() for t in (self.w_router, self.w_gu, self.w_down))       # (w_router: with attached side rows)

    def forward(self, h):
        logits = seqops.gemm_nt(h, self.w_router)                                 # fp32 sums of the products [router | side rows]
        self.side = (logits, self.side_col0)
        ids, weights = seqops.moe_route(logits, self.correction, self.groups, self.keep, self.top, self.renorm, score=self.score,
                                        group_top=self.group_top, renorm_eps=self.renorm_eps, weight_scale=self.weight_scale,
                                        n_out=self.experts + self.identity)
        sorted_tok, slot_pos, tiles, max_tiles, sorted_exp, tm = seqops.moe_align(ids, self.experts, self.tile_m)
        n_slots = ids.numel()
        few = sorted_exp if n_slots <= self.few_rows else None                    # decode steps: weight rows streamed per (row, column)
        if self.fused_act:
            a = seqops.gemm_nt_grouped(h, sorted_tok, self.w_gu, tiles, max_tiles, n_slots, gated=True, out_dtype=h.dtype, row_expert=few, tile_m=tm,
                                       act=self.act, act_alpha=self.act_alpha, act_limit=self.limit)
        else:
            a = seqops.act_mul(seqops.gemm_nt_grouped(h, sorted_tok, self.w_gu, tiles, max_tiles, n_slots, row_expert=few, tile_m=tm), h.dtype,
                               kind=self.act, alpha=self.act_alpha, limit=self.limit, block=16 if self.packed else 0)
        y = seqops.gemm_nt_grouped(a, None, self.w_down, tiles, max_tiles, n_slots, row_expert=few, tile_m=tm)
        return seqops.moe_combine(y, slot_pos, ids, weights, h, self.experts)
