"""Python face of libzhilight_amd_seq.so (include/zhilight_amd_seq.h): the kernels that run a RAGGED step -- portions of prompts and
single decoded tokens of several sequences as one flat list of tokens.  As in `ops`: PyTorch supplies device memory and the stream, every
function enqueues one launcher, and there is no CPU or PyTorch fallback -- without the built library these raise.

The library is built on first use when it is absent (`build.build_seq`: a few files, seconds), so a fresh checkout can serve such a model
without compiling the quantised decode path.
"""
import ctypes as C
import os

import torch

from ._lib import ZLError

BF16, F32 = 1, 2
_HERE = os.path.dirname(os.path.abspath(__file__))
SO_PATH = os.path.join(_HERE, "libzhilight_amd_seq.so")
SYMBOLS = ["zls_version", "zls_gemm_nt", "zls_embed", "zls_token_shift", "zls_add_scalar_norm", "zls_scalar_norm_rows", "zls_polynorm",
           "zls_latent_store", "zls_latent_attention", "zls_latent_attention_workspace_bytes", "zls_latent_attention_prompt", "zls_gemm_nt_gather",
           "zls_conv_silu", "zls_conv_tail_update", "zls_ssm_scan", "zls_ssm_scan_workspace_bytes", "zls_gated_group_norm", "zls_layer_norm",
           "zls_add_layer_norm", "zls_rope_norm_store", "zls_window_attention", "zls_window_attention_prompt", "zls_head_mix_gate", "zls_decay_scan", "zls_exp_gates",
           "zls_linear_attn_finish", "zls_moe_route", "zls_moe_align", "zls_gemm_nt_grouped", "zls_silu_mul", "zls_moe_combine", "zls_rms_norm",
           "zls_add_rms_norm", "zls_scale_softcap", "zls_act_mul", "zls_short_conv", "zls_short_conv_tail", "zls_lowrank_decay", "zls_latent_rope_store",
           "zls_streams_norm", "zls_streams_update", "zls_unary_act"]
_STATUS = {-1: "invalid argument (null pointer / non-positive size)", -2: "shape not supported", -3: "dtype not supported",
           -4: "exceeds a hardware limit"}


class Batch(C.Structure):
    """zls_batch_t"""
    _fields_ = [("n_seq", C.c_int32), ("n_tok", C.c_int32), ("max_pages", C.c_int32), ("page_size", C.c_int32), ("max_count", C.c_int32),
                ("reserved", C.c_int32), ("seq_start", C.c_void_p), ("seq_pos0", C.c_void_p), ("seq_slot", C.c_void_p),
                ("tok_seq", C.c_void_p), ("page_table", C.c_void_p)]


class ScoreForm(C.Structure):
    """zls_score_form_t"""
    _fields_ = [("head_scale", C.c_void_p), ("softcap", C.c_float), ("bias", C.c_void_p), ("bias_rows", C.c_int32), ("offset", C.c_void_p),
                ("chunk", C.c_int32), ("sigmoid", C.c_int32)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(SO_PATH):
            from . import build
            build.build_seq()
        l = C.CDLL(SO_PATH)
        for name in SYMBOLS:
            getattr(l, name)
        l.zls_latent_attention_workspace_bytes.restype = C.c_int64
        l.zls_ssm_scan_workspace_bytes.restype = C.c_int64
        _lib = l
    return _lib


def check(status, what):
    if status != 0:
        raise ZLError(f"{what}: status {status}: {_STATUS.get(status, 'HIP error')}")


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t):
    return C.c_void_p(0 if t is None else t.data_ptr())


def _i(v):
    return C.c_int64(int(v))


def _f(v):
    return C.c_float(float(v))


def dt_code(dtype):
    if dtype == torch.bfloat16:
        return BF16
    if dtype == torch.float32:
        return F32
    raise ZLError(f"the ragged-batch kernels take bfloat16 or float32, not {dtype}")


def _cuda(*ts):
    for t in ts:
        if t is not None and not (t.is_cuda and t.is_contiguous()):
            raise ZLError("tensors must be contiguous device tensors")


def _f32(*ts):
    for t in ts:
        if t is not None and t.dtype != torch.float32:
            raise ZLError("this argument is fp32 in both modes")


class RaggedBatch:
    """The device-side description of one step (zls_batch_t) and the tensors that own its arrays.
    seqs: list of (count, pos0, slot, pages) -- pages: the sequence's page ids, enough for pos0 + count tokens."""

    def __init__(self, seqs, page_size, device):
        n_seq = len(seqs)
        if n_seq == 0:
            raise ZLError("an empty step")
        starts, tok_seq = [0], []
        max_pages = max(1, max(len(s[3]) for s in seqs))
        table = []
        for i, (count, pos0, slot, pages) in enumerate(seqs):
            if count <= 0 or pos0 < 0 or (pos0 + count + page_size - 1) // page_size > len(pages):
                raise ZLError("a portion needs count > 0 and pages for all its positions")
            starts.append(starts[-1] + count)
            tok_seq += [i] * count
            table += list(pages) + [0] * (max_pages - len(pages))
        # the cached rows of every PORTION's whole context, sequence after sequence, each padded to a multiple of 64 rows (the padding
        # points at the sequence's first row): what the prompt attention's up-projection gathers.  ctx_start: -1 for single tokens
        ctx_rows, ctx_start = [], []
        for count, pos0, slot, pages in seqs:
            if count == 1:
                ctx_start.append(-1)
                continue
            ctx_start.append(len(ctx_rows))
            n = pos0 + count
            rows = [pages[j // page_size] * page_size + j % page_size for j in range(n)]
            ctx_rows += rows + [rows[0]] * (-n % 64)
        # query tiles of the portions: (first flat token, rows <= 64, sequence) -- what the matrix-core attention kernels walk
        q_tiles = []
        for i, (count, pos0, slot, pages) in enumerate(seqs):
            if count > 1:
                for r0 in range(0, count, 64):
                    q_tiles += [starts[i] + r0, min(64, count - r0), i]
        # ONE host array, one copy: [seq_start | seq_pos0 | seq_slot | tok_seq | page_table | ctx_start | ctx_rows | q_tiles]
        host = torch.tensor(starts + [s[1] for s in seqs] + [s[2] for s in seqs] + tok_seq + table + ctx_start + ctx_rows + q_tiles,
                            dtype=torch.int32)
        self.dev = host.to(device, non_blocking=False)
        o = [0, n_seq + 1, 2 * n_seq + 1, 3 * n_seq + 1, 3 * n_seq + 1 + starts[-1]]
        base = self.dev.data_ptr()
        self.n_seq, self.n_tok, self.starts = n_seq, starts[-1], starts
        self.counts = [s[0] for s in seqs]
        at = o[4] + len(table)
        self.ctx_start = self.dev[at:at + n_seq]
        self.ctx_rows = self.dev[at + n_seq:at + n_seq + len(ctx_rows)]
        self.n_ctx = len(ctx_rows)
        self.q_tiles = self.dev[at + n_seq + len(ctx_rows):]
        self.n_q_tiles = len(q_tiles) // 3
        self.min_pos0 = min(s[1] for s in seqs)
        self.n_single = sum(1 for c in self.counts if c == 1)
        self.max_ctx = max(s[0] + s[1] for s in seqs)
        self.c = Batch(n_seq, self.n_tok, max_pages, page_size, max(self.counts), 0, *[base + 4 * x for x in o])
        self.ref = C.byref(self.c)
        self._seqs, self._windowed = seqs, {}

    def context(self, window):
        """(ctx_start, ctx_pos0, ctx_rows, n_ctx) for portions that look back `window` positions only: the cached rows from the 64-aligned
        position at or below the oldest key the portion's first token sees, each sequence padded to a multiple of 64 rows.  window 0: the
        whole context (ctx_pos0 None).  One more small host-to-device copy per distinct window of a step."""
        if window <= 0:
            return self.ctx_start, None, self.ctx_rows, self.n_ctx
        if window not in self._windowed:
            ps = self.c.page_size
            ctx_rows, ctx_start, ctx_pos0 = [], [], []
            for count, pos0, slot, pages in self._seqs:
                if count == 1:
                    ctx_start.append(-1)
                    ctx_pos0.append(0)
                    continue
                c0 = max(0, pos0 - window + 1) // 64 * 64
                ctx_start.append(len(ctx_rows))
                ctx_pos0.append(c0)
                rows = [pages[j // ps] * ps + j % ps for j in range(c0, pos0 + count)]
                ctx_rows += rows + [rows[0]] * (-len(rows) % 64)
            dev = torch.tensor(ctx_start + ctx_pos0 + ctx_rows, dtype=torch.int32).to(self.dev.device)
            n = self.n_seq
            self._windowed[window] = (dev[:n], dev[n:2 * n], dev[2 * n:], len(ctx_rows))
        return self._windowed[window]


def gemm_nt(x, w, out=None, out_dtype=torch.float32):
    """x (m, k) . w (n, k)^T -> (m, n); x and w in the serving format, the result fp32 (or that format)."""
    _cuda(w)
    if x.dim() != 2 or x.stride(1) != 1 or not x.is_cuda:
        raise ZLError("gemm_nt: x must be a device matrix with unit column stride")
    m, k = x.shape
    n = w.shape[0]
    if w.shape[1] != k or w.dtype != x.dtype:
        raise ZLError("gemm_nt: size K / dtype mismatch")
    if out is None:
        out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    elif out.shape != (m, n) or not out.is_contiguous():
        raise ZLError("gemm_nt: wrong output")
    check(lib().zls_gemm_nt(_p(x), _i(x.stride(0)), _p(w), _p(out), _i(n), _i(m), _i(n), _i(k), C.c_int(dt_code(x.dtype)),
                            C.c_int(dt_code(out.dtype)), _stream()), "gemm_nt")
    return out


def embed(tokens, table, pos_table, scale, batch, out=None):
    _cuda(tokens, table, pos_table)
    width = table.shape[1]
    if out is None:
        out = torch.empty((batch.n_tok, width), dtype=torch.float32, device=table.device)
    if tokens.dtype != torch.int32 or tokens.numel() != batch.n_tok:
        raise ZLError("embed: tokens must be int32, one per flat token")
    check(lib().zls_embed(_p(tokens), _p(table), _p(pos_table), _i(table.shape[0]), _i(0 if pos_table is None else pos_table.shape[0]),
                          _f(scale), batch.ref, _p(out), _i(width), C.c_int(dt_code(table.dtype)), _stream()), "embed")
    return out


def token_shift(x, mix, prev, batch, dtype):
    _cuda(x, mix, prev)
    _f32(x, mix, prev)
    width = x.shape[1]
    if mix.numel() != width or prev.shape[-1] != width:
        raise ZLError("token_shift: width mismatch")
    h = torch.empty((batch.n_tok, width), dtype=dtype, device=x.device)
    check(lib().zls_token_shift(_p(x), _p(mix), _p(prev), batch.ref, _p(h), _i(width), C.c_int(dt_code(dtype)), _stream()), "token_shift")
    return h


def add_scalar_norm(x, y, gain, eps, out_dtype=None):
    """x += y / rms(y) * gain in place; out_dtype: also return the new x in that format (None: nothing; float32: x itself)"""
    _cuda(x, y)
    _f32(x, y)
    if x.shape != y.shape:
        raise ZLError("add_scalar_norm: shape mismatch")
    xt = torch.empty(x.shape, dtype=out_dtype, device=x.device) if out_dtype not in (None, torch.float32) else None
    check(lib().zls_add_scalar_norm(_p(x), _p(y), _f(gain), _f(eps), _i(x.shape[0]), _i(x.shape[1]), _p(xt),
                                    C.c_int(BF16 if xt is None else dt_code(out_dtype)), _stream()), "add_scalar_norm")
    return x if out_dtype == torch.float32 else xt


def scalar_norm_rows(x, rows, gain, eps, dtype):
    _cuda(x, rows)
    _f32(x)
    if rows.dtype != torch.int32:
        raise ZLError("scalar_norm_rows: rows must be int32")
    out = torch.empty((rows.numel(), x.shape[1]), dtype=dtype, device=x.device)
    check(lib().zls_scalar_norm_rows(_p(x), _p(rows), _f(gain), _f(eps), _i(rows.numel()), _i(x.shape[1]), _p(out), C.c_int(dt_code(dtype)),
                                     _stream()), "scalar_norm_rows")
    return out


def polynorm(z, coef, eps, dtype):
    """coef: four host floats (a, b, c, e)"""
    _cuda(z)
    _f32(z)
    out = torch.empty(z.shape, dtype=dtype, device=z.device)
    arr = (C.c_float * 4)(*[float(v) for v in coef])
    check(lib().zls_polynorm(_p(z), arr, _f(eps), _i(z.shape[0]), _i(z.shape[1]), _p(out), C.c_int(dt_code(dtype)), _stream()), "polynorm")
    return out


def latent_store(proj, col0, weight, eps, rank, batch, cache, rot=0, freq=None, interleaved=True, q_col0=0, heads=0, qdim=0, rot_gain=1.0):
    """normed latent -> the tokens' cache rows; rot > 0: the `rot` columns behind the latent (one key part for all heads) are turned by the
    position and stored behind it, and the last rot of the qdim coordinates of every query head (from q_col0) are turned in place; cos and
    sin times rot_gain"""
    _cuda(proj, weight, cache, freq)
    _f32(proj, weight, freq)
    if cache.dim() != 3 or cache.shape[1] != batch.c.page_size or cache.shape[2] != rank + rot or weight.numel() != rank:
        raise ZLError("latent_store: cache must be (pages, page_size, rank + rot)")
    if rot and (freq is None or freq.numel() != rot // 2):
        raise ZLError("latent_store: one frequency per rotated pair")
    check(lib().zls_latent_rope_store(_p(proj), _i(proj.shape[1]), _i(col0), _p(weight), _f(eps), _i(rank), _i(rot), _p(freq),
                                      C.c_int(int(interleaved)), _i(q_col0), _i(heads), _i(qdim), _f(rot_gain), batch.ref, _p(cache),
                                      C.c_int(dt_code(cache.dtype)), _stream()), "latent_store")


def gemm_nt_gather(x, x_rows, w, w_rows, m, n, out):
    """rows x_rows of x (all of x: None) times rows w_rows of w, transposed -> out (m, n) in its own dtype"""
    k = x.shape[-1]
    if w.shape[-1] != k or x.dtype != w.dtype or out.shape[0] != m or out.shape[1] < n or out.stride(1) != 1:
        raise ZLError("gemm_nt_gather: shapes")
    for r in (x_rows, w_rows):
        if r is not None and (r.dtype != torch.int32 or not r.is_cuda):
            raise ZLError("gemm_nt_gather: int32 device row indices")
    check(lib().zls_gemm_nt_gather(_p(x), _i(k), _p(x_rows), _p(w), _i(k), _p(w_rows), _p(out), _i(out.stride(0)), _i(m), _i(n), _i(k),
                                   C.c_int(dt_code(x.dtype)), C.c_int(dt_code(out.dtype)), _stream()), "gemm_nt_gather")
    return out


def latent_attention_prompt(q, q_col0, gate, g_col0, k, vt, sink, batch, scale, heads, dim, vdim, out, window=0):
    """the portions of the step on the matrix cores; k (n_ctx, heads * dim), vt (heads * vdim, n_ctx) from gemm_nt_gather over the rows of
    batch.context(window); writes its rows of out"""
    _cuda(q, gate, k, vt, sink, out)
    _f32(q, gate, sink)
    ctx_start, ctx_pos0, _, _ = batch.context(window)
    check(lib().zls_latent_attention_prompt(_p(q), _i(q.shape[1]), _i(q_col0), _p(gate), _i(0 if gate is None else gate.shape[1]), _i(g_col0),
                                            _p(k), _i(k.stride(0)), _p(vt), _i(vt.stride(0)), _p(sink), _p(ctx_start), batch.ref, _f(scale),
                                            _i(heads), _i(dim), _i(vdim), _p(out), C.c_int(dt_code(out.dtype)), _i(window), _p(ctx_pos0), _stream()),
          "latent_attention_prompt")
    return out


def latent_attention(q, q_col0, gate, g_col0, w_uk, w_uv, sink, cache, batch, scale, heads, dim, vdim, out=None, single_only=False, mfma=True,
                     n_splits=None, window=0):
    _cuda(q, gate, w_uk, w_uv, sink, cache)
    _f32(q, gate, sink)
    rank = cache.shape[2]
    if w_uk.shape != (heads * dim, rank) or w_uv.shape != (heads * vdim, rank) or w_uk.dtype != cache.dtype or w_uv.dtype != cache.dtype:
        raise ZLError("latent_attention: up-projection shapes / dtypes")
    if sink is not None and sink.numel() != heads:
        raise ZLError("latent_attention: one sink per head")
    if out is None:
        out = torch.empty((batch.n_tok, heads * vdim), dtype=cache.dtype, device=cache.device)
    # enough workgroups to fill the chip (256 CUs, a few per CU), at least 64 keys per split
    groups = batch.n_tok * ((heads + 3) // 4)
    if n_splits is None:
        span = min(batch.max_ctx, window) if window > 0 else batch.max_ctx
        n_splits = max(1, min((span + 63) // 64, (1024 + groups - 1) // groups))
    ws = torch.empty(int(lib().zls_latent_attention_workspace_bytes(_i(batch.n_tok), _i(heads), _i(rank), _i(n_splits))) // 4,
                     dtype=torch.float32, device=cache.device)
    check(lib().zls_latent_attention(_p(q), _i(q.shape[1]), _i(q_col0), _p(gate), _i(0 if gate is None else gate.shape[1]), _i(g_col0), _p(w_uk),
                                     _p(w_uv), _p(sink), _p(cache), batch.ref, _f(scale), _i(heads), _i(dim), _i(vdim), _i(rank), _p(out),
                                     C.c_int(dt_code(cache.dtype)), C.c_int(int(single_only)), _p(ws), _i(n_splits), C.c_int(0 if mfma else 1),
                                     _i(window), _stream()),
          "latent_attention")
    return out


def conv_silu(proj, col0, w, bias, tail, batch):
    """causal convolution + SiLU over `channels` columns of proj from col0, then the carried tail moves on (two launches)"""
    _cuda(proj, w, bias, tail)
    _f32(proj, w, bias, tail)
    channels, taps = w.shape
    if tail is not None and tuple(tail.shape[1:]) != (taps - 1, channels):
        raise ZLError("conv_silu: tail must be (slots, taps - 1, channels)")
    out = torch.empty((batch.n_tok, channels), dtype=torch.float32, device=proj.device)
    check(lib().zls_conv_silu(_p(proj), _i(proj.shape[1]), _i(col0), _p(w), _p(bias), _p(tail), _i(channels), _i(taps), batch.ref, _p(out),
                              _stream()), "conv_silu")
    check(lib().zls_conv_tail_update(_p(proj), _i(proj.shape[1]), _i(col0), _p(tail), _i(channels), _i(taps), batch.ref, _stream()),
          "conv_tail_update")
    return out


def short_conv(proj, col0, w, in_bias, tail, batch, act=False, bias=None):
    """causal convolution over `channels` columns of proj from col0: in_bias joins every input, `bias` the result, act: SiLU; the carried
    tail moves on (two launches)"""
    _cuda(proj, w, bias, in_bias, tail)
    _f32(proj, w, bias, in_bias, tail)
    channels, taps = w.shape
    if tail is not None and tuple(tail.shape[1:]) != (taps - 1, channels):
        raise ZLError("short_conv: tail must be (slots, taps - 1, channels)")
    for t in (bias, in_bias):
        if t is not None and t.numel() != channels:
            raise ZLError("short_conv: one bias per channel")
    out = torch.empty((batch.n_tok, channels), dtype=torch.float32, device=proj.device)
    check(lib().zls_short_conv(_p(proj), _i(proj.shape[1]), _i(col0), _p(w), _p(bias), _p(in_bias), C.c_int(int(act)), _p(tail), _i(channels),
                               _i(taps), batch.ref, _p(out), _stream()), "short_conv")
    check(lib().zls_short_conv_tail(_p(proj), _i(proj.shape[1]), _i(col0), _p(in_bias), _p(tail), _i(channels), _i(taps), batch.ref, _stream()),
          "short_conv_tail")
    return out


SCAN_SEGMENT = 256      # tokens per segment of a long portion (ssm_scan)


def ssm_scan(xbc, proj, dt_col0, dt_bias, a_log, d, state, heads, vdim, n_state, groups, batch, seg_len=None):
    _cuda(xbc, proj, dt_bias, a_log, d, state)
    _f32(xbc, proj, dt_bias, a_log, d, state)
    if xbc.shape[1] != heads * vdim + 2 * groups * n_state or tuple(state.shape[1:]) != (heads, n_state, vdim):
        raise ZLError("ssm_scan: shapes")
    y = torch.empty((batch.n_tok, heads * vdim), dtype=torch.float32, device=xbc.device)
    seg_len = SCAN_SEGMENT if seg_len is None else seg_len
    ws = None
    if seg_len > 0 and batch.c.max_count > seg_len:
        ws = torch.empty(int(lib().zls_ssm_scan_workspace_bytes(_i(batch.n_seq), _i(batch.c.max_count), _i(seg_len), _i(heads), _i(vdim),
                                                                _i(n_state))) // 4, dtype=torch.float32, device=xbc.device)
    check(lib().zls_ssm_scan(_p(xbc), _p(proj), _i(proj.shape[1]), _i(dt_col0), _p(dt_bias), _p(a_log), _p(d), _p(state), _i(heads), _i(vdim),
                             _i(n_state), _i(groups), batch.ref, _p(y), _p(ws), _i(seg_len), _stream()), "ssm_scan")
    return y


def gated_group_norm(y, proj, z_col0, weight, eps, norm_groups, dtype):
    _cuda(y, proj, weight)
    _f32(y, proj, weight)
    out = torch.empty(y.shape, dtype=dtype, device=y.device)
    check(lib().zls_gated_group_norm(_p(y), _p(proj), _i(proj.shape[1]), _i(z_col0), _p(weight), _f(eps), _i(y.shape[0]), _i(y.shape[1]),
                                     _i(norm_groups), _p(out), C.c_int(dt_code(dtype)), _stream()), "gated_group_norm")
    return out


# ---- layer norm ------------------------------------------------------------------------------------------------------------------------
def layer_norm(x, weight, bias, eps, dtype, rows=None):
    """(x - mean) / sqrt(var + eps) * weight + bias of the rows `rows` (int32 device; None: all) of fp32 x, in `dtype`"""
    _cuda(x, weight, bias, rows)
    _f32(x, weight, bias)
    if rows is not None and rows.dtype != torch.int32:
        raise ZLError("layer_norm: rows must be int32")
    n = x.shape[0] if rows is None else rows.numel()
    out = torch.empty((n, x.shape[1]), dtype=dtype, device=x.device)
    check(lib().zls_layer_norm(_p(x), _p(rows), _p(weight), _p(bias), _f(eps), _i(n), _i(x.shape[1]), _p(out), C.c_int(dt_code(dtype)), _stream()),
          "layer_norm")
    return out


def add_layer_norm(x, y, weight, bias, eps, next_weight=None, next_bias=None, dtype=None):
    """x += layer_norm(y) in place; with next_weight also returns layer_norm(new x; next_weight, next_bias) in `dtype`"""
    _cuda(x, y, weight, bias, next_weight, next_bias)
    _f32(x, y, weight, bias, next_weight, next_bias)
    if x.shape != y.shape or weight.numel() != x.shape[1]:
        raise ZLError("add_layer_norm: shape mismatch")
    h2 = torch.empty(x.shape, dtype=dtype, device=x.device) if next_weight is not None else None
    check(lib().zls_add_layer_norm(_p(x), _p(y), _p(weight), _p(bias), _f(eps), _i(x.shape[0]), _i(x.shape[1]), _p(next_weight), _p(next_bias),
                                   _p(h2), C.c_int(dt_code(dtype) if h2 is not None else BF16), _stream()), "add_layer_norm")
    return h2


# ---- weighted RMS norm ------------------------------------------------------------------------------------------------------------------
def rms_norm(x, weight, eps, dtype, rows=None, around_zero=False):
    """x / sqrt(mean(x^2) + eps) * weight (around_zero: * (1 + weight)) of the rows `rows` (int32 device; None: all) of fp32 x, in `dtype`"""
    _cuda(x, weight, rows)
    _f32(x, weight)
    if rows is not None and rows.dtype != torch.int32:
        raise ZLError("rms_norm: rows must be int32")
    if weight.numel() != x.shape[1]:
        raise ZLError("rms_norm: one weight per column")
    n = x.shape[0] if rows is None else rows.numel()
    out = torch.empty((n, x.shape[1]), dtype=dtype, device=x.device)
    check(lib().zls_rms_norm(_p(x), _p(rows), _p(weight), _f(1.0 if around_zero else 0.0), _f(eps), _i(n), _i(x.shape[1]), _p(out),
                             C.c_int(dt_code(dtype)), _stream()), "rms_norm")
    return out


def add_rms_norm(x, y, eps, next_weight=None, dtype=None, around_zero=False):
    """x += y in place; with next_weight also returns the weighted RMS norm of the new x in `dtype`"""
    _cuda(x, y, next_weight)
    _f32(x, y, next_weight)
    if x.shape != y.shape or (next_weight is not None and next_weight.numel() != x.shape[1]):
        raise ZLError("add_rms_norm: shape mismatch")
    h2 = torch.empty(x.shape, dtype=dtype, device=x.device) if next_weight is not None else None
    check(lib().zls_add_rms_norm(_p(x), _p(y), _f(eps), _i(x.shape[0]), _i(x.shape[1]), _p(next_weight), _f(1.0 if around_zero else 0.0), _p(h2),
                                 C.c_int(dt_code(dtype) if h2 is not None else BF16), _stream()), "add_rms_norm")
    return h2


# ---- a residual kept as several streams ------------------------------------------------------------------------------------------------
def streams_norm(xs, n, read_coef, weight, eps, dtype, rows=None, around_zero=False):
    """N(sum_s read_coef[s] x_s) of the rows `rows` (None: all) in `dtype`.  xs fp32: (n_tok, n, width), or (n_tok, width) read as n equal
    streams; read_coef fp32 (n) or None (all 1)"""
    _cuda(xs, read_coef, weight, rows)
    _f32(xs, read_coef, weight)
    width = xs.shape[-1]
    if xs.dim() == 3 and xs.shape[1] != n or (read_coef is not None and read_coef.numel() != n) or weight.numel() != width:
        raise ZLError("streams_norm: shapes")
    if rows is not None and rows.dtype != torch.int32:
        raise ZLError("streams_norm: rows must be int32")
    tok, stream = (n * width, width) if xs.dim() == 3 else (width, 0)
    n_rows = xs.shape[0] if rows is None else rows.numel()
    h = torch.empty((n_rows, width), dtype=dtype, device=xs.device)
    check(lib().zls_streams_norm(_p(xs), _i(tok), _i(stream), _i(n), _p(read_coef), _p(rows), _p(weight), _f(1.0 if around_zero else 0.0),
                                 _f(eps), _i(n_rows), _i(width), _p(h), C.c_int(dt_code(dtype)), _stream()), "streams_norm")
    return h


def streams_update(src, dst, n, y, mix, out_coef, gate=None, g_col0=0, gate_bias=None, next_coef=None, next_weight=None, eps=0.0, dtype=None,
                   around_zero=False):
    """dst_d = sum_s mix[s][d] src_s + out_coef[d] * y * sigmoid(gate[:, g_col0:] + gate_bias) for all streams at once (dst may be src; src
    (n_tok, width) is read as n equal streams); with next_coef also returns N(sum_d next_coef[d] dst_d) in `dtype`"""
    _cuda(src, dst, y, mix, out_coef, gate, gate_bias, next_coef, next_weight)
    _f32(src, dst, y, mix, out_coef, gate, gate_bias, next_coef, next_weight)
    n_tok, width = y.shape
    if tuple(dst.shape) != (n_tok, n, width) or mix.numel() != n * n or out_coef.numel() != n or src.shape[0] != n_tok or src.shape[-1] != width \
            or (src.dim() == 3 and src.shape[1] != n) or (gate_bias is not None and gate_bias.numel() != width):
        raise ZLError("streams_update: shapes")
    tok, stream = (n * width, width) if src.dim() == 3 else (width, 0)
    h = torch.empty((n_tok, width), dtype=dtype, device=y.device) if next_coef is not None else None
    check(lib().zls_streams_update(_p(src), _i(tok), _i(stream), _p(dst), _i(n), _p(y), _p(gate), _i(0 if gate is None else gate.stride(0)),
                                   _i(g_col0), _p(gate_bias), _p(mix), _p(out_coef), _p(next_coef), _p(next_weight),
                                   _f(1.0 if around_zero else 0.0), _f(eps), _i(n_tok), _i(width), _p(h),
                                   C.c_int(dt_code(dtype) if h is not None else BF16), _stream()), "streams_update")
    return h


UNARY_ACTS = {"relu2": 0, "gelu_tanh": 1, "silu": 2}


def unary_act(z, dtype, kind="relu2", cols=None):
    """act(z[:, :cols]) of fp32 rows in `dtype`; see UNARY_ACTS"""
    _f32(z)
    if z.dim() != 2 or z.stride(1) != 1 or not z.is_cuda:
        raise ZLError("unary_act: z must be a device matrix with unit column stride")
    cols = z.shape[1] if cols is None else cols
    out = torch.empty((z.shape[0], cols), dtype=dtype, device=z.device)
    check(lib().zls_unary_act(_p(z), _i(z.stride(0)), _i(z.shape[0]), _i(cols), C.c_int(UNARY_ACTS[kind]), _p(out), C.c_int(dt_code(dtype)),
                              _stream()), "unary_act")
    return out


def scale_softcap(z, scale, cap):
    """z <- cap * tanh(z * scale / cap) in place (cap <= 0: z * scale); fp32"""
    _cuda(z)
    _f32(z)
    check(lib().zls_scale_softcap(_p(z), _i(z.numel()), _f(scale), _f(cap), _stream()), "scale_softcap")
    return z


# ---- softmax attention over paged keys and values -------------------------------------------------------------------------------------------
def rope_norm_store(proj, q_col0, k_col0, v_col0, heads, kv_heads, dim, vdim, qk_freq, rot_dims, v_freq, eps, qk_norm, batch, k_cache, v_cache,
                    interleaved=False, vmix=None, q_norm_w=None, k_norm_w=None):
    """rotate / norm the queries in place in proj; rotate / norm the keys and turn the values into the paged planes (None: queries only).
    interleaved: rotated pairs are neighbours (2i, 2i + 1).  vmix = (src, col0, lam): values <- (1 - lam) values + lam src[t][col0 ..].
    q_norm_w / k_norm_w: fp32 (dim) weights of the norm, shared by the heads"""
    _cuda(proj, qk_freq, v_freq, k_cache, v_cache, q_norm_w, k_norm_w)
    _f32(proj, qk_freq, v_freq, q_norm_w, k_norm_w)
    for t in (q_norm_w, k_norm_w):
        if t is not None and (t.numel() != dim or not qk_norm):
            raise ZLError("rope_norm_store: a norm weight has one number per coordinate of a head")
    vsrc, vcol, vlam = vmix if vmix is not None else (None, 0, 0.0)
    if vsrc is not None and (vsrc.dtype != torch.float32 or vsrc.dim() != 2 or vsrc.stride(1) != 1 or vsrc.shape[0] != batch.n_tok):
        raise ZLError("rope_norm_store: the blended values are fp32 rows, one per token")
    if (qk_freq is not None and qk_freq.numel() != rot_dims // 2) or (v_freq is not None and v_freq.numel() != vdim // 2):
        raise ZLError("rope_norm_store: one frequency per rotated pair")
    if k_cache is not None:
        if tuple(k_cache.shape[1:]) != (batch.c.page_size, kv_heads * dim) or tuple(v_cache.shape[1:]) != (batch.c.page_size, kv_heads * vdim) \
                or k_cache.dtype != v_cache.dtype:
            raise ZLError("rope_norm_store: planes must be (pages, page_size, kv_heads * dim | vdim)")   # (the value plane's pages are
            # written transposed, (kv_heads * vdim, page_size): the same bytes of the same plane)
    code = dt_code(k_cache.dtype) if k_cache is not None else F32
    check(lib().zls_rope_norm_store(_p(proj), _i(proj.shape[1]), _i(q_col0), _i(k_col0), _i(v_col0), _i(heads), _i(kv_heads), _i(dim), _i(vdim),
                                    _p(qk_freq), _i(rot_dims), _p(v_freq), _f(eps), C.c_int(int(qk_norm)), C.c_int(int(interleaved)), _p(vsrc),
                                    _i(0 if vsrc is None else vsrc.stride(0)), _i(vcol), _f(vlam), _p(q_norm_w), _p(k_norm_w), batch.ref, _p(k_cache), _p(v_cache),
                                    C.c_int(code), _stream()), "rope_norm_store")


def score_form(heads, head_scale=None, softcap=0.0, bias=None, offset=None, chunk=0, sigmoid=False):
    """The optional score form of window_attention: per-head factor (heads), tanh cap, distance bias fp32 (heads, rows) -- row min(p - j,
    rows - 1) --, chunked visibility, sigmoid weights with a per-head offset.  Returns an object that keeps the tensors alive."""
    _cuda(head_scale, bias, offset)
    _f32(head_scale, bias, offset)
    for t in (head_scale, offset):
        if t is not None and t.numel() != heads:
            raise ZLError("score_form: one number per head")
    if bias is not None and (bias.dim() != 2 or bias.shape[0] != heads):
        raise ZLError("score_form: the distance bias is (heads, rows)")
    f = ScoreForm(0 if head_scale is None else head_scale.data_ptr(), float(softcap or 0.0), 0 if bias is None else bias.data_ptr(),
                  0 if bias is None else bias.shape[1], 0 if offset is None else offset.data_ptr(), int(chunk), int(bool(sigmoid)))
    f.keep = (head_scale, bias, offset)
    return f


def window_attention(q, q_col0, k_cache, v_cache, batch, scale, window, heads, kv_heads, dim, vdim, all_kv, mfma=True, n_splits=None,
                     keep_first=0, form=None):
    """Every query head's softmax weights applied to its own (all_kv False) or every kv head's values.  Returns (acc, ml, n_splits) for
    head_mix_gate: fp32 partial sums (n_tok, heads, n_splits, nv) and their (maximum, weight sum).  bf16 portions run on the matrix cores
    when the sizes allow (mfma=False: everything on the plain kernel); single tokens are split over their window's pages."""
    _cuda(q, k_cache, v_cache)
    _f32(q)
    ps = batch.c.page_size
    if tuple(k_cache.shape[1:]) != (ps, kv_heads * dim) or tuple(v_cache.shape[1:]) != (ps, kv_heads * vdim) or k_cache.dtype != v_cache.dtype:
        raise ZLError("window_attention: planes must be (pages, page_size, kv_heads * dim | vdim)")
    nv = (kv_heads if all_kv else 1) * vdim
    prompt = mfma and batch.n_q_tiles > 0 and k_cache.dtype == torch.bfloat16 and ps == 64 and dim % 8 == 0 and dim <= 256 and vdim % 16 == 0
    plain_tokens = batch.n_single if prompt else batch.n_tok
    # the pages a window can touch, and enough workgroups to fill the chip (256 CUs, a few per CU) when few tokens take the plain kernel
    span = min(batch.max_ctx, window) if window > 0 else batch.max_ctx
    if form is not None and form.chunk > 0:
        span = min(span, form.chunk)                                 # (a chunk's keys: at most chunk positions, wherever they start in a page)
    fref = C.byref(form) if form is not None else None
    keep_first = int(keep_first) if window > 0 else 0                # (keys 0 .. keep_first - 1 stay visible behind the window)
    pages = min((span + ps - 2) // ps + 1 + (keep_first + ps - 1) // ps, (batch.max_ctx + ps - 1) // ps)
    if n_splits is None:
        n_splits = 1 if plain_tokens == 0 else max(1, min(pages, 1024 // (plain_tokens * heads)))
    n_splits = max(1, min(int(n_splits), pages))
    per = (pages + n_splits - 1) // n_splits
    acc = torch.empty((batch.n_tok, heads, n_splits, nv), dtype=torch.float32, device=q.device)
    ml = torch.empty((batch.n_tok, heads, n_splits, 2), dtype=torch.float32, device=q.device)
    code = C.c_int(dt_code(k_cache.dtype))
    if prompt:
        check(lib().zls_window_attention_prompt(_p(q), _i(q.shape[1]), _i(q_col0), _p(k_cache), _p(v_cache), batch.ref, _p(batch.q_tiles),
                                                _i(batch.n_q_tiles), _f(scale), _i(window), _i(keep_first), _i(heads), _i(kv_heads), _i(dim), _i(vdim),
                                                C.c_int(int(all_kv)), _p(acc), _p(ml), _i(n_splits), fref, code, _stream()), "window_attention_prompt")
    if plain_tokens:
        check(lib().zls_window_attention(_p(q), _i(q.shape[1]), _i(q_col0), _p(k_cache), _p(v_cache), batch.ref, _f(scale), _i(window), _i(keep_first), _i(heads),
                                         _i(kv_heads), _i(dim), _i(vdim), C.c_int(int(all_kv)), _p(acc), _p(ml), _i(n_splits), _i(per),
                                         C.c_int(int(prompt)), fref, code, _stream()), "window_attention")
    return acc, ml, n_splits


def head_mix_gate(acc, ml, n_splits, talk, v_freq, gate, g_col0, batch, heads, kv_heads, vdim, dtype, sink=None, plain_sum=False):
    _cuda(acc, ml, talk, v_freq, gate, sink)
    _f32(acc, ml, talk, v_freq, gate, sink)
    if sink is not None and sink.numel() != heads:
        raise ZLError("head_mix_gate: one sink per head")
    if talk is not None and tuple(talk.shape) != (heads, heads):
        raise ZLError("head_mix_gate: the mixing matrix is (heads, heads)")
    if acc.numel() != batch.n_tok * heads * n_splits * (kv_heads if talk is not None else 1) * vdim or ml.numel() != batch.n_tok * heads * n_splits * 2:
        raise ZLError("head_mix_gate: acc / ml do not fit")
    out = torch.empty((batch.n_tok, heads * vdim), dtype=dtype, device=acc.device)
    check(lib().zls_head_mix_gate(_p(acc), _p(ml), _i(n_splits), _p(talk), _p(v_freq), _p(gate), _i(0 if gate is None else gate.shape[1]),
                                  _i(g_col0), _p(sink), C.c_int(int(plain_sum)), batch.ref, _i(heads), _i(kv_heads), _i(vdim), _p(out), C.c_int(dt_code(dtype)),
                                  _stream()), "head_mix_gate")
    return out


# ---- linear attention with a scalar decay -----------------------------------------------------------------------------------------------------
def decay_scan(proj, q_col0, k_col0, v_col0, act, decay_h, decay_t, gain_t, norm_col, state, heads, dim, vdim, batch, seg_len=None,
               decay_v=None):
    """S <- a S + b k v^T, y = S^T q per head over the step's portions; fp32 y (n_tok, heads * (vdim + norm_col)).  The decay a: a constant
    per head (decay_h), a number per token and head (decay_t), or a vector per token, one number per key channel (decay_v (n_tok, heads * dim))"""
    _cuda(proj, decay_h, decay_t, gain_t, state, decay_v)
    _f32(proj, decay_h, decay_t, gain_t, state, decay_v)
    if decay_v is not None and tuple(decay_v.shape) != (batch.n_tok, heads * dim):
        raise ZLError("decay_scan: per-channel decays are (n_tok, heads * dim)")
    P = vdim + (1 if norm_col else 0)
    if tuple(state.shape[1:]) != (heads, dim, P):
        raise ZLError("decay_scan: state must be (slots, heads, dim, vdim + norm_col)")
    for t in (decay_t, gain_t):
        if t is not None and tuple(t.shape) != (batch.n_tok, heads):
            raise ZLError("decay_scan: per-token decays / gains are (n_tok, heads)")
    y = torch.empty((batch.n_tok, heads * P), dtype=torch.float32, device=proj.device)
    seg_len = SCAN_SEGMENT if seg_len is None else seg_len
    ws = None
    if seg_len > 0 and batch.c.max_count > seg_len:
        ws = torch.empty(int(lib().zls_ssm_scan_workspace_bytes(_i(batch.n_seq), _i(batch.c.max_count), _i(seg_len), _i(heads), _i(P), _i(dim))) // 4,
                         dtype=torch.float32, device=proj.device)
    check(lib().zls_decay_scan(_p(proj), _i(proj.shape[1]), _i(q_col0), _i(k_col0), _i(v_col0), C.c_int(int(act)), _p(decay_h), _p(decay_t),
                               _p(gain_t), C.c_int(int(norm_col)), _p(state), _i(heads), _i(dim), _i(vdim), batch.ref, _p(y), _p(ws), _i(seg_len),
                               _p(decay_v), _stream()), "decay_scan")
    return y


def exp_gates(proj, i_col0, f_col0, i_bias, f_bias, cap, m_state, heads, batch):
    """capped exponential gates with a running maximum: (decay, gain, m) fp32 (n_tok, heads) each; m_state (slots, heads) moves on"""
    _cuda(proj, i_bias, f_bias, m_state)
    _f32(proj, i_bias, f_bias, m_state)
    out = torch.empty((3, batch.n_tok, heads), dtype=torch.float32, device=proj.device)
    check(lib().zls_exp_gates(_p(proj), _i(proj.shape[1]), _i(i_col0), _i(f_col0), _p(i_bias), _p(f_bias), _f(cap), _p(m_state), _i(heads),
                              batch.ref, _p(out[0]), _p(out[1]), _p(out[2]), _stream()), "exp_gates")
    return out[0], out[1], out[2]


def lowrank_decay(proj, u_col0, w2, bias, tau):
    """sigmoid(w2 u + bias)^(1 / tau) per token: u = `low` fp32 columns of proj from u_col0, w2 (channels, low); fp32 (n_tok, channels)"""
    _cuda(proj, w2, bias)
    _f32(proj, bias)
    channels, low = w2.shape
    alpha = torch.empty((proj.shape[0], channels), dtype=torch.float32, device=proj.device)
    check(lib().zls_lowrank_decay(_p(proj), _i(proj.shape[1]), _i(u_col0), _i(low), _p(w2), _p(bias), _f(tau), _i(channels), _i(proj.shape[0]),
                                  _p(alpha), C.c_int(dt_code(w2.dtype)), _stream()), "lowrank_decay")
    return alpha


def linear_attn_finish(y, norm_col, q_scale, m_vals, den_eps, heads, vdim, norm_groups, weight, eps, gate, g_col0, dtype, gate_act="sigmoid"):
    _cuda(y, m_vals, weight, gate)
    _f32(y, m_vals, weight, gate)
    n_tok = y.shape[0]
    if y.shape[1] != heads * (vdim + (1 if norm_col else 0)):
        raise ZLError("linear_attn_finish: y does not fit")
    out = torch.empty((n_tok, heads * vdim), dtype=dtype, device=y.device)
    check(lib().zls_linear_attn_finish(_p(y), _i(int(norm_col)), _f(q_scale), _p(m_vals), _f(den_eps), _i(heads), _i(vdim), _i(norm_groups),
                                       _p(weight), _f(eps), _p(gate), _i(0 if gate is None else gate.shape[1]), _i(g_col0), _i(n_tok), _p(out),
                                       C.c_int(dt_code(dtype)), C.c_int(1 if gate_act == "silu" else 0), _stream()), "linear_attn_finish")
    return out


# ---- mixture of experts ------------------------------------------------------------------------------------------------------------------
MOE_TILE = 64           # rows of an expert's tile in the grouped products; 128 when the average expert gets at least MOE_BIG_SHARE rows
MOE_BIG_SHARE = 256


def moe_route(logits, correction, groups, keep, top, renorm=False, score="softmax", group_top=1, renorm_eps=0.0, weight_scale=1.0, n_out=None):
    """n_out: the router's outputs are the leading n_out columns of wider rows (None: all columns)"""
    _cuda(logits, correction)
    _f32(logits, correction)
    n_tok = logits.shape[0]
    n_out = logits.shape[1] if n_out is None else int(n_out)
    if n_out > logits.shape[1]:
        raise ZLError("moe_route: more router outputs than columns")
    if correction is not None and correction.numel() != n_out:
        raise ZLError("moe_route: one correction per router output")
    ids = torch.empty((n_tok, top), dtype=torch.int32, device=logits.device)
    weights = torch.empty((n_tok, top), dtype=torch.float32, device=logits.device)
    if score not in ("softmax", "sigmoid"):
        raise ZLError("moe_route: scores are softmax or sigmoid")
    check(lib().zls_moe_route(_p(logits), _i(logits.stride(0)), _i(n_tok), _i(n_out), _p(correction), _i(groups), _i(keep), _i(top), C.c_int(int(renorm)),
                              C.c_int(1 if score == "sigmoid" else 0), _i(group_top), _f(renorm_eps), _f(weight_scale), _p(ids), _p(weights), _stream()),
          "moe_route")
    return ids, weights


MOE_FEW_ROWS = 64       # up to this many (token, choice) pairs the grouped products stream weight rows per pair instead of tiling


def moe_align(ids, n_experts, tile_m=None):
    """(sorted_tok, slot_pos, tiles, max_tiles, sorted_exp, tile_m) of the (token, choice) pairs sorted by expert"""
    _cuda(ids)
    n_tok, top = ids.shape
    n_slots = n_tok * top
    if tile_m is None:
        tile_m = 128 if n_slots >= MOE_BIG_SHARE * n_experts else MOE_TILE
    max_tiles = n_slots // tile_m + n_experts
    buf = torch.empty(3 * n_slots + 3 * max_tiles, dtype=torch.int32, device=ids.device)
    sorted_tok, slot_pos, sorted_exp, tiles = buf[:n_slots], buf[n_slots:2 * n_slots], buf[2 * n_slots:3 * n_slots], buf[3 * n_slots:]
    check(lib().zls_moe_align(_p(ids), _i(n_slots), _i(top), _i(n_experts), _i(tile_m), _p(sorted_tok), _p(slot_pos), _p(tiles), _i(max_tiles),
                              _p(sorted_exp), _stream()), "moe_align")
    return sorted_tok, slot_pos, tiles, max_tiles, sorted_exp, tile_m


ACT_KINDS = {"silu": 0, "gelu_tanh": 1, "swish_clamp": 2}


def gemm_nt_grouped(x, x_rows, w, tiles, max_tiles, n_rows, gated=False, out_dtype=torch.float32, row_expert=None, tile_m=MOE_TILE,
                    act="silu", act_alpha=1.0, act_limit=0.0):
    """rows of x (gathered by x_rows, or in sorted order) times their expert's block of w (experts, n, k); (n_rows, n or n / 2 gated).
    row_expert (the sorted positions' experts) selects the few-rows kernel.  act (ACT_KINDS) is the gated form's activation."""
    _cuda(x, x_rows, w, tiles, row_expert)
    E, n, k = w.shape
    if x.shape[1] != k or x.dtype != w.dtype:
        raise ZLError("gemm_nt_grouped: size K / dtype mismatch")
    out = torch.empty((n_rows, n // 2 if gated else n), dtype=out_dtype, device=x.device)
    check(lib().zls_gemm_nt_grouped(_p(x), _i(x.stride(0)), _p(x_rows), _p(w), _p(tiles), _i(max_tiles), _i(tile_m), _p(row_expert), _i(n_rows), _p(out),
                                    _i(out.shape[1]), _i(n), _i(k), C.c_int(int(gated)), C.c_int(dt_code(x.dtype)), C.c_int(dt_code(out_dtype)),
                                    C.c_int(ACT_KINDS[act]), _f(act_alpha), _f(act_limit), _stream()), "gemm_nt_grouped")
    return out


def silu_mul(gu, dtype):
    _cuda(gu)
    _f32(gu)
    rows, two_ff = gu.shape
    out = torch.empty((rows, two_ff // 2), dtype=dtype, device=gu.device)
    check(lib().zls_silu_mul(_p(gu), _i(rows), _i(two_ff // 2), _p(out), C.c_int(dt_code(dtype)), _stream()), "silu_mul")
    return out


def act_mul(gu, dtype, kind="silu", alpha=1.0, limit=0.0, block=0):
    """act(gate, up) of fp32 rows [gates | ups] (block 0) or blocks of `block` gates followed by their ups; see ACT_KINDS"""
    _cuda(gu)
    _f32(gu)
    rows, two_ff = gu.shape
    out = torch.empty((rows, two_ff // 2), dtype=dtype, device=gu.device)
    check(lib().zls_act_mul(_p(gu), _i(rows), _i(two_ff // 2), C.c_int(ACT_KINDS[kind]), _f(alpha), _f(limit), _i(block), _p(out),
                            C.c_int(dt_code(dtype)), _stream()), "act_mul")
    return out


def moe_combine(y, slot_pos, ids, weights, h, n_experts):
    _cuda(y, slot_pos, ids, weights, h)
    _f32(y, weights)
    n_tok, top = ids.shape
    out = torch.empty((n_tok, h.shape[1]), dtype=torch.float32, device=h.device)
    check(lib().zls_moe_combine(_p(y), _p(slot_pos), _p(ids), _p(weights), _p(h), _i(n_tok), _i(top), _i(n_experts), _i(h.shape[1]), _p(out),
                                C.c_int(dt_code(h.dtype)), _stream()), "moe_combine")
    return out
