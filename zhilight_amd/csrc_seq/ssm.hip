// ssm.hip -- the state-space (Mamba-2) mixer's steps over a ragged step: causal short convolution + SiLU with a carried tail, the
// selective recurrence with its fp32 state carried per sequence slot, the gated grouped RMS norm.
//
// k_conv_silu         a thread per (token, channel); taps before the portion come from the slot's tail (oldest row first)
// k_conv_tail_update  after it: a thread per (sequence, channel) shifts the tail by the portion's length (rows in increasing order, each
//                     read before it is overwritten)
// k_ssm_scan          a workgroup per (sequence, head); the state in registers, tokens staged through LDS 16 at a time and walked in order;
//                     dt, the decay and the state are fp32.  The same kernel runs linear attention with a scalar decay per head and token
//                     (zls_decay_scan: x = v, B = k, C = q from columns of one projection, the decay and input scale given per token or
//                     constant per head, optionally one more value column of ones that carries the normaliser).
// k_gated_group_norm  y * silu(z), then each of the row's equal parts divided by its own root mean square, times the weight
#include "seq_common.h"

namespace {

// in_bias (nullable) is added to every INPUT of the convolution (the tail holds inputs with it; before a sequence's start the input is 0,
// not the bias); act 0 leaves out the SiLU
__global__ __launch_bounds__(256) void k_conv_silu(const float* __restrict__ proj, int64_t ld, int col0, const float* __restrict__ w,
                                                   const float* __restrict__ bias, const float* __restrict__ in_bias, int act,
                                                   const float* __restrict__ tail, int channels, int taps, const zls_batch_t b,
                                                   float* __restrict__ out) {
    const int t = blockIdx.x;
    const int sq = b.tok_seq[t];
    const int first = b.seq_start[sq];
    const int i = t - first;                                           // index inside the portion
    const float* tl = tail + (size_t)b.seq_slot[sq] * (taps - 1) * channels;
    for (int c = blockIdx.y * 256 + threadIdx.x; c < channels; c += gridDim.y * 256) {
        float a = bias ? bias[c] : 0.f;
        const float ib = in_bias ? in_bias[c] : 0.f;
        for (int k = 0; k < taps; ++k) {
            const int back = taps - 1 - k;                             // the last column is the current token's
            const int src = i - back;
            const float u = src >= 0 ? proj[(size_t)(first + src) * ld + col0 + c] + ib
                                     : tl[(size_t)(taps - 1 + src) * channels + c];     // src = -1 is the newest tail row
            a = fmaf(w[(size_t)c * taps + k], u, a);
        }
        out[(size_t)t * channels + c] = act ? seq_silu(a) : a;
    }
}

__global__ __launch_bounds__(256) void k_conv_tail_update(const float* __restrict__ proj, int64_t ld, int col0, const float* __restrict__ in_bias,
                                                          float* __restrict__ tail, int channels, int taps, const zls_batch_t b) {
    const int sq = blockIdx.x;
    const int first = b.seq_start[sq], count = b.seq_start[sq + 1] - first;
    float* tl = tail + (size_t)b.seq_slot[sq] * (taps - 1) * channels;
    for (int c = blockIdx.y * 256 + threadIdx.x; c < channels; c += gridDim.y * 256) {
        for (int j = 0; j < taps - 1; ++j) {                           // new row j = input at portion index count - (taps - 1) + j
            const int src = count - (taps - 1) + j;
            tl[(size_t)j * channels + c] = src >= 0 ? proj[(size_t)(first + src) * ld + col0 + c] + (in_bias ? in_bias[c] : 0.f)
                                                    : tl[(size_t)(taps - 1 + src) * channels + c];   // an older row j + count > j
        }
    }
}

struct ScanP {
    const float* xbc; const float* proj; const float* dt_bias; const float* a_log; const float* d; float* state; float* y;
    int64_t ld;
    int dt_col0, heads, vdim, n_state, groups, ngl, npt, kp;
    // long portions in segments: mode 0 = the whole portion in one workgroup; 1 = a segment from a ZERO state, leaving its end state and the
    // product of its decays (no y); 2 = a segment from its true start state (seg_init, or the slot's state for segment 0), writing y
    int mode, seg_len, n_seg;
    float* seg_state; float* seg_prod; float* seg_init;      // (n_seq, n_seg, heads, n_state, vdim) | (n_seq, n_seg, heads) | like seg_state
    // kind 0: the Mamba-2 sources above.  kind 1: linear attention with a scalar decay -- the staged row [v | k | q] comes from columns of
    // `proj` (x = v, B = k, C = q, each head its own), through SiLU when act is set; the input scale is gain_t[t][h] (or 1), the decay
    // decay_t[t][h] (or the constant decay_h[h]); with `ones` the last of the vdim columns is not loaded but 1 for every token
    int kind, act, ones, q_col0, k_col0, v_col0;
    int cols;                                                // value columns per workgroup (all of them, or a part: blockIdx.z picks it)
    const float* decay_h; const float* decay_t; const float* gain_t;
    // vec: the decay is a VECTOR per token, one number per state row (key channel): decay_v (n_tok, heads * n_state) fp32.  The staged row
    // gets a third run [.. | a] laid out like B and C; a segment's decay product is then a vector too (k_seg_decay_prod), seg_prod
    // (n_seq, n_seg, heads, n_state)
    int vec; const float* decay_v;
};

constexpr int kScanSlots = 32;

// thread = (column p of the head's state, g of ngl adjacent lanes): it keeps S[n][p] for the npt <= NPT states n = g * npt .. in registers.
// Tokens go through LDS a chunk at a time, one row [x (vdim) | B (n_state) | C (n_state)] each, plus dt and the decay exp(-e^a_log dt).
// The NEXT chunk's global loads are issued into registers (kScanSlots per thread: slot u = token u / kp, column tid + (u % kp) * threads)
// before the current chunk is walked, and stored to LDS after it: the walk itself has no barrier and waits for no memory -- y_p needs
// only a butterfly over the ngl lanes of the column.
template <int NPT, int MAXT>
__global__ __launch_bounds__(MAXT) void k_ssm_scan(const ScanP p, const zls_batch_t b) {
    extern __shared__ float lds[];
    const int NR = 2 + p.vec;                      // runs of n_state numbers behind x in a staged row
    const int P = p.vdim, N = p.n_state, W = P + NR * N, KP = p.kp, CH = kScanSlots / KP;
    // a staged row in LDS: [x, padded to 4 | B: ngl groups of npt (+ 4 unused) | C: the same]: a thread's states are 16-byte aligned runs, the
    // runs of the ngl lanes of a column start 4 banks apart; everything no token writes (n >= N, the padding) is zero for good
    const int P4 = (P + 3) & ~3, GS = p.npt + 4, WL = P4 + NR * p.ngl * GS;
    float* rows = lds;                             // [CH][WL]
    float* dts = lds + CH * WL;                    // [CH] dt | [CH] decay
    for (int i = threadIdx.x; i < CH * WL; i += blockDim.x) rows[i] = 0.f;
    const int sq = blockIdx.x / p.n_seg, seg = blockIdx.x % p.n_seg, h = blockIdx.y, tid = threadIdx.x, nthr = blockDim.x;
    // (columns never meet in the recurrence: wide heads are cut into column parts, each workgroup stages the whole token row and keeps
    // the states of its own columns)
    const int pp = blockIdx.z * p.cols + tid / p.ngl, g = tid % p.ngl;
    const bool active = tid / p.ngl < p.cols && pp < P;
    const bool lin = p.kind == 1;
    const int grp = lin ? 0 : h / (p.heads / p.groups);
    const int inner = p.heads * P, chan = lin ? (int)p.ld : inner + 2 * p.groups * N;
    const float* srcbase = lin ? p.proj : p.xbc;
    const int whole = b.seq_start[sq + 1] - b.seq_start[sq];
    if (seg * p.seg_len >= whole) return;                               // (workgroup-uniform)
    const int first = b.seq_start[sq] + seg * p.seg_len, count = min(p.seg_len, whole - seg * p.seg_len);
    const bool last_seg = (seg + 1) * p.seg_len >= whole;
    if (p.mode == 1 && last_seg) return;                                // nobody starts from the last segment's end state
    float* st = p.state + ((size_t)b.seq_slot[sq] * p.heads + h) * N * P;
    const size_t seg_at = ((size_t)sq * p.n_seg + seg) * p.heads + h;
    const float* init = (p.mode == 2 && seg > 0) ? p.seg_init + seg_at * N * P : st;
    float S[NPT];
#pragma unroll
    for (int j = 0; j < NPT; ++j) {
        const int n = g * p.npt + j;
        S[j] = (p.mode != 1 && active && j < p.npt && n < N) ? init[(size_t)n * P + pp] : 0.f;
    }
    float prod = 1.0f;
    const float rate = lin ? 0.f : expf(p.a_log[h]), bias = lin ? 0.f : p.dt_bias[h], dskip = lin ? 0.f : p.d[h];
    const float dec_h = (lin && !p.decay_t && p.decay_h) ? p.decay_h[h] : 1.0f;
    // slot u of a thread = (token u / KP of the chunk, column e = tid + (u % KP) * threads of the staged row): where it comes from inside
    // xbc and where it goes in LDS is the same for every chunk, so both offsets are worked out once (a wave64 VALU instruction costs four
    // cycles and this loop runs at one wave per SIMD: index arithmetic per chunk would cost more than the recurrence itself)
    int src_off[kScanSlots], dst_off[kScanSlots];
    uint32_t from_dec = 0;                         // bit u: slot u is read from decay_v (rows of heads * N numbers)
#pragma unroll
    for (int u = 0; u < kScanSlots; ++u) {
        const int i = u / KP, e = tid + (u % KP) * nthr;
        int col = lin ? p.v_col0 + h * (P - p.ones) + e : h * P + e, at = e;
        if (e >= P) {
            const int n = (e - P) % N, half = (e - P) / N;
            col = lin ? (half ? p.q_col0 : p.k_col0) + h * N + n : inner + (half * p.groups + grp) * N + n;
            at = P4 + half * p.ngl * GS + (n / p.npt) * GS + n % p.npt;
            if (half == 2 && e < W) { from_dec |= 1u << u; col = i * (p.heads * N - chan) + h * N + n; }     // (i * chan is added below)
        }
        src_off[u] = e < W ? ((lin && p.ones && e == P - 1) ? -2 : i * chan + col) : -1;      // -2: the column of ones
        dst_off[u] = i * WL + at;
    }
    float pre[kScanSlots], pre_dt = 0.f, pre_dec = 0.f;
    auto fetch = [&](int c0) {
        const int cn = min(CH, count - c0);
        const float* base = srcbase + (size_t)(first + c0) * chan;
        const float* dbase = p.vec ? p.decay_v + (size_t)(first + c0) * p.heads * N : base;
#pragma unroll
        for (int u = 0; u < kScanSlots; ++u)
            pre[u] = (u < cn * KP && src_off[u] >= 0) ? ((from_dec >> u & 1u) ? dbase[src_off[u]] : base[src_off[u]]) : 1.0f;
        if (tid < cn) {
            if (lin) {
                const size_t at = (size_t)(first + c0 + tid) * p.heads + h;
                pre_dt = p.gain_t ? p.gain_t[at] : 1.0f;
                pre_dec = p.decay_t ? p.decay_t[at] : dec_h;
            } else {
                pre_dt = p.proj[(size_t)(first + c0 + tid) * p.ld + p.dt_col0 + h];
            }
        }
    };
    auto publish = [&](int c0) {
        const int cn = min(CH, count - c0);
#pragma unroll
        for (int u = 0; u < kScanSlots; ++u)
            if (u < cn * KP && src_off[u] != -1) rows[dst_off[u]] = (p.act && src_off[u] >= 0 && !(from_dec >> u & 1u)) ? seq_silu(pre[u]) : pre[u];
        if (tid < cn) {
            if (lin) {
                dts[tid] = pre_dt;
                dts[CH + tid] = pre_dec;
            } else {
                const float dt = seq_softplus(pre_dt + bias);
                dts[tid] = dt;
                dts[CH + tid] = expf(-rate * dt);
            }
        }
    };
    fetch(0);
    for (int c0 = 0; c0 < count; c0 += CH) {
        const int cn = min(CH, count - c0);
        __syncthreads();                           // the previous chunk is consumed
        publish(c0);
        __syncthreads();
        if (c0 + CH < count) fetch(c0 + CH);       // in flight during the walk
        if (active) {
            for (int i = 0; i < cn; ++i) {
                const float dt = dts[i], decay = dts[CH + i];
                prod *= decay;
                const float* row = rows + i * WL;
                const float xv = row[pp];
                const float dx = dt * xv;
                const float4* Bv = reinterpret_cast<const float4*>(row + P4 + g * GS);
                const float4* Cv = reinterpret_cast<const float4*>(row + P4 + (p.ngl + g) * GS);
                const float4* Av = reinterpret_cast<const float4*>(row + P4 + (2 * p.ngl + g) * GS);      // (read only with vec)
                float part0 = 0.f, part1 = 0.f;
#pragma unroll
                for (int j = 0; j < NPT; j += 4) {
                    if (j < p.npt) {                               // (npt is a multiple of 4; states past N see B = C = 0 and stay 0)
                        const float4 bq = Bv[j >> 2], cq = Cv[j >> 2];
                        const float4 aq = p.vec ? Av[j >> 2] : make_float4(decay, decay, decay, decay);
                        S[j] = fmaf(aq.x, S[j], bq.x * dx);
                        S[j + 1] = fmaf(aq.y, S[j + 1], bq.y * dx);
                        S[j + 2] = fmaf(aq.z, S[j + 2], bq.z * dx);
                        S[j + 3] = fmaf(aq.w, S[j + 3], bq.w * dx);
                        part0 = fmaf(S[j], cq.x, part0);
                        part1 = fmaf(S[j + 1], cq.y, part1);
                        part0 = fmaf(S[j + 2], cq.z, part0);
                        part1 = fmaf(S[j + 3], cq.w, part1);
                    }
                }
                float part = part0 + part1;
                for (int off = 1; off < p.ngl; off <<= 1) part += __shfl_xor(part, off, 64);
                if (g == 0 && p.mode != 1) p.y[(size_t)(first + c0 + i) * inner + h * P + pp] = fmaf(dskip, xv, part);
            }
        }
    }
    if (!active) return;
    if (p.mode == 2 && !last_seg) return;                               // only the portion's last segment leaves the slot's state
    float* dst = p.mode == 1 ? p.seg_state + seg_at * N * P : st;
#pragma unroll
    for (int j = 0; j < NPT; ++j) {
        const int n = g * p.npt + j;
        if (j < p.npt && n < N) dst[(size_t)n * P + pp] = S[j];
    }
    if (p.mode == 1 && tid == 0 && !p.vec) p.seg_prod[seg_at] = prod;
}

// vector decays: the product of a segment's decays per (sequence, segment, head, state row); the last segment needs none.  The 1024 threads
// are (row, part of the segment's tokens): every part multiplies its tokens in order, the parts meet in LDS and are multiplied in order
__global__ __launch_bounds__(1024) void k_seg_decay_prod(const ScanP p, const zls_batch_t b) {
    __shared__ float part[1024];
    const int sq = blockIdx.x / p.n_seg, seg = blockIdx.x % p.n_seg, h = blockIdx.y, N = p.n_state;
    const int whole = b.seq_start[sq + 1] - b.seq_start[sq];
    if ((seg + 1) * p.seg_len >= whole) return;
    const int first = b.seq_start[sq] + seg * p.seg_len;
    const size_t seg_at = ((size_t)sq * p.n_seg + seg) * p.heads + h;
    int rows = 1;
    while (rows < N && rows < 1024) rows <<= 1;                           // rows per pass (a power of two), 1024 / rows parts
    const int parts = 1024 / rows, r = threadIdx.x % rows, j = threadIdx.x / rows;
    const int per = (p.seg_len + parts - 1) / parts, t0 = j * per, t1 = min(p.seg_len, t0 + per);
    for (int n0 = 0; n0 < N; n0 += rows) {
        const int n = n0 + r;
        float prod = 1.0f;
        if (n < N) {
            const float* a = p.decay_v + (size_t)first * p.heads * N + (size_t)h * N + n;
            for (int i = t0; i < t1; ++i) prod *= a[(size_t)i * p.heads * N];
        }
        part[threadIdx.x] = prod;
        __syncthreads();
        if (j == 0 && n < N) {
            for (int q = 1; q < parts; ++q) prod *= part[q * rows + r];
            p.seg_prod[seg_at * N + n] = prod;
        }
        __syncthreads();
    }
}

// start states of the segments 1 .. of every long portion: S_{k+1} = (product of segment k's decays) S_k + (segment k's end state from zero),
// S_0 = the slot's state.  One workgroup per (sequence, head), threads over the state's elements, segments in order.
__global__ __launch_bounds__(256) void k_ssm_seg_combine(const ScanP p, const zls_batch_t b) {
    const int sq = blockIdx.x, h = blockIdx.y;
    const int whole = b.seq_start[sq + 1] - b.seq_start[sq];
    const int nseg = (whole + p.seg_len - 1) / p.seg_len;
    const int NPs = p.n_state * p.vdim;
    const float* st = p.state + ((size_t)b.seq_slot[sq] * p.heads + h) * NPs;
    for (int e = blockIdx.z * 256 + threadIdx.x; e < NPs; e += gridDim.z * 256) {     // (few heads: the state's elements fill the chip instead)
        float S = st[e];
        for (int k = 0; k + 1 < nseg; ++k) {
            const size_t at = ((size_t)sq * p.n_seg + k) * p.heads + h;
            S = fmaf(p.vec ? p.seg_prod[at * p.n_state + e / p.vdim] : p.seg_prod[at], S, p.seg_state[at * NPs + e]);
            p.seg_init[(at + p.heads) * NPs + e] = S;                   // segment k + 1 of the same sequence and head
        }
    }
}

template <int DT>
__global__ __launch_bounds__(256) void k_gated_group_norm(const float* __restrict__ y, const float* __restrict__ proj, int64_t ld, int z_col0,
                                                          const float* __restrict__ weight, float eps, int inner, int part,
                                                          void* __restrict__ out) {
    __shared__ float red[16];
    const int t = blockIdx.x, c0 = blockIdx.y * part;
    const float* yr = y + (size_t)t * inner + c0;
    const float* zr = proj + (size_t)t * ld + z_col0 + c0;
    float ss = 0.f;
    for (int i = threadIdx.x; i < part; i += 256) { const float v = yr[i] * seq_silu(zr[i]); ss = fmaf(v, v, ss); }
    ss = zl_block_sum(ss, red);
    const float f = 1.0f / sqrtf(ss / (float)part + eps);
    for (int i = threadIdx.x; i < part; i += 256)
        SeqT<DT>::st(out, (size_t)t * inner + c0 + i, yr[i] * seq_silu(zr[i]) * f * weight[c0 + i]);
}

}  // namespace

extern "C" int zls_short_conv(const float* proj, int64_t ld, int64_t col0, const float* w, const float* bias, const float* in_bias, int act,
                              const float* tail, int64_t channels, int64_t taps, const zls_batch_t* b, float* out, zl_stream_t s) {
    ZL_CHECK_ARG(proj && w && out && seq_batch_ok(b) && channels > 0 && taps > 0 && (tail || taps == 1), ZL_EINVAL);
    ZL_CHECK_ARG(col0 >= 0 && col0 + channels <= ld, ZL_ESHAPE);
    const unsigned gy = (unsigned)((channels + 255) / 256 > 64 ? 64 : (channels + 255) / 256);
    hipLaunchKernelGGL(k_conv_silu, dim3(b->n_tok, gy), dim3(256), 0, (hipStream_t)s, proj, ld, (int)col0, w, bias, in_bias, act ? 1 : 0, tail,
                       (int)channels, (int)taps, *b, out);
    return zl_launch_status();
}

extern "C" int zls_conv_silu(const float* proj, int64_t ld, int64_t col0, const float* w, const float* bias, const float* tail, int64_t channels,
                             int64_t taps, const zls_batch_t* b, float* out, zl_stream_t s) {
    return zls_short_conv(proj, ld, col0, w, bias, nullptr, 1, tail, channels, taps, b, out, s);
}

extern "C" int zls_short_conv_tail(const float* proj, int64_t ld, int64_t col0, const float* in_bias, float* tail, int64_t channels, int64_t taps,
                                   const zls_batch_t* b, zl_stream_t s) {
    ZL_CHECK_ARG(proj && seq_batch_ok(b) && channels > 0 && taps > 0, ZL_EINVAL);
    ZL_CHECK_ARG(col0 >= 0 && col0 + channels <= ld, ZL_ESHAPE);
    if (taps == 1) return ZL_OK;
    ZL_CHECK_ARG(tail, ZL_EINVAL);
    const unsigned gy = (unsigned)((channels + 255) / 256 > 64 ? 64 : (channels + 255) / 256);
    hipLaunchKernelGGL(k_conv_tail_update, dim3(b->n_seq, gy), dim3(256), 0, (hipStream_t)s, proj, ld, (int)col0, in_bias, tail, (int)channels,
                       (int)taps, *b);
    return zl_launch_status();
}

extern "C" int zls_conv_tail_update(const float* proj, int64_t ld, int64_t col0, float* tail, int64_t channels, int64_t taps, const zls_batch_t* b,
                                    zl_stream_t s) {
    return zls_short_conv_tail(proj, ld, col0, nullptr, tail, channels, taps, b, s);
}

extern "C" int64_t zls_ssm_scan_workspace_bytes(int64_t n_seq, int64_t max_count, int64_t seg_len, int64_t heads, int64_t vdim, int64_t n_state) {
    if (n_seq <= 0 || max_count <= 0 || seg_len <= 0 || heads <= 0 || vdim <= 0 || n_state <= 0) return ZL_EINVAL;
    const int64_t n_seg = (max_count + seg_len - 1) / seg_len;
    return n_seq * n_seg * heads * (2 * n_state * vdim + n_state + 1) * (int64_t)sizeof(float);      /* (room for a decay product per state row) */
}

// sizes the thread layout for (heads, vdim, n_state) in p and launches the scan (whole portions, or long ones in segments)
static int launch_scan(ScanP& p, int64_t heads, int64_t vdim, int64_t n_state, const zls_batch_t* b, void* workspace, int64_t seg_len,
                       zl_stream_t s) {
    ZL_CHECK_ARG(heads > 0 && vdim > 0 && n_state > 0 && heads <= 65535 && vdim <= 1024, ZL_ESHAPE);
    // ngl lanes share a column: the smallest power of two that leaves a thread at most 32 states
    int64_t ngl = 1;
    while ((n_state + ngl - 1) / ngl > 32) ngl <<= 1;
    ZL_CHECK_ARG(ngl <= 64, ZL_ELIMIT);
    const int64_t cols = ngl * vdim <= 1024 ? vdim : 1024 / ngl, col_parts = (vdim + cols - 1) / cols;
    p.cols = (int)cols;
    const int64_t npt = ((n_state + ngl - 1) / ngl + 3) / 4 * 4;
    const int64_t threads = (ngl * cols + 63) / 64 * 64;
    p.heads = (int)heads; p.vdim = (int)vdim; p.n_state = (int)n_state;
    p.ngl = (int)ngl; p.npt = (int)npt;
    const int64_t runs = 2 + (p.vec ? 1 : 0);
    const int64_t row = vdim + runs * n_state;
    int64_t kp = (row + threads - 1) / threads;                        // register slots a staged token row takes per thread
    const size_t row_bytes = (size_t)((vdim + 3) / 4 * 4 + runs * ngl * (npt + 4) + 2) * sizeof(float);
    while (kp < kScanSlots && (kScanSlots / kp) * row_bytes > 64 * 1024) ++kp;      // long rows: fewer tokens staged at a time
    ZL_CHECK_ARG(kp <= kScanSlots, ZL_ELIMIT);
    p.kp = (int)kp;
    const size_t lds = (kScanSlots / kp) * row_bytes;
    ZL_CHECK_ARG(lds <= 64 * 1024, ZL_ELIMIT);
    // portions longer than seg_len (with a workspace): every segment from a zero state in parallel, the segments' start states by a short
    // serial pass over their end states, then every segment again from its true start state -- twice the arithmetic, 1 / segments of the
    // serial length
    const bool segmented = workspace && seg_len > 0 && b->max_count > seg_len;
    const int64_t n_seg = segmented ? (b->max_count + seg_len - 1) / seg_len : 1;
    p.seg_len = segmented ? (int)seg_len : b->max_count;
    p.n_seg = (int)n_seg;
    const int64_t per = (int64_t)b->n_seq * n_seg * heads;
    p.seg_state = (float*)workspace;
    p.seg_init = p.seg_state + per * n_state * vdim;
    p.seg_prod = p.seg_init + per * n_state * vdim;
    ZL_CHECK_ARG((int64_t)b->n_seq * n_seg <= 0x7fffffff, ZL_ELIMIT);
    const dim3 grid((unsigned)(b->n_seq * n_seg), (unsigned)heads, (unsigned)col_parts), block((unsigned)threads);
    hipStream_t hs = (hipStream_t)s;
    // (up to 256 threads the compiler may use the whole register file for the state and the prefetched chunk, up to 512 half of it: the
    // 32 states, 32 prefetched numbers and 64 offsets of a thread still fit without scratch memory)
#define SCAN(NPT)                                                                                        \
    if (threads <= 256) hipLaunchKernelGGL((k_ssm_scan<NPT, 256>), grid, block, lds, hs, p, *b);         \
    else if (threads <= 512) hipLaunchKernelGGL((k_ssm_scan<NPT, 512>), grid, block, lds, hs, p, *b);    \
    else if (threads <= 640) hipLaunchKernelGGL((k_ssm_scan<NPT, 640>), grid, block, lds, hs, p, *b);    \
    else hipLaunchKernelGGL((k_ssm_scan<NPT, 1024>), grid, block, lds, hs, p, *b);
#define SCAN_ANY if (npt <= 8) { SCAN(8) } else if (npt <= 16) { SCAN(16) } else { SCAN(32) }
    if (!segmented) {
        p.mode = 0;
        SCAN_ANY
    } else {
        p.mode = 1;
        SCAN_ANY
        if (p.vec) hipLaunchKernelGGL(k_seg_decay_prod, dim3((unsigned)(b->n_seq * n_seg), (unsigned)heads), dim3(1024), 0, hs, p, *b);
        const int64_t want_z = (1024 + b->n_seq * heads - 1) / (b->n_seq * heads), have_z = (n_state * vdim + 255) / 256;
        hipLaunchKernelGGL(k_ssm_seg_combine, dim3(b->n_seq, (unsigned)heads, (unsigned)(want_z < have_z ? want_z : have_z)), dim3(256), 0, hs, p, *b);
        p.mode = 2;
        SCAN_ANY
    }
#undef SCAN_ANY
#undef SCAN
    return zl_launch_status();
}

extern "C" int zls_ssm_scan(const float* xbc, const float* proj, int64_t ld, int64_t dt_col0, const float* dt_bias, const float* a_log,
                            const float* d, float* state, int64_t heads, int64_t vdim, int64_t n_state, int64_t groups, const zls_batch_t* b,
                            float* y, void* workspace, int64_t seg_len, zl_stream_t s) {
    ZL_CHECK_ARG(xbc && proj && dt_bias && a_log && d && state && y && seq_batch_ok(b), ZL_EINVAL);
    ZL_CHECK_ARG(heads > 0 && groups > 0 && heads % groups == 0, ZL_ESHAPE);
    ZL_CHECK_ARG(dt_col0 >= 0 && dt_col0 + heads <= ld, ZL_ESHAPE);
    ScanP p = {};
    p.xbc = xbc; p.proj = proj; p.dt_bias = dt_bias; p.a_log = a_log; p.d = d; p.state = state; p.y = y; p.ld = ld;
    p.dt_col0 = (int)dt_col0; p.groups = (int)groups;
    return launch_scan(p, heads, vdim, n_state, b, workspace, seg_len, s);
}

extern "C" int zls_decay_scan(const float* proj, int64_t ld, int64_t q_col0, int64_t k_col0, int64_t v_col0, int act, const float* decay_h,
                              const float* decay_t, const float* gain_t, int norm_col, float* state, int64_t heads, int64_t dim, int64_t vdim,
                              const zls_batch_t* b, float* y, void* workspace, int64_t seg_len, const float* decay_v, zl_stream_t s) {
    ZL_CHECK_ARG(proj && (decay_h || decay_t || decay_v) && state && y && seq_batch_ok(b) && heads > 0 && dim > 0 && vdim > 0, ZL_EINVAL);
    ZL_CHECK_ARG(!decay_v || (!decay_h && !decay_t && heads * dim * (int64_t)kScanSlots < (1LL << 31)), ZL_EINVAL);
    ZL_CHECK_ARG(q_col0 >= 0 && q_col0 + heads * dim <= ld && k_col0 >= 0 && k_col0 + heads * dim <= ld && v_col0 >= 0 &&
                 v_col0 + heads * vdim <= ld && ld * kScanSlots < (1LL << 31), ZL_ESHAPE);
    ScanP p = {};
    p.proj = proj; p.state = state; p.y = y; p.ld = ld; p.groups = (int)heads;
    p.kind = 1; p.act = act ? 1 : 0; p.ones = norm_col ? 1 : 0; p.q_col0 = (int)q_col0; p.k_col0 = (int)k_col0; p.v_col0 = (int)v_col0;
    p.decay_h = decay_h; p.decay_t = decay_t; p.gain_t = gain_t; p.vec = decay_v ? 1 : 0; p.decay_v = decay_v;
    return launch_scan(p, heads, vdim + p.ones, dim, b, workspace, seg_len, s);
}

extern "C" int zls_gated_group_norm(const float* y, const float* proj, int64_t ld, int64_t z_col0, const float* weight, float eps, int64_t rows,
                                    int64_t inner, int64_t norm_groups, void* out, int dtype, zl_stream_t s) {
    ZL_CHECK_ARG(y && proj && weight && out && rows > 0 && inner > 0 && norm_groups > 0, ZL_EINVAL);
    ZL_CHECK_ARG(inner % norm_groups == 0 && z_col0 >= 0 && z_col0 + inner <= ld && norm_groups <= 65535, ZL_ESHAPE);
    const int part = (int)(inner / norm_groups);
#define CALL(DT) hipLaunchKernelGGL((k_gated_group_norm<DT>), dim3((unsigned)rows, (unsigned)norm_groups), dim3(256), 0, (hipStream_t)s, y, proj, ld, \
                                    (int)z_col0, weight, eps, (int)inner, part, out);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}
