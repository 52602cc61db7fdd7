// latent_attn.hip -- attention over a PAGED cache of normed low-rank latents, for every token of a ragged step.
//
// Beside csrc/mla_attn.hip (DeepSeek's geometry: 512 + 64 rotated columns, 16-bit, decode rows only, no sink): any rank / head sizes, a
// learned per-head sink in the softmax denominator, a per-head sigmoid output gate, causal portions of prompts at any offset, an optional
// sliding window, and a 32-bit mode.  Only the latent is cached; for single tokens keys and values are never materialised:
//     score_j = (W_uk,h^T q_h) . c_j * scale          o_h = W_uv,h . (sum_j w_j c_j)
// A rotated key part shared by all heads rides in the same cached row behind the latent: the row is [c | k_rot], the up-projections get
// identity columns for it (W_uk) or zeros (W_uv) on the host, and every kernel below sees one longer "latent".
// k_latent_store        RMS norm (plain weight) of the down-projection -> the token's cache row; the rotated key part behind it and the
//                       queries' rotated parts (in place), turned by the token's position
// k_latent_absorb       the query folded through W_uk (and the scale), once per token and head
// k_latent_split        single tokens (and, in 32-bit serving, every token): the keys split over workgroups, fp32 VALU
// k_latent_decode_mfma  the same split pass for bf16 on the matrix cores
// k_latent_combine      merges the splits with the sink (it counts once, unscaled, with no value), applies W_uv and the gate
// k_latent_fa           portions of prompts in bf16 on the matrix cores, over keys and values up-projected for the step
#include "seq_common.h"

namespace {

// rot > 0: the down-projection has rot more columns behind the latent, one rotated key part for all heads: pair (2i, 2i + 1) (interleaved)
// or (i, i + rot / 2) is turned by pos * freq[i] and stored behind the normed latent (cache rows hold rank + rot numbers); the last rot
// coordinates of every query head (q_col0, heads x qdim) are turned the same way in place.  A thread owns a whole pair.
template <int DT>
__global__ __launch_bounds__(256) void k_latent_store(float* __restrict__ proj, int64_t ld, int col0, const float* __restrict__ weight,
                                                      float eps, int rank, int rot, const float* __restrict__ freq, int interleaved, int q_col0,
                                                      int heads, int qdim, const zls_batch_t b, void* __restrict__ cache, float rot_gain) {
    __shared__ float red[16];
    const int t = blockIdx.x;
    const int sq = b.tok_seq[t];
    const int pos = b.seq_pos0[sq] + (t - b.seq_start[sq]);
    const int page = b.page_table[(size_t)sq * b.max_pages + pos / b.page_size];
    const size_t dst = ((size_t)page * b.page_size + pos % b.page_size) * (rank + rot);
    float* row = proj + (size_t)t * ld;
    const float* u = row + col0;
    float ss = 0.f;
    for (int i = threadIdx.x; i < rank; i += 256) ss = fmaf(u[i], u[i], ss);
    ss = zl_block_sum(ss, red);
    const float f = 1.0f / sqrtf(ss / (float)rank + eps);
    for (int i = threadIdx.x; i < rank; i += 256) SeqT<DT>::st(cache, dst + i, u[i] * f * weight[i]);
    const int half = rot >> 1;
    for (int w = threadIdx.x; w < (heads + 1) * half; w += 256) {          // vector 0: the key part; 1 ..: the heads' query parts
        const int vec = w / half, i = w % half;
        const int a = interleaved ? 2 * i : i, c = interleaved ? 2 * i + 1 : i + half;
        float sn, cs;
        seq_sincos((float)pos * freq[i], &sn, &cs);
        sn *= rot_gain; cs *= rot_gain;                                    // (rescaled frequencies come with a gain on cos and sin)
        float* src = vec == 0 ? row + col0 + rank : row + q_col0 + (size_t)(vec - 1) * qdim + (qdim - rot);
        const float x = src[a], y = src[c];
        const float xr = x * cs - y * sn, yr = y * cs + x * sn;
        if (vec == 0) { SeqT<DT>::st(cache, dst + rank + a, xr); SeqT<DT>::st(cache, dst + rank + c, yr); }
        else { src[a] = xr; src[c] = yr; }
    }
}

struct AttnP {
    const float* q; const float* gate; const void* w_uk; const void* w_uv; const float* sink; const void* cache; void* out;
    int64_t ldq, ldg;
    int q_col0, g_col0, heads, dim, vdim, rank, single_only, vec;
    float scale;
    int window;                                    // > 0: a token at position p sees the keys p - window < j <= p only
};

// Split over keys: workgroup = (token, group of 4 heads, split), a wave per head.  A tile of 16 cached rows is staged once in LDS as fp32
// (row stride rank + 4) and shared by the four heads.  Scores: lane = (key, quarter of the latent columns), two butterflies; weighted sum:
// a lane owns the latent columns lane, lane + 64, ... (RPL of them, in registers).  Every split leaves (max, denominator, sums) in the
// workspace; k_latent_combine merges them WITH the sink (m = max(sink, m_i), l = e^(sink - m) + sum l_i e^(m_i - m)), applies W_uv and the
// gate.  LDS: ct[16][rank + 4] | qk[4][rank]
// q'_h = scale * W_uk,h^T q_h, once per (token, head): workgroup = 64 latent columns (lanes: coalesced rows of W_uk), the four waves
// take every fourth query dimension, eight loads in flight each; the partial sums meet in LDS.  qa (n_tok, heads, rank) fp32
template <int DT>
__global__ __launch_bounds__(256) void k_latent_absorb(const AttnP p, const zls_batch_t b, float* __restrict__ qa) {
    __shared__ float part[4][64];
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sq = b.tok_seq[t];
    if (p.single_only && b.seq_start[sq + 1] - b.seq_start[sq] > 1) return;
    const float* qh = p.q + (size_t)t * p.ldq + p.q_col0 + (size_t)h * p.dim;
    const int r = blockIdx.z * 64 + lane;
    float acc = 0.f;
    if (r < p.rank) {
        for (int d0 = wave; d0 < p.dim; d0 += 32) {
            float w[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int d = d0 + 4 * u;
                w[u] = d < p.dim ? SeqT<DT>::ld(p.w_uk, ((size_t)h * p.dim + d) * p.rank + r) : 0.f;
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int d = d0 + 4 * u;
                acc = fmaf(d < p.dim ? qh[d] : 0.f, w[u], acc);
            }
        }
    }
    part[wave][lane] = acc;
    __syncthreads();
    if (wave == 0 && r < p.rank)
        qa[((size_t)t * p.heads + h) * p.rank + r] = (part[0][lane] + part[1][lane] + part[2][lane] + part[3][lane]) * p.scale;
}

template <int DT, int RPL>
__global__ __launch_bounds__(256) void k_latent_split(const AttnP p, const zls_batch_t b, const float* __restrict__ qa, float* __restrict__ ws,
                                                      int n_splits) {
    extern __shared__ float lds[];
    const int RP = p.rank + 4;                     // rows 16-byte aligned; 4 banks between neighbouring keys
    float* ct = lds;
    float* qk = lds + 16 * RP + (threadIdx.x >> 6) * p.rank;
    const int t = blockIdx.x, split = blockIdx.z, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int h = blockIdx.y * 4 + wave;
    const bool hvalid = h < p.heads;
    const int sq = b.tok_seq[t];
    if (p.single_only && b.seq_start[sq + 1] - b.seq_start[sq] > 1) return;      // portions go to the prompt kernel (workgroup-uniform)
    const int pos = b.seq_pos0[sq] + (t - b.seq_start[sq]);
    const int key_lo = p.window > 0 ? max(0, pos - p.window + 1) : 0;
    const int nkeys = pos + 1 - key_lo;
    const int chunk = ((nkeys + n_splits - 1) / n_splits + 15) & ~15;
    const int k0 = key_lo + split * chunk, k1 = min(pos + 1, k0 + chunk);
    const int32_t* pages = b.page_table + (size_t)sq * b.max_pages;
    if (hvalid)
        for (int r = lane; r < p.rank; r += 64) qk[r] = qa[((size_t)t * p.heads + h) * p.rank + r];
    float acc[RPL];
#pragma unroll
    for (int i = 0; i < RPL; ++i) acc[i] = 0.f;
    float m = -INFINITY, l = 0.f;
    const int key = lane & 15, quarter = lane >> 4;
    // tile fill: 16 threads per key; with aligned rows the NEXT tile's 16-byte loads are issued into registers before the current tile is
    // worked on and written to LDS after it (8 slots of 16 bytes cover rank <= 1024)
    constexpr int V = DT == ZL_BF16 ? 8 : 4;
    const int fk = threadIdx.x >> 4, fc = threadIdx.x & 15;
    uint4 raw[8];
    auto row_base = [&](int j) { return ((size_t)pages[j / b.page_size] * b.page_size + j % b.page_size) * p.rank; };
    auto prefetch = [&](int j0) {
        const int j = j0 + fk;
        if (!p.vec || j >= k1) return;
        const size_t base = row_base(j);
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int r = (fc + 16 * u) * V;
            if (r < p.rank) {
                if constexpr (DT == ZL_BF16) raw[u] = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(p.cache) + base + r);
                else raw[u] = *reinterpret_cast<const uint4*>(reinterpret_cast<const float*>(p.cache) + base + r);
            }
        }
    };
    auto publish = [&](int j0) {
        const int j = j0 + fk;
        float* dst = ct + fk * RP;
        if (j >= k1) {
            for (int r = fc; r < p.rank; r += 16) dst[r] = 0.f;
        } else if (p.vec) {
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int r = (fc + 16 * u) * V;
                if (r < p.rank) {
                    if constexpr (DT == ZL_BF16) {
                        const uint32_t w4[4] = {raw[u].x, raw[u].y, raw[u].z, raw[u].w};
                        float v[8];
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            v[2 * e] = __builtin_bit_cast(float, w4[e] << 16);
                            v[2 * e + 1] = __builtin_bit_cast(float, w4[e] & 0xffff0000u);
                        }
                        *reinterpret_cast<float4*>(dst + r) = make_float4(v[0], v[1], v[2], v[3]);
                        *reinterpret_cast<float4*>(dst + r + 4) = make_float4(v[4], v[5], v[6], v[7]);
                    } else {
                        *reinterpret_cast<uint4*>(dst + r) = raw[u];
                    }
                }
            }
        } else {
            const size_t base = row_base(j);
            for (int r = fc; r < p.rank; r += 16) dst[r] = SeqT<DT>::ld(p.cache, base + r);
        }
    };
    prefetch(k0);
    for (int j0 = k0; j0 < k1; j0 += 16) {
        __syncthreads();
        publish(j0);
        __syncthreads();
        if (j0 + 16 < k1) prefetch(j0 + 16);
        if (!hvalid) continue;
        float sc = 0.f;
        for (int r = quarter; r < p.rank; r += 4) sc = fmaf(qk[r], ct[key * RP + r], sc);    // (key, quarter): 32 banks, two lanes each
        sc += __shfl_xor(sc, 16, 64);
        sc += __shfl_xor(sc, 32, 64);
        const bool valid = j0 + key < k1;
        sc = valid ? sc : -INFINITY;
        float mx = sc;
#pragma unroll
        for (int off = 1; off < 16; off <<= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
        const float mnew = fmaxf(m, mx);                               // finite: key j0 is valid
        const float corr = expf(m - mnew);                             // m = -inf at the first tile: 0
        const float pj = valid ? expf(sc - mnew) : 0.f;
        float ps = pj;
#pragma unroll
        for (int off = 1; off < 16; off <<= 1) ps += __shfl_xor(ps, off, 64);
        l = l * corr + ps;
        m = mnew;
        float pk[16];
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) pk[kk] = __shfl(pj, kk, 64);
#pragma unroll
        for (int i = 0; i < RPL; ++i) {
            const int r = lane + 64 * i;
            if (r < p.rank) {
                float a = acc[i] * corr;
#pragma unroll
                for (int kk = 0; kk < 16; ++kk) a = fmaf(pk[kk], ct[kk * RP + r], a);
                acc[i] = a;
            }
        }
    }
    if (!hvalid) return;
    float* out = ws + (((size_t)t * p.heads + h) * n_splits + split) * (p.rank + 2);
    if (lane == 0) { out[0] = m; out[1] = l; }
#pragma unroll
    for (int i = 0; i < RPL; ++i) {
        const int r = lane + 64 * i;
        if (r < p.rank) out[2 + r] = acc[i];
    }
}

// LDS: acc[rank] | wgt[n_splits]
template <int DT>
__global__ __launch_bounds__(256) void k_latent_combine(const AttnP p, const zls_batch_t b, const float* __restrict__ ws, int n_splits) {
    extern __shared__ float lds[];
    __shared__ float red[16];
    float* wgt = lds + p.rank;
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sq = b.tok_seq[t];
    if (p.single_only && b.seq_start[sq + 1] - b.seq_start[sq] > 1) return;
    const float* part = ws + ((size_t)t * p.heads + h) * n_splits * (p.rank + 2);
    float mloc = p.sink ? p.sink[h] : -INFINITY;                       // threads along the splits: loads in parallel
    for (int s2 = threadIdx.x; s2 < n_splits; s2 += 256) mloc = fmaxf(mloc, part[(size_t)s2 * (p.rank + 2)]);
    const float m = zl_block_max(mloc, red);
    float lloc = 0.f;
    for (int s2 = threadIdx.x; s2 < n_splits; s2 += 256) {
        const float ms = part[(size_t)s2 * (p.rank + 2)];
        const float w = ms == -INFINITY ? 0.f : expf(ms - m);
        wgt[s2] = w;
        lloc = fmaf(part[(size_t)s2 * (p.rank + 2) + 1], w, lloc);
    }
    const float l = zl_block_sum(lloc, red) + (p.sink ? expf(p.sink[h] - m) : 0.f);      // (its barriers also publish wgt)
    for (int r = threadIdx.x; r < p.rank; r += 256) {
        float a = 0.f;
#pragma unroll 8
        for (int s2 = 0; s2 < n_splits; ++s2) a = fmaf(part[(size_t)s2 * (p.rank + 2) + 2 + r], wgt[s2], a);
        lds[r] = a;
    }
    __syncthreads();
    const float g = p.gate ? seq_sigmoid(p.gate[(size_t)t * p.ldg + p.g_col0 + h]) : 1.0f;
    const float inv = g / l;
    // a wave per output value, lanes along the latent (coalesced W_uv rows), four values per pass so that their loads are in flight
    // together; the workgroups of blockIdx.z share the head's outputs
    for (int d0 = (blockIdx.z * 4 + wave) * 4; d0 < p.vdim; d0 += gridDim.z * 16) {
        float a[4] = {0.f, 0.f, 0.f, 0.f};
        for (int r = lane; r < p.rank; r += 64) {
            const float c = lds[r];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (d0 + u < p.vdim) a[u] = fmaf(SeqT<DT>::ld(p.w_uv, ((size_t)h * p.vdim + d0 + u) * p.rank + r), c, a[u]);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const float v = zl_wave_sum(a[u]);
            if (lane == 0 && d0 + u < p.vdim) SeqT<DT>::st(p.out, ((size_t)t * p.heads + h) * p.vdim + d0 + u, v * inv);
        }
    }
}

// ---- prompt portions on the matrix cores (bf16 serving) -----------------------------------------------------------------------------
// Keys and values of a portion's whole context are up-projected once per step into dense K (n_ctx, heads * dim) and V^T (heads * vdim,
// n_ctx) (zls_gemm_nt_gather over the cached rows; each sequence's rows start at a multiple of 64).  A workgroup = 64 queries of one
// sequence x one head, a wave = 16 of them.  Per 64-key tile (K and V^T staged in LDS, shared by the four waves):
//   S^T (16 keys x 16 queries) = K_tile . Q^T on v_mfma_f32_16x16x32_bf16 -- a lane then holds 4 consecutive keys of ONE query; two such
//   blocks side by side are a B operand of the same instruction with the 32 keys in a permuted order, and V^T is read in that order too,
//   so the weights never travel through LDS:
//   O^T (vdim x 16 queries) += V^T_tile . P^T, with P = hi + lo (two bf16 halves: the weights keep 16 bits of mantissa).
// Scores, running maximum / denominator (starting at the sink: m = sink, l = 1) and the output sums are fp32, per lane = per query; the
// exponentials are the hardware's exp2 of the fp32 argument times log2 e (the softmax VALU work, not the MFMAs, bounds this kernel).
typedef __bf16 fa_b8 __attribute__((ext_vector_type(8)));
typedef short fa_s4 __attribute__((ext_vector_type(4)));
typedef float fa_f4 __attribute__((ext_vector_type(4)));

// a non-negative fp32 weight as two bf16 halves, hi + lo = the weight to 2^-16 relative: hi is its upper 16 bits (truncation), lo the upper
// 16 bits of the exact remainder -- three instructions where two round-to-nearest conversions cost a dozen
__device__ __forceinline__ void fa_split(float pv, uint16_t& hb, uint16_t& lb) {
    const uint32_t u = __builtin_bit_cast(uint32_t, pv);
    hb = (uint16_t)(u >> 16);
    lb = (uint16_t)(__builtin_bit_cast(uint32_t, pv - __builtin_bit_cast(float, u & 0xffff0000u)) >> 16);
}

struct FaP {
    const float* q; const float* gate; const uint16_t* k; const uint16_t* vt; const float* sink; const int32_t* ctx_start; uint16_t* out;
    int64_t ldq, ldg, ldk, ldv;
    int q_col0, g_col0, heads, dim, vdim, tiles_per_seq, vec_k;
    float scale;
    int window; const int32_t* ctx_pos0;           // window > 0: keys p - window < j <= p; ctx_pos0 (nullable: 0): the position of a sequence's
};                                                 // first up-projected row (a windowed step does not bring its whole context)

template <int DK, int DV>
__global__ __launch_bounds__(256) void k_latent_fa(const FaP p, const zls_batch_t b) {
    constexpr int KR = DK * 32 + 8, VR = 64 + 8;
    __shared__ __attribute__((aligned(16))) uint16_t Ks[64 * KR];
    __shared__ __attribute__((aligned(16))) uint16_t Vs[DV * 16 * VR];
    // (the last query tiles see the most keys: they are dispatched first, so the launch does not end on its longest workgroups)
    const int sq = blockIdx.x % b.n_seq, tile = p.tiles_per_seq - 1 - blockIdx.x / b.n_seq, h = blockIdx.y;
    const int first = b.seq_start[sq], count = b.seq_start[sq + 1] - first;
    const int cs = p.ctx_start[sq];
    if (cs < 0 || tile * 64 >= count) return;
    // positions below are counted from the sequence's first up-projected row (position c0): a key's index there is its row in K / V^T
    const int c0 = p.ctx_pos0 ? p.ctx_pos0[sq] : 0;
    const int pos0 = b.seq_pos0[sq] - c0;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nrow = lane & 15, kq = lane >> 4;
    const int qi = tile * 64 + wave * 16 + nrow;
    const bool qvalid = qi < count;
    const int qpos = pos0 + qi;
    const int j_first = p.window > 0 ? max(0, pos0 + tile * 64 - p.window + 1) & ~63 : 0;     // the tile of the oldest key the first query sees
    const int wave_last = pos0 + min(count, tile * 64 + wave * 16 + 16) - 1;       // the last key any query of this wave sees
    const int block_last = pos0 + min(count, tile * 64 + 64) - 1;

    uint4 qf[DK];
    {
        const float* qr = p.q + (size_t)(first + (qvalid ? qi : 0)) * p.ldq + p.q_col0 + (size_t)h * p.dim;
#pragma unroll
        for (int kk = 0; kk < DK; ++kk) {
            uint32_t w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int d = 32 * kk + 8 * kq + 2 * i;
                const float a = (qvalid && d < p.dim) ? qr[d] : 0.f, c = (qvalid && d + 1 < p.dim) ? qr[d + 1] : 0.f;
                w[i] = ZT<ZL_BF16>::from_f32(a) | (uint32_t)ZT<ZL_BF16>::from_f32(c) << 16;
            }
            qf[kk] = make_uint4(w[0], w[1], w[2], w[3]);
        }
    }
    fa_f4 o[DV];
#pragma unroll
    for (int dt = 0; dt < DV; ++dt) o[dt] = (fa_f4){0.f, 0.f, 0.f, 0.f};
    float m = p.sink ? p.sink[h] : -INFINITY, l = p.sink ? 1.0f : 0.0f;

    // K and V^T tiles: the NEXT tile's 16-byte loads are issued into registers before the current tile's MFMAs and written to LDS after them
    constexpr int KU = DK, VU = (DV + 1) / 2;                                      // 16-byte units per thread: 64 DK 4 / 256 and DV 16 8 / 256
    uint4 kreg[KU], vreg[VU];
    auto fetch_tiles = [&](int j0) {
#pragma unroll
        for (int u = 0; u < KU; ++u) {
            const int idx = tid + 256 * u;
            const int key = idx / (DK * 4), d = (idx % (DK * 4)) * 8;
            const uint16_t* src = p.k + (size_t)(cs + j0 + key) * p.ldk + (size_t)h * p.dim + d;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (d + 8 <= p.dim && p.vec_k) v = *reinterpret_cast<const uint4*>(src);
            else if (d < p.dim) {
                uint16_t e[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) e[i] = d + i < p.dim ? src[i] : (uint16_t)0;
                v = make_uint4(e[0] | (uint32_t)e[1] << 16, e[2] | (uint32_t)e[3] << 16, e[4] | (uint32_t)e[5] << 16, e[6] | (uint32_t)e[7] << 16);
            }
            kreg[u] = v;
        }
#pragma unroll
        for (int u = 0; u < VU; ++u) {
            const int idx = tid + 256 * u;
            const int d = idx >> 3, c8 = (idx & 7) * 8;
            uint4 v = make_uint4(0, 0, 0, 0);
            if (idx < DV * 16 * 8 && d < p.vdim) v = *reinterpret_cast<const uint4*>(p.vt + ((size_t)h * p.vdim + d) * p.ldv + cs + j0 + c8);
            vreg[u] = v;
        }
    };
    auto publish_tiles = [&]() {
#pragma unroll
        for (int u = 0; u < KU; ++u) {
            const int idx = tid + 256 * u;
            *reinterpret_cast<uint4*>(Ks + (idx / (DK * 4)) * KR + (idx % (DK * 4)) * 8) = kreg[u];
        }
#pragma unroll
        for (int u = 0; u < VU; ++u) {
            const int idx = tid + 256 * u;
            if (idx < DV * 16 * 8) *reinterpret_cast<uint4*>(Vs + (idx >> 3) * VR + (idx & 7) * 8) = vreg[u];
        }
    };
    fetch_tiles(j_first);
    for (int j0 = j_first; j0 <= block_last; j0 += 64) {
        __syncthreads();                                                           // the previous tile is consumed
        publish_tiles();
        __syncthreads();
        if (j0 + 64 <= block_last) fetch_tiles(j0 + 64);                           // in flight during this tile's MFMAs
        if (j0 > wave_last) continue;                                              // wave-uniform; the barriers above stay in step
        fa_f4 sc[4];
        float mx = -INFINITY;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            sc[c] = (fa_f4){0.f, 0.f, 0.f, 0.f};
            if (j0 + 16 * c <= wave_last) {
#pragma unroll
                for (int kk = 0; kk < DK; ++kk) {
                    const uint4 a = *reinterpret_cast<const uint4*>(Ks + (16 * c + nrow) * KR + 32 * kk + 8 * kq);
                    sc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(fa_b8, a), __builtin_bit_cast(fa_b8, qf[kk]), sc[c], 0, 0, 0);
                }
            }
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int key = j0 + 16 * c + 4 * kq + r;
                const float v = (qvalid && key <= qpos && (p.window <= 0 || qpos - key < p.window)) ? sc[c][r] * p.scale : -INFINITY;
                sc[c][r] = v;
                mx = fmaxf(mx, v);
            }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float mnew = fmaxf(m, mx);
        const bool dead = mnew == -INFINITY;                                       // nothing seen yet and no sink: keep zeros
        const float corr = dead ? 1.0f : __expf(m - mnew);
        float ps = 0.f;
        // the 32-key contraction of v_mfma_f32_16x16x32_bf16 may run over the keys in ANY order as long as both operands use the same one:
        // slot s of lane group kq stands for key 16 (s / 4) + 4 kq + s % 4 of the pair of 16-key blocks, which is how the scores lie here
        uint32_t hi[2][4], lo[2][4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
#pragma unroll
            for (int r = 0; r < 4; r += 2) {
                uint16_t hb[2], lb[2];
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const float pv = (dead || sc[c][r + e] == -INFINITY) ? 0.f : __expf(sc[c][r + e] - mnew);
                    ps += pv;
                    fa_split(pv, hb[e], lb[e]);
                }
                hi[c >> 1][2 * (c & 1) + (r >> 1)] = hb[0] | (uint32_t)hb[1] << 16;
                lo[c >> 1][2 * (c & 1) + (r >> 1)] = lb[0] | (uint32_t)lb[1] << 16;
            }
        }
        ps += __shfl_xor(ps, 16, 64);
        ps += __shfl_xor(ps, 32, 64);
        l = l * corr + ps;
        m = mnew;
#pragma unroll
        for (int dt = 0; dt < DV; ++dt) {
            o[dt] *= corr;
#pragma unroll
            for (int c2 = 0; c2 < 2; ++c2) {
                if (j0 + 32 * c2 <= wave_last) {                                    // (a block past the wave's last key has weights 0)
                    const uint2 a0 = *reinterpret_cast<const uint2*>(Vs + (16 * dt + nrow) * VR + 32 * c2 + 4 * kq);
                    const uint2 a1 = *reinterpret_cast<const uint2*>(Vs + (16 * dt + nrow) * VR + 32 * c2 + 16 + 4 * kq);
                    const fa_b8 a = __builtin_bit_cast(fa_b8, make_uint4(a0.x, a0.y, a1.x, a1.y));
                    const fa_b8 ph = __builtin_bit_cast(fa_b8, make_uint4(hi[c2][0], hi[c2][1], hi[c2][2], hi[c2][3]));
                    const fa_b8 pl = __builtin_bit_cast(fa_b8, make_uint4(lo[c2][0], lo[c2][1], lo[c2][2], lo[c2][3]));
                    o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, ph, o[dt], 0, 0, 0);
                    o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pl, o[dt], 0, 0, 0);
                }
            }
        }
    }
    if (!qvalid) return;
    const float g = p.gate ? seq_sigmoid(p.gate[(size_t)(first + qi) * p.ldg + p.g_col0 + h]) : 1.0f;
    const float inv = l > 0.f ? g / l : 0.f;
    uint16_t* orow = p.out + ((size_t)(first + qi) * p.heads + h) * p.vdim;
#pragma unroll
    for (int dt = 0; dt < DV; ++dt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int d = 16 * dt + 4 * kq + r;
            if (d < p.vdim) orow[d] = ZT<ZL_BF16>::from_f32(o[dt][r] * inv);
        }
}

// ---- single tokens in bf16 on the matrix cores --------------------------------------------------------------------------------------
// One wave = one token x 16 heads x one split of the keys.  Per 32 keys: the latent rows go from the pages straight into A operands
// (lane = key, 8 consecutive latent columns per 16-byte load), S^T (16 keys x 16 heads) = C . Q'^T with the folded queries as B operands
// held in registers; softmax per lane (= per head) as in the prompt kernel; the rows are then parked in LDS and read back column-wise for
// O^T (latent x 16 heads) += C^T . P^T (the contraction runs over the 32 keys in the order the scores lie in the lanes; two bf16 halves
// per weight).  Leaves (max, denominator, sums) per split in the workspace of k_latent_split's format: k_latent_combine finishes both.
template <int RT>                                                                  // rank <= 32 RT
__global__ __launch_bounds__(64) void k_latent_decode_mfma(const AttnP p, const zls_batch_t b, const float* __restrict__ qa,
                                                           float* __restrict__ ws, int n_splits) {
    constexpr int CR = RT * 32 + 8;
    __shared__ __attribute__((aligned(16))) uint16_t ct[32 * CR];
    const int t = blockIdx.x, split = blockIdx.z, lane = threadIdx.x, nrow = lane & 15, kq = lane >> 4;
    const int head = blockIdx.y * 16 + nrow;
    const bool hvalid = head < p.heads;
    const int sq = b.tok_seq[t];
    if (p.single_only && b.seq_start[sq + 1] - b.seq_start[sq] > 1) return;
    const int pos = b.seq_pos0[sq] + (t - b.seq_start[sq]);
    const int key_lo = p.window > 0 ? max(0, pos - p.window + 1) : 0;
    const int nkeys = pos + 1 - key_lo;
    const int chunk = ((nkeys + n_splits - 1) / n_splits + 31) & ~31;
    const int k0 = key_lo + split * chunk, k1 = min(pos + 1, k0 + chunk);
    const int32_t* pages = b.page_table + (size_t)sq * b.max_pages;
    const uint16_t* cache = reinterpret_cast<const uint16_t*>(p.cache);

    uint4 qf[RT];
    {
        const float* qr = qa + ((size_t)t * p.heads + (hvalid ? head : 0)) * p.rank;
#pragma unroll
        for (int kk = 0; kk < RT; ++kk) {
            uint32_t w[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int r = 32 * kk + 8 * kq + 2 * i;
                const float a = (hvalid && r < p.rank) ? qr[r] : 0.f, c = (hvalid && r + 1 < p.rank) ? qr[r + 1] : 0.f;
                w[i] = ZT<ZL_BF16>::from_f32(a) | (uint32_t)ZT<ZL_BF16>::from_f32(c) << 16;
            }
            qf[kk] = make_uint4(w[0], w[1], w[2], w[3]);
        }
    }
    fa_f4 o[2 * RT];
#pragma unroll
    for (int rt = 0; rt < 2 * RT; ++rt) o[rt] = (fa_f4){0.f, 0.f, 0.f, 0.f};
    float m = -INFINITY, l = 0.f;

    for (int j0 = k0; j0 < k1; j0 += 32) {
        uint4 cr[2][RT];
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            const int j = j0 + 16 * c + nrow;
            const bool valid = j < k1;
            const size_t base = valid ? ((size_t)pages[j / b.page_size] * b.page_size + j % b.page_size) * p.rank : 0;
#pragma unroll
            for (int kk = 0; kk < RT; ++kk) {
                const int r = 32 * kk + 8 * kq;
                cr[c][kk] = (valid && r < p.rank) ? *reinterpret_cast<const uint4*>(cache + base + r) : make_uint4(0, 0, 0, 0);
            }
        }
        fa_f4 sc[2];
        float mx = -INFINITY;
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            sc[c] = (fa_f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int kk = 0; kk < RT; ++kk)
                sc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(fa_b8, cr[c][kk]), __builtin_bit_cast(fa_b8, qf[kk]), sc[c], 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float v = (j0 + 16 * c + 4 * kq + r < k1) ? sc[c][r] : -INFINITY;        // (the folded query carries the scale)
                sc[c][r] = v;
                mx = fmaxf(mx, v);
            }
        }
        mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float mnew = fmaxf(m, mx);                                           // finite: key j0 is valid
        const float corr = __expf(m - mnew);                                       // m = -inf at the first block: 0
        float ps = 0.f;
        uint32_t hi[4], lo[4];
#pragma unroll
        for (int c = 0; c < 2; ++c) {
#pragma unroll
            for (int r = 0; r < 4; r += 2) {
                uint16_t hb[2], lb[2];
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const float pv = sc[c][r + e] == -INFINITY ? 0.f : __expf(sc[c][r + e] - mnew);
                    ps += pv;
                    fa_split(pv, hb[e], lb[e]);
                }
                hi[2 * c + (r >> 1)] = hb[0] | (uint32_t)hb[1] << 16;
                lo[2 * c + (r >> 1)] = lb[0] | (uint32_t)lb[1] << 16;
            }
        }
        ps += __shfl_xor(ps, 16, 64);
        ps += __shfl_xor(ps, 32, 64);
        l = l * corr + ps;
        m = mnew;
        const fa_b8 ph = __builtin_bit_cast(fa_b8, make_uint4(hi[0], hi[1], hi[2], hi[3]));
        const fa_b8 pl = __builtin_bit_cast(fa_b8, make_uint4(lo[0], lo[1], lo[2], lo[3]));
        __syncthreads();                                                           // the previous block's column reads are done
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int kk = 0; kk < RT; ++kk) *reinterpret_cast<uint4*>(ct + (16 * c + nrow) * CR + 32 * kk + 8 * kq) = cr[c][kk];
        __syncthreads();
#pragma unroll
        for (int rt = 0; rt < 2 * RT; ++rt) {
            // slot s of lane group kq <-> key 16 (s / 4) + 4 kq + s % 4 of the block; this lane's column of the latent: 16 rt + nrow
            uint32_t w[4];
#pragma unroll
            for (int s2 = 0; s2 < 4; ++s2) {
                const int ka = 16 * (s2 >> 1) + 4 * kq + 2 * (s2 & 1);
                w[s2] = ct[ka * CR + 16 * rt + nrow] | (uint32_t)ct[(ka + 1) * CR + 16 * rt + nrow] << 16;
            }
            const fa_b8 a = __builtin_bit_cast(fa_b8, make_uint4(w[0], w[1], w[2], w[3]));
            o[rt] *= corr;
            o[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, ph, o[rt], 0, 0, 0);
            o[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pl, o[rt], 0, 0, 0);
        }
    }
    if (!hvalid) return;
    float* out = ws + (((size_t)t * p.heads + head) * n_splits + split) * (p.rank + 2);
    if (kq == 0) { out[0] = m; out[1] = l; }
#pragma unroll
    for (int rt = 0; rt < 2 * RT; ++rt)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int r = 16 * rt + 4 * kq + i;
            if (r < p.rank) out[2 + r] = o[rt][i];
        }
}

}  // namespace

extern "C" int zls_latent_rope_store(float* proj, int64_t ld, int64_t col0, const float* weight, float eps, int64_t rank, int64_t rot,
                                     const float* freq, int interleaved, int64_t q_col0, int64_t heads, int64_t qdim, float rot_gain,
                                     const zls_batch_t* b, void* cache, int dtype, zl_stream_t s) {
    ZL_CHECK_ARG(proj && weight && cache && seq_batch_ok(b) && b->page_table && b->page_size > 0 && b->max_pages > 0 && rank > 0 && rot >= 0, ZL_EINVAL);
    ZL_CHECK_ARG(col0 >= 0 && col0 + rank + rot <= ld && rot % 2 == 0, ZL_ESHAPE);
    ZL_CHECK_ARG(rot == 0 || (freq && heads > 0 && qdim >= rot && q_col0 >= 0 && q_col0 + heads * qdim <= ld), ZL_ESHAPE);
#define CALL(DT) hipLaunchKernelGGL((k_latent_store<DT>), dim3(b->n_tok), dim3(256), 0, (hipStream_t)s, proj, ld, (int)col0, weight, eps, (int)rank, \
                                    (int)rot, freq, interleaved ? 1 : 0, (int)q_col0, (int)(rot ? heads : 0), (int)qdim, *b, cache, rot_gain);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}

extern "C" int zls_latent_store(const float* proj, int64_t ld, int64_t col0, const float* weight, float eps, int64_t rank, const zls_batch_t* b,
                                void* cache, int dtype, zl_stream_t s) {
    return zls_latent_rope_store(const_cast<float*>(proj), ld, col0, weight, eps, rank, 0, nullptr, 0, 0, 0, 0, 1.0f, b, cache, dtype, s);
}

extern "C" int64_t zls_latent_attention_workspace_bytes(int64_t n_tok, int64_t heads, int64_t rank, int64_t n_splits) {
    if (n_tok <= 0 || heads <= 0 || rank <= 0 || n_splits <= 0) return ZL_EINVAL;
    return (n_tok * heads * n_splits * (rank + 2) + n_tok * heads * rank) * (int64_t)sizeof(float);    /* partials | folded queries */
}

extern "C" int zls_latent_attention(const float* q, int64_t ldq, int64_t q_col0, const float* gate, int64_t ldg, int64_t g_col0, const void* w_uk,
                                    const void* w_uv, const float* sink, const void* cache, const zls_batch_t* b, float scale, int64_t heads,
                                    int64_t dim, int64_t vdim, int64_t rank, void* out, int dtype, int single_only, void* workspace,
                                    int64_t n_splits, int no_mfma, int64_t window, zl_stream_t s) {
    ZL_CHECK_ARG(q && w_uk && w_uv && cache && out && workspace && seq_batch_ok(b) && b->page_table && b->page_size > 0 && b->max_pages > 0, ZL_EINVAL);
    ZL_CHECK_ARG(heads > 0 && dim > 0 && vdim > 0 && rank > 0 && heads <= 65535 && n_splits > 0 && n_splits <= 65535, ZL_EINVAL);
    ZL_CHECK_ARG(q_col0 >= 0 && q_col0 + heads * dim <= ldq && (!gate || (g_col0 >= 0 && g_col0 + heads <= ldg)), ZL_ESHAPE);
    const size_t lds = (16 * ((size_t)rank + 4) + 4 * (size_t)rank) * sizeof(float);
    ZL_CHECK_ARG(rank <= 1024 && lds <= 64 * 1024, ZL_ELIMIT);
    AttnP p;
    p.q = q; p.gate = gate; p.w_uk = w_uk; p.w_uv = w_uv; p.sink = sink; p.cache = cache; p.out = out;
    p.ldq = ldq; p.ldg = ldg; p.q_col0 = (int)q_col0; p.g_col0 = (int)g_col0;
    p.heads = (int)heads; p.dim = (int)dim; p.vdim = (int)vdim; p.rank = (int)rank; p.scale = scale; p.single_only = single_only;
    ZL_CHECK_ARG(window < (1 << 30), ZL_ESHAPE);
    p.window = window > 0 ? (int)window : 0;
    // (the split kernel's eight 16-byte slots per thread cover 1024 bf16 or 512 fp32 columns of a row; longer fp32 rows are read singly)
    p.vec = (rank % (dtype == ZL_BF16 ? 8 : 4) == 0 && ((uintptr_t)cache & 15) == 0 && (dtype == ZL_BF16 || rank <= 512)) ? 1 : 0;
    const dim3 grid(b->n_tok, (unsigned)((heads + 3) / 4), (unsigned)n_splits);
    hipStream_t hs = (hipStream_t)s;
    float* ws = (float*)workspace;
    float* qa = ws + (size_t)b->n_tok * heads * n_splits * (rank + 2);
    const int ns = (int)n_splits;
    // bf16 with aligned rows of at most 640 latent columns (512 + a rotated part): the split pass on the matrix cores (absorb and combine
    // are shared)
    const bool mfma = dtype == ZL_BF16 && p.vec && rank <= 640 && !no_mfma;
    const dim3 mgrid(b->n_tok, (unsigned)((heads + 15) / 16), (unsigned)n_splits);
#define MSPLIT(RT) hipLaunchKernelGGL((k_latent_decode_mfma<RT>), mgrid, dim3(64), 0, hs, p, *b, qa, ws, ns)
#define SPLIT(DT, RPL) hipLaunchKernelGGL((k_latent_split<DT, RPL>), grid, dim3(256), lds, hs, p, *b, qa, ws, ns)
#define CALL(DT)                                  \
    hipLaunchKernelGGL((k_latent_absorb<DT>), dim3(b->n_tok, (unsigned)heads, (unsigned)((rank + 63) / 64)), dim3(256), 0, hs, p, *b, qa); \
    if (mfma) {                                   \
        if (rank <= 64) MSPLIT(2);                \
        else if (rank <= 128) MSPLIT(4);          \
        else if (rank <= 256) MSPLIT(8);          \
        else if (rank <= 512) MSPLIT(16);         \
        else MSPLIT(20);                          \
    } else if (rank <= 64) SPLIT(DT, 1);          \
    else if (rank <= 128) SPLIT(DT, 2);           \
    else if (rank <= 256) SPLIT(DT, 4);           \
    else if (rank <= 512) SPLIT(DT, 8);           \
    else SPLIT(DT, 16);                           \
    hipLaunchKernelGGL((k_latent_combine<DT>), dim3(b->n_tok, (unsigned)heads, (unsigned)((vdim + 31) / 32 > 4 ? 4 : (vdim + 31) / 32)), dim3(256), (size_t)(rank + n_splits) * sizeof(float), hs, p, *b, ws, ns);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
#undef SPLIT
#undef MSPLIT
    return zl_launch_status();
}

extern "C" int zls_latent_attention_prompt(const float* q, int64_t ldq, int64_t q_col0, const float* gate, int64_t ldg, int64_t g_col0,
                                           const void* k, int64_t ldk, const void* vt, int64_t ldv, const float* sink, const int32_t* ctx_start,
                                           const zls_batch_t* b, float scale, int64_t heads, int64_t dim, int64_t vdim, void* out, int dtype,
                                           int64_t window, const int32_t* ctx_pos0, zl_stream_t s) {
    ZL_CHECK_ARG(q && k && vt && ctx_start && out && seq_batch_ok(b) && window < (1 << 30), ZL_EINVAL);
    ZL_CHECK_ARG(dtype == ZL_BF16, ZL_EDTYPE);
    ZL_CHECK_ARG(heads > 0 && heads <= 65535 && dim > 0 && vdim > 0 && dim <= 256 && vdim <= 256, ZL_ESHAPE);
    ZL_CHECK_ARG(q_col0 >= 0 && q_col0 + heads * dim <= ldq && (!gate || (g_col0 >= 0 && g_col0 + heads <= ldg)), ZL_ESHAPE);
    ZL_CHECK_ARG(ldk >= heads * dim && ldv % 8 == 0 && ((uintptr_t)vt & 15) == 0, ZL_ESHAPE);
    FaP p;
    p.q = q; p.gate = gate; p.k = (const uint16_t*)k; p.vt = (const uint16_t*)vt; p.sink = sink; p.ctx_start = ctx_start; p.out = (uint16_t*)out;
    p.ldq = ldq; p.ldg = ldg; p.ldk = ldk; p.ldv = ldv; p.q_col0 = (int)q_col0; p.g_col0 = (int)g_col0;
    p.heads = (int)heads; p.dim = (int)dim; p.vdim = (int)vdim; p.scale = scale; p.window = window > 0 ? (int)window : 0; p.ctx_pos0 = ctx_pos0;
    p.tiles_per_seq = (b->max_count + 63) / 64;
    p.vec_k = (dim % 8 == 0 && ldk % 8 == 0 && ((uintptr_t)k & 15) == 0) ? 1 : 0;
    const dim3 grid((unsigned)(b->n_seq * p.tiles_per_seq), (unsigned)heads);
    hipStream_t hs = (hipStream_t)s;
    // the smallest instantiation that holds both the key size (32 DK) and the value size (16 DV): heads with a rotated part have keys
    // longer than their values
#define FA(DK, DV) if (dim <= 32 * DK && vdim <= 16 * DV) { hipLaunchKernelGGL((k_latent_fa<DK, DV>), grid, dim3(256), 0, hs, p, *b); return zl_launch_status(); }
    FA(1, 2) FA(2, 2) FA(2, 4) FA(4, 4) FA(4, 8) FA(6, 8) FA(8, 8) FA(8, 16)
#undef FA
    return ZL_ESHAPE;
}
