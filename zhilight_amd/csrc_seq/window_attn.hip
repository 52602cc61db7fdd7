// window_attn.hip -- softmax attention over a paged key / value cache for a ragged step: rotary positions on a part of every query and key
// head (pairs half a part apart, or neighbouring coordinates), unit-RMS queries and keys, values turned by their own position and the sums
// turned back, values blended with another layer's values of the same token, a sliding window that may keep the sequence's first keys, a
// learned sink in the softmax denominator, weights mixed across heads after the softmax, a sigmoid gate per output coordinate.
// A general score form (FORM = 1 instantiations) serves relatives: weighted query / key norms, a factor per head, scores capped by tanh, a
// bias by the distance between query and key, queries confined to their chunk of positions, and weights that are sigmoids instead of a
// softmax (every key on its own; the splits of a token are then plain sums).
//
// k_rope_norm_store    a workgroup per token, a wave per head in turn: the head's coordinates in registers, rotated, normed, written back
//                      (queries, fp32, in place) or to the token's row of the paged planes (keys, values; serving format)
// k_window_attention   a workgroup per (token, query head, split of the window's pages): a page of keys at a time -- a wave per key for the
//                      scores (butterfly over the head size), running maximum and sum, then a thread per output coordinate for P.V over the
//                      page's transposed values.  Single decoded tokens in both formats, and everything in fp32.
// k_window_attention_mfma  bf16 portions on the matrix cores, 64 queries x one head per workgroup (described at the kernel)
//                      With all_kv both apply the weights of a query head to the values of EVERY key / value head: mixing the heads'
//                      weights afterwards is then a small product per token (k_head_mix_gate), sum_g T[h][g] acc[g][c(h)], and no weight
//                      ever has to wait for another head's normaliser.
// k_head_mix_gate      a workgroup per (token, kv head): the splits merged, the mix over heads, the turn back by the token's own position, the gate
// Positions, angles, scores, weights, sums: fp32.  exp is the accurate library version (the bf16 matrix-core kernel: the hardware's exp2);
// sin / cos take an angle reduced in double (seq_sincos).
#include "seq_common.h"

namespace {

constexpr int kMaxE = 8;            // coordinates of a head per lane: dim, vdim <= 64 * kMaxE
constexpr int kChunk = 128;         // the largest page k_window_attention walks
constexpr int kMaxV = 8;            // output coordinates per thread: (all_kv ? kv_heads : 1) * vdim <= 256 * kMaxV

// one head of `size` coordinates in the lanes' registers (coordinate i in lane i % 64, register i / 64): rotate the first n_rot (pairs
// i, i + n_rot / 2; interleaved: pairs 2i, 2i + 1) by pos * freq[i], optionally divide by the root mean square; the result stays in v[]
__device__ __forceinline__ void rope_head(float* v, const float* src, int size, int n_rot, const float* __restrict__ freq, float pos, bool norm,
                                          float eps, int lane, bool interleaved = false, const float* __restrict__ w = nullptr) {
    const int half = n_rot >> 1;
    float ss = 0.f;
#pragma unroll
    for (int r = 0; r < kMaxE; ++r) {
        const int i = lane + 64 * r;
        float o = 0.f;
        if (i < size) {
            o = src[i];
            if (i < n_rot) {
                const bool lo = interleaved ? (i & 1) == 0 : i < half;
                const float other = src[interleaved ? (i ^ 1) : (lo ? i + half : i - half)];
                float sn, cs;
                seq_sincos(pos * freq[interleaved ? (i >> 1) : (lo ? i : i - half)], &sn, &cs);
                o = lo ? o * cs - other * sn : o * cs + other * sn;
            }
            ss = fmaf(o, o, ss);
        }
        v[r] = o;
    }
    if (norm) {
        const float f = 1.0f / sqrtf(zl_wave_sum(ss) / (float)size + eps);
#pragma unroll
        for (int r = 0; r < kMaxE; ++r) v[r] *= (w && lane + 64 * r < size) ? f * w[lane + 64 * r] : f;
    }
}

struct RopeP {
    float* proj; int64_t ld;
    int q_col0, k_col0, v_col0, heads, kv_heads, dim, vdim, rot_dims, qk_norm;
    const float* qk_freq; const float* v_freq;
    float eps;
    void* k_cache; void* v_cache;
    int interleaved;
    const float* vmix_src; int64_t vmix_ld; int vmix_col0; float vmix_lambda;     // values <- (1 - lambda) values + lambda vmix_src[t][col0 ..]
    const float* q_w; const float* k_w;             // nullable (dim): weights of the query / key norm, shared by the heads
};

template <int DT>
__global__ __launch_bounds__(256) void k_rope_norm_store(const RopeP p, const zls_batch_t b) {
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sq = b.tok_seq[t];
    const int posi = b.seq_pos0[sq] + (t - b.seq_start[sq]);
    const float pos = (float)posi;
    float* row = p.proj + (size_t)t * p.ld;
    const size_t cpage = (size_t)b.page_table[(size_t)sq * b.max_pages + posi / b.page_size];
    const size_t crow = cpage * b.page_size + posi % b.page_size;
    const int n_kv = p.k_cache ? p.kv_heads : 0;
    float v[kMaxE];
    for (int h = wave; h < p.heads + 2 * n_kv; h += 4) {                 // (a wave owns its heads: no two waves touch the same numbers)
        if (h < p.heads) {
            float* q = row + p.q_col0 + h * p.dim;
            rope_head(v, q, p.dim, p.rot_dims, p.qk_freq, pos, p.qk_norm != 0, p.eps, lane, p.interleaved != 0, p.q_w);
#pragma unroll
            for (int r = 0; r < kMaxE; ++r)
                if (lane + 64 * r < p.dim) q[lane + 64 * r] = v[r];
        } else if (h < p.heads + n_kv) {
            const int c = h - p.heads;
            rope_head(v, row + p.k_col0 + c * p.dim, p.dim, p.rot_dims, p.qk_freq, pos, p.qk_norm != 0, p.eps, lane, p.interleaved != 0, p.k_w);
#pragma unroll
            for (int r = 0; r < kMaxE; ++r)
                if (lane + 64 * r < p.dim) SeqT<DT>::st(p.k_cache, (crow * p.kv_heads + c) * p.dim + lane + 64 * r, v[r]);
        } else {
            const int c = h - p.heads - n_kv;
            rope_head(v, row + p.v_col0 + c * p.vdim, p.vdim, p.v_freq ? p.vdim : 0, p.v_freq, pos, false, 0.f, lane);
            if (p.vmix_src) {
                const float* other = p.vmix_src + (size_t)t * p.vmix_ld + p.vmix_col0 + c * p.vdim;
#pragma unroll
                for (int r = 0; r < kMaxE; ++r)
                    if (lane + 64 * r < p.vdim) v[r] = (1.0f - p.vmix_lambda) * v[r] + p.vmix_lambda * other[lane + 64 * r];
            }
#pragma unroll
            for (int r = 0; r < kMaxE; ++r)
                if (lane + 64 * r < p.vdim)                             // values lie transposed inside a page: (kv head, coordinate, key)
                    SeqT<DT>::st(p.v_cache, ((cpage * p.kv_heads + c) * p.vdim + lane + 64 * r) * b.page_size + posi % b.page_size, v[r]);
        }
    }
}

// 8 consecutive cached numbers as fp32
template <int DT> struct Ld8;
template <> struct Ld8<ZL_BF16> {
    static __device__ __forceinline__ void ld(const void* p, size_t i, float* v) {
        const uint4 u = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(p) + i);
        const uint32_t q[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            v[2 * j] = __builtin_bit_cast(float, q[j] << 16);
            v[2 * j + 1] = __builtin_bit_cast(float, q[j] & 0xffff0000u);
        }
    }
};
template <> struct Ld8<ZL_F32> {
    static __device__ __forceinline__ void ld(const void* p, size_t i, float* v) {
        const float4 a = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p) + i);
        const float4 c = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p) + i + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = c.x; v[5] = c.y; v[6] = c.z; v[7] = c.w;
    }
};

struct AttnP {
    const float* q; int64_t ldq; int q_col0;
    const void* k_cache; const void* v_cache;
    float scale; int window, keep_first, heads, kv_heads, dim, vdim, all_kv;    // keep_first: keys 0 .. keep_first - 1 stay visible behind the window
    float* acc; float* ml;                 // (n_tok, heads, n_splits, nv) partial sums | (n_tok, heads, n_splits, 2) their maximum and weight sum
    int n_splits, pages_per_split, single_only;
    const int32_t* tiles;                  // the matrix-core kernel: (first flat token, rows, sequence) per query tile
    // the general score form (kernels instantiated with FORM = 1; all of it optional):
    const float* head_scale;               // (heads) the score of head g is also multiplied by head_scale[g]
    float softcap;                         // > 0: score <- softcap * tanh(score / softcap)
    const float* bias; int bias_rows;      // (heads, bias_rows): bias[g][min(p - j, bias_rows - 1)] is added to the (capped) score
    const float* offset;                   // (heads) sigmoid weights: w = sigmoid(score + offset[g])
    int chunk;                             // > 0: a query only sees the keys of its own chunk of `chunk` positions, counted from position 0
    int sigmoid;                           // weights are sigmoids, each key on its own: no maximum, no normaliser (ml = (0, 1) for a split with keys)
};

// the score of the general form from the scaled product
__device__ __forceinline__ float form_score(const AttnP& p, float s, int g, int dist) {
    if (p.softcap > 0.f) s = p.softcap * tanhf(s / p.softcap);
    if (p.bias) s += p.bias[(size_t)g * p.bias_rows + min(dist, p.bias_rows - 1)];
    return s;
}

// A token's pages: those that only hold kept first keys (before the page of the window's oldest key), then the window's.  Split s walks
// pages_per_split of that list from s * pages_per_split, a page at a
// time: scores of the page's keys (a wave per key), weights with the running maximum -- 0 for keys outside the window or after the
// token -- then every thread adds the WHOLE page of its value coordinates (the plane holds values transposed, 8 keys per 16-byte load).
// What a split leaves is unnormalised: sum_j e^(s_j - m) v_j with m and sum_j e^(s_j - m); k_head_mix_gate merges the splits.
template <int DT, int FORM>
__global__ __launch_bounds__(256) void k_window_attention(const AttnP p, const zls_batch_t b) {
    extern __shared__ float lds[];
    __shared__ float red[16];
    __shared__ __attribute__((aligned(16))) float sc[kChunk];
    float* qs = lds;                                                      // [dim], already times scale
    const int t = blockIdx.x, g = blockIdx.y, sp = blockIdx.z, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int sq = b.tok_seq[t];
    if (p.single_only && b.seq_start[sq + 1] - b.seq_start[sq] > 1) return;
    const int ps = b.page_size;
    const int pos = b.seq_pos0[sq] + (t - b.seq_start[sq]);
    int lo = p.window > 0 ? max(0, pos - p.window + 1) : 0;
    if (FORM && p.chunk > 0) lo = max(lo, pos / p.chunk * p.chunk);
    const int wp0 = lo / ps, nkp = min((p.keep_first + ps - 1) / ps, wp0);   // kept pages before the window's first page
    const int c = g / (p.heads / p.kv_heads);
    const int nv = p.all_kv ? p.kv_heads * p.vdim : p.vdim, voff = p.all_kv ? 0 : c * p.vdim;
    const int32_t* pages = b.page_table + (size_t)sq * b.max_pages;
    const int li0 = sp * p.pages_per_split, li1 = min(nkp + pos / ps - wp0, li0 + p.pages_per_split - 1);
    const float qscale = (FORM && p.head_scale) ? p.scale * p.head_scale[g] : p.scale;
    for (int i = tid; i < p.dim; i += 256) qs[i] = p.q[(size_t)t * p.ldq + p.q_col0 + g * p.dim + i] * qscale;
    float A[kMaxV];
#pragma unroll
    for (int r = 0; r < kMaxV; ++r) A[r] = 0.f;
    float m = -INFINITY, l = 0.f;
    __syncthreads();
    for (int li = li0; li <= li1; ++li) {
        const int pg = li < nkp ? li : wp0 + li - nkp;
        const size_t page = (size_t)pages[pg];
        const int j0 = pg * ps;
        for (int jj = wave; jj < ps; jj += 4) {
            const int j = j0 + jj;
            float part = -INFINITY;
            if (j <= pos && (j >= lo || j < p.keep_first)) {              // (wave-uniform)
                const size_t at = ((page * ps + jj) * p.kv_heads + c) * p.dim;
                part = 0.f;
                for (int i = lane; i < p.dim; i += 64) part = fmaf(qs[i], SeqT<DT>::ld(p.k_cache, at + i), part);
                part = zl_wave_sum(part);
                if (FORM) part = form_score(p, part, g, pos - j);
            }
            if (lane == 0) sc[jj] = part;
        }
        __syncthreads();
        if (FORM && p.sigmoid) {                                          // every key on its own: no maximum, nothing to correct
            const float off = p.offset ? p.offset[g] : 0.f;
            for (int jj = tid; jj < ps; jj += 256) sc[jj] = sc[jj] == -INFINITY ? 0.f : seq_sigmoid(sc[jj] + off);
            m = 0.f; l = 1.f;
            __syncthreads();
#pragma unroll
            for (int r = 0; r < kMaxV; ++r) {
                const int e = tid + 256 * r;
                if (e < nv) {
                    float a = A[r];
                    const size_t at = (page * p.kv_heads * p.vdim + voff + e) * ps;
                    for (int j8 = 0; j8 < ps; j8 += 8) {
                        float v[8];
                        Ld8<DT>::ld(p.v_cache, at + j8, v);
                        const float4 w0 = *reinterpret_cast<const float4*>(sc + j8), w1 = *reinterpret_cast<const float4*>(sc + j8 + 4);
                        a = fmaf(w0.x, v[0], a); a = fmaf(w0.y, v[1], a); a = fmaf(w0.z, v[2], a); a = fmaf(w0.w, v[3], a);
                        a = fmaf(w1.x, v[4], a); a = fmaf(w1.y, v[5], a); a = fmaf(w1.z, v[6], a); a = fmaf(w1.w, v[7], a);
                    }
                    A[r] = a;
                }
            }
            __syncthreads();
            continue;
        }
        float cm = -INFINITY;
        for (int jj = tid; jj < ps; jj += 256) cm = fmaxf(cm, sc[jj]);
        const float m_new = fmaxf(m, zl_block_max(cm, red));              // finite: the page holds a visible key
        float psum = 0.f;
        for (int jj = tid; jj < ps; jj += 256) { const float e = expf(sc[jj] - m_new); sc[jj] = e; psum += e; }      // e^(-inf) = 0
        const float corr = expf(m - m_new);                               // (first page: 0, on sums that are 0)
        l = l * corr + zl_block_sum(psum, red);                           // (its barriers also publish the weights in sc[])
        m = m_new;
#pragma unroll
        for (int r = 0; r < kMaxV; ++r) {
            const int e = tid + 256 * r;
            if (e < nv) {
                float a = A[r] * corr;
                const size_t at = (page * p.kv_heads * p.vdim + voff + e) * ps;
                for (int j8 = 0; j8 < ps; j8 += 8) {
                    float v[8];
                    Ld8<DT>::ld(p.v_cache, at + j8, v);
                    const float4 w0 = *reinterpret_cast<const float4*>(sc + j8), w1 = *reinterpret_cast<const float4*>(sc + j8 + 4);
                    a = fmaf(w0.x, v[0], a); a = fmaf(w0.y, v[1], a); a = fmaf(w0.z, v[2], a); a = fmaf(w0.w, v[3], a);
                    a = fmaf(w1.x, v[4], a); a = fmaf(w1.y, v[5], a); a = fmaf(w1.z, v[6], a); a = fmaf(w1.w, v[7], a);
                }
                A[r] = a;
            }
        }
        __syncthreads();                                                  // sc[] is free for the next page
    }
    const size_t at = ((size_t)t * p.heads + g) * p.n_splits + sp;
    float* out = p.acc + at * nv;
#pragma unroll
    for (int r = 0; r < kMaxV; ++r)
        if (tid + 256 * r < nv) out[tid + 256 * r] = A[r];
    if (tid == 0) { p.ml[2 * at] = m; p.ml[2 * at + 1] = l; }            // (a split without pages: -inf, 0, sums 0)
}

// ---- portions on the matrix cores (bf16, 64-key pages) ------------------------------------------------------------------------------------
// A workgroup = a tile of up to 64 consecutive queries of one sequence x one query head (x a part of the output coordinates when they
// are many); wave w owns queries 16 w .. for the scores and the softmax, and a share of the (kv head, 16 value coordinates) output blocks
// for ALL 64 queries.  Per page of keys:
//   S^T = K Q^T      v_mfma_f32_16x16x32_bf16, A = 16 keys x 32 coordinates straight from the cache rows (16 bytes a lane), B = the wave's
//                    queries, split once into bf16 halves hi + lo (two MFMAs: the scores keep the fp32 queries' bits)
//   softmax          a lane holds 16 scores of one query (keys 4 kq + r of the page's four 16-key blocks); maximum and sum over the four
//                    lanes of the query by two butterflies; running maximum, correction e^(m_old - m_new)
//   P -> LDS         the weights, split into bf16 halves, in exactly the registers' order: a lane's 8 numbers for 32 keys ARE the B operand
//                    of O^T = V^T P^T if slot i of quarter kq means key 4 kq + i (i < 4) or 16 + 4 kq + i - 4 -- so the A operand takes V^T
//                    in that order: two 8-byte loads from the transposed value plane
//   O^T += V^T P^T   every wave: its output blocks x 4 query blocks x 2 key halves x (hi, lo), after scaling by the queries' corrections
// Two P buffers alternate, so one barrier per page is enough.
typedef __bf16 b8v __attribute__((ext_vector_type(8)));
typedef float f4v __attribute__((ext_vector_type(4)));
constexpr int kItems = 8;               // output blocks (16 value coordinates of one kv head) per wave: 4 waves x 8 x 16 = 512 per workgroup

__device__ __forceinline__ uint32_t bf16_bits(float f) {                 // round to nearest even; finite inputs
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    u += 0x7fffu + ((u >> 16) & 1u);
    return u >> 16;
}
__device__ __forceinline__ void split8(const float* v, uint4& hi, uint4& lo) {
    uint32_t h[8], l[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        h[i] = bf16_bits(v[i]);
        l[i] = bf16_bits(v[i] - __builtin_bit_cast(float, h[i] << 16));
    }
    hi = make_uint4(h[0] | h[1] << 16, h[2] | h[3] << 16, h[4] | h[5] << 16, h[6] | h[7] << 16);
    lo = make_uint4(l[0] | l[1] << 16, l[2] | l[3] << 16, l[4] | l[5] << 16, l[6] | l[7] << 16);
}

constexpr int kBiasLds = 2048;          // rows of a head's distance bias that the matrix-core kernel keeps in LDS (longer tables: the rest from memory)

// tanh and the logistic function on the hardware's exp2 and reciprocal: 1 ulp each, far inside what bf16 keys leave (bf16 kernel only)
__device__ __forceinline__ float fast_sigmoid(float x) {
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x));
}
__device__ __forceinline__ float fast_tanh(float x) { return 2.0f * fast_sigmoid(2.0f * x) - 1.0f; }

template <int KS, int FORM>             // 32-coordinate steps of the head size: dim <= 32 KS; FORM 1: the general score form of AttnP with a
                                        // softmax, 2: with sigmoid weights (no maximum, no correction of the sums, no normaliser)
__global__ __launch_bounds__(256) void k_window_attention_mfma(const AttnP p, const zls_batch_t b) {
    __shared__ uint4 pfrag[2][4][2][2][64];                              // [buffer][query block][key half][hi, lo][lane]
    __shared__ float corr_s[2][64], l_s[64], m_s[64];
    __shared__ float bias_s[FORM ? kBiasLds : 1];
    const int tile = blockIdx.x, g = blockIdx.y, part = blockIdx.z;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nrow = lane & 15, kq = lane >> 4;
    const int t0 = p.tiles[3 * tile], rows = p.tiles[3 * tile + 1], sq = p.tiles[3 * tile + 2];
    const int pos0 = b.seq_pos0[sq] + (t0 - b.seq_start[sq]);
    const int G = p.kv_heads, d = p.dim, vd = p.vdim;
    const int c = g / (p.heads / G);
    const int nv = p.all_kv ? G * vd : vd;
    const int32_t* pages = b.page_table + (size_t)sq * b.max_pages;
    const uint16_t* kc = reinterpret_cast<const uint16_t*>(p.k_cache);
    const uint16_t* vc = reinterpret_cast<const uint16_t*>(p.v_cache);
    // the wave's own query (for the scores): tile row 16 wave + nrow
    const int qi = 16 * wave + nrow;
    const bool qok = qi < rows;
    const int pq = pos0 + qi;
    const float qscale = (FORM && p.head_scale) ? p.scale * p.head_scale[g] : p.scale;
    const int chunk0 = (FORM && p.chunk > 0) ? pq / p.chunk * p.chunk : 0;          // the first position of the query's chunk
    const float off = (FORM && p.offset) ? p.offset[g] : 0.f;
    const float inv_cap = (FORM && p.softcap > 0.f) ? 1.0f / p.softcap : 0.f;
    const bool bias_lds = FORM && p.bias && p.bias_rows <= kBiasLds;     // (uniform: the whole row of the head sits in LDS)
    // Sigmoid weights (FORM 2) in as few instructions per score as the form allows.  With r = 1 / (1 + 2^(k1 s)), k1 = -2 log2(e) / cap,
    // the capped score is 2 cap r - cap, so the weight is 1 / (1 + 2^z) with z = A r + b[distance]: A = -2 cap log2(e) and
    // b = -log2(e) (bias + offset - cap), which is what the LDS row holds here; without a cap r = s and A = -log2(e).
    constexpr float kL2e = 1.4426950408889634f;
    const bool has_cap = FORM && p.softcap > 0.f;
    const float sg_k1 = has_cap ? -2.0f * kL2e * inv_cap : 0.f, sg_a = has_cap ? -2.0f * kL2e * p.softcap : -kL2e;
    const float sg_c0 = -kL2e * (off - (has_cap ? p.softcap : 0.f));
    // a key at distance dq = pq - j is visible iff 0 <= dq <= dmax (chunk and window in one unsigned comparison); kept first keys
    // need the general test
    const bool fast_vis = FORM == 2 && p.keep_first == 0;
    const int pq_eff = qok ? pq : -(1 << 30);
    const unsigned dmax = qok ? (unsigned)min(pq - chunk0, p.window > 0 ? p.window - 1 : pq) : 0u;
    if (FORM && p.bias) {
        for (int i = tid; i < min(p.bias_rows, kBiasLds); i += 256) {
            const float bv = p.bias[(size_t)g * p.bias_rows + i];
            bias_s[i] = FORM == 2 ? fmaf(-kL2e, bv, sg_c0) : bv;
        }
        __syncthreads();
    }
    uint4 qh[KS], ql[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int x = 32 * ks + 8 * kq + i;
            v[i] = (qok && x < d) ? p.q[(size_t)(t0 + qi) * p.ldq + p.q_col0 + g * d + x] * qscale : 0.f;
        }
        split8(v, qh[ks], ql[ks]);
    }
    // this wave's output blocks: block index nb = (part * 4 * kItems) + wave + 4 i  ->  (kv head, 16 coordinates)
    const int n_blocks = nv / 16, vb_per = vd / 16;
    f4v acc[kItems][4];
#pragma unroll
    for (int i = 0; i < kItems; ++i)
#pragma unroll
        for (int qb = 0; qb < 4; ++qb) acc[i][qb] = (f4v){0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY, l_run = 0.f;
    int lo_key = p.window > 0 ? max(0, pos0 - p.window + 1) : 0;
    if (FORM && p.chunk > 0) lo_key = max(lo_key, pos0 / p.chunk * p.chunk);        // (the tile's first query has the oldest chunk)
    const int hi_key = pos0 + rows - 1;
    int buf = 0;
    const int pg_last = hi_key / 64;
    // the key fragments of a page: A operands straight from the cache rows; the NEXT page's are requested as soon as this page's scores
    // are issued, and arrive during the softmax and the second product
    uint4 kf[4][KS];
    auto load_keys = [&](int pg) {
        const size_t page = (size_t)pages[pg];
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) {
            const uint16_t* kr = kc + ((page * 64 + kb * 16 + nrow) * G + c) * d + 8 * kq;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks)
                kf[kb][ks] = (32 * ks + 8 * kq < d) ? *reinterpret_cast<const uint4*>(kr + 32 * ks) : make_uint4(0, 0, 0, 0);
        }
    };
    // the tile's pages: those that only hold kept first keys, then the pages from the oldest key any of its queries sees in its window
    const int wp0 = lo_key / 64, nkp = min((p.keep_first + 63) / 64, wp0), li_last = nkp + pg_last - wp0;
    auto page_of = [&](int li) { return li < nkp ? li : wp0 + li - nkp; };
    load_keys(page_of(0));
    for (int li = 0; li <= li_last; ++li, buf ^= 1) {
        const int pg = page_of(li);
        const size_t page = (size_t)pages[pg];
        // ---- scores of the wave's 16 queries against the page's 64 keys
        f4v st[4];
#pragma unroll
        for (int kb = 0; kb < 4; ++kb) {
            st[kb] = (f4v){0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                st[kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(b8v, kf[kb][ks]), __builtin_bit_cast(b8v, qh[ks]), st[kb], 0, 0, 0);
                st[kb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(b8v, kf[kb][ks]), __builtin_bit_cast(b8v, ql[ks]), st[kb], 0, 0, 0);
            }
        }
        if (li < li_last) load_keys(page_of(li + 1));
        // st[kb][r]: key pg * 64 + 16 kb + 4 kq + r, query nrow
        float cm = -INFINITY;
        bool vis[4][4];
        float pw[4][4], psum = 0.f;
        if (FORM == 2) {
#pragma unroll
            for (int kb = 0; kb < 4; ++kb)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int j = pg * 64 + 16 * kb + 4 * kq + r;
                    const int dq = pq_eff - j;
                    const bool v = fast_vis ? (unsigned)dq <= dmax
                                            : (qok && j <= pq && (p.window <= 0 || pq - j < p.window || j < p.keep_first) && j >= chunk0);
                    const unsigned bi = min((unsigned)dq, (unsigned)(p.bias_rows - 1));
                    const float rr = has_cap ? __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(sg_k1 * st[kb][r])) : st[kb][r];
                    const float bb = bias_lds ? bias_s[bi] : (p.bias ? fmaf(-kL2e, p.bias[(size_t)g * p.bias_rows + bi], sg_c0) : sg_c0);
                    pw[kb][r] = v ? __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(fmaf(sg_a, rr, bb))) : 0.f;
                }
        }
#pragma unroll
        for (int kb = 0; FORM != 2 && kb < 4; ++kb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int j = pg * 64 + 16 * kb + 4 * kq + r;
                vis[kb][r] = qok && j <= pq && (p.window <= 0 || pq - j < p.window || j < p.keep_first) && (!FORM || j >= chunk0);
                if (FORM && vis[kb][r]) {
                    float sv = st[kb][r];
                    if (p.softcap > 0.f) sv = p.softcap * fast_tanh(sv * inv_cap);
                    if (bias_lds) sv += bias_s[min(pq - j, p.bias_rows - 1)];
                    else if (p.bias) {
                        const int bi = min(pq - j, p.bias_rows - 1);
                        sv += bi < kBiasLds ? bias_s[bi] : p.bias[(size_t)g * p.bias_rows + bi];
                    }
                    st[kb][r] = sv;
                }
                if (FORM != 2 && vis[kb][r]) cm = fmaxf(cm, st[kb][r]);
            }
        constexpr bool sig = FORM == 2;
        if (!sig) {
            cm = fmaxf(cm, __shfl_xor(cm, 16, 64));
            cm = fmaxf(cm, __shfl_xor(cm, 32, 64));
        }
        const float m_new = sig ? 0.f : fmaxf(m_run, cm);
        // (this kernel serves bf16 only: the hardware's exp2 is accurate to 1 ulp of the fp32 result, far inside what the bf16 keys leave)
        constexpr float kLog2e = 1.4426950408889634f;
        const float corr = (sig || m_new == -INFINITY) ? 1.0f : __builtin_amdgcn_exp2f((m_run - m_new) * kLog2e);
#pragma unroll
        for (int kb = 0; !sig && kb < 4; ++kb)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                pw[kb][r] = !vis[kb][r] ? 0.f : __builtin_amdgcn_exp2f((st[kb][r] - m_new) * kLog2e);
                psum += pw[kb][r];
            }
        if (!sig) {
            psum += __shfl_xor(psum, 16, 64);
            psum += __shfl_xor(psum, 32, 64);
        }
        l_run = sig ? 1.0f : l_run * corr + psum;                         // (sigmoid weights: nothing to normalise, ml = (0, 1))
        m_run = m_new;
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) {
            const float v[8] = {pw[2 * h2][0], pw[2 * h2][1], pw[2 * h2][2], pw[2 * h2][3],
                                pw[2 * h2 + 1][0], pw[2 * h2 + 1][1], pw[2 * h2 + 1][2], pw[2 * h2 + 1][3]};
            uint4 hi, lo;
            split8(v, hi, lo);
            pfrag[buf][wave][h2][0][lane] = hi;
            pfrag[buf][wave][h2][1][lane] = lo;
        }
        if (!sig && kq == 0) corr_s[buf][qi] = corr;
        __syncthreads();
        // ---- O^T += V^T P^T for this wave's output blocks and all four query blocks
        if (!sig) {
            float cq[4];
#pragma unroll
            for (int qb = 0; qb < 4; ++qb) cq[qb] = corr_s[buf][16 * qb + nrow];
#pragma unroll
            for (int i = 0; i < kItems; ++i)
#pragma unroll
                for (int qb = 0; qb < 4; ++qb) acc[i][qb] *= cq[qb];
        }
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) {
            uint4 vf[kItems];
#pragma unroll
            for (int i = 0; i < kItems; ++i) {
                const int nb = part * 4 * kItems + wave + 4 * i;
                vf[i] = make_uint4(0, 0, 0, 0);
                if (nb < n_blocks) {
                    const int cc = p.all_kv ? nb / vb_per : c, x = (nb % vb_per) * 16 + nrow;
                    const uint16_t* vr = vc + ((page * G + cc) * vd + x) * 64 + 32 * h2 + 4 * kq;
                    const uint2 a0 = *reinterpret_cast<const uint2*>(vr), a1 = *reinterpret_cast<const uint2*>(vr + 16);
                    vf[i] = make_uint4(a0.x, a0.y, a1.x, a1.y);
                }
            }
#pragma unroll
            for (int qb = 0; qb < 4; ++qb) {
                const uint4 bh = pfrag[buf][qb][h2][0][lane], bl = pfrag[buf][qb][h2][1][lane];
#pragma unroll
                for (int i = 0; i < kItems; ++i) {
                    acc[i][qb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(b8v, vf[i]), __builtin_bit_cast(b8v, bh), acc[i][qb], 0, 0, 0);
                    acc[i][qb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(b8v, vf[i]), __builtin_bit_cast(b8v, bl), acc[i][qb], 0, 0, 0);
                }
            }
        }
    }
    if (kq == 0) { l_s[qi] = l_run; m_s[qi] = m_run; }
    __syncthreads();
    // acc[i][qb][r]: value coordinate 16 (block) + 4 kq + r of query 16 qb + nrow; split 0 of the token's partial sums, unnormalised as the
    // plain kernel leaves them, with (maximum, weight sum): k_head_mix_gate normalises (and counts a sink)
#pragma unroll
    for (int qb = 0; qb < 4; ++qb) {
        const int row = 16 * qb + nrow;
        if (row >= rows) continue;
        const float inv = 1.0f;
        float* out = p.acc + (((size_t)(t0 + row) * p.heads + g) * p.n_splits) * nv;
#pragma unroll
        for (int i = 0; i < kItems; ++i) {
            const int nb = part * 4 * kItems + wave + 4 * i;
            if (nb < n_blocks)
                *reinterpret_cast<float4*>(out + nb * 16 + 4 * kq) = make_float4(acc[i][qb][0] * inv, acc[i][qb][1] * inv, acc[i][qb][2] * inv, acc[i][qb][3] * inv);
        }
    }
    if (part == 0)
        for (int e = tid; e < rows * p.n_splits; e += 256) {
            const int row = e / p.n_splits, sp = e % p.n_splits;
            float* mlp = p.ml + 2 * ((((size_t)(t0 + row) * p.heads + g) * p.n_splits) + sp);
            mlp[0] = sp == 0 ? m_s[row] : -INFINITY;
            mlp[1] = sp == 0 ? l_s[row] : 0.f;
        }
}

struct MixP {
    const float* acc; const float* ml; const float* talk; const float* v_freq; const float* gate; int64_t ldg; int g_col0;
    int heads, kv_heads, vdim, n_splits;
    void* out;
    const float* sink;                                                    // (heads) nullable: exp(sink_h) joins head h's denominator
    int plain_sum;                                                        // the splits hold finished weights (sigmoids): they are added, not normalised
};

// a workgroup per (token, key / value head c): the splits of every source head merged into LDS (for c's values only), then for the heads of
// c's group the mix over source heads, the turn back by the token's own position, the gate.  Without a mixing matrix a head's only source
// is itself.
template <int DT>
__global__ __launch_bounds__(256) void k_head_mix_gate(const MixP p, const zls_batch_t b) {
    extern __shared__ float sh[];
    const int t = blockIdx.x, c = blockIdx.y;
    const int sq = b.tok_seq[t];
    const float pos = (float)(b.seq_pos0[sq] + (t - b.seq_start[sq]));
    const int per = p.heads / p.kv_heads, half = p.vdim >> 1, S = p.n_splits, vd = p.vdim;
    const int nv = p.talk ? p.kv_heads * vd : vd;                         // a head's stride in a split of acc
    const int src0 = p.talk ? 0 : c * per, n_src = p.talk ? p.heads : per, col0 = p.talk ? c * vd : 0;
    float* wsp = sh;                                                      // [n_src][S] weights of the splits
    float* mg = sh + n_src * S;                                           // [n_src][vd] merged sums
    float* tk = mg + n_src * vd;                                          // [per][heads] this group's rows of the mixing matrix
    const float* a = p.acc + (size_t)t * p.heads * S * nv;
    const int lane = threadIdx.x & 63;
    if (S > 1)
        for (int k = threadIdx.x >> 6; k < n_src; k += 4) {               // a wave per source head, a lane per split: all loads at once
            const float2* mlp = reinterpret_cast<const float2*>(p.ml) + ((size_t)t * p.heads + src0 + k) * S;
            if (p.plain_sum) {
                for (int s = lane; s < S; s += 64) wsp[k * S + s] = mlp[s].y > 0.f ? 1.0f : 0.f;
                continue;
            }
            float M = p.sink ? p.sink[src0 + k] : -INFINITY;
            for (int s = lane; s < S; s += 64) M = fmaxf(M, mlp[s].x);
            M = zl_wave_max(M);
            float L = 0.f;
            for (int s = lane; s < S; s += 64) { const float2 v = mlp[s]; L += v.y > 0.f ? v.y * expf(v.x - M) : 0.f; }
            L = zl_wave_sum(L) + (p.sink ? expf(p.sink[src0 + k] - M) : 0.f);
            for (int s = lane; s < S; s += 64) { const float2 v = mlp[s]; wsp[k * S + s] = v.y > 0.f ? expf(v.x - M) / L : 0.f; }
        }
    if (p.talk)
        for (int i = threadIdx.x; i < per * p.heads; i += 256) tk[i] = p.talk[(size_t)c * per * p.heads + i];
    __syncthreads();
    // merged sums: 8 elements per thread at a time, their loads of one split in flight together
    for (int e0 = 0; e0 < n_src * vd; e0 += 8 * 256) {
        float v[8];
        const float* src[8];
        int kk[8];
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const int e = min(e0 + 256 * r + (int)threadIdx.x, n_src * vd - 1);
            kk[r] = e / vd;
            src[r] = a + (size_t)(src0 + kk[r]) * S * nv + col0 + e % vd;
            v[r] = 0.f;
        }
        if (S == 1) {                                                     // one split: its own weight sum (and the sink) normalises it
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                const float* mlp = p.ml + 2 * ((size_t)t * p.heads + src0 + kk[r]);
                float f = p.plain_sum ? 1.0f : 1.0f / mlp[1];
                if (p.sink && !p.plain_sum) {
                    const float sk = p.sink[src0 + kk[r]], M = fmaxf(mlp[0], sk), e = expf(mlp[0] - M);
                    f = e / (mlp[1] * e + expf(sk - M));
                }
                v[r] = f * *src[r];
            }
        } else {
            for (int s = 0; s < S; ++s) {
                float x[8];
#pragma unroll
                for (int r = 0; r < 8; ++r) x[r] = src[r][(size_t)s * nv];
#pragma unroll
                for (int r = 0; r < 8; ++r) {
                    const float w = wsp[kk[r] * S + s];
                    v[r] = w != 0.f ? fmaf(w, x[r], v[r]) : v[r];         // (a split without weight may hold anything)
                }
            }
        }
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            const int e = e0 + 256 * r + (int)threadIdx.x;
            if (e < n_src * vd) mg[e] = v[r];
        }
    }
    __syncthreads();
    // a thread owns a PAIR (m, m + vdim / 2) of one head (an odd vdim without rotation: the last coordinate alone)
    const int pairs = p.v_freq ? half : (vd + 1) / 2;
    for (int w = threadIdx.x; w < per * pairs; w += 256) {
        const int h = c * per + w / pairs, mm = w % pairs;
        const int i0 = mm, i1 = mm + pairs;
        float u = 0.f, v = 0.f;
        if (p.talk) {
            for (int g = 0; g < p.heads; ++g) {
                const float tw = tk[(h - c * per) * p.heads + g];
                u = fmaf(tw, mg[g * vd + i0], u);
                if (i1 < vd) v = fmaf(tw, mg[g * vd + i1], v);
            }
        } else {
            u = mg[(h - src0) * vd + i0];
            if (i1 < vd) v = mg[(h - src0) * vd + i1];
        }
        if (p.v_freq) {
            float sn, cs;
            seq_sincos(pos * p.v_freq[mm], &sn, &cs);                        // turned by -pos: (u cs + v sn, v cs - u sn)
            const float u2 = u * cs + v * sn, v2 = v * cs - u * sn;
            u = u2; v = v2;
        }
        const size_t o = (size_t)t * p.heads * vd + (size_t)h * vd;
        if (p.gate) {
            const float* gr = p.gate + (size_t)t * p.ldg + p.g_col0 + h * vd;
            u *= seq_sigmoid(gr[i0]);
            if (i1 < vd) v *= seq_sigmoid(gr[i1]);
        }
        SeqT<DT>::st(p.out, o + i0, u);
        if (i1 < vd) SeqT<DT>::st(p.out, o + i1, v);
    }
}

}  // namespace

extern "C" int zls_rope_norm_store(float* proj, int64_t ld, int64_t q_col0, int64_t k_col0, int64_t v_col0, int64_t heads, int64_t kv_heads,
                                   int64_t dim, int64_t vdim, const float* qk_freq, int64_t rot_dims, const float* v_freq, float eps, int qk_norm,
                                   int interleaved, const float* vmix_src, int64_t vmix_ld, int64_t vmix_col0, float vmix_lambda,
                                   const float* q_norm_w, const float* k_norm_w, const zls_batch_t* b, void* k_cache, void* v_cache, int dtype,
                                   zl_stream_t s) {
    ZL_CHECK_ARG(proj && seq_batch_ok(b) && b->page_table && b->page_size > 0 && heads > 0 && kv_heads > 0 && dim > 0 && vdim > 0, ZL_EINVAL);
    ZL_CHECK_ARG((k_cache == nullptr) == (v_cache == nullptr), ZL_EINVAL);
    ZL_CHECK_ARG(rot_dims >= 0 && rot_dims <= dim && rot_dims % 2 == 0 && (rot_dims == 0 || qk_freq) && (!v_freq || vdim % 2 == 0), ZL_ESHAPE);
    ZL_CHECK_ARG(dim <= 64 * kMaxE && vdim <= 64 * kMaxE, ZL_ELIMIT);
    ZL_CHECK_ARG(q_col0 >= 0 && q_col0 + heads * dim <= ld, ZL_ESHAPE);
    ZL_CHECK_ARG(!k_cache || (k_col0 >= 0 && k_col0 + kv_heads * dim <= ld && v_col0 >= 0 && v_col0 + kv_heads * vdim <= ld), ZL_ESHAPE);
    RopeP p;
    p.proj = proj; p.ld = ld; p.q_col0 = (int)q_col0; p.k_col0 = (int)k_col0; p.v_col0 = (int)v_col0; p.heads = (int)heads;
    p.kv_heads = (int)kv_heads; p.dim = (int)dim; p.vdim = (int)vdim; p.rot_dims = (int)rot_dims; p.qk_norm = qk_norm; p.qk_freq = qk_freq;
    p.v_freq = v_freq; p.eps = eps; p.k_cache = k_cache; p.v_cache = v_cache;
    ZL_CHECK_ARG(!vmix_src || (vmix_col0 >= 0 && vmix_col0 + kv_heads * vdim <= vmix_ld), ZL_ESHAPE);
    p.q_w = qk_norm ? q_norm_w : nullptr; p.k_w = qk_norm ? k_norm_w : nullptr;
    p.interleaved = interleaved ? 1 : 0; p.vmix_src = vmix_src; p.vmix_ld = vmix_ld; p.vmix_col0 = (int)vmix_col0; p.vmix_lambda = vmix_lambda;
#define CALL(DT) hipLaunchKernelGGL((k_rope_norm_store<DT>), dim3(b->n_tok), dim3(256), 0, (hipStream_t)s, p, *b);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}

// the optional score form of a launch (NULL: plain scaled scores and a softmax)
static int set_form(AttnP& p, const zls_score_form_t* f) {
    if (!f) return ZL_OK;
    ZL_CHECK_ARG((!f->bias || f->bias_rows > 0) && f->chunk >= 0 && f->chunk < (1 << 30), ZL_ESHAPE);
    ZL_CHECK_ARG(!(f->chunk > 0 && p.keep_first > 0), ZL_ESHAPE);        // (kept first keys belong to a sliding window, not to chunks)
    p.head_scale = f->head_scale; p.softcap = f->softcap; p.bias = f->bias; p.bias_rows = f->bias_rows; p.offset = f->offset;
    p.chunk = f->chunk; p.sigmoid = f->sigmoid ? 1 : 0;
    return ZL_OK;
}

extern "C" int zls_window_attention(const float* q, int64_t ldq, int64_t q_col0, const void* k_cache, const void* v_cache, const zls_batch_t* b,
                                    float scale, int64_t window, int64_t keep_first, int64_t heads, int64_t kv_heads, int64_t dim, int64_t vdim,
                                    int all_kv, float* acc, float* ml, int64_t n_splits, int64_t pages_per_split, int single_only,
                                    const zls_score_form_t* form, int dtype, zl_stream_t s) {
    ZL_CHECK_ARG(q && k_cache && v_cache && acc && ml && seq_batch_ok(b) && b->page_table && b->page_size > 0, ZL_EINVAL);
    ZL_CHECK_ARG(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && dim > 0 && vdim > 0 && heads <= 65535, ZL_ESHAPE);
    ZL_CHECK_ARG(q_col0 >= 0 && q_col0 + heads * dim <= ldq && window < (1 << 30) && n_splits >= 1 && n_splits <= 65535 && pages_per_split >= 1 &&
                 keep_first >= 0 && keep_first < (1 << 30), ZL_ESHAPE);
    ZL_CHECK_ARG((all_kv ? kv_heads : 1) * vdim <= 256 * kMaxV && dim <= 8192 && b->page_size <= kChunk && b->page_size % 8 == 0, ZL_ELIMIT);
    AttnP p = {};
    p.q = q; p.ldq = ldq; p.q_col0 = (int)q_col0; p.k_cache = k_cache; p.v_cache = v_cache; p.scale = scale; p.window = (int)window;
    p.heads = (int)heads; p.kv_heads = (int)kv_heads; p.dim = (int)dim; p.vdim = (int)vdim; p.all_kv = all_kv ? 1 : 0; p.acc = acc; p.ml = ml;
    p.n_splits = (int)n_splits; p.pages_per_split = (int)pages_per_split; p.single_only = single_only ? 1 : 0;
    p.keep_first = p.window > 0 ? (int)keep_first : 0;
    const int st = set_form(p, form);
    if (st != ZL_OK) return st;
    const size_t lds = (size_t)dim * sizeof(float);
    const dim3 grid(b->n_tok, (unsigned)heads, (unsigned)n_splits);
#define CALL(DT)                                                                                            \
    if (form) hipLaunchKernelGGL((k_window_attention<DT, 1>), grid, dim3(256), lds, (hipStream_t)s, p, *b); \
    else hipLaunchKernelGGL((k_window_attention<DT, 0>), grid, dim3(256), lds, (hipStream_t)s, p, *b);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}

extern "C" int zls_window_attention_prompt(const float* q, int64_t ldq, int64_t q_col0, const void* k_cache, const void* v_cache,
                                           const zls_batch_t* b, const int32_t* tiles, int64_t n_tiles, float scale, int64_t window,
                                           int64_t keep_first, int64_t heads, int64_t kv_heads, int64_t dim, int64_t vdim, int all_kv, float* acc, float* ml, int64_t n_splits,
                                           const zls_score_form_t* form, int dtype, zl_stream_t s) {
    ZL_CHECK_ARG(q && k_cache && v_cache && acc && ml && tiles && n_tiles > 0 && seq_batch_ok(b) && b->page_table, ZL_EINVAL);
    ZL_CHECK_ARG(dtype == ZL_BF16, ZL_EDTYPE);
    ZL_CHECK_ARG(heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && heads <= 65535 && n_splits >= 1 && q_col0 >= 0 && q_col0 + heads * dim <= ldq,
                 ZL_ESHAPE);
    ZL_CHECK_ARG(b->page_size == 64 && dim > 0 && dim % 8 == 0 && dim <= 256 && vdim > 0 && vdim % 16 == 0 && window < (1 << 30) &&
                 keep_first >= 0 && keep_first < (1 << 30), ZL_ESHAPE);
    AttnP p = {};
    p.q = q; p.ldq = ldq; p.q_col0 = (int)q_col0; p.k_cache = k_cache; p.v_cache = v_cache; p.scale = scale; p.window = (int)window;
    p.heads = (int)heads; p.kv_heads = (int)kv_heads; p.dim = (int)dim; p.vdim = (int)vdim; p.all_kv = all_kv ? 1 : 0; p.acc = acc; p.ml = ml;
    p.n_splits = (int)n_splits; p.tiles = tiles; p.keep_first = p.window > 0 ? (int)keep_first : 0;
    const int st = set_form(p, form);
    if (st != ZL_OK) return st;
    const int64_t n_blocks = (all_kv ? kv_heads : 1) * vdim / 16, parts = (n_blocks + 4 * kItems - 1) / (4 * kItems);
    ZL_CHECK_ARG(parts <= 65535, ZL_ELIMIT);
    const dim3 grid((unsigned)n_tiles, (unsigned)heads, (unsigned)parts);
    hipStream_t hs = (hipStream_t)s;
    const int ks = (int)((dim + 31) / 32);
#define PROMPT(KS)                                                                                      \
    if (form && form->sigmoid) hipLaunchKernelGGL((k_window_attention_mfma<KS, 2>), grid, dim3(256), 0, hs, p, *b); \
    else if (form) hipLaunchKernelGGL((k_window_attention_mfma<KS, 1>), grid, dim3(256), 0, hs, p, *b); \
    else hipLaunchKernelGGL((k_window_attention_mfma<KS, 0>), grid, dim3(256), 0, hs, p, *b)
    if (ks <= 1) { PROMPT(1); }
    else if (ks <= 2) { PROMPT(2); }
    else if (ks <= 3) { PROMPT(3); }
    else if (ks <= 4) { PROMPT(4); }
    else if (ks <= 6) { PROMPT(6); }
    else { PROMPT(8); }
#undef PROMPT
    return zl_launch_status();
}

extern "C" int zls_head_mix_gate(const float* acc, const float* ml, int64_t n_splits, const float* talk, const float* v_freq, const float* gate,
                                 int64_t ldg, int64_t g_col0, const float* sink, int plain_sum, const zls_batch_t* b, int64_t heads,
                                 int64_t kv_heads, int64_t vdim, void* out, int dtype, zl_stream_t s) {
    ZL_CHECK_ARG(acc && ml && out && seq_batch_ok(b) && heads > 0 && kv_heads > 0 && heads % kv_heads == 0 && vdim > 0 && n_splits >= 1, ZL_EINVAL);
    ZL_CHECK_ARG((!v_freq || vdim % 2 == 0) && (!gate || (g_col0 >= 0 && g_col0 + heads * vdim <= ldg)), ZL_ESHAPE);
    const int64_t n_src = talk ? heads : heads / kv_heads;
    const size_t lds = (size_t)(n_src * (n_splits + vdim) + (talk ? heads / kv_heads * heads : 0)) * sizeof(float);
    ZL_CHECK_ARG(lds <= 64 * 1024 && kv_heads <= 65535, ZL_ELIMIT);
    MixP p;
    p.acc = acc; p.ml = ml; p.n_splits = (int)n_splits; p.talk = talk; p.v_freq = v_freq; p.gate = gate; p.ldg = ldg; p.g_col0 = (int)g_col0;
    p.heads = (int)heads; p.kv_heads = (int)kv_heads; p.vdim = (int)vdim; p.out = out; p.sink = sink;
    p.plain_sum = plain_sum ? 1 : 0;
#define CALL(DT) hipLaunchKernelGGL((k_head_mix_gate<DT>), dim3(b->n_tok, (unsigned)kv_heads), dim3(256), lds, (hipStream_t)s, p, *b);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}
