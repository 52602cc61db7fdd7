// seq_elem.hip -- the per-token steps between the matrix products of a ragged step: embedding with learned positions, token shift with
// its carried row, the scalar-gain RMS norm fused with the residual sum, the gathered final norm, PolyNorm, layer norm, the weighted RMS
// norm before a sub-layer (alone, or fused with the residual sum that precedes it), scaled and soft-capped logits, and the same two steps
// for a residual kept as SEVERAL streams (k_streams_norm, k_streams_update): a sub-layer reads a weighted sum of the streams, its result --
// optionally gated by a sigmoid -- goes to every stream with a factor of its own while the streams are mixed by a small matrix.
// One workgroup per token row; every sum of squares is fp32 (butterfly inside a wave, waves in order).
#include "seq_common.h"

namespace {

constexpr int kT = 256;

template <int DT>
__global__ __launch_bounds__(kT) void k_embed(const int32_t* __restrict__ tokens, const void* __restrict__ table, const void* __restrict__ pos_table,
                                              int vocab, int max_pos, float scale, const zls_batch_t b, float* __restrict__ x, int width) {
    const int t = blockIdx.x;
    const int sq = b.tok_seq[t];
    int pos = b.seq_pos0[sq] + (t - b.seq_start[sq]);
    int tok = tokens[t];
    tok = tok < 0 ? 0 : (tok >= vocab ? vocab - 1 : tok);
    pos = pos >= max_pos ? max_pos - 1 : pos;                       // (the host refuses such a step; never an out-of-bounds read)
    for (int i = threadIdx.x; i < width; i += kT) {
        float v = SeqT<DT>::ld(table, (size_t)tok * width + i) * scale;
        if (pos_table) v += SeqT<DT>::ld(pos_table, (size_t)pos * width + i);
        x[(size_t)t * width + i] = v;
    }
}

// the workgroup of a portion's FIRST token reads prev[slot] and, once it has, replaces it with the portion's last row: no other workgroup
// touches that slot's row, and each thread reads its own elements before it writes them
template <int DT>
__global__ __launch_bounds__(kT) void k_token_shift(const float* __restrict__ x, const float* __restrict__ mix, float* __restrict__ prev,
                                                    const zls_batch_t b, void* __restrict__ h, int width) {
    const int t = blockIdx.x;
    const int sq = b.tok_seq[t];
    const int first = b.seq_start[sq], last = b.seq_start[sq + 1] - 1;
    const bool head = t == first;
    float* pr = prev + (size_t)b.seq_slot[sq] * width;
    const float* before = head ? pr : x + (size_t)(t - 1) * width;
    for (int i = threadIdx.x; i < width; i += kT) {
        const float cur = x[(size_t)t * width + i];
        const float pv = before[i];
        SeqT<DT>::st(h, (size_t)t * width + i, cur + (pv - cur) * mix[i]);
        if (head) pr[i] = x[(size_t)last * width + i];
    }
}

template <int DT>
__global__ __launch_bounds__(kT) void k_add_scalar_norm(float* __restrict__ x, const float* __restrict__ y, float gain, float eps, int width,
                                                        void* __restrict__ xt) {
    __shared__ float red[16];
    const size_t row = (size_t)blockIdx.x * width;
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += kT) { const float v = y[row + i]; ss = fmaf(v, v, ss); }
    ss = zl_block_sum(ss, red);
    const float f = gain / sqrtf(ss / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += kT) {
        const float v = x[row + i] + y[row + i] * f;
        x[row + i] = v;
        if (xt) SeqT<DT>::st(xt, row + i, v);                   // the sum once more in the serving format, for the next matrix product
    }
}

template <int DT>
__global__ __launch_bounds__(kT) void k_scalar_norm_rows(const float* __restrict__ x, const int32_t* __restrict__ rows, float gain, float eps,
                                                         int width, void* __restrict__ out) {
    __shared__ float red[16];
    const size_t row = (size_t)rows[blockIdx.x] * width, orow = (size_t)blockIdx.x * width;
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += kT) { const float v = x[row + i]; ss = fmaf(v, v, ss); }
    ss = zl_block_sum(ss, red);
    const float f = gain / sqrtf(ss / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += kT) SeqT<DT>::st(out, orow + i, x[row + i] * f);
}

template <int DT>
__global__ __launch_bounds__(kT) void k_polynorm(const float* __restrict__ z, float a, float bq, float c, float e, float eps, int ff,
                                                 void* __restrict__ out) {
    __shared__ float red[16];
    const size_t row = (size_t)blockIdx.x * ff;
    float s1 = 0.f, s2 = 0.f, s3 = 0.f;
    for (int i = threadIdx.x; i < ff; i += kT) {
        const float v = z[row + i], v2 = v * v, v3 = v2 * v;
        s1 = fmaf(v, v, s1); s2 = fmaf(v2, v2, s2); s3 = fmaf(v3, v3, s3);
    }
    s1 = zl_block_sum(s1, red);
    s2 = zl_block_sum(s2, red);
    s3 = zl_block_sum(s3, red);
    const float f1 = a / sqrtf(s1 / (float)ff + eps), f2 = bq / sqrtf(s2 / (float)ff + eps), f3 = c / sqrtf(s3 / (float)ff + eps);
    for (int i = threadIdx.x; i < ff; i += kT) {
        const float v = z[row + i], v2 = v * v;
        SeqT<DT>::st(out, row + i, v * f1 + v2 * f2 + v2 * v * f3 + e);
    }
}

// mean first, then the mean of the squared deviations (both fp32): the row is read three times, from L1 / L2 after the first
__device__ __forceinline__ void ln_moments(const float* __restrict__ r, int width, float eps, float* red, float& mean, float& inv) {
    float sum = 0.f;
    for (int i = threadIdx.x; i < width; i += kT) sum += r[i];
    mean = zl_block_sum(sum, red) / (float)width;
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += kT) { const float d = r[i] - mean; ss = fmaf(d, d, ss); }
    inv = 1.0f / sqrtf(zl_block_sum(ss, red) / (float)width + eps);
}

template <int DT>
__global__ __launch_bounds__(kT) void k_layer_norm(const float* __restrict__ x, const int32_t* __restrict__ rows, const float* __restrict__ w,
                                                   const float* __restrict__ bias, float eps, int width, void* __restrict__ out) {
    __shared__ float red[16];
    const float* r = x + (size_t)(rows ? rows[blockIdx.x] : (int)blockIdx.x) * width;
    const size_t orow = (size_t)blockIdx.x * width;
    float mean, inv;
    ln_moments(r, width, eps, red, mean, inv);
    for (int i = threadIdx.x; i < width; i += kT) SeqT<DT>::st(out, orow + i, (r[i] - mean) * inv * w[i] + (bias ? bias[i] : 0.f));
}

// x += LN(y); optionally the NEXT sub-layer's input LN2(x) in the serving format from the same workgroup (the new row is in L1)
template <int DT>
__global__ __launch_bounds__(kT) void k_add_layer_norm(float* __restrict__ x, const float* __restrict__ y, const float* __restrict__ w,
                                                       const float* __restrict__ bias, float eps, int width, const float* __restrict__ w2,
                                                       const float* __restrict__ bias2, void* __restrict__ h2) {
    __shared__ float red[16];
    const size_t row = (size_t)blockIdx.x * width;
    float mean, inv;
    ln_moments(y + row, width, eps, red, mean, inv);
    for (int i = threadIdx.x; i < width; i += kT) x[row + i] += (y[row + i] - mean) * inv * w[i] + (bias ? bias[i] : 0.f);
    if (!w2) return;
    __syncthreads();                                             // (each thread re-reads rows that other threads wrote)
    ln_moments(x + row, width, eps, red, mean, inv);
    for (int i = threadIdx.x; i < width; i += kT) SeqT<DT>::st(h2, row + i, (x[row + i] - mean) * inv * w2[i] + (bias2 ? bias2[i] : 0.f));
}

// x / sqrt(mean(x^2) + eps) * (w + shift): shift 1 for weights stored around zero, 0 for plain weights
template <int DT>
__global__ __launch_bounds__(kT) void k_rms_norm(const float* __restrict__ x, const int32_t* __restrict__ rows, const float* __restrict__ w,
                                                 float shift, float eps, int width, void* __restrict__ out) {
    __shared__ float red[16];
    const float* r = x + (size_t)(rows ? rows[blockIdx.x] : (int)blockIdx.x) * width;
    const size_t orow = (size_t)blockIdx.x * width;
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += kT) ss = fmaf(r[i], r[i], ss);
    const float f = 1.0f / sqrtf(zl_block_sum(ss, red) / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += kT) SeqT<DT>::st(out, orow + i, r[i] * f * (w[i] + shift));
}

// x += y (fp32, in place); optionally the NEXT sub-layer's input, the weighted RMS norm of the new row, in the serving format
template <int DT>
__global__ __launch_bounds__(kT) void k_add_rms_norm(float* __restrict__ x, const float* __restrict__ y, float eps, int width,
                                                     const float* __restrict__ w2, float shift, void* __restrict__ h2) {
    __shared__ float red[16];
    const size_t row = (size_t)blockIdx.x * width;
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += kT) {          // (a thread re-reads below only what it wrote itself)
        const float v = x[row + i] + y[row + i];
        x[row + i] = v;
        ss = fmaf(v, v, ss);
    }
    if (!w2) return;
    const float f = 1.0f / sqrtf(zl_block_sum(ss, red) / (float)width + eps);
    for (int i = threadIdx.x; i < width; i += kT) SeqT<DT>::st(h2, row + i, x[row + i] * f * (w2[i] + shift));
}

// z <- cap * tanh(z * scale / cap) (cap <= 0: z * scale)
__global__ __launch_bounds__(kT) void k_scale_softcap(float* __restrict__ z, int64_t n, float scale, float cap) {
    const int64_t i = (int64_t)blockIdx.x * kT + threadIdx.x;
    if (i >= n) return;
    const float v = z[i] * scale;
    z[i] = cap > 0.f ? cap * tanhf(v / cap) : v;
}

constexpr int kMaxStreams = 8;

struct StreamsP {
    const float* src; int64_t src_tok, src_stream;      // the streams that are read: element (t, s, i) at t * src_tok + s * src_stream + i
    float* dst;                                         // the streams that are written, (n_tok, n, width) -- may be src
    int n, width;
    const float* y;                                     // the sub-layer's result (n_tok, width)
    const float* gate; int64_t ldg; int g_col0;         // nullable: y *= sigmoid(gate[t][g_col0 + i] + gate_bias[i])
    const float* gate_bias;
    const float* mix; const float* out_coef;            // (n, n) indexed [from][to]; (n)
    const float* read_coef;                             // (n) nullable: the coefficients of the sum that is normed (NULL in k_streams_norm: all 1)
    const int32_t* rows;                                // k_streams_norm: nullable gather
    const float* w; float shift, eps;
    void* h;                                            // the normed sum, (rows, width) in the serving format
};

// h[r] = norm(sum_s read_coef[s] x_s[row]) * (w + shift); the sum is taken in the order of the streams, fp32
template <int DT>
__global__ __launch_bounds__(kT) void k_streams_norm(const StreamsP p) {
    extern __shared__ float u[];
    __shared__ float red[16];
    float rc[kMaxStreams];
#pragma unroll
    for (int s = 0; s < kMaxStreams; ++s) rc[s] = s < p.n ? (p.read_coef ? p.read_coef[s] : 1.0f) : 0.f;
    const size_t row = p.rows ? (size_t)p.rows[blockIdx.x] : (size_t)blockIdx.x;
    const float* x = p.src + row * p.src_tok;
    float ss = 0.f;
    for (int i = threadIdx.x; i < p.width; i += kT) {
        float a = 0.f;
#pragma unroll
        for (int s = 0; s < kMaxStreams; ++s)
            if (s < p.n) a = fmaf(rc[s], x[(size_t)s * p.src_stream + i], a);
        u[i] = a;
        ss = fmaf(a, a, ss);
    }
    const float f = 1.0f / sqrtf(zl_block_sum(ss, red) / (float)p.width + p.eps);
    for (int i = threadIdx.x; i < p.width; i += kT) SeqT<DT>::st(p.h, (size_t)blockIdx.x * p.width + i, u[i] * f * (p.w[i] + p.shift));
}

// V consecutive fp32 numbers (V = 4: one 16-byte access)
template <int V> struct VecF;
template <> struct VecF<1> {
    static __device__ __forceinline__ void ld(const float* p, float* v) { v[0] = *p; }
    static __device__ __forceinline__ void st(float* p, const float* v) { *p = v[0]; }
};
template <> struct VecF<4> {
    static __device__ __forceinline__ void ld(const float* p, float* v) {
        const float4 a = *reinterpret_cast<const float4*>(p);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    }
    static __device__ __forceinline__ void st(float* p, const float* v) { *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]); }
};

// x_t <- sum_s mix[s][t] x_s + out_coef[t] * y * sigmoid(gate + bias), all streams from the old ones (a thread holds its elements of every
// stream in registers before it writes); with read_coef also the NEXT sub-layer's input, the normed weighted sum of the new streams.
// N streams (the coefficients sit in registers, every loop unrolled), V elements per thread and access.
template <int DT, int N, int V>
__global__ __launch_bounds__(kT) void k_streams_update(const StreamsP p) {
    extern __shared__ float u[];
    __shared__ float red[16];
    float cm[N][N], co[N], cr[N];
#pragma unroll
    for (int s = 0; s < N; ++s) {
#pragma unroll
        for (int d = 0; d < N; ++d) cm[s][d] = p.mix[s * N + d];
        co[s] = p.out_coef[s];
        cr[s] = p.read_coef ? p.read_coef[s] : 0.f;
    }
    const size_t t = blockIdx.x;
    const float* x = p.src + t * p.src_tok;
    float* o = p.dst + t * (size_t)N * p.width;
    float ss = 0.f;
    for (int i = threadIdx.x * V; i < p.width; i += kT * V) {
        float old[N][V], yv[V];
#pragma unroll
        for (int s = 0; s < N; ++s) VecF<V>::ld(x + (size_t)s * p.src_stream + i, old[s]);
        VecF<V>::ld(p.y + t * p.width + i, yv);
        if (p.gate) {
            float g[V], gb[V];
            VecF<V>::ld(p.gate + t * p.ldg + p.g_col0 + i, g);
#pragma unroll
            for (int e = 0; e < V; ++e) gb[e] = 0.f;
            if (p.gate_bias) VecF<V>::ld(p.gate_bias + i, gb);
#pragma unroll
            for (int e = 0; e < V; ++e) yv[e] *= seq_sigmoid(g[e] + gb[e]);
        }
        float a[V];
#pragma unroll
        for (int e = 0; e < V; ++e) a[e] = 0.f;
#pragma unroll
        for (int d = 0; d < N; ++d) {
            float v[V];
#pragma unroll
            for (int e = 0; e < V; ++e) {
                float acc = 0.f;
#pragma unroll
                for (int s = 0; s < N; ++s) acc = fmaf(cm[s][d], old[s][e], acc);
                v[e] = fmaf(co[d], yv[e], acc);
                a[e] = fmaf(cr[d], v[e], a[e]);
            }
            VecF<V>::st(o + (size_t)d * p.width + i, v);
        }
#pragma unroll
        for (int e = 0; e < V; ++e) { u[i + e] = a[e]; ss = fmaf(a[e], a[e], ss); }
    }
    if (!p.read_coef) return;
    const float f = 1.0f / sqrtf(zl_block_sum(ss, red) / (float)p.width + p.eps);
    for (int i = threadIdx.x; i < p.width; i += kT) SeqT<DT>::st(p.h, t * p.width + i, u[i] * f * (p.w[i] + p.shift));
}

// out = act(z): kind 0 relu(z)^2, 1 gelu_tanh(z), 2 silu(z); V consecutive elements of a row per thread
template <int DT, int V>
__global__ __launch_bounds__(kT) void k_unary_act(const float* __restrict__ z, int64_t ldz, int64_t rows, int64_t cols, int kind, void* __restrict__ out) {
    const int64_t e = ((int64_t)blockIdx.x * kT + threadIdx.x) * V;
    if (e >= rows * cols) return;
    float v[V];
    VecF<V>::ld(z + (e / cols) * ldz + e % cols, v);
#pragma unroll
    for (int i = 0; i < V; ++i) {
        float r;
        if (kind == 0) { const float m = fmaxf(v[i], 0.f); r = m * m; }
        else if (kind == 1) r = 0.5f * v[i] * (1.0f + tanhf(0.7978845608028654f * (v[i] + 0.044715f * v[i] * v[i] * v[i])));
        else r = seq_silu(v[i]);
        SeqT<DT>::st(out, (size_t)e + i, r);
    }
}

}  // namespace

extern "C" int zls_embed(const int32_t* tokens, const void* table, const void* pos_table, int64_t vocab, int64_t max_positions, float scale,
                         const zls_batch_t* b, float* x, int64_t width, int dtype, zl_stream_t s) {
    ZL_CHECK_ARG(tokens && table && x && seq_batch_ok(b) && width > 0 && vocab > 0, ZL_EINVAL);
    ZL_CHECK_ARG(!pos_table || max_positions > 0, ZL_EINVAL);
#define CALL(DT) hipLaunchKernelGGL((k_embed<DT>), dim3(b->n_tok), dim3(kT), 0, (hipStream_t)s, tokens, table, pos_table, (int)vocab, \
                                    (int)max_positions, scale, *b, x, (int)width);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}

extern "C" int zls_token_shift(const float* x, const float* mix, float* prev, const zls_batch_t* b, void* h, int64_t width, int dtype,
                               zl_stream_t s) {
    ZL_CHECK_ARG(x && mix && prev && h && seq_batch_ok(b) && width > 0, ZL_EINVAL);
#define CALL(DT) hipLaunchKernelGGL((k_token_shift<DT>), dim3(b->n_tok), dim3(kT), 0, (hipStream_t)s, x, mix, prev, *b, h, (int)width);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}

extern "C" int zls_add_scalar_norm(float* x, const float* y, float gain, float eps, int64_t rows, int64_t width, void* xt, int dtype,
                                   zl_stream_t s) {
    ZL_CHECK_ARG(x && y && rows > 0 && width > 0, ZL_EINVAL);
#define CALL(DT) hipLaunchKernelGGL((k_add_scalar_norm<DT>), dim3((unsigned)rows), dim3(kT), 0, (hipStream_t)s, x, y, gain, eps, (int)width, xt);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}

extern "C" int zls_scalar_norm_rows(const float* x, const int32_t* rows, float gain, float eps, int64_t n_rows, int64_t width, void* out,
                                    int dtype, zl_stream_t s) {
    ZL_CHECK_ARG(x && rows && out && n_rows > 0 && width > 0, ZL_EINVAL);
#define CALL(DT) hipLaunchKernelGGL((k_scalar_norm_rows<DT>), dim3((unsigned)n_rows), dim3(kT), 0, (hipStream_t)s, x, rows, gain, eps, (int)width, out);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}

extern "C" int zls_polynorm(const float* z, const float* coef, float eps, int64_t rows, int64_t ff, void* out, int dtype, zl_stream_t s) {
    ZL_CHECK_ARG(z && coef && out && rows > 0 && ff > 0, ZL_EINVAL);
#define CALL(DT) hipLaunchKernelGGL((k_polynorm<DT>), dim3((unsigned)rows), dim3(kT), 0, (hipStream_t)s, z, coef[0], coef[1], coef[2], coef[3], eps, (int)ff, out);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}

extern "C" int zls_layer_norm(const float* x, const int32_t* rows, const float* w, const float* b, float eps, int64_t n_rows, int64_t width,
                              void* out, int dtype, zl_stream_t s) {
    ZL_CHECK_ARG(x && w && out && n_rows > 0 && width > 0, ZL_EINVAL);
#define CALL(DT) hipLaunchKernelGGL((k_layer_norm<DT>), dim3((unsigned)n_rows), dim3(kT), 0, (hipStream_t)s, x, rows, w, b, eps, (int)width, out);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}

extern "C" int zls_add_layer_norm(float* x, const float* y, const float* w, const float* b, float eps, int64_t rows, int64_t width,
                                  const float* w2, const float* b2, void* h2, int dtype, zl_stream_t s) {
    ZL_CHECK_ARG(x && y && w && rows > 0 && width > 0 && (!w2 || h2), ZL_EINVAL);
#define CALL(DT) hipLaunchKernelGGL((k_add_layer_norm<DT>), dim3((unsigned)rows), dim3(kT), 0, (hipStream_t)s, x, y, w, b, eps, (int)width, w2, b2, h2);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}

extern "C" int zls_rms_norm(const float* x, const int32_t* rows, const float* w, float shift, float eps, int64_t n_rows, int64_t width, void* out,
                            int dtype, zl_stream_t s) {
    ZL_CHECK_ARG(x && w && out && n_rows > 0 && width > 0, ZL_EINVAL);
#define CALL(DT) hipLaunchKernelGGL((k_rms_norm<DT>), dim3((unsigned)n_rows), dim3(kT), 0, (hipStream_t)s, x, rows, w, shift, eps, (int)width, out);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}

extern "C" int zls_add_rms_norm(float* x, const float* y, float eps, int64_t rows, int64_t width, const float* w2, float shift, void* h2, int dtype,
                                zl_stream_t s) {
    ZL_CHECK_ARG(x && y && rows > 0 && width > 0 && (!w2 || h2), ZL_EINVAL);
#define CALL(DT) hipLaunchKernelGGL((k_add_rms_norm<DT>), dim3((unsigned)rows), dim3(kT), 0, (hipStream_t)s, x, y, eps, (int)width, w2, shift, h2);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}

extern "C" int zls_scale_softcap(float* z, int64_t n, float scale, float cap, zl_stream_t s) {
    ZL_CHECK_ARG(z && n > 0 && n < (1LL << 40), ZL_EINVAL);
    hipLaunchKernelGGL(k_scale_softcap, dim3((unsigned)((n + kT - 1) / kT)), dim3(kT), 0, (hipStream_t)s, z, n, scale, cap);
    return zl_launch_status();
}

extern "C" int zls_streams_norm(const float* src, int64_t src_tok, int64_t src_stream, int64_t n, const float* read_coef, const int32_t* rows,
                                const float* w, float shift, float eps, int64_t n_rows, int64_t width, void* h, int dtype, zl_stream_t s) {
    ZL_CHECK_ARG(src && w && h && n_rows > 0 && width > 0 && n > 0 && src_tok >= 0 && src_stream >= 0, ZL_EINVAL);
    ZL_CHECK_ARG(n <= kMaxStreams && width * sizeof(float) <= 64 * 1024, ZL_ELIMIT);
    StreamsP p = {};
    p.src = src; p.src_tok = src_tok; p.src_stream = src_stream; p.n = (int)n; p.width = (int)width; p.read_coef = read_coef; p.rows = rows;
    p.w = w; p.shift = shift; p.eps = eps; p.h = h;
#define CALL(DT) hipLaunchKernelGGL((k_streams_norm<DT>), dim3((unsigned)n_rows), dim3(kT), (size_t)width * sizeof(float), (hipStream_t)s, p);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}

extern "C" int zls_streams_update(const float* src, int64_t src_tok, int64_t src_stream, float* dst, int64_t n, const float* y, const float* gate,
                                  int64_t ldg, int64_t g_col0, const float* gate_bias, const float* mix, const float* out_coef,
                                  const float* read_coef, const float* w, float shift, float eps, int64_t n_tok, int64_t width, void* h, int dtype,
                                  zl_stream_t s) {
    ZL_CHECK_ARG(src && dst && y && mix && out_coef && n_tok > 0 && width > 0 && n > 0 && src_tok >= 0 && src_stream >= 0, ZL_EINVAL);
    ZL_CHECK_ARG((!read_coef || (w && h)) && (!gate || (g_col0 >= 0 && g_col0 + width <= ldg)), ZL_ESHAPE);
    ZL_CHECK_ARG(n <= kMaxStreams && width * sizeof(float) <= 64 * 1024, ZL_ELIMIT);
    StreamsP p = {};
    p.src = src; p.src_tok = src_tok; p.src_stream = src_stream; p.dst = dst; p.n = (int)n; p.width = (int)width; p.y = y; p.gate = gate;
    p.ldg = ldg; p.g_col0 = (int)g_col0; p.gate_bias = gate_bias; p.mix = mix; p.out_coef = out_coef; p.read_coef = read_coef; p.w = w;
    p.shift = shift; p.eps = eps; p.h = h;
    // 16-byte accesses when every row that is read or written starts on a 16-byte boundary
    auto al = [](const void* q) { return ((uintptr_t)q & 15) == 0; };
    const bool vec = width % 4 == 0 && src_tok % 4 == 0 && src_stream % 4 == 0 && al(src) && al(dst) && al(y) &&
                     (!gate || (ldg % 4 == 0 && g_col0 % 4 == 0 && al(gate))) && (!gate_bias || al(gate_bias));
    const dim3 grid((unsigned)n_tok);
    const size_t lds = (size_t)width * sizeof(float);
#define GO(DT, N)                                                                                          \
    if (vec) hipLaunchKernelGGL((k_streams_update<DT, N, 4>), grid, dim3(kT), lds, (hipStream_t)s, p);     \
    else hipLaunchKernelGGL((k_streams_update<DT, N, 1>), grid, dim3(kT), lds, (hipStream_t)s, p);
#define CALL(DT)                                                                                           \
    switch (n) {                                                                                           \
        case 1: GO(DT, 1) break; case 2: GO(DT, 2) break; case 3: GO(DT, 3) break; case 4: GO(DT, 4) break; \
        case 5: GO(DT, 5) break; case 6: GO(DT, 6) break; case 7: GO(DT, 7) break; default: GO(DT, 8) break; \
    }
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
#undef GO
    return zl_launch_status();
}

extern "C" int zls_unary_act(const float* z, int64_t ldz, int64_t rows, int64_t cols, int kind, void* out, int dtype, zl_stream_t s) {
    ZL_CHECK_ARG(z && out && rows > 0 && cols > 0 && ldz >= cols && kind >= 0 && kind <= 2, ZL_EINVAL);
    const int64_t n = rows * cols;
    ZL_CHECK_ARG(n < (1LL << 40), ZL_ELIMIT);
    const bool vec = cols % 4 == 0 && ldz % 4 == 0 && ((uintptr_t)z & 15) == 0;
    hipStream_t hs = (hipStream_t)s;
#define CALL(DT)                                                                                                                     \
    if (vec) hipLaunchKernelGGL((k_unary_act<DT, 4>), dim3((unsigned)((n / 4 + kT - 1) / kT)), dim3(kT), 0, hs, z, ldz, rows, cols, kind, out); \
    else hipLaunchKernelGGL((k_unary_act<DT, 1>), dim3((unsigned)((n + kT - 1) / kT)), dim3(kT), 0, hs, z, ldz, rows, cols, kind, out);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}
