// linear_attn.hip -- what stands around the decayed outer-product recurrence (zls_decay_scan in ssm.hip) in a linear-attention mixer:
//
// k_exp_gates           exponential input / forget gates with a soft cap and a running maximum m: a workgroup per (sequence, head) walks the
//                       portion 256 tokens at a time -- every thread the capped gates of its token, one thread the max-recurrence over the
//                       chunk (an add and a max per token), every thread the decay exp(f + m_prev - m) and the gain exp(i - m) of its token.
//                       m is carried per sequence slot.
// k_linear_attn_finish  a workgroup per (token, norm group): the optional division by max(|n . q|, exp(-m)) + den_eps per head, the RMS norm
//                       over the group (all heads together, or each head alone), the weight, the sigmoid gate.
// k_lowrank_decay      a decay per key channel from a low-rank projection: alpha = sigmoid(W2 u + bias)^(1 / tau), u the token's `low`
//                       numbers; a workgroup per token, u in LDS, a thread per channel walks its row of W2 (fp32 sums)
// Everything here is fp32; only the finished row is written in the serving format.
#include "seq_common.h"

namespace {

constexpr int kG = 256;

__device__ __forceinline__ float log_sigmoid(float v) { return fminf(v, 0.f) - log1pf(expf(-fabsf(v))); }

__global__ __launch_bounds__(kG) void k_exp_gates(const float* __restrict__ proj, int64_t ld, int i_col0, int f_col0, const float* __restrict__ i_bias,
                                                  const float* __restrict__ f_bias, float cap, float* __restrict__ m_state, int heads,
                                                  const zls_batch_t b, float* __restrict__ decay, float* __restrict__ gain, float* __restrict__ m_out) {
    __shared__ float gi[kG], gf[kG], mm[kG + 1];
    const int sq = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
    const int first = b.seq_start[sq], count = b.seq_start[sq + 1] - first;
    float* ms = m_state + (size_t)b.seq_slot[sq] * heads + h;
    const float bi = i_bias ? i_bias[h] : 0.f, bf = f_bias ? f_bias[h] : 0.f;
    if (tid == 0) mm[0] = *ms;
    for (int c0 = 0; c0 < count; c0 += kG) {
        const int cn = min(kG, count - c0);
        if (tid < cn) {
            const float* row = proj + (size_t)(first + c0 + tid) * ld;
            float zi = row[i_col0 + h] + bi, zf = row[f_col0 + h] + bf;
            if (cap > 0.f) { zi = cap * tanhf(zi / cap); zf = cap * tanhf(zf / cap); }
            gi[tid] = zi;
            gf[tid] = log_sigmoid(zf);
        }
        __syncthreads();
        if (tid == 0) {
            float m = mm[0];
            for (int i = 0; i < cn; ++i) { m = fmaxf(gf[i] + m, gi[i]); mm[i + 1] = m; }
        }
        __syncthreads();
        if (tid < cn) {
            const float m = mm[tid + 1];
            const size_t at = (size_t)(first + c0 + tid) * heads + h;
            decay[at] = expf(gf[tid] + mm[tid] - m);
            gain[at] = expf(gi[tid] - m);
            m_out[at] = m;
        }
        __syncthreads();
        if (tid == 0) mm[0] = mm[cn];
    }
    __syncthreads();
    if (tid == 0) *ms = mm[0];
}

// alpha[t][c] = exp(log_sigmoid(sum_j w2[c][j] u[t][j] + bias[c]) / tau): the logarithm of the decay never leaves fp32
template <int DT>
__global__ __launch_bounds__(kG) void k_lowrank_decay(const float* __restrict__ proj, int64_t ld, int u_col0, int low, const void* __restrict__ w2,
                                                      const float* __restrict__ bias, float inv_tau, int channels, float* __restrict__ alpha) {
    extern __shared__ float us[];
    const size_t t = blockIdx.x;
    for (int j = threadIdx.x; j < low; j += kG) us[j] = proj[t * ld + u_col0 + j];
    __syncthreads();
    for (int c = threadIdx.x; c < channels; c += kG) {
        float z = 0.f;
        for (int j = 0; j < low; ++j) z = fmaf(SeqT<DT>::ld(w2, (size_t)c * low + j), us[j], z);
        z += bias ? bias[c] : 0.f;
        alpha[t * channels + c] = expf(log_sigmoid(z) * inv_tau);
    }
}

struct FinP {
    const float* y; const float* m_vals; const float* weight; const float* gate; int64_t ldg;
    int norm_col, heads, vdim, part, g_col0, gate_kind;       // gate_kind 0: sigmoid(gate); 1: silu(gate)
    float q_scale, den_eps, eps;
    void* out;
};

template <int DT>
__global__ __launch_bounds__(kG) void k_linear_attn_finish(const FinP p) {
    __shared__ float red[16];
    const int t = blockIdx.x, c0 = blockIdx.y * p.part, hp = p.vdim + p.norm_col;
    const float* yr = p.y + (size_t)t * p.heads * hp;
    auto value = [&](int c) {
        const int h = c / p.vdim, i = c % p.vdim;
        float v = yr[h * hp + i];
        if (!p.m_vals) v *= p.q_scale;
        if (p.m_vals) {
            const float nq = yr[h * hp + p.vdim] * p.q_scale;
            v = v * p.q_scale / (fmaxf(fabsf(nq), expf(-p.m_vals[(size_t)t * p.heads + h])) + p.den_eps);
        }
        return v;
    };
    float ss = 0.f;
    for (int i = threadIdx.x; i < p.part; i += blockDim.x) { const float v = value(c0 + i); ss = fmaf(v, v, ss); }
    ss = zl_block_sum(ss, red);
    const float f = 1.0f / sqrtf(ss / (float)p.part + p.eps);
    for (int i = threadIdx.x; i < p.part; i += blockDim.x) {
        const int c = c0 + i;
        float v = value(c) * f;
        if (p.weight) v *= p.weight[c];
        if (p.gate) {
            const float gv = p.gate[(size_t)t * p.ldg + p.g_col0 + c];
            v *= p.gate_kind == 1 ? seq_silu(gv) : seq_sigmoid(gv);
        }
        SeqT<DT>::st(p.out, (size_t)t * p.heads * p.vdim + c, v);
    }
}

}  // namespace

extern "C" int zls_exp_gates(const float* proj, int64_t ld, int64_t i_col0, int64_t f_col0, const float* i_bias, const float* f_bias, float cap,
                             float* m_state, int64_t heads, const zls_batch_t* b, float* decay, float* gain, float* m_out, zl_stream_t s) {
    ZL_CHECK_ARG(proj && m_state && decay && gain && m_out && seq_batch_ok(b) && heads > 0 && heads <= 65535, ZL_EINVAL);
    ZL_CHECK_ARG(i_col0 >= 0 && i_col0 + heads <= ld && f_col0 >= 0 && f_col0 + heads <= ld, ZL_ESHAPE);
    hipLaunchKernelGGL(k_exp_gates, dim3(b->n_seq, (unsigned)heads), dim3(kG), 0, (hipStream_t)s, proj, ld, (int)i_col0, (int)f_col0, i_bias,
                       f_bias, cap, m_state, (int)heads, *b, decay, gain, m_out);
    return zl_launch_status();
}

extern "C" int zls_linear_attn_finish(const float* y, int64_t norm_col, float q_scale, const float* m_vals, float den_eps, int64_t heads,
                                      int64_t vdim, int64_t norm_groups, const float* weight, float eps, const float* gate, int64_t ldg,
                                      int64_t g_col0, int64_t n_tok, void* out, int dtype, int gate_kind, zl_stream_t s) {
    ZL_CHECK_ARG(y && out && heads > 0 && vdim > 0 && norm_groups > 0 && n_tok > 0 && (!m_vals || norm_col), ZL_EINVAL);
    ZL_CHECK_ARG((heads * vdim) % norm_groups == 0 && norm_groups <= 65535 && (!gate || (g_col0 >= 0 && g_col0 + heads * vdim <= ldg)), ZL_ESHAPE);
    FinP p;
    p.y = y; p.m_vals = m_vals; p.weight = weight; p.gate = gate; p.ldg = ldg; p.norm_col = norm_col ? 1 : 0; p.heads = (int)heads;
    p.vdim = (int)vdim; p.part = (int)(heads * vdim / norm_groups); p.g_col0 = (int)g_col0; p.q_scale = q_scale; p.den_eps = den_eps;
    p.eps = eps; p.out = out; p.gate_kind = gate_kind == 1 ? 1 : 0;
    // (a norm group per workgroup: short groups -- a head each -- get no more waves than they have elements for)
    const unsigned threads = p.part >= kG ? kG : (unsigned)((p.part + 63) / 64 * 64);
#define CALL(DT) hipLaunchKernelGGL((k_linear_attn_finish<DT>), dim3((unsigned)n_tok, (unsigned)norm_groups), dim3(threads), 0, (hipStream_t)s, p);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}

extern "C" int zls_lowrank_decay(const float* proj, int64_t ld, int64_t u_col0, int64_t low, const void* w2, const float* bias, float tau,
                                 int64_t channels, int64_t n_tok, float* alpha, int dtype, zl_stream_t s) {
    ZL_CHECK_ARG(proj && w2 && alpha && low > 0 && channels > 0 && n_tok > 0 && tau > 0.f, ZL_EINVAL);
    ZL_CHECK_ARG(u_col0 >= 0 && u_col0 + low <= ld && low <= 8192, ZL_ESHAPE);
#define CALL(DT) hipLaunchKernelGGL((k_lowrank_decay<DT>), dim3((unsigned)n_tok), dim3(kG), (size_t)low * sizeof(float), (hipStream_t)s, proj, ld, \
                                    (int)u_col0, (int)low, w2, bias, 1.0f / tau, (int)channels, alpha);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}
