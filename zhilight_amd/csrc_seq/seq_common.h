// seq_common.h -- helpers shared by the ragged-batch kernels (gfx950, wave64).
#pragma once
#include "../csrc/zl_common.h"
#include "../../include/zhilight_amd_seq.h"

// element access of the two storage formats: bf16 as raw 16-bit patterns, fp32 as is
template <int DT> struct SeqT;
template <> struct SeqT<ZL_BF16> {
    typedef uint16_t type;
    static __device__ __forceinline__ float ld(const void* p, size_t i) { return ZT<ZL_BF16>::to_f32(reinterpret_cast<const uint16_t*>(p)[i]); }
    static __device__ __forceinline__ void st(void* p, size_t i, float v) { reinterpret_cast<uint16_t*>(p)[i] = ZT<ZL_BF16>::from_f32(v); }
};
template <> struct SeqT<ZL_F32> {
    typedef float type;
    static __device__ __forceinline__ float ld(const void* p, size_t i) { return reinterpret_cast<const float*>(p)[i]; }
    static __device__ __forceinline__ void st(void* p, size_t i, float v) { reinterpret_cast<float*>(p)[i] = v; }
};

__device__ __forceinline__ float seq_silu(float v) { return v / (1.0f + expf(-v)); }
__device__ __forceinline__ float seq_sigmoid(float v) { return 1.0f / (1.0f + expf(-v)); }
__device__ __forceinline__ float seq_softplus(float v) { return v > 20.0f ? v : log1pf(expf(v)); }
// the gated activations of the feed-forwards
// kind 0: silu(g) u; 1: gelu_tanh(g) u; 2: g' sigmoid(alpha g') (u' + 1) with g' = min(g, limit), u' = clamp(u, -limit, limit)
__device__ __forceinline__ float gated_act(float g, float u, int kind, float alpha, float limit) {
    if (kind == 1) return 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g))) * u;
    if (kind == 2) {
        g = fminf(g, limit);
        u = fminf(fmaxf(u, -limit), limit);
        return g * seq_sigmoid(alpha * g) * (u + 1.0f);
    }
    return seq_silu(g) * u;
}
// sine and cosine of an fp32 angle of any size (positions times frequencies reach thousands of radians): the angle is brought into
// [-pi, pi] in double (exact to 1e-9 for angles up to 2^24), where the fp32 functions take their short path
__device__ __forceinline__ void seq_sincos(float a, float* sn, float* cs) {
    const double t = (double)a;
    const double k = rint(t * 0.15915494309189535);
    const float r = (float)fma(-k, 6.283185307179586, t);
    *sn = sinf(r);
    *cs = cosf(r);
}

static inline bool seq_batch_ok(const zls_batch_t* b) {
    return b && b->n_seq > 0 && b->n_tok > 0 && b->seq_start && b->seq_pos0 && b->seq_slot && b->tok_seq && b->max_count > 0 &&
           b->max_count <= b->n_tok;
}

#define ZLS_DISPATCH(dtype, CALL)                     \
    if ((dtype) == ZL_BF16) { CALL(ZL_BF16) }         \
    else if ((dtype) == ZL_F32) { CALL(ZL_F32) }      \
    else return ZL_EDTYPE;
