// moe_seq.hip -- the routing side of a mixture-of-experts feed-forward over a ragged step (the products are zls_gemm_nt_grouped):
//
// k_moe_route    a wave per token: fp32 scores over all router outputs (softmax, or a sigmoid of each logit), choice scores = scores +
//                correction, group-limited choice (a group's score = its best choice score, or the sum of its `group_top` best; outputs
//                outside the best `keep` groups count as minus infinity), `top` picks by repeated arg-max (ties: the lower index),
//                weights = the scores of the picks (optionally divided by their sum + renorm_eps), times weight_scale
// k_moe_align    one workgroup: counts per expert, their prefix, every (token, choice) pair's place in the expert-sorted order, and the list of
//                (expert, first, end) row tiles that the grouped product walks.  Identity outputs (id >= n_experts) take no place.
// k_silu_mul     silu(gate) * up
// k_act_mul      the gated activations of the feed-forwards: silu(g) u, gelu_tanh(g) u, or the clamped g sigmoid(a g) (u + 1)
// k_moe_combine  a workgroup per token: the weighted sum of its picks' rows in the order of the picks; an identity pick adds the input row
#include "seq_common.h"

namespace {

__device__ __forceinline__ void wave_argmax(float& v, int& i) {          // largest value, lowest index among equals; result in every lane
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(v, off, 64);
        const int oi = __shfl_xor(i, off, 64);
        if (ov > v || (ov == v && oi < i)) { v = ov; i = oi; }
    }
}

__global__ __launch_bounds__(64) void k_moe_route(const float* __restrict__ logits, int64_t ld, int n_out, const float* __restrict__ correction, int groups,
                                                  int keep, int top, int renorm, int score_kind, int group_top, float renorm_eps,
                                                  float weight_scale, int32_t* __restrict__ ids, float* __restrict__ weights) {
    __shared__ float prob[1024], choice[1024], gscore[1024];
    const int t = blockIdx.x, lane = threadIdx.x;
    const float* z = logits + (size_t)t * ld;                          // (the router's columns may lead wider rows)
    float mx = -INFINITY;
    for (int i = lane; i < n_out; i += 64) mx = fmaxf(mx, z[i]);
    mx = zl_wave_max(mx);
    float sum = 0.f;
    if (score_kind == 1) {                                               // every output on its own: sigmoid of its logit
        for (int i = lane; i < n_out; i += 64) prob[i] = seq_sigmoid(z[i]);
        sum = 1.0f;
    } else {
        for (int i = lane; i < n_out; i += 64) { const float e = expf(z[i] - mx); prob[i] = e; sum += e; }
        sum = zl_wave_sum(sum);
    }
    for (int i = lane; i < n_out; i += 64) {
        const float pr = prob[i] / sum;
        prob[i] = pr;
        choice[i] = pr + (correction ? correction[i] : 0.f);
    }
    __syncthreads();
    if (groups > 1 && keep < groups) {
        const int size = n_out / groups;
        for (int g = lane; g < groups; g += 64) {
            float best = -INFINITY;
            if (group_top <= 1) {
                for (int i = 0; i < size; ++i) best = fmaxf(best, choice[g * size + i]);
            } else {                                                     // the sum of the group's group_top largest choice scores
                best = 0.f;
                float bound = INFINITY; int bound_i = -1;                // the last one taken: the next is the largest below it (index order among equals)
                for (int k = 0; k < group_top && k < size; ++k) {
                    float bv = -INFINITY; int bi = -1;
                    for (int i = 0; i < size; ++i) {
                        const float v = choice[g * size + i];
                        const bool below = v < bound || (v == bound && i > bound_i);
                        if (below && (v > bv || bi < 0)) { bv = v; bi = i; }
                    }
                    best += bv; bound = bv; bound_i = bi;
                }
            }
            gscore[g] = best;
        }
        __syncthreads();
        for (int k = 0; k < keep; ++k) {                                 // the kept groups are marked by +inf, then everything else drops out
            float bv = -INFINITY; int bi = 0x7fffffff;
            for (int g = lane; g < groups; g += 64) {
                const float v = gscore[g];
                if (v != INFINITY && (v > bv || (v == bv && g < bi))) { bv = v; bi = g; }
            }
            wave_argmax(bv, bi);
            __syncthreads();
            if (lane == 0 && bi < groups) gscore[bi] = INFINITY;
            __syncthreads();
        }
        for (int i = lane; i < n_out; i += 64)
            if (gscore[i / size] != INFINITY) choice[i] = -INFINITY;
        __syncthreads();
    }
    float wsum = 0.f;
    for (int k = 0; k < top; ++k) {
        float bv = -INFINITY; int bi = 0x7fffffff;
        for (int i = lane; i < n_out; i += 64) {
            const float v = choice[i];
            if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
        }
        wave_argmax(bv, bi);
        if (bi >= n_out) bi = 0;                                         // (fewer finite choices than picks: never with top <= kept outputs)
        __syncthreads();
        if (lane == 0) {
            ids[(size_t)t * top + k] = bi;
            weights[(size_t)t * top + k] = prob[bi];
            choice[bi] = -INFINITY;
        }
        wsum += prob[bi];
        __syncthreads();
    }
    if (renorm || weight_scale != 1.0f) {
        __syncthreads();
        for (int k = lane; k < top; k += 64) {
            float w = weights[(size_t)t * top + k];
            if (renorm) w /= wsum + renorm_eps;
            weights[(size_t)t * top + k] = w * weight_scale;
        }
    }
}

__global__ __launch_bounds__(1024) void k_moe_align(const int32_t* __restrict__ ids, int n_slots, int top, int n_experts, int tile_m,
                                                    int32_t* __restrict__ sorted_tok, int32_t* __restrict__ slot_pos, int32_t* __restrict__ tiles,
                                                    int max_tiles, int32_t* __restrict__ sorted_exp) {
    extern __shared__ int sh[];
    int* count = sh;                       // [n_experts]
    int* start = sh + n_experts;           // [n_experts + 1]
    int* tile0 = start + n_experts + 1;    // [n_experts + 1]
    const int tid = threadIdx.x;
    for (int e = tid; e < n_experts; e += 1024) count[e] = 0;
    __syncthreads();
    for (int i = tid; i < n_slots; i += 1024) {
        const int e = ids[i];
        if (e >= 0 && e < n_experts) atomicAdd(&count[e], 1);
    }
    __syncthreads();
    if (tid == 0) {
        int at = 0, tl = 0;
        for (int e = 0; e < n_experts; ++e) {
            start[e] = at; tile0[e] = tl;
            at += count[e];
            tl += (count[e] + tile_m - 1) / tile_m;
        }
        start[n_experts] = at; tile0[n_experts] = tl;
    }
    __syncthreads();
    for (int e = tid; e < n_experts; e += 1024) {
        const int n = count[e], s0 = start[e];
        for (int k = 0, tl = tile0[e]; k < n && tl < max_tiles; k += tile_m, ++tl) {
            tiles[3 * tl] = e; tiles[3 * tl + 1] = s0 + k; tiles[3 * tl + 2] = s0 + min(n, k + tile_m);
        }
        count[e] = 0;                                                    // becomes the fill counter below
    }
    for (int tl = tile0[n_experts] + tid; tl < max_tiles; tl += 1024) { tiles[3 * tl] = -1; tiles[3 * tl + 1] = 0; tiles[3 * tl + 2] = 0; }
    __syncthreads();
    // a pair's place inside its expert's run: the number of earlier pairs of the same expert -- in the order of the pairs, so that the sorted
    // order does not depend on which thread came first.  A wave per expert walks the list 64 pairs at a time (ballot + prefix count)
    const int lane = tid & 63;
    for (int e = tid >> 6; e < n_experts; e += 16) {
        int at = start[e];
        const int end = start[e + 1];
        for (int i0 = 0; i0 < n_slots && at < end; i0 += 64) {
            const int i = i0 + lane;
            const bool hit = i < n_slots && ids[i] == e;
            const unsigned long long mask = __ballot(hit);
            if (hit) {
                const int pos = at + __popcll(mask & ((1ull << lane) - 1ull));
                sorted_tok[pos] = i / top;
                slot_pos[i] = pos;
                if (sorted_exp) sorted_exp[pos] = e;
            }
            at += __popcll(mask);
        }
    }
    for (int i = tid; i < n_slots; i += 1024) {
        const int e = ids[i];
        if (e < 0 || e >= n_experts) slot_pos[i] = -1;
        if (sorted_exp && i >= start[n_experts]) sorted_exp[i] = -1;       // sorted positions that no pair takes
    }
}

template <int DT>
__global__ __launch_bounds__(256) void k_silu_mul(const float* __restrict__ gu, int ff, void* __restrict__ out) {
    const size_t r = blockIdx.x;
    for (int c = threadIdx.x; c < ff; c += 256) SeqT<DT>::st(out, r * ff + c, seq_silu(gu[r * 2 * ff + c]) * gu[r * 2 * ff + ff + c]);
}

// block > 0: the row holds blocks of `block` gate columns followed by their `block` up columns; 0: all gates, then all ups
template <int DT>
__global__ __launch_bounds__(256) void k_act_mul(const float* __restrict__ gu, int ff, int kind, float alpha, float limit, int block,
                                                 void* __restrict__ out) {
    const size_t r = blockIdx.x;
    for (int c = threadIdx.x; c < ff; c += 256) {
        const int gi = block > 0 ? (c / block) * 2 * block + c % block : c, ui = block > 0 ? gi + block : ff + c;
        SeqT<DT>::st(out, r * ff + c, gated_act(gu[r * 2 * ff + gi], gu[r * 2 * ff + ui], kind, alpha, limit));
    }
}

template <int DT>
__global__ __launch_bounds__(256) void k_moe_combine(const float* __restrict__ y, const int32_t* __restrict__ slot_pos, const int32_t* __restrict__ ids,
                                                     const float* __restrict__ weights, const void* __restrict__ h, int top, int n_experts, int width,
                                                     float* __restrict__ out) {
    const size_t t = blockIdx.x;
    for (int c = threadIdx.x; c < width; c += 256) {
        float a = 0.f;
        for (int k = 0; k < top; ++k) {
            const int e = ids[t * top + k];
            const float w = weights[t * top + k];
            const float v = e >= n_experts ? SeqT<DT>::ld(h, t * width + c) : y[(size_t)slot_pos[t * top + k] * width + c];
            a = fmaf(w, v, a);
        }
        out[t * width + c] = a;
    }
}

}  // namespace

extern "C" int zls_moe_route(const float* logits, int64_t ld, int64_t n_tok, int64_t n_out, const float* correction, int64_t groups, int64_t keep, int64_t top,
                             int renorm, int score_kind, int64_t group_top, float renorm_eps, float weight_scale, int32_t* ids, float* weights,
                             zl_stream_t s) {
    ZL_CHECK_ARG(logits && ids && weights && n_tok > 0 && n_out > 0 && top > 0 && ld >= n_out, ZL_EINVAL);
    ZL_CHECK_ARG(n_out <= 1024 && top <= n_out, ZL_ELIMIT);
    if (groups < 1) groups = 1;
    ZL_CHECK_ARG(n_out % groups == 0 && keep >= 1 && keep <= groups && top <= keep * (n_out / groups), ZL_ESHAPE);
    ZL_CHECK_ARG((score_kind == 0 || score_kind == 1) && group_top >= 1, ZL_EINVAL);
    hipLaunchKernelGGL(k_moe_route, dim3((unsigned)n_tok), dim3(64), 0, (hipStream_t)s, logits, ld, (int)n_out, correction, (int)groups, (int)keep,
                       (int)top, renorm, score_kind, (int)group_top, renorm_eps, weight_scale, ids, weights);
    return zl_launch_status();
}

extern "C" int zls_moe_align(const int32_t* ids, int64_t n_slots, int64_t top, int64_t n_experts, int64_t tile_m, int32_t* sorted_tok,
                             int32_t* slot_pos, int32_t* tiles, int64_t max_tiles, int32_t* sorted_exp, zl_stream_t s) {
    ZL_CHECK_ARG(ids && sorted_tok && slot_pos && tiles && n_slots > 0 && top > 0 && n_experts > 0 && tile_m > 0, ZL_EINVAL);
    ZL_CHECK_ARG(n_experts <= 4096 && n_slots < (1 << 30), ZL_ELIMIT);
    ZL_CHECK_ARG(max_tiles >= n_slots / tile_m + n_experts, ZL_ESHAPE);
    const size_t lds = (size_t)(3 * n_experts + 2) * sizeof(int);
    hipLaunchKernelGGL(k_moe_align, dim3(1), dim3(1024), lds, (hipStream_t)s, ids, (int)n_slots, (int)top, (int)n_experts, (int)tile_m, sorted_tok,
                       slot_pos, tiles, (int)max_tiles, sorted_exp);
    return zl_launch_status();
}

extern "C" int zls_silu_mul(const float* gu, int64_t rows, int64_t ff, void* out, int dtype, zl_stream_t s) {
    ZL_CHECK_ARG(gu && out && rows > 0 && ff > 0, ZL_EINVAL);
#define CALL(DT) hipLaunchKernelGGL((k_silu_mul<DT>), dim3((unsigned)rows), dim3(256), 0, (hipStream_t)s, gu, (int)ff, out);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}

extern "C" int zls_act_mul(const float* gu, int64_t rows, int64_t ff, int kind, float alpha, float limit, int64_t block, void* out, int dtype,
                           zl_stream_t s) {
    ZL_CHECK_ARG(gu && out && rows > 0 && ff > 0 && kind >= 0 && kind <= 2 && block >= 0 && (block == 0 || ff % block == 0), ZL_EINVAL);
#define CALL(DT) hipLaunchKernelGGL((k_act_mul<DT>), dim3((unsigned)rows), dim3(256), 0, (hipStream_t)s, gu, (int)ff, kind, alpha, limit, (int)block, out);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}

extern "C" int zls_moe_combine(const float* y, const int32_t* slot_pos, const int32_t* ids, const float* weights, const void* h, int64_t n_tok,
                               int64_t top, int64_t n_experts, int64_t width, float* out, int dtype, zl_stream_t s) {
    ZL_CHECK_ARG(y && slot_pos && ids && weights && h && out && n_tok > 0 && top > 0 && width > 0, ZL_EINVAL);
#define CALL(DT) hipLaunchKernelGGL((k_moe_combine<DT>), dim3((unsigned)n_tok), dim3(256), 0, (hipStream_t)s, y, slot_pos, ids, weights, h, (int)top, \
                                    (int)n_experts, (int)width, out);
    ZLS_DISPATCH(dtype, CALL)
#undef CALL
    return zl_launch_status();
}
