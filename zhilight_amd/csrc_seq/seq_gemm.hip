// seq_gemm.hip -- y = x . W^T for ANY m, n, k in bf16 or true fp32, fp32 accumulation and (by default) fp32 output.
//
// The other dense products of this library (csrc/dense_gemm.hip, dense_gemv.hip) want k % 128 == 0 and 16-bit types; models whose sizes
// come from a configuration file (widths like 320, projections like 582 columns) and the 32-bit serving mode need a product without
// shape conditions.  Two kernels:
//   k_seq_gemv  m <= 8 rows (decode steps): a wave streams the weight rows of 1 / 2 / 4 output columns (for <= 2 / 4 / 8 activation rows)
//               once, 16-byte loads, all sums in registers, butterflies at the end -- the weight matrix is read exactly once.
//   k_seq_gemv_mfma  3 .. 16 rows in bf16: the same streaming with the products on the matrix cores (see there).
//   k_seq_gemm  more rows (prompt portions, mixed steps): 128 x 128 or 64 x 64 output tile per workgroup of 4 waves (2 x 2; a wave =
//               4 x 4 or 2 x 2 MFMA tiles of 16 x 16), 32-k slices of x and W staged through LDS (zero-filled past the edges), the next slice's global
//               loads issued before the current slice's MFMAs.  bf16: v_mfma_f32_16x16x32_bf16; fp32: v_mfma_f32_16x16x4_f32.
#include "seq_common.h"

namespace {

typedef __bf16 b8 __attribute__((ext_vector_type(8)));
typedef float f4 __attribute__((ext_vector_type(4)));

constexpr int kBK = 32;

struct GemmP {
    const void* x; const void* w; void* y;
    int64_t ldx, ldw, ldy;
    int m, n, k, vec;
    const int32_t* x_rows;                                     // row r of x is x[x_rows[r]] (NULL: r); the same for w
    const int32_t* w_rows;
    // grouped form (a mixture of experts): row tile i of the launch is tiles[3 i ..] = (expert, first row, end row) with rows counted in
    // the expert-sorted order, w = the expert's (n, k) block of a stacked (experts, n, k) array; expert < 0: the tile is unused
    const int32_t* tiles;
    int64_t w_stride;
    int act; float act_alpha, act_limit;                       // the gated epilogue's activation (gated_act in seq_common.h)
};

// ---- tiles in LDS -----------------------------------------------------------------------------------------------------------------
template <int DT> struct Tile;
template <> struct Tile<ZL_BF16> {
    static constexpr int kRow = kBK + 8;                       // 80-byte rows: 16-byte aligned fragments, conflict-free enough
    typedef uint16_t elem;
    uint4 r;                                                   // 8 values of one row
    __device__ __forceinline__ void load(const void* base, int64_t ld, int row, int rows, int k0, int kc, int k, int vec) {
        const uint16_t* p = reinterpret_cast<const uint16_t*>(base) + (size_t)row * ld + k0 + kc;
        if (row < rows && vec && k0 + kc + 8 <= k) { r = *reinterpret_cast<const uint4*>(p); return; }
        uint16_t v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = (row < rows && k0 + kc + i < k) ? p[i] : (uint16_t)0;
        r = make_uint4(v[0] | (uint32_t)v[1] << 16, v[2] | (uint32_t)v[3] << 16, v[4] | (uint32_t)v[5] << 16, v[6] | (uint32_t)v[7] << 16);
    }
    __device__ __forceinline__ void store(elem* lds, int row, int kc) { *reinterpret_cast<uint4*>(lds + row * kRow + kc) = r; }
};
template <> struct Tile<ZL_F32> {
    static constexpr int kRow = kBK + 4;
    typedef float elem;
    float4 r[2];
    __device__ __forceinline__ void load(const void* base, int64_t ld, int row, int rows, int k0, int kc, int k, int vec) {
        const float* p = reinterpret_cast<const float*>(base) + (size_t)row * ld + k0 + kc;
        if (row < rows && vec && k0 + kc + 8 <= k) {
            r[0] = *reinterpret_cast<const float4*>(p);
            r[1] = *reinterpret_cast<const float4*>(p + 4);
            return;
        }
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = (row < rows && k0 + kc + i < k) ? p[i] : 0.f;
        r[0] = make_float4(v[0], v[1], v[2], v[3]);
        r[1] = make_float4(v[4], v[5], v[6], v[7]);
    }
    __device__ __forceinline__ void store(elem* lds, int row, int kc) {
        *reinterpret_cast<float4*>(lds + row * kRow + kc) = r[0];
        *reinterpret_cast<float4*>(lds + row * kRow + kc + 4) = r[1];
    }
};

// WT x WT MFMA tiles per wave: the workgroup's output tile is (32 WT) x (32 WT)
// GATED: the weight rows come in blocks of 16 gate rows followed by their 16 up rows, so that a wave's even column tiles are gates and the
// odd ones the up projections of the same 16 outputs; the epilogue writes act(gate, up) (gated_act: silu(gate) * up and others), half as many columns
template <int DT, int ODT, int WT, bool GATED = false>
__global__ __launch_bounds__(256) void k_seq_gemm(const GemmP p) {
    typedef typename Tile<DT>::elem E;
    constexpr int RS = Tile<DT>::kRow;
    constexpr int kBM = 32 * WT, kBN = 32 * WT, PASS = kBM / 64;
    __shared__ __attribute__((aligned(16))) E xs[kBM * RS];
    __shared__ __attribute__((aligned(16))) E ws[kBN * RS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int nrow = lane & 15, kq = lane >> 4;
    const int wm = wave >> 1, wn = wave & 1;
    int m0 = blockIdx.y * kBM, mlim = p.m;
    const int n0 = blockIdx.x * kBN;
    const void* wbase = p.w;
    if (p.tiles) {
        const int e = p.tiles[3 * blockIdx.y];
        if (e < 0) return;                                      // (the whole workgroup)
        m0 = p.tiles[3 * blockIdx.y + 1];
        mlim = p.tiles[3 * blockIdx.y + 2];
        wbase = reinterpret_cast<const E*>(p.w) + (size_t)e * p.w_stride;
    }
    const int lrow = tid >> 2, lkc = (tid & 3) * 8;

    f4 acc[WT][WT];
#pragma unroll
    for (int i = 0; i < WT; ++i)
#pragma unroll
        for (int j = 0; j < WT; ++j) acc[i][j] = (f4){0.f, 0.f, 0.f, 0.f};

    Tile<DT> tx[PASS], tw[PASS];
    // a gathered operand: the tile row's source row, looked up once (rows past the edge keep their own, unread, index)
    int xr[PASS], wr[PASS], xlim[PASS], wlim[PASS];
#pragma unroll
    for (int u = 0; u < PASS; ++u) {
        const int mr = m0 + lrow + 64 * u, nr = n0 + lrow + 64 * u;
        xr[u] = (p.x_rows && mr < mlim) ? p.x_rows[mr] : mr;
        wr[u] = (p.w_rows && nr < p.n) ? p.w_rows[nr] : nr;
        xlim[u] = mr < mlim ? xr[u] + 1 : 0;
        wlim[u] = nr < p.n ? wr[u] + 1 : 0;
        tx[u].load(p.x, p.ldx, xr[u], xlim[u], 0, lkc, p.k, p.vec);
        tw[u].load(wbase, p.ldw, wr[u], wlim[u], 0, lkc, p.k, p.vec);
    }
    for (int k0 = 0; k0 < p.k; k0 += kBK) {
        __syncthreads();                                        // the previous slice's fragments are consumed
#pragma unroll
        for (int u = 0; u < PASS; ++u) {
            tx[u].store(xs, lrow + 64 * u, lkc);
            tw[u].store(ws, lrow + 64 * u, lkc);
        }
        __syncthreads();
        if (k0 + kBK < p.k) {                                   // next slice in flight during the MFMAs
#pragma unroll
            for (int u = 0; u < PASS; ++u) {
                tx[u].load(p.x, p.ldx, xr[u], xlim[u], k0 + kBK, lkc, p.k, p.vec);
                tw[u].load(wbase, p.ldw, wr[u], wlim[u], k0 + kBK, lkc, p.k, p.vec);
            }
        }
        if constexpr (DT == ZL_BF16) {
            uint4 a[WT], b[WT];
#pragma unroll
            for (int i = 0; i < WT; ++i) a[i] = *reinterpret_cast<const uint4*>(xs + (wm * 16 * WT + i * 16 + nrow) * RS + 8 * kq);
#pragma unroll
            for (int j = 0; j < WT; ++j) b[j] = *reinterpret_cast<const uint4*>(ws + (wn * 16 * WT + j * 16 + nrow) * RS + 8 * kq);
#pragma unroll
            for (int i = 0; i < WT; ++i)
#pragma unroll
                for (int j = 0; j < WT; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(b8, a[i]), __builtin_bit_cast(b8, b[j]), acc[i][j], 0, 0, 0);
        } else {
#pragma unroll
            for (int kk = 0; kk < kBK / 4; ++kk) {
                float a[WT], b[WT];
#pragma unroll
                for (int i = 0; i < WT; ++i) a[i] = xs[(wm * 16 * WT + i * 16 + nrow) * RS + 4 * kk + kq];
#pragma unroll
                for (int j = 0; j < WT; ++j) b[j] = ws[(wn * 16 * WT + j * 16 + nrow) * RS + 4 * kk + kq];
#pragma unroll
                for (int i = 0; i < WT; ++i)
#pragma unroll
                    for (int j = 0; j < WT; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i], b[j], acc[i][j], 0, 0, 0);
            }
        }
    }
    if constexpr (GATED) {
        static_assert(WT % 2 == 0, "the gated epilogue pairs a wave's column tiles: even ones are gates, odd ones their up projections");
#pragma unroll
        for (int jj = 0; jj < WT / 2; ++jj) {
            const int wcol = n0 + wn * 16 * WT + jj * 32 + nrow;            // the gate's weight row; its output column is half the block offset
            const int col = (n0 + wn * 16 * WT) / 2 + jj * 16 + nrow;
#pragma unroll
            for (int i = 0; i < WT; ++i)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int row = m0 + wm * 16 * WT + i * 16 + 4 * kq + r;
                    if (row < mlim && wcol < p.n)
                        SeqT<ODT>::st(p.y, (size_t)row * p.ldy + col, gated_act(acc[i][2 * jj][r], acc[i][2 * jj + 1][r], p.act, p.act_alpha, p.act_limit));
                }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < WT; ++i)
#pragma unroll
        for (int j = 0; j < WT; ++j) {
            const int col = n0 + wn * 16 * WT + j * 16 + nrow;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int row = m0 + wm * 16 * WT + i * 16 + 4 * kq + r;
                if (row < mlim && col < p.n) SeqT<ODT>::st(p.y, (size_t)row * p.ldy + col, acc[i][j][r]);
            }
        }
}

// ---- a few rows: the weights are the traffic -----------------------------------------------------------------------------------------
template <int DT> struct Vec8;
template <> struct Vec8<ZL_BF16> {
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
template <> struct Vec8<ZL_F32> {
    static __device__ __forceinline__ void ld(const void* p, size_t i, float* v) {
        const float4 a = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p) + i);
        const float4 b = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p) + i + 4);
        v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
    }
};

// CPW output columns per wave: the activation rows (L2) are read once per CPW weight rows (HBM) -- with 8 rows and one column per wave
// the activations would be eight times the weight traffic
template <int DT, int ODT, int MR, int CPW>
__global__ __launch_bounds__(256) void k_seq_gemv(const GemmP p) {
    const int lane = threadIdx.x & 63;
    const int col0 = (blockIdx.x * 4 + (threadIdx.x >> 6)) * CPW;
    if (col0 >= p.n) return;
    float acc[MR][CPW];
#pragma unroll
    for (int r = 0; r < MR; ++r)
#pragma unroll
        for (int c = 0; c < CPW; ++c) acc[r][c] = 0.f;
    size_t wrow[CPW];
#pragma unroll
    for (int c = 0; c < CPW; ++c) wrow[c] = (size_t)min(col0 + c, p.n - 1) * p.k;      // (a column past the edge: the last one, never stored)
    if (p.vec && (p.k & 7) == 0) {
        for (int k = lane * 8; k < p.k; k += 512) {
            float wv[CPW][8];
#pragma unroll
            for (int c = 0; c < CPW; ++c) Vec8<DT>::ld(p.w, wrow[c] + k, wv[c]);
#pragma unroll
            for (int r = 0; r < MR; ++r) {
                if (r < p.m) {
                    float xv[8];
                    Vec8<DT>::ld(p.x, (size_t)r * p.ldx + k, xv);
#pragma unroll
                    for (int c = 0; c < CPW; ++c)
#pragma unroll
                        for (int i = 0; i < 8; ++i) acc[r][c] = fmaf(wv[c][i], xv[i], acc[r][c]);
                }
            }
        }
    } else {
        for (int k = lane; k < p.k; k += 64) {
            float wv[CPW];
#pragma unroll
            for (int c = 0; c < CPW; ++c) wv[c] = SeqT<DT>::ld(p.w, wrow[c] + k);
#pragma unroll
            for (int r = 0; r < MR; ++r)
                if (r < p.m) {
                    const float xv = SeqT<DT>::ld(p.x, (size_t)r * p.ldx + k);
#pragma unroll
                    for (int c = 0; c < CPW; ++c) acc[r][c] = fmaf(wv[c], xv, acc[r][c]);
                }
        }
    }
#pragma unroll
    for (int r = 0; r < MR; ++r)
#pragma unroll
        for (int c = 0; c < CPW; ++c) {
            const float v = zl_wave_sum(acc[r][c]);
            if (lane == 0 && r < p.m && col0 + c < p.n) SeqT<ODT>::st(p.y, (size_t)r * p.ldy + col0 + c, v);
        }
}

// 3 .. 16 activation rows in bf16 on the matrix cores without LDS staging: a workgroup owns 16 output columns, its four waves take every
// fourth 32-k step; per step a lane loads 16 bytes of ITS weight row (A operand: lane = column, 8 consecutive k) and 16 bytes of ITS
// activation row (B operand: lane = row; rows past m are zero), eight steps in flight, one v_mfma_f32_16x16x32_bf16 each.  The weights are
// read exactly once, the activations cost half the weight bytes at 8 rows (L2), and no VALU multiply is spent.  The four partial tiles
// meet in LDS.
template <int ODT>
__global__ __launch_bounds__(256) void k_seq_gemv_mfma(const GemmP p) {
    __shared__ float red[4][16][17];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nrow = lane & 15, kq = lane >> 4;
    const int col0 = blockIdx.x * 16;
    const uint16_t* wp = reinterpret_cast<const uint16_t*>(p.w) + (size_t)min(col0 + nrow, p.n - 1) * p.k + 8 * kq;
    const bool xok = nrow < p.m;
    const uint16_t* xp = reinterpret_cast<const uint16_t*>(p.x) + (size_t)(xok ? nrow : 0) * p.ldx + 8 * kq;
    f4 acc = (f4){0.f, 0.f, 0.f, 0.f};
    const int steps = (p.k + 31) / 32;
    constexpr int U = 8;
    for (int s0 = wave; s0 < steps; s0 += 4 * U) {
        uint4 wf[U], xf[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k0 = 32 * (s0 + 4 * u);
            const bool ok = k0 + 8 * kq < p.k;                          // (k is a multiple of 8: a lane's 8 values are all in or all out)
            wf[u] = ok ? zl_load_nt(reinterpret_cast<const uint4*>(wp + k0)) : make_uint4(0, 0, 0, 0);
            xf[u] = (ok && xok) ? *reinterpret_cast<const uint4*>(xp + k0) : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(b8, wf[u]), __builtin_bit_cast(b8, xf[u]), acc, 0, 0, 0);
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][4 * kq + r][nrow] = acc[r];   // acc[r] = sum for column col0 + 4 kq + r, row nrow
    __syncthreads();
    const int c = threadIdx.x >> 4, m = threadIdx.x & 15;
    if (m < p.m && col0 + c < p.n)
        SeqT<ODT>::st(p.y, (size_t)m * p.ldy + col0 + c, red[0][c][m] + red[1][c][m] + red[2][c][m] + red[3][c][m]);
}

// the grouped product for a FEW rows (decode steps of a mixture of experts): a wave per (sorted row, output column) streams the column's
// weight row of the row's expert once, 16-byte loads -- a 64-row tile per expert would multiply 63 rows of zeros and leave most of the
// chip idle.  GATED: the gate row and its up row (16 rows further in the packed block), act(gate, up).
template <int DT, int ODT, bool GATED>
__global__ __launch_bounds__(256) void k_seq_gemv_grouped(const GemmP p, const int32_t* __restrict__ row_expert, int n_rows) {
    const int lane = threadIdx.x & 63;
    const int col = blockIdx.x * 4 + (threadIdx.x >> 6), row = blockIdx.y;
    const int n_cols = GATED ? p.n / 2 : p.n;
    if (col >= n_cols || row >= n_rows) return;
    const int e = row_expert[row];
    if (e < 0) return;
    const size_t xr = (size_t)(p.x_rows ? p.x_rows[row] : row) * p.ldx;
    const size_t w0 = (size_t)e * p.w_stride + (size_t)(GATED ? (col / 16) * 32 + col % 16 : col) * p.k;
    const size_t w1 = w0 + (size_t)16 * p.k;
    float a0 = 0.f, a1 = 0.f;
    if (p.vec && (p.k & 7) == 0) {
        for (int k = lane * 8; k < p.k; k += 512) {
            float xv[8], wv[8];
            Vec8<DT>::ld(p.x, xr + k, xv);
            Vec8<DT>::ld(p.w, w0 + k, wv);
#pragma unroll
            for (int i = 0; i < 8; ++i) a0 = fmaf(wv[i], xv[i], a0);
            if constexpr (GATED) {
                Vec8<DT>::ld(p.w, w1 + k, wv);
#pragma unroll
                for (int i = 0; i < 8; ++i) a1 = fmaf(wv[i], xv[i], a1);
            }
        }
    } else {
        for (int k = lane; k < p.k; k += 64) {
            const float xv = SeqT<DT>::ld(p.x, xr + k);
            a0 = fmaf(SeqT<DT>::ld(p.w, w0 + k), xv, a0);
            if constexpr (GATED) a1 = fmaf(SeqT<DT>::ld(p.w, w1 + k), xv, a1);
        }
    }
    a0 = zl_wave_sum(a0);
    if constexpr (GATED) a0 = gated_act(a0, zl_wave_sum(a1), p.act, p.act_alpha, p.act_limit);
    if (lane == 0) SeqT<ODT>::st(p.y, (size_t)row * p.ldy + col, a0);
}

// 128 x 128 tiles (four times the MFMAs per LDS fragment) when they still fill the chip, 64 x 64 otherwise
template <int DT, int ODT>
void launch_tiled(const GemmP& p, hipStream_t hs) {
    const int64_t big = (int64_t)((p.m + 127) / 128) * ((p.n + 127) / 128);
    if (big >= 256) {
        const dim3 grid((unsigned)((p.n + 127) / 128), (unsigned)((p.m + 127) / 128));
        hipLaunchKernelGGL((k_seq_gemm<DT, ODT, 4>), grid, dim3(256), 0, hs, p);
    } else {
        const dim3 grid((unsigned)((p.n + 63) / 64), (unsigned)((p.m + 63) / 64));
        hipLaunchKernelGGL((k_seq_gemm<DT, ODT, 2>), grid, dim3(256), 0, hs, p);
    }
}

template <int DT, int ODT>
int launch(const GemmP& p, hipStream_t hs) {
    if constexpr (DT == ZL_BF16) {
        if (p.m >= 3 && p.m <= 16 && p.vec && (p.k & 7) == 0) {
            hipLaunchKernelGGL((k_seq_gemv_mfma<ODT>), dim3((unsigned)((p.n + 15) / 16)), dim3(256), 0, hs, p);
            return zl_launch_status();
        }
    }
    if (p.m <= 8) {
        if (p.m <= 2) hipLaunchKernelGGL((k_seq_gemv<DT, ODT, 2, 1>), dim3((unsigned)((p.n + 3) / 4)), dim3(256), 0, hs, p);
        else if (p.m <= 4) hipLaunchKernelGGL((k_seq_gemv<DT, ODT, 4, 2>), dim3((unsigned)((p.n + 7) / 8)), dim3(256), 0, hs, p);
        else hipLaunchKernelGGL((k_seq_gemv<DT, ODT, 8, 4>), dim3((unsigned)((p.n + 15) / 16)), dim3(256), 0, hs, p);
    } else {
        launch_tiled<DT, ODT>(p, hs);
    }
    return zl_launch_status();
}

}  // namespace

extern "C" int zls_version(void) { return 1; }

extern "C" int zls_gemm_nt(const void* x, int64_t ldx, const void* w, void* y, int64_t ldy, int64_t m, int64_t n, int64_t k, int dtype,
                           int out_dtype, zl_stream_t s) {
    ZL_CHECK_ARG(x && w && y && m > 0 && n > 0 && k > 0, ZL_EINVAL);
    ZL_CHECK_ARG(ldx >= k && ldy >= n && m < (1 << 30) && n < (1 << 30) && k < (1 << 30), ZL_ESHAPE);
    ZL_CHECK_ARG((m + 63) / 64 <= 65535, ZL_ELIMIT);
    ZL_CHECK_ARG(dtype == ZL_BF16 || dtype == ZL_F32, ZL_EDTYPE);
    ZL_CHECK_ARG(out_dtype == ZL_F32 || out_dtype == dtype, ZL_EDTYPE);
    GemmP p = {};
    p.x = x; p.w = w; p.y = y; p.ldx = ldx; p.ldw = k; p.ldy = ldy; p.m = (int)m; p.n = (int)n; p.k = (int)k;
    p.x_rows = p.w_rows = nullptr; p.tiles = nullptr; p.w_stride = 0;
    const int64_t unit = dtype == ZL_BF16 ? 8 : 4;
    p.vec = (k % unit == 0 && ldx % unit == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0) ? 1 : 0;
    hipStream_t hs = (hipStream_t)s;
    if (dtype == ZL_BF16) return out_dtype == ZL_F32 ? launch<ZL_BF16, ZL_F32>(p, hs) : launch<ZL_BF16, ZL_BF16>(p, hs);
    return launch<ZL_F32, ZL_F32>(p, hs);
}

// the same product with GATHERED rows of x and / or w (x_rows / w_rows: device int32 row indices, NULL: the rows in order), always on the
// tiled matrix-core kernel -- the up-projection of cached rows that lie scattered over pages
extern "C" int zls_gemm_nt_gather(const void* x, int64_t ldx, const int32_t* x_rows, const void* w, int64_t ldw, const int32_t* w_rows, void* y,
                                  int64_t ldy, int64_t m, int64_t n, int64_t k, int dtype, int out_dtype, zl_stream_t s) {
    ZL_CHECK_ARG(x && w && y && m > 0 && n > 0 && k > 0, ZL_EINVAL);
    ZL_CHECK_ARG(ldx >= k && ldw >= k && ldy >= n && m < (1 << 30) && n < (1 << 30) && k < (1 << 30), ZL_ESHAPE);
    ZL_CHECK_ARG((m + 63) / 64 <= 65535, ZL_ELIMIT);
    ZL_CHECK_ARG(dtype == ZL_BF16 || dtype == ZL_F32, ZL_EDTYPE);
    ZL_CHECK_ARG(out_dtype == ZL_F32 || out_dtype == dtype, ZL_EDTYPE);
    GemmP p = {};
    p.x = x; p.w = w; p.y = y; p.ldx = ldx; p.ldw = ldw; p.ldy = ldy; p.m = (int)m; p.n = (int)n; p.k = (int)k;
    p.x_rows = x_rows; p.w_rows = w_rows; p.tiles = nullptr; p.w_stride = 0;
    const int64_t unit = dtype == ZL_BF16 ? 8 : 4;
    p.vec = (k % unit == 0 && ldx % unit == 0 && ldw % unit == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0) ? 1 : 0;
    hipStream_t hs = (hipStream_t)s;
    if (dtype == ZL_BF16) {
        if (out_dtype == ZL_F32) launch_tiled<ZL_BF16, ZL_F32>(p, hs);
        else launch_tiled<ZL_BF16, ZL_BF16>(p, hs);
    } else {
        launch_tiled<ZL_F32, ZL_F32>(p, hs);
    }
    return zl_launch_status();
}

// the grouped product of a mixture of experts: one launch over the (expert, row tile) list that zls_moe_align left on the device -- the host
// never learns how many rows an expert got, the grid covers the upper bound and unused tiles return at once.  64- or 128-row tiles (the
// caller aligns with the same size: 128 when the experts' shares are long enough to fill them).
extern "C" int zls_gemm_nt_grouped(const void* x, int64_t ldx, const int32_t* x_rows, const void* w, const int32_t* tiles, int64_t max_tiles,
                                   int64_t tile_m, const int32_t* row_expert, int64_t n_rows, void* y, int64_t ldy, int64_t n, int64_t k, int gated,
                                   int dtype, int out_dtype, int act, float act_alpha, float act_limit, zl_stream_t s) {
    ZL_CHECK_ARG(act >= 0 && act <= 2, ZL_EINVAL);
    ZL_CHECK_ARG(x && w && tiles && y && max_tiles > 0 && n > 0 && k > 0, ZL_EINVAL);
    ZL_CHECK_ARG(tile_m == 64 || tile_m == 128, ZL_ESHAPE);
    ZL_CHECK_ARG(!row_expert || (n_rows > 0 && n_rows <= 65535), ZL_ESHAPE);
    ZL_CHECK_ARG(ldx >= k && n < (1 << 30) && k < (1 << 30) && max_tiles <= 65535, ZL_ESHAPE);
    ZL_CHECK_ARG(dtype == ZL_BF16 || dtype == ZL_F32, ZL_EDTYPE);
    ZL_CHECK_ARG(out_dtype == ZL_F32 || out_dtype == dtype, ZL_EDTYPE);
    ZL_CHECK_ARG(gated ? (n % 32 == 0 && ldy >= n / 2) : ldy >= n, ZL_ESHAPE);
    GemmP p = {};
    p.x = x; p.w = w; p.y = y; p.ldx = ldx; p.ldw = k; p.ldy = ldy; p.m = 0; p.n = (int)n; p.k = (int)k;
    p.x_rows = x_rows; p.w_rows = nullptr; p.tiles = tiles; p.w_stride = n * k;
    p.act = act; p.act_alpha = act_alpha; p.act_limit = act_limit;
    const int64_t unit = dtype == ZL_BF16 ? 8 : 4;
    p.vec = (k % unit == 0 && ldx % unit == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0) ? 1 : 0;
    hipStream_t hs = (hipStream_t)s;
    const dim3 grid((unsigned)((n + tile_m - 1) / tile_m), (unsigned)max_tiles);
    const int64_t n_cols = gated ? n / 2 : n;
    const dim3 vgrid((unsigned)((n_cols + 3) / 4), (unsigned)(row_expert ? n_rows : 1));
#define GROUPED(DT, ODT)                                                                                                        \
    if (row_expert && gated) hipLaunchKernelGGL((k_seq_gemv_grouped<DT, ODT, true>), vgrid, dim3(256), 0, hs, p, row_expert, (int)n_rows);   \
    else if (row_expert) hipLaunchKernelGGL((k_seq_gemv_grouped<DT, ODT, false>), vgrid, dim3(256), 0, hs, p, row_expert, (int)n_rows);      \
    else if (gated && tile_m == 128) hipLaunchKernelGGL((k_seq_gemm<DT, ODT, 4, true>), grid, dim3(256), 0, hs, p);             \
    else if (gated) hipLaunchKernelGGL((k_seq_gemm<DT, ODT, 2, true>), grid, dim3(256), 0, hs, p);                              \
    else if (tile_m == 128) hipLaunchKernelGGL((k_seq_gemm<DT, ODT, 4, false>), grid, dim3(256), 0, hs, p);                     \
    else hipLaunchKernelGGL((k_seq_gemm<DT, ODT, 2, false>), grid, dim3(256), 0, hs, p);
    if (dtype == ZL_BF16) {
        if (out_dtype == ZL_F32) { GROUPED(ZL_BF16, ZL_F32) } else { GROUPED(ZL_BF16, ZL_BF16) }
    } else {
        GROUPED(ZL_F32, ZL_F32)
    }
#undef GROUPED
    return zl_launch_status();
}
