// FP8 LayerNorm forward / backward for gfx950, without and with affine parameters.
//
// Reference: coat/activation/real_quantization/func_layernorm_noparam.py (_layer_norm_fwd_fused :53-115,
// _layer_norm_bwd_dx_fused :122-185) and func_layernorm_param.py (_layer_norm_fwd_fused :52-119,
// _layer_norm_bwd_dx_fused :128-209, _fp8_layer_norm_bwd_dwdb :214-240).
//
// Same organisation as the RMSNorm kernels: one 256-thread block per row, the dequantized row stays in registers
// for the mean pass, the variance pass (two-pass variance, as the reference computes it) and the output pass.
// The forward output is fp32 (the reference allocates y as float32 and lets the per-tensor division read that).
// dw / db use per-block fp32 partial rows and a column reduction in block order instead of the reference's
// lock-guarded accumulation in the weight dtype.
#include <math.h>

#include "coat_host.h"
#include "norm_common.h"

namespace coat {

constexpr int kNoParam = 3;  // WMODE: 0..2 = dtype of w and b, 3 = no affine parameters

template <int WMODE> __device__ __forceinline__ void load_wb16(const void* w, int col, float* o) {
    if (WMODE == kNoParam) {
#pragma unroll
        for (int i = 0; i < 16; i++) o[i] = 1.0f;
    } else {
        load_w16<WMODE == kNoParam ? kF32 : WMODE>(w, col, o);
    }
}
// Forward: y = (x - mean) * rstd (* w + b) in fp32, mean[row], rstd[row], row scale (max|y| + 1e-10)/fp8max (bf16),
// tensor max of the row scales.
template <int KIND, int WMODE, int ITERS>
__global__ __launch_bounds__(256) void k_layernorm_fwd(const uint8_t* __restrict__ q, const void* __restrict__ s, int s_dt,
                                                        const void* __restrict__ w, const void* __restrict__ b,
                                                        float* __restrict__ y, void* __restrict__ s_row,
                                                        float* __restrict__ mean_out, float* __restrict__ rstd_out,
                                                        float* __restrict__ s_max, int N, int qb, float eps) {
    __shared__ float smem[4];
    const int64_t row = blockIdx.x;
    const int64_t row_off = row * N, srow_off = row * (N / qb);
    float x[ITERS][16];
    float sum = 0.0f;
#pragma unroll
    for (int it = 0; it < ITERS; it++) {
        const int col = (threadIdx.x + it * 256) * 16;
        if (col < N) {
            dequant16<KIND>(q, s, s_dt, row_off, srow_off, col, qb, x[it]);
#pragma unroll
            for (int i = 0; i < 16; i++) sum += x[it][i];
        }
    }
    const float mean = block_sum_256(sum, smem) / (float)N;
    float ss = 0.0f;
#pragma unroll
    for (int it = 0; it < ITERS; it++) {
        const int col = (threadIdx.x + it * 256) * 16;
        if (col < N) {
#pragma unroll
            for (int i = 0; i < 16; i++) {
                const float d = x[it][i] - mean;
                ss += d * d;
            }
        }
    }
    const float var = block_sum_256(ss, smem) / (float)N;
    const float rstd = 1 / sqrtf(var + eps);
    float amax = 0.0f;
#pragma unroll
    for (int it = 0; it < ITERS; it++) {
        const int col = (threadIdx.x + it * 256) * 16;
        if (col < N) {
            float wv[16], bv[16], yv[16];
            if (WMODE != kNoParam) {
                load_wb16<WMODE>(w, col, wv);
                load_wb16<WMODE>(b, col, bv);
            }
#pragma unroll
            for (int i = 0; i < 16; i++) {
                float v = (x[it][i] - mean) * rstd;
                if (WMODE != kNoParam) v = v * wv[i] + bv[i];
                yv[i] = v;
                amax = fmaxf(amax, fabsf(v));
            }
            if (y) {  // NULL: statistics only (the division recomputes y)
                float4* dst = (float4*)(y + row_off + col);
#pragma unroll
                for (int i = 0; i < 4; i++) dst[i] = make_float4(yv[4 * i], yv[4 * i + 1], yv[4 * i + 2], yv[4 * i + 3]);
            }
        }
    }
    amax = block_max_256(amax, smem);
    if (threadIdx.x == 0) {
        const float sr = group_scale<KIND>(amax);
        ((uint16_t*)s_row)[row] = (uint16_t)f2bf16(sr);
        mean_out[row] = mean;
        rstd_out[row] = rstd;
        atomic_max_nonneg(max_slot(s_max), sr);
    }
}

// Backward: wdy = w * dy; dx = bf16((wdy - (xhat * mean(xhat * wdy) + mean(wdy))) * rstd);
// per-block partials of dw = sum_rows dy * xhat and db = sum_rows dy (affine variant only).
// ADD: the residual-gradient addition that follows in the block (reference add_bwd.py:107-135 after
// func_layernorm_noparam.py:248-297, coat/models/coat_olmo.py:318-339) happens here: dx is rounded to bf16 as it would be
// stored, `radd` (bf16 [M, N]) is added in fp32, and what goes out is bf16 of the sum, the bf16 scale (amax + 1e-10) / fp8max of
// every 1 x qb group of the fp32 sum and the maximum of those scales (fp32) for the per-tensor division that follows.
struct LnAddArgs {
    const void* radd;   // bf16 [M, N]
    void* s_pg;         // bf16 [M, N / qb]
    float* s_max;       // COAT_MAX_WORDS
    int kind_out;       // kE4M3 / kE5M2: the FP8 format the scales are for
};
template <int KIND, int WMODE, int ITERS, bool ADD>
__device__ __forceinline__ void layernorm_bwd_body(const uint8_t* __restrict__ q, const void* __restrict__ s, int s_dt,
                                                    const void* __restrict__ dy, const void* __restrict__ w,
                                                    const float* __restrict__ mean_in, const float* __restrict__ rstd_in,
                                                    void* __restrict__ dx, float* __restrict__ dw_partial,
                                                    float* __restrict__ db_partial, int64_t M, int N, int qb, const LnAddArgs& A) {
    __shared__ float smem[4];
    float block_max = 0.0f;  // ADD: largest group scale this thread has seen
    constexpr bool kAffine = WMODE != kNoParam;
    float accw[kAffine ? ITERS : 1][16], accb[kAffine ? ITERS : 1][16];
    if (kAffine) {
#pragma unroll
        for (int it = 0; it < ITERS; it++)
#pragma unroll
            for (int i = 0; i < 16; i++) accw[it][i] = accb[it][i] = 0.0f;
    }
    for (int64_t row = blockIdx.x; row < M; row += gridDim.x) {
        const int64_t row_off = row * N, srow_off = row * (N / qb);
        const float mean = mean_in[row], rstd = rstd_in[row];
        float xhat[ITERS][16], wdy[ITERS][16];
        uint4 ra[ADD ? ITERS : 1][2];  // ADD: the residual gradient's chunks, requested before the row is reduced
        float dot = 0.0f, sum = 0.0f;
#pragma unroll
        for (int it = 0; it < ITERS; it++) {
            const int col = (threadIdx.x + it * 256) * 16;
            if (ADD) {  // unconditional load from a clamped column (a load under a branch is waited for on the spot)
                const uint4* rp = (const uint4*)((const uint16_t*)A.radd + row_off + (col < N ? col : 0));
                ra[it][0] = rp[0];
                ra[it][1] = rp[1];
            }
            if (col < N) {
                float xv[16], wv[16], gv[16];
                dequant16<KIND>(q, s, s_dt, row_off, srow_off, col, qb, xv);
                load_wb16<WMODE>(w, col, wv);
                load_bf16_16(dy, row_off + col, gv);
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    xhat[it][i] = (xv[i] - mean) * rstd;
                    wdy[it][i] = kAffine ? wv[i] * gv[i] : gv[i];
                    dot += xhat[it][i] * wdy[it][i];
                    sum += wdy[it][i];
                    if (kAffine) {
                        accw[it][i] += gv[i] * xhat[it][i];
                        accb[it][i] += gv[i];
                    }
                }
            }
        }
        const float c1 = block_sum_256(dot, smem) / (float)N;
        const float c2 = block_sum_256(sum, smem) / (float)N;
#pragma unroll
        for (int it = 0; it < ITERS; it++) {
            const int col = (threadIdx.x + it * 256) * 16;
            float gm = 0.0f;  // ADD: max |sum| of this thread's chunk (0 past the row's end)
            if (col < N) {
                float o[16];
#pragma unroll
                for (int i = 0; i < 16; i++) o[i] = (wdy[it][i] - (xhat[it][i] * c1 + c2)) * rstd;
                if (ADD) {
                    const uint32_t rw[8] = {ra[it][0].x, ra[it][0].y, ra[it][0].z, ra[it][0].w,
                                            ra[it][1].x, ra[it][1].y, ra[it][1].z, ra[it][1].w};
#pragma unroll
                    for (int i = 0; i < 8; i++) {
                        o[2 * i] = bf16lo(rw[i]) + round_to<kBF16>(o[2 * i]);
                        o[2 * i + 1] = bf16hi(rw[i]) + round_to<kBF16>(o[2 * i + 1]);
                    }
                }
                store_bf16_16(dx, row_off + col, o);
                if (ADD) {
                    float am = fmaxf(fabsf(o[0]), fabsf(o[1]));
#pragma unroll
                    for (int i = 2; i < 16; i++) am = fmaxf(am, fabsf(o[i]));
                    gm = am;
                }
            }
            if (ADD) {  // neighbouring threads hold neighbouring chunks: a group of qb columns is qb / 16 lanes
                const int lpg = qb >> 4;
                const float am = cluster_max_rt(gm, lpg);
                const float sg = A.kind_out == kE5M2 ? group_scale<kE5M2>(am) : group_scale<kE4M3>(am);
                if (col < N) {
                    if ((threadIdx.x & (lpg - 1)) == 0) ((uint16_t*)A.s_pg)[row * (N / qb) + col / qb] = (uint16_t)f2bf16(sg);
                    block_max = fmaxf(block_max, sg);
                }
            }
        }
    }
    if (ADD) {
        __syncthreads();  // the last row's sums may still be read from smem
        block_atomic_max_nonneg(A.s_max, block_max, smem);
    }
    if (kAffine) {
#pragma unroll
        for (int it = 0; it < ITERS; it++) {
            const int col = (threadIdx.x + it * 256) * 16;
            if (col < N) {
                float4* dw = (float4*)(dw_partial + (int64_t)blockIdx.x * N + col);
                float4* db = (float4*)(db_partial + (int64_t)blockIdx.x * N + col);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    dw[i] = make_float4(accw[it][4 * i], accw[it][4 * i + 1], accw[it][4 * i + 2], accw[it][4 * i + 3]);
                    db[i] = make_float4(accb[it][4 * i], accb[it][4 * i + 1], accb[it][4 * i + 2], accb[it][4 * i + 3]);
                }
            }
        }
    }
}

template <int KIND, int WMODE, int ITERS>
__global__ __launch_bounds__(256) void k_layernorm_bwd(const uint8_t* __restrict__ q, const void* __restrict__ s, int s_dt,
                                                        const void* __restrict__ dy, const void* __restrict__ w,
                                                        const float* __restrict__ mean_in, const float* __restrict__ rstd_in,
                                                        void* __restrict__ dx, float* __restrict__ dw_partial,
                                                        float* __restrict__ db_partial, int64_t M, int N, int qb) {
    layernorm_bwd_body<KIND, WMODE, ITERS, false>(q, s, s_dt, dy, w, mean_in, rstd_in, dx, dw_partial, db_partial, M, N, qb, LnAddArgs{});
}
template <int KIND, int WMODE, int ITERS>
__global__ __launch_bounds__(256) void k_layernorm_bwd_add(const uint8_t* __restrict__ q, const void* __restrict__ s, int s_dt,
                                                            const void* __restrict__ dy, const void* __restrict__ w,
                                                            const float* __restrict__ mean_in, const float* __restrict__ rstd_in,
                                                            void* __restrict__ dx, float* __restrict__ dw_partial,
                                                            float* __restrict__ db_partial, int64_t M, int N, int qb, LnAddArgs A) {
    layernorm_bwd_body<KIND, WMODE, ITERS, true>(q, s, s_dt, dy, w, mean_in, rstd_in, dx, dw_partial, db_partial, M, N, qb, A);
}

}  // namespace coat

using namespace coat;

static int ln_check(int64_t M, int64_t N, int QB) {
    if (M < 0 || N < 0) return COAT_EINVAL;
    if (QB < 16 || (QB & (QB - 1)) || N % QB != 0 || N % 16 != 0) return COAT_ESHAPE;
    if (N > 16384) return COAT_ESHAPE;  // a row is held in registers: 4 chunks of 16 per lane at most
    return COAT_OK;
}

// w_dtype < 0: no affine parameters
#define LN_CASE(KERNEL, GRID, K, W, I, ...)                                                           \
    case ((K * 4 + W) * 3 + (I == 1 ? 0 : (I == 2 ? 1 : 2))):                                          \
        hipLaunchKernelGGL((KERNEL<K, W, I>), dim3((unsigned)(GRID)), dim3(256), 0, st, __VA_ARGS__);  \
        break;
#define LN_CASES_W(KERNEL, GRID, K, W, ...) \
    LN_CASE(KERNEL, GRID, K, W, 1, __VA_ARGS__) LN_CASE(KERNEL, GRID, K, W, 2, __VA_ARGS__) LN_CASE(KERNEL, GRID, K, W, 4, __VA_ARGS__)
#define LN_CASES_K(KERNEL, GRID, K, ...)                                                          \
    LN_CASES_W(KERNEL, GRID, K, 0, __VA_ARGS__) LN_CASES_W(KERNEL, GRID, K, 1, __VA_ARGS__)       \
    LN_CASES_W(KERNEL, GRID, K, 2, __VA_ARGS__) LN_CASES_W(KERNEL, GRID, K, 3, __VA_ARGS__)
#define LN_DISPATCH(KERNEL, GRID, ...)                                                            \
    {                                                                                             \
        const int iters = N <= 4096 ? 1 : (N <= 8192 ? 2 : 4);                                    \
        const int wmode = w_dtype < 0 ? kNoParam : w_dtype;                                       \
        if (fp8 != COAT_E4M3 && fp8 != COAT_E5M2) return COAT_EINVAL;                             \
        if (wmode > kNoParam) return COAT_EDTYPE;                                                 \
        switch ((fp8 * 4 + wmode) * 3 + (iters == 1 ? 0 : (iters == 2 ? 1 : 2))) {                \
            LN_CASES_K(KERNEL, GRID, 0, __VA_ARGS__)                                              \
            LN_CASES_K(KERNEL, GRID, 1, __VA_ARGS__)                                              \
            default: return COAT_EINVAL;                                                          \
        }                                                                                         \
    }

extern "C" int coat_fp8_layernorm_forward(const void* x, int fp8, const void* s_x, int s_dtype, const void* w,
                                          const void* b, int w_dtype, float* y, void* s_row, float* mean, float* rstd,
                                          float* s_max, int64_t M, int64_t N, int QB, float eps, void* stream) {
    if (int e = ln_check(M, N, QB)) return e;
    if (M * N == 0) return COAT_OK;
    if (!x || !s_x || !s_row || !mean || !rstd || !s_max) return COAT_EINVAL;  // y may be NULL
    if (w_dtype >= 0 && (!w || !b)) return COAT_EINVAL;
    if (s_dtype < 0 || s_dtype > 2) return COAT_EDTYPE;
    if (!coat_aligned16(x) || !coat_aligned16(y) || !coat_aligned16(w) || !coat_aligned16(b)) return COAT_EALIGN;
    hipStream_t st = (hipStream_t)stream;
    LN_DISPATCH(k_layernorm_fwd, M, (const uint8_t*)x, s_x, s_dtype, w, b, y, s_row, mean, rstd, s_max, (int)N, QB, eps)
    return coat_launch_status();
}

static int layernorm_backward_common(const void* x, int fp8, const void* s_x, int s_dtype, const void* dy, const void* w,
                                     int w_dtype, const float* mean, const float* rstd, void* dx, void* dw, void* db,
                                     float* dw_partial, float* db_partial, int n_partial, int64_t M, int64_t N, int QB,
                                     const LnAddArgs* add, void* stream) {
    if (int e = ln_check(M, N, QB)) return e;
    if (add && QB > 1024) return COAT_ESHAPE;  // a group's chunks sit in the lanes of one wave
    if (M * N == 0) return COAT_OK;
    if (!x || !s_x || !dy || !mean || !rstd || !dx) return COAT_EINVAL;
    if (add && (!add->radd || !add->s_pg || !add->s_max || !coat_aligned16(add->radd))) return add->radd && add->s_pg && add->s_max ? COAT_EALIGN : COAT_EINVAL;
    if (w_dtype >= 0 && (!w || !dw || !db || !dw_partial || !db_partial || n_partial <= 0)) return COAT_EINVAL;
    if (s_dtype < 0 || s_dtype > 2) return COAT_EDTYPE;
    if (!coat_aligned16(x) || !coat_aligned16(w) || !coat_aligned16(dy) || !coat_aligned16(dx) ||
        !coat_aligned16(dw_partial) || !coat_aligned16(db_partial))
        return COAT_EALIGN;
    hipStream_t st = (hipStream_t)stream;
    int64_t grid = w_dtype >= 0 ? (n_partial < M ? n_partial : M) : (M < 2048 ? M : 2048);
    if (add) {
        LN_DISPATCH(k_layernorm_bwd_add, grid, (const uint8_t*)x, s_x, s_dtype, dy, w, mean, rstd, dx, dw_partial, db_partial, M, (int)N, QB, *add)
    } else {
        LN_DISPATCH(k_layernorm_bwd, grid, (const uint8_t*)x, s_x, s_dtype, dy, w, mean, rstd, dx, dw_partial, db_partial, M, (int)N, QB)
    }
    if (int e = coat_launch_status()) return e;
    if (w_dtype < 0) return COAT_OK;
    const int cols_blocks = (int)((N + kColsumCols - 1) / kColsumCols);
    switch (w_dtype) {
        case COAT_F32:
            hipLaunchKernelGGL((k_norm_colsum<kF32>), dim3(cols_blocks), dim3(kColsumThreads), 0, st, dw_partial, dw, (int)grid, (int)N);
            hipLaunchKernelGGL((k_norm_colsum<kF32>), dim3(cols_blocks), dim3(kColsumThreads), 0, st, db_partial, db, (int)grid, (int)N);
            break;
        case COAT_BF16:
            hipLaunchKernelGGL((k_norm_colsum<kBF16>), dim3(cols_blocks), dim3(kColsumThreads), 0, st, dw_partial, dw, (int)grid, (int)N);
            hipLaunchKernelGGL((k_norm_colsum<kBF16>), dim3(cols_blocks), dim3(kColsumThreads), 0, st, db_partial, db, (int)grid, (int)N);
            break;
        default:
            hipLaunchKernelGGL((k_norm_colsum<kF16>), dim3(cols_blocks), dim3(kColsumThreads), 0, st, dw_partial, dw, (int)grid, (int)N);
            hipLaunchKernelGGL((k_norm_colsum<kF16>), dim3(cols_blocks), dim3(kColsumThreads), 0, st, db_partial, db, (int)grid, (int)N);
            break;
    }
    return coat_launch_status();
}

extern "C" int coat_fp8_layernorm_backward(const void* x, int fp8, const void* s_x, int s_dtype, const void* dy,
                                           const void* w, int w_dtype, const float* mean, const float* rstd, void* dx,
                                           void* dw, void* db, float* dw_partial, float* db_partial, int n_partial,
                                           int64_t M, int64_t N, int QB, void* stream) {
    return layernorm_backward_common(x, fp8, s_x, s_dtype, dy, w, w_dtype, mean, rstd, dx, dw, db, dw_partial, db_partial,
                                     n_partial, M, N, QB, nullptr, stream);
}

extern "C" int coat_fp8_layernorm_backward_add(const void* x, int fp8, const void* s_x, int s_dtype, const void* dy,
                                               const void* w, int w_dtype, const float* mean, const float* rstd,
                                               const void* residual_grad, void* y, void* s_pg, float* s_max, int fp8_out,
                                               void* dw, void* db, float* dw_partial, float* db_partial, int n_partial,
                                               int64_t M, int64_t N, int QB, void* stream) {
    if (fp8_out != COAT_E4M3 && fp8_out != COAT_E5M2) return COAT_EINVAL;
    const LnAddArgs add{residual_grad, s_pg, s_max, fp8_out == COAT_E5M2 ? kE5M2 : kE4M3};
    return layernorm_backward_common(x, fp8, s_x, s_dtype, dy, w, w_dtype, mean, rstd, y, dw, db, dw_partial, db_partial,
                                     n_partial, M, N, QB, &add, stream);
}
