// FP8 RMSNorm forward / backward for gfx950.
//
// Reference: coat/activation/real_quantization/func_rmsnorm.py (_rms_norm_fwd_fused :54-111,
// _rms_norm_bwd_dx_fused :121-196, _rms_norm_bwd_dwdb :200-220).
//
// One 256-thread block per row; a lane owns 16-element chunks `lane + 256*it` of the row (16 B of FP8 codes,
// 2 x 16 B of bf16 per chunk), so a row of up to 16384 columns lives in registers for the two passes over it
// (statistic, then normalise).  Row sums are reduced in a fixed order (in-lane, DPP butterfly per wave, then
// the four wave partials in index order), so results are deterministic, unlike the reference's lock-ordered dw.
// dw is a two-stage reduction: every block accumulates the rows it owns into fp32 registers and writes one
// partial row; a second kernel sums the partials in block order.
#include <math.h>

#include <atomic>

#include "coat_host.h"
#include "norm_common.h"

namespace coat {

// Forward: y = bf16(x * rstd * w), rstd[row], row scale (max|y| + 1e-10)/fp8max (bf16), tensor max of the row scales.
template <int KIND, int WDT, int ITERS>
__global__ __launch_bounds__(256) void k_rmsnorm_fwd(const uint8_t* __restrict__ q, const void* __restrict__ s, int s_dt,
                                                      const void* __restrict__ w, void* __restrict__ y,
                                                      void* __restrict__ s_row, float* __restrict__ rstd_out,
                                                      float* __restrict__ s_max, int N, int qb, float eps) {
    __shared__ float smem[4];
    const int64_t row = blockIdx.x;
    const int64_t row_off = row * N, srow_off = row * (N / qb);
    float x[ITERS][16];
    float ss = 0.0f;
#pragma unroll
    for (int it = 0; it < ITERS; it++) {
        const int col = (threadIdx.x + it * 256) * 16;
        if (col < N) {
            dequant16<KIND>(q, s, s_dt, row_off, srow_off, col, qb, x[it]);
#pragma unroll
            for (int i = 0; i < 16; i++) ss += x[it][i] * x[it][i];
        }
    }
    const float var = block_sum_256(ss, smem) / (float)N;
    const float rstd = 1 / sqrtf(var + eps);
    float amax = 0.0f;
#pragma unroll
    for (int it = 0; it < ITERS; it++) {
        const int col = (threadIdx.x + it * 256) * 16;
        if (col < N) {
            float wv[16], yv[16];
            load_w16<WDT>(w, col, wv);
#pragma unroll
            for (int i = 0; i < 16; i++) {
                yv[i] = (x[it][i] * rstd) * wv[i];
                amax = fmaxf(amax, fabsf(yv[i]));
            }
            if (y) store_bf16_16(y, row_off + col, yv);  // NULL: statistics only (the division recomputes y)
        }
    }
    amax = block_max_256(amax, smem);
    if (threadIdx.x == 0) {
        const float sr = group_scale<KIND>(amax);
        ((uint16_t*)s_row)[row] = (uint16_t)f2bf16(sr);
        rstd_out[row] = rstd;
        atomic_max_nonneg(s_max, sr);
    }
}

// Backward: dx = bf16((w*dy - xhat * mean(xhat*w*dy)) * rstd); per-block partial of dw = sum_rows dy * xhat.
template <int KIND, int WDT, int ITERS>
__global__ __launch_bounds__(256) void k_rmsnorm_bwd(const uint8_t* __restrict__ q, const void* __restrict__ s, int s_dt,
                                                      const void* __restrict__ dy, const void* __restrict__ dy2,
                                                      const void* __restrict__ dy3, const void* __restrict__ w,
                                                      const float* __restrict__ rstd_in, void* __restrict__ dx,
                                                      float* __restrict__ dw_partial, int64_t M, int N, int qb) {
    __shared__ float smem[4];
    float acc[ITERS][16];
#pragma unroll
    for (int it = 0; it < ITERS; it++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[it][i] = 0.0f;
    for (int64_t row = blockIdx.x; row < M; row += gridDim.x) {
        const int64_t row_off = row * N, srow_off = row * (N / qb);
        const float rstd = rstd_in[row];
        float xhat[ITERS][16], wdy[ITERS][16];
        float dot = 0.0f;
#pragma unroll
        for (int it = 0; it < ITERS; it++) {
            const int col = (threadIdx.x + it * 256) * 16;
            if (col < N) {
                float xv[16], wv[16], gv[16];
                dequant16<KIND>(q, s, s_dt, row_off, srow_off, col, qb, xv);
                load_w16<WDT>(w, col, wv);
                load_bf16_16(dy, row_off + col, gv);
                // optional further gradients of the same tensor, summed the way a chain of bf16 tensor additions
                // would: (dy + dy2) rounded to bf16, then + dy3 rounded to bf16 (block-uniform branches)
                if (dy2) {
                    float g2[16];
                    load_bf16_16(dy2, row_off + col, g2);
#pragma unroll
                    for (int i = 0; i < 16; i++) gv[i] = round_to<kBF16>(gv[i] + g2[i]);
                    if (dy3) {
                        load_bf16_16(dy3, row_off + col, g2);
#pragma unroll
                        for (int i = 0; i < 16; i++) gv[i] = round_to<kBF16>(gv[i] + g2[i]);
                    }
                }
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    xhat[it][i] = xv[i] * rstd;
                    wdy[it][i] = wv[i] * gv[i];
                    dot += xhat[it][i] * wdy[it][i];
                    acc[it][i] += gv[i] * xhat[it][i];
                }
            }
        }
        const float c1 = block_sum_256(dot, smem) / (float)N;
#pragma unroll
        for (int it = 0; it < ITERS; it++) {
            const int col = (threadIdx.x + it * 256) * 16;
            if (col < N) {
                float o[16];
#pragma unroll
                for (int i = 0; i < 16; i++) o[i] = (wdy[it][i] - (xhat[it][i] * c1)) * rstd;
                store_bf16_16(dx, row_off + col, o);
            }
        }
    }
#pragma unroll
    for (int it = 0; it < ITERS; it++) {
        const int col = (threadIdx.x + it * 256) * 16;
        if (col < N) {
            float4* dst = (float4*)(dw_partial + (int64_t)blockIdx.x * N + col);
#pragma unroll
            for (int i = 0; i < 4; i++) dst[i] = make_float4(acc[it][4 * i], acc[it][4 * i + 1], acc[it][4 * i + 2], acc[it][4 * i + 3]);
        }
    }
}

}  // namespace coat

using namespace coat;

static int rms_check(int64_t M, int64_t N, int QB) {
    if (M < 0 || N < 0) return COAT_EINVAL;
    if (QB < 16 || (QB & (QB - 1)) || N % QB != 0 || N % 16 != 0) return COAT_ESHAPE;
    if (N > 16384) return COAT_ESHAPE;  // a row is held in registers: 4 chunks of 16 per lane at most
    return COAT_OK;
}

#define RMS_DISPATCH(KERNEL, GRID, ...)                                                                                \
    {                                                                                                                  \
        const int iters = N <= 4096 ? 1 : (N <= 8192 ? 2 : 4);                                                         \
        if (fp8 != COAT_E4M3 && fp8 != COAT_E5M2) return COAT_EINVAL;                                                  \
        if (w_dtype != COAT_BF16 && w_dtype != COAT_F32 && w_dtype != COAT_F16) return COAT_EDTYPE;                    \
        switch ((fp8 * 3 + w_dtype) * 3 + (iters == 1 ? 0 : (iters == 2 ? 1 : 2))) {                                   \
            RMS_CASES(KERNEL, GRID, __VA_ARGS__)                                                                       \
            default: return COAT_EINVAL;                                                                               \
        }                                                                                                              \
    }
#define RMS_CASE(KERNEL, GRID, K, W, I, ...)                                                                           \
    case ((K * 3 + W) * 3 + (I == 1 ? 0 : (I == 2 ? 1 : 2))):                                                          \
        hipLaunchKernelGGL((KERNEL<K, W, I>), dim3((unsigned)(GRID)), dim3(256), 0, st, __VA_ARGS__);                  \
        break;
#define RMS_CASES(KERNEL, GRID, ...)                                                                                   \
    RMS_CASE(KERNEL, GRID, 0, 0, 1, __VA_ARGS__) RMS_CASE(KERNEL, GRID, 0, 0, 2, __VA_ARGS__) RMS_CASE(KERNEL, GRID, 0, 0, 4, __VA_ARGS__) \
    RMS_CASE(KERNEL, GRID, 0, 1, 1, __VA_ARGS__) RMS_CASE(KERNEL, GRID, 0, 1, 2, __VA_ARGS__) RMS_CASE(KERNEL, GRID, 0, 1, 4, __VA_ARGS__) \
    RMS_CASE(KERNEL, GRID, 0, 2, 1, __VA_ARGS__) RMS_CASE(KERNEL, GRID, 0, 2, 2, __VA_ARGS__) RMS_CASE(KERNEL, GRID, 0, 2, 4, __VA_ARGS__) \
    RMS_CASE(KERNEL, GRID, 1, 0, 1, __VA_ARGS__) RMS_CASE(KERNEL, GRID, 1, 0, 2, __VA_ARGS__) RMS_CASE(KERNEL, GRID, 1, 0, 4, __VA_ARGS__) \
    RMS_CASE(KERNEL, GRID, 1, 1, 1, __VA_ARGS__) RMS_CASE(KERNEL, GRID, 1, 1, 2, __VA_ARGS__) RMS_CASE(KERNEL, GRID, 1, 1, 4, __VA_ARGS__) \
    RMS_CASE(KERNEL, GRID, 1, 2, 1, __VA_ARGS__) RMS_CASE(KERNEL, GRID, 1, 2, 2, __VA_ARGS__) RMS_CASE(KERNEL, GRID, 1, 2, 4, __VA_ARGS__)

extern "C" int coat_fp8_rmsnorm_forward(const void* x, int fp8, const void* s_x, int s_dtype, const void* w, int w_dtype,
                                        void* y, void* s_row, float* rstd, float* s_max, int64_t M, int64_t N, int QB,
                                        float eps, void* stream) {
    if (int e = rms_check(M, N, QB)) return e;
    if (M * N == 0) return COAT_OK;
    if (!x || !s_x || !w || !s_row || !rstd || !s_max) return COAT_EINVAL;  // y may be NULL
    if (!coat_aligned16(x) || !coat_aligned16(w) || !coat_aligned16(y)) return COAT_EALIGN;
    hipStream_t st = (hipStream_t)stream;
    RMS_DISPATCH(k_rmsnorm_fwd, M, (const uint8_t*)x, s_x, s_dtype, w, y, s_row, rstd, s_max, (int)N, QB, eps)
    return coat_launch_status();
}

// Shared by the two backward entry points: dx kernel on min(n_partial, M) blocks, then the column sum of their partial rows.
static int rms_backward_launch(const void* x, int fp8, const void* s_x, int s_dtype, const void* dy, const void* dy2,
                               const void* dy3, const void* w, int w_dtype, const float* rstd, void* dx, void* dw,
                               float* dw_partial, int64_t n_partial, int64_t M, int64_t N, int QB, hipStream_t st) {
    const int64_t grid = n_partial < M ? n_partial : M;
    RMS_DISPATCH(k_rmsnorm_bwd, grid, (const uint8_t*)x, s_x, s_dtype, dy, dy2, dy3, w, rstd, dx, dw_partial, M, (int)N, QB)
    if (int e = coat_launch_status()) return e;
    const int cols_blocks = (int)((N + 15) / 16);
    switch (w_dtype) {
        case COAT_F32: hipLaunchKernelGGL((k_norm_colsum<kF32>), dim3(cols_blocks), dim3(256), 0, st, dw_partial, dw, (int)grid, (int)N); break;
        case COAT_BF16: hipLaunchKernelGGL((k_norm_colsum<kBF16>), dim3(cols_blocks), dim3(256), 0, st, dw_partial, dw, (int)grid, (int)N); break;
        default: hipLaunchKernelGGL((k_norm_colsum<kF16>), dim3(cols_blocks), dim3(256), 0, st, dw_partial, dw, (int)grid, (int)N); break;
    }
    return coat_launch_status();
}

static int rms_backward_check(const void* x, const void* s_x, const void* dy, const void* dy2, const void* dy3, const void* w,
                              const float* rstd, void* dx, void* dw) {
    if (!x || !s_x || !dy || !w || !rstd || !dx || !dw) return COAT_EINVAL;
    if (!coat_aligned16(x) || !coat_aligned16(w) || !coat_aligned16(dy) || !coat_aligned16(dx) || !coat_aligned16(dy2) ||
        !coat_aligned16(dy3))
        return COAT_EALIGN;
    if (dy3 && !dy2) return COAT_EINVAL;
    return COAT_OK;
}

extern "C" int coat_fp8_rmsnorm_backward(const void* x, int fp8, const void* s_x, int s_dtype, const void* dy,
                                         const void* dy2, const void* dy3, const void* w, int w_dtype, const float* rstd,
                                         void* dx, void* dw, float* dw_partial, int n_partial, int64_t M, int64_t N,
                                         int QB, void* stream) {
    if (int e = rms_check(M, N, QB)) return e;
    if (M * N == 0) return COAT_OK;
    if (!dw_partial || n_partial <= 0) return COAT_EINVAL;
    if (int e = rms_backward_check(x, s_x, dy, dy2, dy3, w, rstd, dx, dw)) return e;
    if (!coat_aligned16(dw_partial)) return COAT_EALIGN;
    return rms_backward_launch(x, fp8, s_x, s_dtype, dy, dy2, dy3, w, w_dtype, rstd, dx, dw, dw_partial, n_partial, M, N, QB,
                               (hipStream_t)stream);
}

// ------------------------------------------------------------------------------------------------ no allocation
// The weight-gradient partial rows of the entry point below live in this array instead of a caller-provided workspace:
// 16 MiB per GPU, held from the moment the library is loaded until the process ends.  In host code `dw_scratch` is only a
// handle for hipGetSymbolAddress; the device address is looked up once per device (each GPU has its own copy of the array at
// its own address) and only that pointer is ever passed to a kernel.
constexpr int64_t kDwScratchFloats = (int64_t)COAT_RMSNORM_STATIC_PARTIALS * COAT_RMSNORM_STATIC_FULL_N;
static __device__ __align__(256) float dw_scratch[kDwScratchFloats];
static std::atomic<float*> dw_scratch_ptr[kCoatMaxDevices];

static int dw_scratch_address(float** out) {
    const int dev = coat_device_index();
    if (dev < 0) return COAT_EINVAL;
    float* p = dw_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        // the current device is `dev`: the address returned is that device's copy.  Two threads racing here store the same value.
        hipError_t e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(dw_scratch));
        if (e != hipSuccess) return (int)e;
        if (!p) return COAT_EINVAL;
        dw_scratch_ptr[dev].store(p, std::memory_order_release);
    }
    *out = p;
    return COAT_OK;
}

extern "C" int coat_fp8_rmsnorm_backward_static(const void* x, int fp8, const void* s_x, int s_dtype, const void* dy,
                                                const void* dy2, const void* dy3, const void* w, int w_dtype,
                                                const float* rstd, void* dx, void* dw, int64_t M, int64_t N, int QB,
                                                void* stream) {
    if (int e = rms_check(M, N, QB)) return e;  // N > 16384 is beyond what the scratch rows (and the kernels) hold
    if (M * N == 0) return COAT_OK;
    if (int e = rms_backward_check(x, s_x, dy, dy2, dy3, w, rstd, dx, dw)) return e;
    float* partial = nullptr;
    if (int e = dw_scratch_address(&partial)) return e;
    // every block writes its whole partial row and the column sum reads only the rows of this launch's blocks, so
    // nothing has to be cleared between calls
    return rms_backward_launch(x, fp8, s_x, s_dtype, dy, dy2, dy3, w, w_dtype, rstd, dx, dw, partial,
                               coat_rmsnorm_static_partials(N), M, N, QB, (hipStream_t)stream);
}
