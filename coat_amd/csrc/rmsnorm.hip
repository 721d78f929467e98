// FP8 RMSNorm forward / backward for gfx950.
//
// Reference: coat/activation/real_quantization/func_rmsnorm.py (_rms_norm_fwd_fused :54-111,
// _rms_norm_bwd_dx_fused :121-196, _rms_norm_bwd_dwdb :200-220).
//
// Rows up to 8192 columns: one wave per row (k_rmsnorm_fwd / k_rmsnorm_bwd below).  Wider rows, up to 16384 columns: one
// 256-thread block per row (k_rmsnorm_*_block); a lane owns 16-element chunks `lane + 256*it` of the row (16 B of FP8
// codes, 2 x 16 B of bf16 per chunk), so the row lives in registers for the two passes over it (statistic, then
// normalise).  Row sums are reduced in a fixed order (in-lane, DPP butterfly per wave, then the four wave partials in
// index order) in both layouts, so results are deterministic and independent of the layout, unlike the reference's
// lock-ordered dw.  dw is a two-stage reduction: every block accumulates the rows it owns into fp32 registers and writes
// one partial row; a second kernel sums the partials in block order.
#include <math.h>

#include <atomic>

#include "coat_host.h"
#include "norm_common.h"

namespace coat {

// Forward: y = bf16(x * rstd * w), rstd[row], row scale (max|y| + 1e-10)/fp8max (bf16), tensor max of the row scales.
template <int KIND, int WDT, int ITERS>
__global__ __launch_bounds__(256) void k_rmsnorm_fwd_block(const uint8_t* __restrict__ q, const void* __restrict__ s, int s_dt,
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
        atomic_max_nonneg(max_slot(s_max), sr);
    }
}

// Backward: dx = bf16((w*dy - xhat * mean(xhat*w*dy)) * rstd); per-block partial of dw = sum_rows dy * xhat.
template <int KIND, int WDT, int ITERS>
__global__ __launch_bounds__(256) void k_rmsnorm_bwd_block(const uint8_t* __restrict__ q, const void* __restrict__ s, int s_dt,
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


// ------------------------------------------------------------------------------------------------ one wave per row
// Rows up to 8192 columns.  A wave owns whole rows: lane l holds the 16-element chunks c * 64 + l (c < CH), so every load
// instruction of the wave covers 1 KiB of consecutive codes, all loads of a row are in flight before the first
// conversion, the next row's codes are requested before the current row is reduced (forward), and nothing waits at a
// block-wide barrier.  The weight stays in registers for all rows of the wave.
// The row sums are formed exactly as the block-per-row kernels above form them (chunk c belongs to "wave" c & 3 of that
// kernel: in-lane running sum over c, c + 4, ..., one butterfly per partial, the four partials added in index order),
// so rstd, dx and every code derived from them are bit-identical between the two layouts.
template <int CH> struct RowRaw {
    uint4 codes[CH];
    uint32_t sc[CH];
};
template <int CH>
__device__ __forceinline__ void load_row(const uint8_t* __restrict__ q, const void* __restrict__ s, int s_dt, int64_t row, int N,
                                         int qb, int lane, RowRaw<CH>& r) {
    const uint8_t* qr = q + row * N;
    const int64_t srow = row * (N / qb);
#pragma unroll
    for (int c = 0; c < CH; c++) {
        const int col = (c * 64 + lane) * 16;
        if (col < N) {
            r.codes[c] = *(const uint4*)(qr + col);
            const int64_t si = srow + col / qb;
            r.sc[c] = s_dt == kF32 ? ((const uint32_t*)s)[si] : (uint32_t)((const uint16_t*)s)[si];
        }
    }
}
__device__ __forceinline__ float scale_from_raw(uint32_t u, int s_dt) {
    if (s_dt == kBF16) return u2f(u << 16);
    if (s_dt == kF32) return u2f(u);
    return f16lo(u);
}
template <int KIND> __device__ __forceinline__ void decode16(const uint4& c, float sc, float* v) {
    const uint32_t w[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
    for (int k = 0; k < 4; k++) {
        float f[4];
        fp8x4_to_f32<KIND>(w[k], f);
#pragma unroll
        for (int i = 0; i < 4; i++) v[4 * k + i] = f[i] * sc;
    }
}
template <int WDT> __device__ __forceinline__ void unpack_w16(const uint4* p, float* o) {
    const uint32_t u[8] = {p[0].x, p[0].y, p[0].z, p[0].w, p[1].x, p[1].y, p[1].z, p[1].w};
#pragma unroll
    for (int k = 0; k < 8; k++) {
        o[2 * k] = WDT == kBF16 ? bf16lo(u[k]) : f16lo(u[k]);
        o[2 * k + 1] = WDT == kBF16 ? bf16hi(u[k]) : f16hi(u[k]);
    }
}
// the four partial sums of a row, reduced and added in the block-per-row kernel's order
__device__ __forceinline__ float row_sum4(float* part) {
#pragma unroll
    for (int k = 0; k < 4; k++) part[k] = cluster_sum<64>(part[k]);
    return ((part[0] + part[1]) + part[2]) + part[3];
}

template <int KIND, int WDT, int CH>
__global__ __launch_bounds__(256) void k_rmsnorm_fwd(const uint8_t* __restrict__ q, const void* __restrict__ s, int s_dt,
                                                      const void* __restrict__ w, void* __restrict__ y,
                                                      void* __restrict__ s_row, float* __restrict__ rstd_out,
                                                      float* __restrict__ s_max, int64_t M, int N, int qb, float eps) {
    constexpr bool HOLD_W = WDT != kF32;  // 8 registers per chunk; an fp32 weight is re-read from the cache per row
    const int lane = threadIdx.x & 63;
    const int64_t nwaves = (int64_t)gridDim.x * 4;
    int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    uint4 wreg[HOLD_W ? CH : 1][2];
    if (HOLD_W) {
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int col = (c * 64 + lane) * 16;
            if (col < N) {
                const uint4* wp = (const uint4*)((const uint16_t*)w + col);
                wreg[c][0] = wp[0];
                wreg[c][1] = wp[1];
            }
        }
    }
    RowRaw<CH> cur, nxt;
    if (row < M) load_row<CH>(q, s, s_dt, row, N, qb, lane, cur);
    float wave_max = 0.0f;
    while (row < M) {
        const int64_t nrow = row + nwaves;
        if (nrow < M) load_row<CH>(q, s, s_dt, nrow, N, qb, lane, nxt);
        float part[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int c = 0; c < CH; c++) {
            if ((c * 64 + lane) * 16 < N) {
                float x[16];
                decode16<KIND>(cur.codes[c], scale_from_raw(cur.sc[c], s_dt), x);
#pragma unroll
                for (int i = 0; i < 16; i++) part[c & 3] += x[i] * x[i];
            }
        }
        const float var = row_sum4(part) / (float)N;
        const float rstd = 1 / sqrtf(var + eps);
        float amax = 0.0f;
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int col = (c * 64 + lane) * 16;
            if (col < N) {
                float x[16], wv[16], yv[16];
                decode16<KIND>(cur.codes[c], scale_from_raw(cur.sc[c], s_dt), x);
                if (HOLD_W) unpack_w16<WDT>(wreg[c], wv);
                else load_w16<WDT>(w, col, wv);
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    yv[i] = (x[i] * rstd) * wv[i];
                    amax = fmaxf(amax, fabsf(yv[i]));
                }
                if (y) store_bf16_16(y, row * N + col, yv);  // NULL: statistics only (the division recomputes y)
            }
        }
        amax = cluster_max<64>(amax);
        const float sr = group_scale<KIND>(amax);
        wave_max = fmaxf(wave_max, sr);
        if (lane == 0) {
            ((uint16_t*)s_row)[row] = (uint16_t)f2bf16(sr);
            rstd_out[row] = rstd;
        }
        cur = nxt;
        row = nrow;
    }
    // one lazy atomic per block (waves without rows hold 0)
    __shared__ float wmax[4];
    if (lane == 0) wmax[threadIdx.x >> 6] = wave_max;
    __syncthreads();
    if (threadIdx.x == 0) atomic_max_nonneg(max_slot(s_max), fmaxf(fmaxf(wmax[0], wmax[1]), fmaxf(wmax[2], wmax[3])));
}

// Backward, one wave per row.  A block's four waves keep fp32 weight-gradient sums for the rows they walked; at the end
// they are added in wave order through LDS, 1024 columns at a time, into the block's partial row.
// MULTI: up to two further gradients of the same tensor are added to dy (dy2, dy3).  A variant of its own, because the
// extra loads in flight cost it the second resident block per CU, which the single-gradient kernel keeps.
// Five chunks (the 5120 columns of the 13B shape) with several gradients need 268 registers; held to 256, i.e. to two
// waves per SIMD with 12 registers spilled, the kernel takes 91 us per call in the 13B layer against 104 us with one wave
// per SIMD and no spill (128.7 us as 5 of 8 chunks, loaded chunk by chunk).
// ADD: the residual-gradient addition that follows in the layer (reference add_bwd.py:107-135 after
// func_rmsnorm.py:121-196) happens here: dx is rounded to bf16 as it would be stored, `radd` (bf16 [M, N]) is added in
// fp32, and what goes out is bf16 of the sum, the bf16 scale (amax + 1e-10) / fp8max of every 1 x qb group of the fp32 sum
// and the maximum of those scales (fp32) for the per-tensor division that follows.
struct RmsAddArgs {
    const void* radd;   // bf16 [M, N]
    void* s_pg;         // bf16 [M, N / qb]
    float* s_max;       // COAT_MAX_WORDS
    int kind_out;       // kE4M3 / kE5M2: the FP8 format the scales are for
};
template <int KIND, int WDT, int CH, bool MULTI, bool ADD = false>
__global__ __launch_bounds__(256, ((CH == 5 && MULTI) || (ADD && CH == 4)) ? 2 : 1) void k_rmsnorm_bwd(const uint8_t* __restrict__ q, const void* __restrict__ s, int s_dt,
                                                      const void* __restrict__ dy, const void* __restrict__ dy2,
                                                      const void* __restrict__ dy3, const void* __restrict__ w,
                                                      const float* __restrict__ rstd_in, void* __restrict__ dx,
                                                      float* __restrict__ dw_partial, int64_t M, int N, int qb,
                                                      RmsAddArgs A) {
    // MULTI spends those registers on gradient loads in flight; with five chunks they decide between one and two waves per
    // SIMD (61.3 -> 50.1 us at [8192, 5120]), with eight there is one wave either way and re-reading the weight costs 20 %
    constexpr bool HOLD_W = WDT != kF32 && !MULTI && CH != 5 && !ADD;
    __shared__ float red[4][64 * 16];
    const int lane = threadIdx.x & 63, wv_id = threadIdx.x >> 6;
    const int64_t nwaves = (int64_t)gridDim.x * 4;
    uint4 wreg[HOLD_W ? CH : 1][2];
    if (HOLD_W) {
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int col = (c * 64 + lane) * 16;
            if (col < N) {
                const uint4* wp = (const uint4*)((const uint16_t*)w + col);
                wreg[c][0] = wp[0];
                wreg[c][1] = wp[1];
            }
        }
    }
    float acc[CH][16];
#pragma unroll
    for (int c = 0; c < CH; c++)
#pragma unroll
        for (int i = 0; i < 16; i++) acc[c][i] = 0.0f;
    float wave_max = 0.0f;  // ADD: largest group scale this lane has seen
    for (int64_t row = (int64_t)blockIdx.x * 4 + wv_id; row < M; row += nwaves) {
        const int64_t row_off = row * N;
        RowRaw<CH> raw;
        uint4 g[CH][2];  // the (summed) gradient as packed bf16: exact, it is a bf16 value
        load_row<CH>(q, s, s_dt, row, N, qb, lane, raw);
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int col = (c * 64 + lane) * 16;
            if (col < N) {
                const uint4* gp = (const uint4*)((const uint16_t*)dy + row_off + col);
                g[c][0] = gp[0];
                g[c][1] = gp[1];
            }
        }
        // ADD: the residual gradient, two chunks in flight: chunk 0 is requested before the row is reduced, chunk c + 1
        // before chunk c is used (a whole row of it in registers costs the kernel its second wave per SIMD).
        uint4 ra[2][2];
        auto load_radd = [&](int c) {
            const int col = min((c * 64 + lane) * 16, N - 16);
            const uint4* p = (const uint4*)((const uint16_t*)A.radd + row_off + col);
            ra[c & 1][0] = p[0]; ra[c & 1][1] = p[1];
        };
        const float rstd = rstd_in[row];
        if constexpr (MULTI) {
            // further gradients of the same tensor, summed the way a chain of bf16 tensor additions would:
            // (dy + dy2) rounded to bf16, then + dy3 rounded to bf16.  Their loads are unconditional (a chunk past the
            // row's end re-reads its last 16 columns and is dropped; without a third gradient the second is read again,
            // from the cache) and issued ahead of the additions: loaded and converted chunk by chunk, every one of the
            // up to 2 x CH loads was a round trip of its own.
            const void* const d3 = dy3 ? dy3 : dy2;
            auto add_to = [&](int c, const uint4* r2, const uint4* r3) {  // adds both (as loaded) to chunk c of g
                float a[16], b[16];
                unpack_w16<kBF16>(g[c], a);
                unpack_w16<kBF16>(r2, b);
#pragma unroll
                for (int i = 0; i < 16; i++) a[i] = round_to<kBF16>(a[i] + b[i]);
                if (dy3) {  // wave-uniform
                    unpack_w16<kBF16>(r3, b);
#pragma unroll
                    for (int i = 0; i < 16; i++) a[i] = round_to<kBF16>(a[i] + b[i]);
                }
                uint32_t pk[8];
#pragma unroll
                for (int k = 0; k < 8; k++) pk[k] = pack_bf16x2(a[2 * k], a[2 * k + 1]);
                g[c][0] = make_uint4(pk[0], pk[1], pk[2], pk[3]);
                g[c][1] = make_uint4(pk[4], pk[5], pk[6], pk[7]);
            };
            if constexpr (CH <= 5) {  // a whole row of one gradient at a time: two round trips instead of 2 x CH
                uint4 r[CH][2];
                auto load_all = [&](const void* src) {
#pragma unroll
                    for (int c = 0; c < CH; c++) {
                        const int col = min((c * 64 + lane) * 16, N - 16);
                        const uint4* p = (const uint4*)((const uint16_t*)src + row_off + col);
                        r[c][0] = p[0]; r[c][1] = p[1];
                    }
                };
                auto add_all = [&]() {
#pragma unroll
                    for (int c = 0; c < CH; c++) {
                        if ((c * 64 + lane) * 16 < N) {
                            float a[16], b[16];
                            unpack_w16<kBF16>(g[c], a);
                            unpack_w16<kBF16>(r[c], b);
                            uint32_t pk[8];
#pragma unroll
                            for (int k = 0; k < 8; k++)
                                pk[k] = pack_bf16x2(round_to<kBF16>(a[2 * k] + b[2 * k]), round_to<kBF16>(a[2 * k + 1] + b[2 * k + 1]));
                            g[c][0] = make_uint4(pk[0], pk[1], pk[2], pk[3]);
                            g[c][1] = make_uint4(pk[4], pk[5], pk[6], pk[7]);
                        }
                    }
                };
                load_all(dy2);
                add_all();
                if (dy3) {  // wave-uniform
                    load_all(dy3);
                    add_all();
                }
            } else {  // eight chunks: one chunk's four loads at a time
#pragma unroll
                for (int c = 0; c < CH; c++) {
                    const int col = (c * 64 + lane) * 16, lcol = min(col, N - 16);
                    const uint4* p2 = (const uint4*)((const uint16_t*)dy2 + row_off + lcol);
                    const uint4* p3 = (const uint4*)((const uint16_t*)d3 + row_off + lcol);
                    const uint4 r2[2] = {p2[0], p2[1]}, r3[2] = {p3[0], p3[1]};
                    if (col < N) add_to(c, r2, r3);
                }
            }
        }
        if constexpr (ADD) load_radd(0);
        float part[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int col = (c * 64 + lane) * 16;
            if (col < N) {
                float xv[16], wvv[16], gv[16];
                decode16<KIND>(raw.codes[c], scale_from_raw(raw.sc[c], s_dt), xv);
                if (HOLD_W) unpack_w16<WDT>(wreg[c], wvv);
                else load_w16<WDT>(w, col, wvv);
                unpack_w16<kBF16>(g[c], gv);
#pragma unroll
                for (int i = 0; i < 16; i++) {
                    const float xhat = xv[i] * rstd;
                    const float wdy = wvv[i] * gv[i];
                    part[c & 3] += xhat * wdy;
                    acc[c][i] += gv[i] * xhat;
                }
            }
        }
        const float c1 = row_sum4(part) / (float)N;
        float gmax[ADD ? CH : 1] = {};  // ADD: max |sum| of the lane's chunk c (0 for a chunk past the row's end)
#pragma unroll
        for (int c = 0; c < CH; c++) {
            const int col = (c * 64 + lane) * 16;
            if constexpr (ADD) {
                if (c + 1 < CH) load_radd(c + 1);
            }
            if (col < N) {
                float xv[16], wvv[16], gv[16], o[16];
                decode16<KIND>(raw.codes[c], scale_from_raw(raw.sc[c], s_dt), xv);
                if (HOLD_W) unpack_w16<WDT>(wreg[c], wvv);
                else load_w16<WDT>(w, col, wvv);
                unpack_w16<kBF16>(g[c], gv);
#pragma unroll
                for (int i = 0; i < 16; i++) o[i] = ((wvv[i] * gv[i]) - ((xv[i] * rstd) * c1)) * rstd;
                if constexpr (ADD) {
                    float rg[16];
                    unpack_w16<kBF16>(ra[c & 1], rg);
#pragma unroll
                    for (int i = 0; i < 16; i++) o[i] = rg[i] + round_to<kBF16>(o[i]);
                    float am = fmaxf(fabsf(o[0]), fabsf(o[1]));
#pragma unroll
                    for (int i = 2; i < 16; i++) am = fmaxf(am, fabsf(o[i]));
                    gmax[c] = am;
                }
                store_bf16_16(dx, row_off + col, o);
            }
        }
        if constexpr (ADD) {
            const int lpg = qb >> 4;  // lanes per group: neighbouring lanes hold neighbouring chunks
#pragma unroll
            for (int c = 0; c < CH; c++) {
                const float am = cluster_max_rt(gmax[c], lpg);
                const float sg = A.kind_out == kE5M2 ? group_scale<kE5M2>(am) : group_scale<kE4M3>(am);
                const int col = (c * 64 + lane) * 16;
                if (col < N) {
                    if ((lane & (lpg - 1)) == 0) ((uint16_t*)A.s_pg)[row * (N / qb) + col / qb] = (uint16_t)f2bf16(sg);
                    wave_max = fmaxf(wave_max, sg);
                }
            }
        }
    }
    if constexpr (ADD) {  // one lazy atomic per block
        __shared__ float wmax[4];
        wave_max = cluster_max<64>(wave_max);
        if (lane == 0) wmax[wv_id] = wave_max;
        __syncthreads();
        if (threadIdx.x == 0) atomic_max_nonneg(max_slot(A.s_max), fmaxf(fmaxf(wmax[0], wmax[1]), fmaxf(wmax[2], wmax[3])));
    }
    // the block's partial row: waves added in index order, 1024 columns per round
#pragma unroll
    for (int c = 0; c < CH; c++) {
        float4* mine = (float4*)&red[wv_id][lane * 16];
#pragma unroll
        for (int k = 0; k < 4; k++) mine[k] = make_float4(acc[c][4 * k], acc[c][4 * k + 1], acc[c][4 * k + 2], acc[c][4 * k + 3]);
        __syncthreads();
        const int e = threadIdx.x * 4, col = c * 1024 + e;
        if (col < N) {
            const float4 a0 = *(const float4*)&red[0][e], a1 = *(const float4*)&red[1][e], a2 = *(const float4*)&red[2][e],
                         a3 = *(const float4*)&red[3][e];
            *(float4*)(dw_partial + (int64_t)blockIdx.x * N + col) =
                make_float4(((a0.x + a1.x) + a2.x) + a3.x, ((a0.y + a1.y) + a2.y) + a3.y, ((a0.z + a1.z) + a2.z) + a3.z,
                            ((a0.w + a1.w) + a2.w) + a3.w);
        }
        __syncthreads();
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

// Rows up to 8192 columns go to the wave-per-row kernels (CH = 4, 5 or 8 chunks of 16 per lane; 5 is the 5120 columns of
// the 13B shape, which as 5 of 8 chunks ran at 0.6 of the rate of the 4096-column rows), wider rows (up to 16384) to
// the block-per-row kernels.  The forward changes over at 5120 columns already: with eight chunks a wave holds 256
// registers and is alone on its SIMD, and the block-per-row kernel is faster ([8192, 8192]: 22 against 41 us); the
// backward is faster wave by wave up to 8192 (110 against 136 us).  Both layouts give the same bits.  KW = fp8 kind * 3 + weight dtype.
#ifndef COAT_RMS_FWD_BLOCKS
#define COAT_RMS_FWD_BLOCKS 768
#endif
// three resident blocks (12 waves) on each of 256 CUs: 13.2 us at [8192, 4096] against 15.2 / 15.0 / 15.8 us with 512 / 1024 /
// 2048 blocks; a wave walks its rows with the next one prefetched under the current one
constexpr int kRmsFwdMaxBlocks = COAT_RMS_FWD_BLOCKS;
#define RMS_KW_CASES(X) X(0, 0) X(0, 1) X(0, 2) X(1, 0) X(1, 1) X(1, 2)
#define RMS_CHECK_ENUMS()                                                                                   \
    if (fp8 != COAT_E4M3 && fp8 != COAT_E5M2) return COAT_EINVAL;                                           \
    if (w_dtype != COAT_BF16 && w_dtype != COAT_F32 && w_dtype != COAT_F16) return COAT_EDTYPE;
extern "C" int coat_fp8_rmsnorm_forward(const void* x, int fp8, const void* s_x, int s_dtype, const void* w, int w_dtype,
                                        void* y, void* s_row, float* rstd, float* s_max, int64_t M, int64_t N, int QB,
                                        float eps, void* stream) {
    if (int e = rms_check(M, N, QB)) return e;
    if (M * N == 0) return COAT_OK;
    if (!x || !s_x || !w || !s_row || !rstd || !s_max) return COAT_EINVAL;  // y may be NULL
    if (!coat_aligned16(x) || !coat_aligned16(w) || !coat_aligned16(y)) return COAT_EALIGN;
    hipStream_t st = (hipStream_t)stream;
    RMS_CHECK_ENUMS()
    const int64_t wave_blocks = (M + 3) / 4 < kRmsFwdMaxBlocks ? (M + 3) / 4 : kRmsFwdMaxBlocks;
#define RMS_FWD(K, W)                                                                                                  \
    case K * 3 + W:                                                                                                    \
        if (N <= 4096)                                                                                                 \
            hipLaunchKernelGGL((k_rmsnorm_fwd<K, W, 4>), dim3((unsigned)wave_blocks), dim3(256), 0, st, (const uint8_t*)x, s_x, \
                               s_dtype, w, y, s_row, rstd, s_max, M, (int)N, QB, eps);                                 \
        else if (N <= 5120)                                                                                            \
            hipLaunchKernelGGL((k_rmsnorm_fwd<K, W, 5>), dim3((unsigned)wave_blocks), dim3(256), 0, st, (const uint8_t*)x, s_x, \
                               s_dtype, w, y, s_row, rstd, s_max, M, (int)N, QB, eps);                                 \
        else                                                                                                           \
            hipLaunchKernelGGL((k_rmsnorm_fwd_block<K, W, 4>), dim3((unsigned)M), dim3(256), 0, st, (const uint8_t*)x, s_x, \
                               s_dtype, w, y, s_row, rstd, s_max, (int)N, QB, eps);                                    \
        break;
    switch (fp8 * 3 + w_dtype) {
        RMS_KW_CASES(RMS_FWD)
        default: return COAT_EINVAL;
    }
#undef RMS_FWD
    return coat_launch_status();
}

// Shared by the two backward entry points: dx kernel on min(n_partial, M) blocks, then the column sum of their partial rows.
static int rms_backward_launch(const void* x, int fp8, const void* s_x, int s_dtype, const void* dy, const void* dy2,
                               const void* dy3, const void* w, int w_dtype, const float* rstd, void* dx, void* dw,
                               float* dw_partial, int64_t n_partial, int64_t M, int64_t N, int QB, hipStream_t st,
                               const RmsAddArgs* add = nullptr) {
    RMS_CHECK_ENUMS()
    // one partial row per block: min(n_partial, M) blocks of the block-per-row kernel, min(n_partial, ceil(M / 4)) blocks
    // of four row-owning waves otherwise
    const int64_t rows_per_block = N <= 8192 ? 4 : 1;
    const int64_t want = (M + rows_per_block - 1) / rows_per_block;
    const int64_t grid = n_partial < want ? n_partial : want;
    if (add && N > 8192) return COAT_ESHAPE;  // the fused addition exists in the wave-per-row kernels only
    const RmsAddArgs no_add = {};
#define RMS_BWD_WAVE(K, W, CHV, MU)                                                                                    \
    {                                                                                                                  \
        if (add)                                                                                                       \
            hipLaunchKernelGGL((k_rmsnorm_bwd<K, W, CHV, MU, true>), dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t*)x, s_x, \
                               s_dtype, dy, dy2, dy3, w, rstd, dx, dw_partial, M, (int)N, QB, *add);                   \
        else                                                                                                           \
            hipLaunchKernelGGL((k_rmsnorm_bwd<K, W, CHV, MU, false>), dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t*)x, s_x, \
                               s_dtype, dy, dy2, dy3, w, rstd, dx, dw_partial, M, (int)N, QB, no_add);                 \
    }
#define RMS_BWD(K, W)                                                                                                  \
    case K * 3 + W:                                                                                                    \
        if (N <= 4096) {                                                                                               \
            if (dy2) RMS_BWD_WAVE(K, W, 4, true)                                                                       \
            else RMS_BWD_WAVE(K, W, 4, false)                                                                          \
        } else if (N <= 5120) {                                                                                        \
            if (dy2) RMS_BWD_WAVE(K, W, 5, true)                                                                       \
            else RMS_BWD_WAVE(K, W, 5, false)                                                                          \
        } else if (N <= 8192) {                                                                                        \
            if (dy2) RMS_BWD_WAVE(K, W, 8, true)                                                                       \
            else RMS_BWD_WAVE(K, W, 8, false)                                                                          \
        } else {                                                                                                       \
            hipLaunchKernelGGL((k_rmsnorm_bwd_block<K, W, 4>), dim3((unsigned)grid), dim3(256), 0, st, (const uint8_t*)x, s_x, \
                               s_dtype, dy, dy2, dy3, w, rstd, dx, dw_partial, M, (int)N, QB);                         \
        }                                                                                                              \
        break;
    switch (fp8 * 3 + w_dtype) {
        RMS_KW_CASES(RMS_BWD)
        default: return COAT_EINVAL;
    }
#undef RMS_BWD
#undef RMS_BWD_WAVE
    if (int e = coat_launch_status()) return e;
    const int cols_blocks = (int)((N + kColsumCols - 1) / kColsumCols);
    switch (w_dtype) {
        case COAT_F32: hipLaunchKernelGGL((k_norm_colsum<kF32>), dim3(cols_blocks), dim3(kColsumThreads), 0, st, dw_partial, dw, (int)grid, (int)N); break;
        case COAT_BF16: hipLaunchKernelGGL((k_norm_colsum<kBF16>), dim3(cols_blocks), dim3(kColsumThreads), 0, st, dw_partial, dw, (int)grid, (int)N); break;
        default: hipLaunchKernelGGL((k_norm_colsum<kF16>), dim3(cols_blocks), dim3(kColsumThreads), 0, st, dw_partial, dw, (int)grid, (int)N); break;
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

extern "C" int coat_fp8_rmsnorm_backward_add(const void* x, int fp8, const void* s_x, int s_dtype, const void* dy,
                                             const void* dy2, const void* dy3, const void* w, int w_dtype,
                                             const float* rstd, const void* residual_grad, void* y, void* s_pg,
                                             float* s_max, int fp8_out, void* dw, float* dw_partial, int n_partial,
                                             int64_t M, int64_t N, int QB, void* stream) {
    if (int e = rms_check(M, N, QB)) return e;
    if (N > 8192 || QB > 1024) return COAT_ESHAPE;
    if (M * N == 0) return COAT_OK;
    if (!dw_partial || n_partial <= 0 || !residual_grad || !s_pg || !s_max) return COAT_EINVAL;
    if (fp8_out != COAT_E4M3 && fp8_out != COAT_E5M2) return COAT_EINVAL;
    if (int e = rms_backward_check(x, s_x, dy, dy2, dy3, w, rstd, y, dw)) return e;
    if (!coat_aligned16(dw_partial) || !coat_aligned16(residual_grad)) return COAT_EALIGN;
    const RmsAddArgs add = {residual_grad, s_pg, s_max, fp8_out == COAT_E5M2 ? kE5M2 : kE4M3};
    return rms_backward_launch(x, fp8, s_x, s_dtype, dy, dy2, dy3, w, w_dtype, rstd, y, dw, dw_partial, n_partial, M, N, QB,
                               (hipStream_t)stream, &add);
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
