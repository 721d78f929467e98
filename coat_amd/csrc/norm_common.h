// Helpers shared by the RMSNorm and LayerNorm kernels: 256-thread block reductions in a fixed order, dequantization
// of 16 FP8 codes with their group scale, 16-element weight loads / bf16 stores, and the column reduction that turns
// per-block fp32 partial rows into a weight gradient.
#pragma once
#include "coat_device.h"

namespace coat {

__device__ __forceinline__ float block_sum_256(float v, float* smem) {
    v = cluster_sum<64>(v);
    const int wave = threadIdx.x >> 6;
    __syncthreads();  // smem may still be read from a previous call
    if ((threadIdx.x & 63) == 0) smem[wave] = v;
    __syncthreads();
    return ((smem[0] + smem[1]) + smem[2]) + smem[3];
}
__device__ __forceinline__ float block_max_256(float v, float* smem) {
    v = cluster_max<64>(v);
    const int wave = threadIdx.x >> 6;
    __syncthreads();
    if ((threadIdx.x & 63) == 0) smem[wave] = v;
    __syncthreads();
    return fmaxf(fmaxf(smem[0], smem[1]), fmaxf(smem[2], smem[3]));
}

template <int KIND> __device__ __forceinline__ void dequant16(const uint8_t* q, const void* s, int s_dt, int64_t row_off,
                                                             int64_t srow_off, int col, int qb, float* v) {
    uint4 c = *(const uint4*)(q + row_off + col);
    float sc;
    const int64_t si = srow_off + col / qb;
    if (s_dt == kBF16) sc = u2f((uint32_t)((const uint16_t*)s)[si] << 16);
    else if (s_dt == kF32) sc = ((const float*)s)[si];
    else sc = f16lo(((const uint16_t*)s)[si]);
    uint32_t w[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
    for (int k = 0; k < 4; k++) {
        float f[4];
        fp8x4_to_f32<KIND>(w[k], f);
#pragma unroll
        for (int i = 0; i < 4; i++) v[4 * k + i] = f[i] * sc;
    }
}
template <int WDT> __device__ __forceinline__ void load_w16(const void* w, int col, float* o) {
    if (WDT == kF32) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float4 t = ((const float4*)((const float*)w + col))[i];
            o[4 * i] = t.x; o[4 * i + 1] = t.y; o[4 * i + 2] = t.z; o[4 * i + 3] = t.w;
        }
    } else {
        const uint4* src = (const uint4*)((const uint16_t*)w + col);
        uint4 a = src[0], b = src[1];
        uint32_t u[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int k = 0; k < 8; k++) {
            o[2 * k] = WDT == kBF16 ? bf16lo(u[k]) : f16lo(u[k]);
            o[2 * k + 1] = WDT == kBF16 ? bf16hi(u[k]) : f16hi(u[k]);
        }
    }
}
__device__ __forceinline__ void load_bf16_16(const void* p, int64_t off, float* v) {
    const uint4* src = (const uint4*)((const uint16_t*)p + off);
    const uint4 a = src[0], b = src[1];
    const uint32_t u[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
    for (int k = 0; k < 8; k++) {
        v[2 * k] = bf16lo(u[k]);
        v[2 * k + 1] = bf16hi(u[k]);
    }
}
__device__ __forceinline__ void store_bf16_16(void* p, int64_t off, const float* v) {
    uint32_t w[8];
#pragma unroll
    for (int k = 0; k < 8; k++) w[k] = pack_bf16x2(v[2 * k], v[2 * k + 1]);
    uint4* dst = (uint4*)((uint16_t*)p + off);
    dst[0] = make_uint4(w[0], w[1], w[2], w[3]);
    dst[1] = make_uint4(w[4], w[5], w[6], w[7]);
}

// dw[col] = sum of the partial rows in a fixed order (deterministic), stored in the weight's dtype.
// 32 columns per block: one 128-byte line of every partial row, so no line is fetched by two blocks (blocks sit on
// different XCDs with an L2 each; 16-column blocks fetched every line twice).  The rows are split over 16 thread slices,
// slice s taking rows 8 s .. 8 s + 7 of every 128, with 32 loads in flight per thread.
constexpr int kColsumCols = 32, kColsumThreads = 512;
template <int WDT>
__global__ __launch_bounds__(kColsumThreads) void k_norm_colsum(const float* __restrict__ partial, void* __restrict__ dw,
                                                                 int nblocks, int N) {
    __shared__ float red[16][kColsumCols];
    const int c = threadIdx.x & (kColsumCols - 1), slice = threadIdx.x / kColsumCols;
    const int col = blockIdx.x * kColsumCols + c;
    float acc[8];
#pragma unroll
    for (int u = 0; u < 8; u++) acc[u] = 0.0f;
    if (col < N) {
        // four rounds of rows at a time: all 32 loads are issued before the first addition (rows past the end are read
        // from the last row and add 0), the additions keep their order
        for (int b0 = slice * 8; b0 < nblocks; b0 += 512) {
            float v[4][8];
#pragma unroll
            for (int k = 0; k < 4; k++)
#pragma unroll
                for (int u = 0; u < 8; u++)
                    v[k][u] = partial[(int64_t)min(b0 + 128 * k + u, nblocks - 1) * N + col];
#pragma unroll
            for (int k = 0; k < 4; k++)
#pragma unroll
                for (int u = 0; u < 8; u++) acc[u] += (b0 + 128 * k + u < nblocks) ? v[k][u] : 0.0f;
        }
    }
    red[slice][c] = ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
    __syncthreads();
    if (slice == 0 && col < N) {
        float s = 0.0f;
#pragma unroll
        for (int k = 0; k < 16; k++) s += red[k][c];
        store_from_f32<WDT>(dw, col, s);
    }
}

}  // namespace coat
