// Softmax cross-entropy of the LM head: per-row loss and, written over the logits, the gradient of the reduced loss.
//
// Restates the reference's liger_cross_entropy_kernel (coat/activation/liger/cross_entropy.py:24-198) and
// element_mul_kernel (coat/activation/liger/utils.py) for gfx950.  One block owns one row of V logits:
//   * V <= 512 * VEC * 16: the row is loaded once into registers (16-byte loads), reduced twice (max, then sum of
//     exponentials) and overwritten once: 1 read + 1 write of the row, the algorithmic minimum;
//   * longer rows: online softmax in a first sweep (running max and rescaled sum per thread, merged across the block),
//     gradient in a second sweep that re-reads the row (from L2 / Infinity Cache when it is still there).
// loss = lse - x_y, optionally label-smoothed, plus lse_square_scale * lse^2; with reduction "mean" loss and gradient
// are divided by the number of non-ignored rows, which is read from device memory (no host synchronisation).
// Rows whose target equals ignore_index get a zero gradient and a zero loss.  All arithmetic is fp32.
#include "coat_device.h"
#include "coat_host.h"

namespace coat {

struct CeArgs {
    void* x;
    const int64_t* target;
    void* loss;
    void* z_loss;  // may be NULL
    const int64_t* n_non_ignore;
    int64_t n_rows, n_cols, x_stride, ignore_index;
    float lse_square_scale, label_smoothing, softcap;
    int mean, has_softcap;
};

constexpr float kLog2e = 1.4426950408889634f;

template <int XDT> struct ElemSize { static constexpr int kBytes = XDT == kF32 ? 4 : 2; };

// The VEC values of a whole chunk from its 16 bytes.
template <int XDT, int VEC> __device__ __forceinline__ void unpack_chunk(const uint4& t, float* v) {
    const uint32_t w[4] = {t.x, t.y, t.z, t.w};
    if (XDT == kF32) {
#pragma unroll
        for (int i = 0; i < 4; i++) v[i % VEC] = u2f(w[i]);
    } else {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            v[(2 * i) % VEC] = XDT == kBF16 ? bf16lo(w[i]) : f16lo(w[i]);
            v[(2 * i + 1) % VEC] = XDT == kBF16 ? bf16hi(w[i]) : f16hi(w[i]);
        }
    }
}
// Chunk j of a row = elements [j * VEC, j * VEC + VEC); elements at or beyond V read as `fill`.
template <int XDT, int VEC> __device__ __forceinline__ void load_chunk(const void* row, int64_t j, int64_t V, float fill, float* v) {
    const int64_t e0 = j * VEC;
    if (VEC > 1 && e0 + VEC <= V) {
        if (XDT == kF32) {
            const uint4 tu = ld_stream16((const float*)row + e0);
            const float4 t = make_float4(u2f(tu.x), u2f(tu.y), u2f(tu.z), u2f(tu.w));
            v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
        } else {
            const uint4 t = ld_stream16((const uint16_t*)row + e0);
            const uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
            for (int i = 0; i < 4; i++) {
                v[(2 * i) % VEC] = XDT == kBF16 ? bf16lo(w[i]) : f16lo(w[i]);
                v[(2 * i + 1) % VEC] = XDT == kBF16 ? bf16hi(w[i]) : f16hi(w[i]);
            }
        }
    } else {
#pragma unroll
        for (int k = 0; k < VEC; k++) v[k] = e0 + k < V ? load_as_f32<XDT>(row, e0 + k) : fill;
    }
}
template <int XDT, int VEC> __device__ __forceinline__ void store_chunk(void* row, int64_t j, int64_t V, const float* v) {
    const int64_t e0 = j * VEC;
    if (VEC > 1 && e0 + VEC <= V) {
        if (XDT == kF32) {
            *(float4*)((float*)row + e0) = make_float4(v[0], v[1 % VEC], v[2 % VEC], v[3 % VEC]);
        } else {
            uint32_t w[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float lo = v[(2 * i) % VEC], hi = v[(2 * i + 1) % VEC];
                w[i] = XDT == kBF16 ? pack_bf16x2(lo, hi) : (f2f16(lo) | (f2f16(hi) << 16));
            }
            *(uint4*)((uint16_t*)row + e0) = make_uint4(w[0], w[1], w[2], w[3]);
        }
    } else {
#pragma unroll
        for (int k = 0; k < VEC; k++)
            if (e0 + k < V) store_from_f32<XDT>(row, e0 + k, v[k]);
    }
}

// Reduction over the waves of the block; every thread calls, every thread gets the result.
template <bool MAX, int kCeThreads> __device__ __forceinline__ float ce_block_reduce(float v, float* smem) {
    v = MAX ? cluster_max<64>(v) : cluster_sum<64>(v);
    __syncthreads();  // the previous reduction's readers are done with smem
    if ((threadIdx.x & 63) == 0) smem[threadIdx.x >> 6] = v;
    __syncthreads();
    float r = smem[0];
#pragma unroll
    for (int i = 1; i < kCeThreads / 64; i++) r = MAX ? fmaxf(r, smem[i]) : r + smem[i];
    return r;
}

__device__ __forceinline__ float ce_exp(float x_minus_m) { return __builtin_amdgcn_exp2f(x_minus_m * kLog2e); }

// ITERS > 0: chunks per thread held in registers (the whole row);  ITERS == 0: two sweeps over memory.
template <int XDT, int VEC, int ITERS, int kCeThreads, bool CAP>
__global__ __launch_bounds__(kCeThreads) void k_cross_entropy(CeArgs a) {
    __shared__ float smem[kCeThreads / 64];
    const int tid = threadIdx.x;
    const int64_t row = blockIdx.x, V = a.n_cols;
    void* xrow = (uint8_t*)a.x + row * a.x_stride * ElemSize<XDT>::kBytes;
    const int64_t y = a.target[row];
    const int64_t nchunk = (V + VEC - 1) / VEC;
    const float ninf = -__builtin_inff();

    if (y == a.ignore_index) {  // block-uniform
        float z[VEC];
#pragma unroll
        for (int k = 0; k < VEC; k++) z[k] = 0.0f;
        for (int64_t j = tid; j < nchunk; j += kCeThreads) store_chunk<XDT, VEC>(xrow, j, V, z);
        if (tid == 0) {
            store_from_f32<XDT>(a.loss, row, 0.0f);
            if (a.z_loss) store_from_f32<XDT>(a.z_loss, row, 0.0f);
        }
        return;
    }

    constexpr bool cap = CAP;
    const float sc = a.softcap;
    const float ls = a.label_smoothing;
    const float eps = ls / (float)V;
    // the target's logit, read before any thread overwrites the row (stores start after the block reductions)
    float xy = __builtin_nanf("");
    if (tid == 0 && y >= 0 && y < V) {
        xy = load_as_f32<XDT>(xrow, y);
        if (cap) xy = sc * tanhf(xy / sc);
    }

    float v[ITERS > 0 ? ITERS : 1][VEC];
    float m = ninf, d = 0.0f, sx = 0.0f;
    if (ITERS > 0) {
        // All 16-byte loads of the row first, unconditionally (a chunk that is not a whole chunk of the row re-reads the
        // row's last whole chunk and is replaced below): under a condition, or with a conversion between them, the
        // compiler makes the wave wait for each load before it issues the next.
        uint4 raw[ITERS > 0 ? ITERS : 1];
        const int64_t nfull = V / VEC;  // whole chunks
        if (VEC > 1 && nfull > 0) {
#pragma unroll
            for (int it = 0; it < ITERS; it++) {
                const int64_t j = min((int64_t)it * kCeThreads + tid, nfull - 1);
                raw[it] = ld_stream16((const uint8_t*)xrow + j * 16);
            }
        }
#pragma unroll
        for (int it = 0; it < ITERS; it++) {
            const int64_t j = (int64_t)it * kCeThreads + tid;
            if (j < nchunk) {
                if (VEC > 1 && j < nfull) unpack_chunk<XDT, VEC>(raw[it], v[it]);
                else load_chunk<XDT, VEC>(xrow, j, V, ninf, v[it]);
#pragma unroll
                for (int k = 0; k < VEC; k++) {
                    const bool valid = j * VEC + k < V;
                    if (cap && valid) v[it][k] = sc * tanhf(v[it][k] / sc);
                    m = fmaxf(m, v[it][k]);
                    if (ls > 0.0f && valid) sx += -eps * v[it][k];
                }
            } else {
#pragma unroll
                for (int k = 0; k < VEC; k++) v[it][k] = ninf;
            }
        }
        m = ce_block_reduce<true, kCeThreads>(m, smem);
#pragma unroll
        for (int it = 0; it < ITERS; it++)
#pragma unroll
            for (int k = 0; k < VEC; k++) d += ce_exp(v[it][k] - m);
        d = ce_block_reduce<false, kCeThreads>(d, smem);
    } else {
        // online softmax per thread: (m, d) with d = sum exp(x - m) over the elements seen so far
        for (int64_t j = tid; j < nchunk; j += kCeThreads) {
            float t[VEC];
            load_chunk<XDT, VEC>(xrow, j, V, ninf, t);
            float bm = ninf;
#pragma unroll
            for (int k = 0; k < VEC; k++) {
                const bool valid = j * VEC + k < V;
                if (cap && valid) t[k] = sc * tanhf(t[k] / sc);
                bm = fmaxf(bm, t[k]);
                if (ls > 0.0f && valid) sx += -eps * t[k];
            }
            if (bm > ninf) {
                const float mn = fmaxf(m, bm);
                float acc = d * ce_exp(m - mn);  // m == -inf: d == 0 and exp2(-inf) == 0
#pragma unroll
                for (int k = 0; k < VEC; k++) acc += ce_exp(t[k] - mn);
                d = acc;
                m = mn;
            }
        }
        const float mt = ce_block_reduce<true, kCeThreads>(m, smem);
        d = ce_block_reduce<false, kCeThreads>(m > ninf ? d * ce_exp(m - mt) : 0.0f, smem);
        m = mt;
    }
    if (ls > 0.0f) sx = ce_block_reduce<false, kCeThreads>(sx, smem);

    const float lse = m + logf(d);
    const float n = a.mean ? (float)*a.n_non_ignore : 1.0f;
    const float rd = 1.0f / d;
    const float zk = 2.0f * a.lse_square_scale * lse;
    const float one_minus_ls = 1.0f - ls;

    auto grad_chunk = [&](int64_t j, float* t) {
#pragma unroll
        for (int k = 0; k < VEC; k++) {
            const float p = ce_exp(t[k] - m) * rd;
            float g = p + zk * p;
            g += -eps;
            if (j * VEC + k == y) g -= one_minus_ls;
            if (a.mean) g = g / n;
            if (cap) {
                const float th = t[k] / sc;  // tanh(x / softcap), recovered from the capped value
                g = g * (1.0f - th * th);
            }
            t[k] = g;
        }
        store_chunk<XDT, VEC>(xrow, j, V, t);
    };
    if (ITERS > 0) {
#pragma unroll
        for (int it = 0; it < ITERS; it++) {
            const int64_t j = (int64_t)it * kCeThreads + tid;
            if (j < nchunk) grad_chunk(j, v[it]);
        }
    } else {
        for (int64_t j = tid; j < nchunk; j += kCeThreads) {
            float t[VEC];
            load_chunk<XDT, VEC>(xrow, j, V, ninf, t);
            if (cap) {
#pragma unroll
                for (int k = 0; k < VEC; k++)
                    if (j * VEC + k < V) t[k] = sc * tanhf(t[k] / sc);
            }
            grad_chunk(j, t);
        }
    }

    if (tid == 0) {
        float loss = lse - xy;
        if (ls > 0.0f) loss = loss * one_minus_ls + (sx + ls * lse);
        float z = a.lse_square_scale * lse * lse;
        loss += z;
        if (a.mean) {
            z = z / n;
            loss = loss / n;
        }
        store_from_f32<XDT>(a.loss, row, loss);
        if (a.z_loss) store_from_f32<XDT>(a.z_loss, row, z);
    }
}

// x *= *g over [n_rows, n_cols]; returns at once when *g == 1 (the loss was the last node of the graph).
template <int XDT, int VEC>
__global__ __launch_bounds__(256) void k_ce_scale(void* x, const void* g, int g_dtype, int64_t n_rows, int64_t n_cols,
                                                   int64_t x_stride) {
    const float gs = load_rt_f32(g, 0, g_dtype);
    if (gs == 1.0f) return;
    const int64_t nchunk = (n_cols + VEC - 1) / VEC, total = n_rows * nchunk;
    for (int64_t job = (int64_t)blockIdx.x * 256 + threadIdx.x; job < total; job += (int64_t)gridDim.x * 256) {
        const int64_t row = job / nchunk, j = job % nchunk;
        void* xrow = (uint8_t*)x + row * x_stride * ElemSize<XDT>::kBytes;
        float t[VEC];
        load_chunk<XDT, VEC>(xrow, j, n_cols, 0.0f, t);
#pragma unroll
        for (int k = 0; k < VEC; k++) t[k] = t[k] * gs;
        store_chunk<XDT, VEC>(xrow, j, n_cols, t);
    }
}

// Rows of up to 512 * VEC * 16 elements (32768 fp32, 65536 bf16) stay in registers: 512-thread blocks, two per CU, so
// that one block's stores overlap the other's loads (measured faster than one 1024-thread block per CU and than
// 256-thread blocks with 32 chunks per thread).  Longer rows, and rows without 16-byte alignment, take two sweeps.
template <int XDT, int VEC, bool CAP> static int ce_launch(const CeArgs& a, hipStream_t st) {
    const dim3 grid((unsigned)a.n_rows);
    const int64_t cap1 = (int64_t)512 * VEC;
    if (VEC == 1 || a.n_cols > 16 * cap1) hipLaunchKernelGGL((k_cross_entropy<XDT, VEC, 0, 1024, CAP>), grid, dim3(1024), 0, st, a);
    else if (a.n_cols <= 2 * cap1) hipLaunchKernelGGL((k_cross_entropy<XDT, VEC, 2, 512, CAP>), grid, dim3(512), 0, st, a);
    else if (a.n_cols <= 4 * cap1) hipLaunchKernelGGL((k_cross_entropy<XDT, VEC, 4, 512, CAP>), grid, dim3(512), 0, st, a);
    else if (a.n_cols <= 8 * cap1) hipLaunchKernelGGL((k_cross_entropy<XDT, VEC, 8, 512, CAP>), grid, dim3(512), 0, st, a);
    else hipLaunchKernelGGL((k_cross_entropy<XDT, VEC, 16, 512, CAP>), grid, dim3(512), 0, st, a);
    return coat_launch_status();
}

template <int XDT> static int ce_dispatch(const CeArgs& a, hipStream_t st) {
    constexpr int VEC = XDT == kF32 ? 4 : 8;
    // 16-byte accesses need every row to start on a 16-byte boundary
    const bool vec = coat_aligned16(a.x) && a.x_stride % VEC == 0;
    if (a.has_softcap) return vec ? ce_launch<XDT, VEC, true>(a, st) : ce_launch<XDT, 1, true>(a, st);
    return vec ? ce_launch<XDT, VEC, false>(a, st) : ce_launch<XDT, 1, false>(a, st);
}

template <int XDT> static int ce_scale_dispatch(void* x, const void* g, int g_dtype, int64_t n_rows, int64_t n_cols,
                                                int64_t x_stride, hipStream_t st) {
    constexpr int VEC = XDT == kF32 ? 4 : 8;
    const bool vec = coat_aligned16(x) && x_stride % VEC == 0;
    const int64_t total = n_rows * ((n_cols + (vec ? VEC : 1) - 1) / (vec ? VEC : 1));
    int64_t blocks = (total + 255) / 256;
    if (blocks > 8192) blocks = 8192;
    if (vec) hipLaunchKernelGGL((k_ce_scale<XDT, VEC>), dim3((unsigned)blocks), dim3(256), 0, st, x, g, g_dtype, n_rows, n_cols, x_stride);
    else hipLaunchKernelGGL((k_ce_scale<XDT, 1>), dim3((unsigned)blocks), dim3(256), 0, st, x, g, g_dtype, n_rows, n_cols, x_stride);
    return coat_launch_status();
}

}  // namespace coat

using namespace coat;

extern "C" int coat_cross_entropy_forward(void* x, int x_dtype, int64_t x_stride, const int64_t* target, void* loss,
                                          void* z_loss, const int64_t* n_non_ignore, int64_t n_rows, int64_t n_cols,
                                          int64_t ignore_index, float lse_square_scale, float label_smoothing,
                                          int reduction, float softcap, int has_softcap, void* stream) {
    if (n_rows < 0 || n_cols <= 0 || x_stride < n_cols) return COAT_EINVAL;
    if (reduction < 0 || reduction > 2) return COAT_EINVAL;
    if (n_rows == 0) return COAT_OK;
    if (!x || !target || !loss || (reduction == 1 && !n_non_ignore)) return COAT_EINVAL;
    if (n_rows > 0x7FFFFFFF) return COAT_ESHAPE;
    if (has_softcap && !(softcap > 0.0f)) return COAT_EINVAL;
    CeArgs a{x, target, loss, z_loss, n_non_ignore, n_rows, n_cols, x_stride, ignore_index,
             lse_square_scale, label_smoothing, softcap, reduction == 1, has_softcap};
    hipStream_t st = (hipStream_t)stream;
    switch (x_dtype) {
        case kF32: return ce_dispatch<kF32>(a, st);
        case kBF16: return ce_dispatch<kBF16>(a, st);
        case kF16: return ce_dispatch<kF16>(a, st);
    }
    return COAT_EINVAL;
}

extern "C" int coat_cross_entropy_scale_grad(void* x, int x_dtype, int64_t x_stride, const void* grad_output,
                                             int g_dtype, int64_t n_rows, int64_t n_cols, void* stream) {
    if (n_rows < 0 || n_cols <= 0 || x_stride < n_cols) return COAT_EINVAL;
    if (n_rows == 0) return COAT_OK;
    if (!x || !grad_output || g_dtype < 0 || g_dtype > 2) return COAT_EINVAL;
    hipStream_t st = (hipStream_t)stream;
    switch (x_dtype) {
        case kF32: return ce_scale_dispatch<kF32>(x, grad_output, g_dtype, n_rows, n_cols, x_stride, st);
        case kBF16: return ce_scale_dispatch<kBF16>(x, grad_output, g_dtype, n_rows, n_cols, x_stride, st);
        case kF16: return ce_scale_dispatch<kF16>(x, grad_output, g_dtype, n_rows, n_cols, x_stride, st);
    }
    return COAT_EINVAL;
}
