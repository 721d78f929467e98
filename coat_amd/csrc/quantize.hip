// Streaming FP8 quantize family for gfx950: per-group quantize (+transpose), per-group scales with a
// device-wide maximum, per-tensor division (+transpose), byte transpose, dequantize, abs-max.
//
// All of these are HBM-bound.  Layout rules used throughout:
//   * every lane moves 16 bytes per global load (8 two-byte elements or 4 fp32), consecutive lanes
//     touch consecutive 16-byte chunks, so a wave instruction covers 1 KiB of contiguous memory;
//   * a 1 x QB group is QB/VEC consecutive lanes; its amax is a DPP reduction inside one 16-lane row;
//   * transposed outputs are staged through LDS tiles so that global stores are 16 bytes per lane
//     with neighbouring lanes writing neighbouring chunks of one output row.
#include "coat_device.h"
#include "coat_host.h"
#include "norm_common.h"

namespace coat {

template <int XDT> struct VecOf { static constexpr int kVec = (XDT == kF32) ? 4 : 8; };

// The division kernels are second passes: a kernel before them has just read or written the same tensor from its first
// row to its last, so what the 256 MB memory-side cache still holds of it is its end.  Their blocks therefore walk the
// tensor from the end (measured on one box: SiLU * mul chain at [8192, 11008] 524.7 -> 518.7 us, fp8_division_transpose
// [8192, 4096] 25.0 -> 23.9 us, 7B layer step 5.80 -> 5.79 ms).
__device__ __forceinline__ int64_t block_from_end() { return (int64_t)gridDim.x - 1 - blockIdx.x; }

// 16-byte load of VEC elements starting at element index e (e % VEC == 0) converted to fp32.
template <int XDT> __device__ __forceinline__ void load_vec(const void* x, int64_t e, float* v) {
    if (XDT == kF32) {
        float4 t = *(const float4*)((const float*)x + e);
        v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    } else {
        uint4 t = *(const uint4*)((const uint16_t*)x + e);
        uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            v[2 * i] = XDT == kBF16 ? bf16lo(w[i]) : f16lo(w[i]);
            v[2 * i + 1] = XDT == kBF16 ? bf16hi(w[i]) : f16hi(w[i]);
        }
    }
}

// the same conversion for 16 bytes already in registers
template <int XDT> __device__ __forceinline__ void unpack_vec(const uint4& t, float* v) {
    if (XDT == kF32) {
        v[0] = u2f(t.x); v[1] = u2f(t.y); v[2] = u2f(t.z); v[3] = u2f(t.w);
    } else {
        uint32_t w[4] = {t.x, t.y, t.z, t.w};
#pragma unroll
        for (int i = 0; i < 4; i++) {
            v[2 * i] = XDT == kBF16 ? bf16lo(w[i]) : f16lo(w[i]);
            v[2 * i + 1] = XDT == kBF16 ? bf16hi(w[i]) : f16hi(w[i]);
        }
    }
}

template <int VEC> __device__ __forceinline__ float vec_amax(const float* v) {
    float a = fmaxf(fabsf(v[0]), fabsf(v[1]));
#pragma unroll
    for (int i = 2; i < VEC; i++) a = fmaxf(a, fabsf(v[i]));
    return a;
}

// VEC fp32 -> VEC FP8 codes (VEC/4 dwords), dividing by s through the reciprocal r.
template <int KIND, int VEC> __device__ __forceinline__ void quantize_vec(const float* v, float s, float r, uint32_t* out) {
#pragma unroll
    for (int i = 0; i < VEC / 4; i++)
        out[i] = cvt4_fp8<KIND>(div_by_scale(v[4 * i], s, r), div_by_scale(v[4 * i + 1], s, r),
                                div_by_scale(v[4 * i + 2], s, r), div_by_scale(v[4 * i + 3], s, r));
}
template <int KIND, int VEC> __device__ __forceinline__ void quantize_vec_slow(const float* v, float s, uint32_t* out) {
#pragma unroll
    for (int i = 0; i < VEC / 4; i++)
        out[i] = cvt4_fp8<KIND>(v[4 * i] / s, v[4 * i + 1] / s, v[4 * i + 2] / s, v[4 * i + 3] / s);
}
// Stochastic variant: the quotient of element (e0 + k) is perturbed with Philox noise drawn at that linear index.
template <int KIND, int VEC, bool FAST>
__device__ __forceinline__ void quantize_vec_sr_impl(const float* v, float s, float r, uint32_t e0, uint32_t k0,
                                                     uint32_t k1, uint32_t* out) {
    float t[VEC];
#pragma unroll
    for (int k = 0; k < VEC; k++) {
        const float qv = FAST ? div_by_scale(v[k], s, r) : v[k] / s;
        t[k] = stochastic_perturb<KIND>(qv, uniform_from_word(philox4x32_10_word0(e0 + (uint32_t)k, k0, k1)));
    }
#pragma unroll
    for (int i = 0; i < VEC / 4; i++) out[i] = cvt4_fp8<KIND>(t[4 * i], t[4 * i + 1], t[4 * i + 2], t[4 * i + 3]);
}
template <int KIND, int VEC>
__device__ __forceinline__ void quantize_vec_sr(const float* v, float s, float r, bool fast, uint32_t e0, uint32_t k0,
                                                uint32_t k1, uint32_t* out) {
    if (fast) quantize_vec_sr_impl<KIND, VEC, true>(v, s, r, e0, k0, k1, out);  // `fast` is uniform across the grid
    else quantize_vec_sr_impl<KIND, VEC, false>(v, s, r, e0, k0, k1, out);
}
template <int VEC> __device__ __forceinline__ void store_codes(void* q, int64_t e, const uint32_t* c) {
    if (VEC == 8) *(uint2*)((uint8_t*)q + e) = make_uint2(c[0], c[1]);
    else *(uint32_t*)((uint8_t*)q + e) = c[0];
}

// ------------------------------------------------------------------------------------------------
// K1 / K3: per-group quantize over the flat [M*N] array (groups never straddle rows since N % QB == 0).
//   WRITE_Q   store the FP8 codes
//   WRITE_S   store the per-group scales
//   WITH_MAX  accumulate the maximum fp32 group scale into *s_max (atomic, order independent)
template <int XDT, int SDT, int KIND, int QB, bool WRITE_Q, bool WRITE_S, bool WITH_MAX, int UNROLL>
__global__ __launch_bounds__(256) void k_quantize_pg(const void* __restrict__ x, void* __restrict__ q,
                                                      void* __restrict__ s_out, float* __restrict__ s_max,
                                                      int64_t nvec, int qb_rt) {
    constexpr int VEC = VecOf<XDT>::kVec;
    const int LPG = (QB ? QB : qb_rt) / VEC;  // lanes per group (QB == 0: group size given at run time)
    __shared__ float smem_max[4];
    enable_fp8_saturation();
    float wmax = 0.0f;
    for (int64_t blk = blockIdx.x; blk * (UNROLL * 256) < nvec; blk += gridDim.x) {
    const int64_t base = (blk * UNROLL) * 256 + threadIdx.x;
    float v[UNROLL][VEC];
    bool ok[UNROLL];
#pragma unroll
    // Loads are unconditional (a lane past the end re-reads the last vector and its results are dropped): under a
    // condition the compiler makes the wave wait for each load before it issues the next.
    for (int u = 0; u < UNROLL; u++) {
        int64_t i = base + (int64_t)u * 256;
        ok[u] = i < nvec;
        load_vec<XDT>(x, (ok[u] ? i : nvec - 1) * VEC, v[u]);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        int64_t i = base + (int64_t)u * 256;
        float amax = QB ? cluster_max<(QB ? QB : 16) / VEC>(vec_amax<VEC>(v[u])) : cluster_max_rt(vec_amax<VEC>(v[u]), LPG);
        float s = group_scale<KIND>(amax);
        if (WITH_MAX) wmax = fmaxf(wmax, ok[u] ? s : 0.0f);
        if (WRITE_Q) {
            float r = 1.0f / s;
            uint32_t c[VEC / 4];
            quantize_vec<KIND, VEC>(v[u], s, r, c);
            if (ok[u]) store_codes<VEC>(q, i * VEC, c);
        }
        if (WRITE_S && ok[u] && (threadIdx.x % LPG) == 0) store_from_f32<SDT>(s_out, i / LPG, s);
    }
    }
    if (WITH_MAX) block_atomic_max_nonneg(s_max, wmax, smem_max);
}

// ------------------------------------------------------------------------------------------------
// Q5: max|x| over a flat array (atomic into *amax, which the caller zeroed).
template <int XDT, int UNROLL>
__global__ __launch_bounds__(256) void k_absmax(const void* __restrict__ x, float* __restrict__ amax, int64_t nvec,
                                                 int64_t numel) {
    constexpr int VEC = VecOf<XDT>::kVec;
    __shared__ float smem_max[4];
    float m = 0.0f;
    for (int64_t blk = blockIdx.x; blk * (UNROLL * 256) < nvec; blk += gridDim.x) {
        const int64_t base = (blk * UNROLL) * 256 + threadIdx.x;
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {  // unconditional loads (see k_quantize_pg): the last vector counts twice, harmless
            const int64_t i = min(base + (int64_t)u * 256, nvec - 1);
            float v[VEC];
            load_vec<XDT>(x, i * VEC, v);
            m = fmaxf(m, vec_amax<VEC>(v));
        }
    }
    // ragged tail (numel % VEC elements), handled by the first threads of block 0
    if (blockIdx.x == 0 && threadIdx.x < numel - nvec * VEC) m = fmaxf(m, fabsf(load_as_f32<XDT>(x, nvec * VEC + threadIdx.x)));
    block_atomic_max_nonneg(amax, m, smem_max);
}

// The per-tensor scale of a division kernel.  s_out == NULL: *s_ptr is the scale, an element of dtype SDT.  Otherwise
// s_ptr holds the slots of the fp32 maximum of the group scales left by the producer kernel's atomics (max over the slots =
// the maximum): it is rounded to SDT here (what
// the reference's ``s.max()`` over the stored scales gives, rounding being monotone) and the first thread of the grid
// stores the rounded value to s_out for the consumers, which saves a separate conversion launch per tensor.
template <int SDT> __device__ __forceinline__ float load_scale_or_max(const void* s_ptr, void* s_out) {
    if (!s_out) return load_as_f32<SDT>(s_ptr, 0);
    const float s = round_to<SDT>(load_max((const float*)s_ptr));
    if (blockIdx.x == 0 && threadIdx.x == 0) store_from_f32<SDT>(s_out, 0, s);
    return s;
}

// ------------------------------------------------------------------------------------------------
// K4: per-tensor division over the flat array, q = fp8(x / float(*s)).  SR: stochastic rounding with the
// Philox key (k0, k1) (the reference's branch, coat/activation/real_quantization/_division.py:96-112).
template <int XDT, int SDT, int KIND, int UNROLL, bool SR>
__global__ __launch_bounds__(256) void k_division(const void* __restrict__ x, const void* __restrict__ s_ptr,
                                                   void* __restrict__ q, int64_t nvec, int64_t numel, uint32_t k0,
                                                   uint32_t k1, void* __restrict__ s_out) {
    constexpr int VEC = VecOf<XDT>::kVec;
    enable_fp8_saturation();
    const float s = load_scale_or_max<SDT>(s_ptr, s_out);
    const float r = 1.0f / s;
    const bool fast = s >= kMinFastDivScale && s < 0x1p100f;  // uniform across the grid
    const int64_t base = (block_from_end() * UNROLL) * 256 + threadIdx.x;
    float v[UNROLL][VEC];
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {  // unconditional loads (see k_quantize_pg)
        int64_t i = base + (int64_t)u * 256;
        if (nvec > 0) load_vec<XDT>(x, min(i, nvec - 1) * VEC, v[u]);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        int64_t i = base + (int64_t)u * 256;
        if (i < nvec) {
            uint32_t c[VEC / 4];
            if (SR) quantize_vec_sr<KIND, VEC>(v[u], s, r, fast, (uint32_t)(i * VEC), k0, k1, c);
            else if (fast) quantize_vec<KIND, VEC>(v[u], s, r, c);
            else quantize_vec_slow<KIND, VEC>(v[u], s, c);
            store_codes<VEC>(q, i * VEC, c);
        }
    }
    if (blockIdx.x == 0 && threadIdx.x < numel - nvec * VEC) {
        int64_t e = nvec * VEC + threadIdx.x;
        float qv = load_as_f32<XDT>(x, e) / s;
        if (SR) qv = stochastic_perturb<KIND>(qv, uniform_from_word(philox4x32_10_word0((uint32_t)e, k0, k1)));
        uint32_t w = cvt_pk_fp8<KIND>(qv, 0.0f, 0u, false);
        ((uint8_t*)q)[e] = (uint8_t)(w & 0xFF);
    }
}

// ------------------------------------------------------------------------------------------------
// K7: y = bf16(float(q) * float(s_group)).  One lane: 16 codes (one 16-byte load), two 16-byte stores.
template <int SDT, int KIND>
__global__ __launch_bounds__(256) void k_dequantize(const void* __restrict__ q, const void* __restrict__ s,
                                                     void* __restrict__ y, int64_t nchunk, int QB) {
    int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;  // chunk of 16 elements
    if (i >= nchunk) return;
    uint4 c = *(const uint4*)((const uint8_t*)q + i * 16);
    float sc = load_as_f32<SDT>(s, (i * 16) / QB);
    uint32_t w[4] = {c.x, c.y, c.z, c.w};
    uint32_t o[8];
#pragma unroll
    for (int k = 0; k < 4; k++) {
        float f[4];
        fp8x4_to_f32<KIND>(w[k], f);
        o[2 * k] = pack_bf16x2(f[0] * sc, f[1] * sc);
        o[2 * k + 1] = pack_bf16x2(f[2] * sc, f[3] * sc);
    }
    uint4* yo = (uint4*)((uint16_t*)y + i * 16);
    yo[0] = make_uint4(o[0], o[1], o[2], o[3]);
    yo[1] = make_uint4(o[4], o[5], o[6], o[7]);
}

// ------------------------------------------------------------------------------------------------
// Byte-tile transpose helpers.  A block owns a TM x 128 tile of FP8 codes in LDS (row pitch 33 dwords: odd, so
// that the column-quad reads below spread evenly over the banks).  128 x 128 tiles give whole 128-byte lines in both
// output orientations and keep all 256 lanes busy in the transposed store; measured against 64 x 64 tiles on
// bf16 [8192, 11008] -> q + q^T: 74.7 us instead of 89.5 us.
constexpr int kTileN = 128;
constexpr int kPitchDw = kTileN / 4 + 1;
// threads per block of the dividing / transposing kernels: 512 = two 16-element jobs per thread on a 128 x 128 tile
// (bf16 [8192, 4096] -> q + q^T: 26 us against 28-31 us with 256 threads; 1024 threads: no further gain)
constexpr int kDivTThreads = 512;

// 4x4 byte transpose: r[j] holds row j (4 columns); returns c[j] = column j (4 rows).
__device__ __forceinline__ void transpose4x4_bytes(const uint32_t* r, uint32_t* c) {
    // v_perm_b32(hi, lo, sel): byte k of the result = byte sel[k] of {hi:7..4, lo:3..0}
    uint32_t t0 = __builtin_amdgcn_perm(r[1], r[0], 0x05010400u);  // r0b0 r1b0 r0b1 r1b1
    uint32_t t1 = __builtin_amdgcn_perm(r[3], r[2], 0x05010400u);  // r2b0 r3b0 r2b1 r3b1
    uint32_t t2 = __builtin_amdgcn_perm(r[1], r[0], 0x07030602u);  // r0b2 r1b2 r0b3 r1b3
    uint32_t t3 = __builtin_amdgcn_perm(r[3], r[2], 0x07030602u);
    c[0] = __builtin_amdgcn_perm(t1, t0, 0x05040100u);  // r0b0 r1b0 r2b0 r3b0
    c[1] = __builtin_amdgcn_perm(t1, t0, 0x07060302u);
    c[2] = __builtin_amdgcn_perm(t3, t2, 0x05040100u);
    c[3] = __builtin_amdgcn_perm(t3, t2, 0x07060302u);
}

// Write the transposed TM x 128 byte tile held in LDS to yt[N, M] (row pitch M bytes).
// Lane job = (column quad nq, 16-row chunk mc): 16 dword reads, four 16-byte stores.
template <int TM>
__device__ __forceinline__ void store_tile_transposed(const uint32_t* tile, void* __restrict__ yt, int64_t M, int64_t N,
                                                      int64_t m0, int64_t n0) {
    constexpr int MC = TM / 16;              // 16-row chunks per tile
    constexpr int JOBS = MC * (kTileN / 4);  // (mc, nq) pairs
    for (int job = threadIdx.x; job < JOBS; job += blockDim.x) {
        int mc = job % MC, nq = job / MC;
        int64_t m = m0 + mc * 16, n = n0 + nq * 4;
        if (m >= M || n >= N) continue;  // M % 16 == 0 and N % 4 == 0: chunks are whole or absent
        uint32_t col[4][4];
#pragma unroll
        for (int b = 0; b < 4; b++) {
            uint32_t r[4], c[4];
#pragma unroll
            for (int j = 0; j < 4; j++) r[j] = tile[(mc * 16 + b * 4 + j) * kPitchDw + nq];
            transpose4x4_bytes(r, c);
#pragma unroll
            for (int j = 0; j < 4; j++) col[j][b] = c[j];
        }
#pragma unroll
        for (int j = 0; j < 4; j++)
            *(uint4*)((uint8_t*)yt + (n + j) * M + m) = make_uint4(col[j][0], col[j][1], col[j][2], col[j][3]);
    }
}

// K5 / K6: q = fp8(x / *s) and/or its transpose; RAW = input already FP8 bytes (pure transpose).
// Requires N % 16 == 0 and M % 16 == 0.
// SR: stochastic rounding, noise index = the element's linear index in x
// (coat/activation/real_quantization/_division_transpose.py:103-119).
template <int XDT, int SDT, int KIND, bool RAW, bool WRITE_Q, int TM, bool SR>
__global__ __launch_bounds__(kDivTThreads) void k_division_transpose(const void* __restrict__ x, const void* __restrict__ s_ptr,
                                                             void* __restrict__ q, void* __restrict__ qt, int64_t M,
                                                             int64_t N, uint32_t k0, uint32_t k1, void* __restrict__ s_out) {
    __shared__ uint32_t tile[TM * kPitchDw];
    enable_fp8_saturation();
    const int64_t tiles_n = (N + kTileN - 1) / kTileN;
    const int64_t m0 = (block_from_end() / tiles_n) * TM, n0 = (block_from_end() % tiles_n) * kTileN;
    float s = 1.0f, r = 1.0f;
    bool fast = true;
    if (!RAW) {
        s = load_scale_or_max<SDT>(s_ptr, s_out);
        r = 1.0f / s;
        fast = s >= kMinFastDivScale && s < 0x1p100f;
    }
    // phase 1: each job converts 16 consecutive elements of one row into 4 dwords of the tile.  All loads of the
    // thread's jobs are issued before the first conversion.
    constexpr int JOBS = TM * (kTileN / 16);
    static_assert(JOBS % kDivTThreads == 0, "whole iterations");
    constexpr int NIT = JOBS / kDivTThreads;
    constexpr int VEC = VecOf<XDT>::kVec;
    constexpr int LPJ = RAW ? 1 : 16 / VEC;        // 16-byte loads per job
    constexpr int ESIZE = RAW ? 1 : 16 / VEC;      // bytes per input element
    uint4 raw[NIT][LPJ];
#pragma unroll
    for (int it = 0; it < NIT; it++) {
        const int job = threadIdx.x + it * kDivTThreads;
        const int64_t m = m0 + job / (kTileN / 16), n = n0 + (job % (kTileN / 16)) * 16;
        const bool ok = m < M && n < N;
#pragma unroll
        for (int h = 0; h < LPJ; h++)
            raw[it][h] = ok ? *(const uint4*)((const uint8_t*)x + (m * N + n) * ESIZE + h * 16) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int it = 0; it < NIT; it++) {
        const int job = threadIdx.x + it * kDivTThreads;
        const int row = job / (kTileN / 16), c16 = job % (kTileN / 16);
        const int64_t m = m0 + row, n = n0 + c16 * 16;
        uint32_t c[4] = {0, 0, 0, 0};
        if (m < M && n < N) {
            if (RAW) {
                c[0] = raw[it][0].x; c[1] = raw[it][0].y; c[2] = raw[it][0].z; c[3] = raw[it][0].w;
            } else {
#pragma unroll
                for (int h = 0; h < 16 / VEC; h++) {
                    float v[VEC];
                    unpack_vec<XDT>(raw[it][RAW ? 0 : h], v);
                    if (SR) quantize_vec_sr<KIND, VEC>(v, s, r, fast, (uint32_t)(m * N + n + h * VEC), k0, k1, c + h * (VEC / 4));
                    else if (fast) quantize_vec<KIND, VEC>(v, s, r, c + h * (VEC / 4));
                    else quantize_vec_slow<KIND, VEC>(v, s, c + h * (VEC / 4));
                }
                if (WRITE_Q) *(uint4*)((uint8_t*)q + m * N + n) = make_uint4(c[0], c[1], c[2], c[3]);
            }
        }
#pragma unroll
        for (int k = 0; k < 4; k++) tile[row * kPitchDw + c16 * 4 + k] = c[k];
    }
    __syncthreads();
    store_tile_transposed<TM>(tile, qt, M, N, m0, n0);
}

// ------------------------------------------------------------------------------------------------
// Division + transpose of a bf16 tensor that is never stored: the tile's values are recomputed from the inputs of
// the kernel that produced the tensor's statistics (same expressions, same roundings, so the codes equal those of
// "write the bf16 tensor, then divide it"), which trades a bf16 write and read for a second read of FP8 inputs.
// A source provides  struct Raw,  load(m, n, Raw&)  (16 elements of row m from column n, loads only),  struct Col,
// load_col(n, Col&)  (what depends on the column only: a thread's jobs all lie in one 16-column strip, so it is loaded
// once per thread) and  value(Raw, Col, float v[16])  (the 16 values, already rounded to bf16).

// bf16((x * rstd[row]) * w[col]) of k_rmsnorm_fwd (coat/activation/real_quantization/func_rmsnorm.py:92-108)
template <int KIND, int WDT> struct RmsNormSource {
    const uint8_t* q; const void* s; const void* w; const float* rstd;
    int s_dt, qb; int64_t N;
    struct Raw { uint4 codes; uint32_t sc; float rstd; };  // sc: the scale as loaded, converted in value()
    struct Col { uint4 w[WDT == kF32 ? 4 : 2]; };
    __device__ __forceinline__ void load(int64_t m, int64_t n, Raw& r) const {
        r.codes = *(const uint4*)(q + m * N + n);
        r.sc = load_rt_raw(s, m * (N / qb) + n / qb, s_dt);
        r.rstd = rstd[m];
    }
    __device__ __forceinline__ void load_col(int64_t n, Col& c) const {
        const uint4* wp = (const uint4*)((const uint8_t*)w + n * (WDT == kF32 ? 4 : 2));
#pragma unroll
        for (int i = 0; i < (WDT == kF32 ? 4 : 2); i++) c.w[i] = wp[i];
    }
    __device__ __forceinline__ void value(const Raw& r, const Col& col, float* v) const {
        const uint32_t c[4] = {r.codes.x, r.codes.y, r.codes.z, r.codes.w};
        const float sc = rt_raw_to_f32(r.sc, s_dt);
        float wv[16];
        if constexpr (WDT == kF32) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                wv[4 * i] = u2f(col.w[i].x); wv[4 * i + 1] = u2f(col.w[i].y); wv[4 * i + 2] = u2f(col.w[i].z); wv[4 * i + 3] = u2f(col.w[i].w);
            }
        } else {
            const uint32_t u[8] = {col.w[0].x, col.w[0].y, col.w[0].z, col.w[0].w, col.w[1].x, col.w[1].y, col.w[1].z, col.w[1].w};
#pragma unroll
            for (int k = 0; k < 8; k++) {
                wv[2 * k] = WDT == kBF16 ? bf16lo(u[k]) : f16lo(u[k]);
                wv[2 * k + 1] = WDT == kBF16 ? bf16hi(u[k]) : f16hi(u[k]);
            }
        }
#pragma unroll
        for (int k = 0; k < 4; k++) {
            float f[4];
            fp8x4_to_f32<KIND>(c[k], f);
#pragma unroll
            for (int i = 0; i < 4; i++) v[4 * k + i] = round_to<kBF16>(((f[i] * sc) * r.rstd) * wv[4 * k + i]);
        }
    }
};

// (x - mean[row]) * rstd[row] (* w[col] + b[col]) of k_layernorm_fwd, kept in fp32 as the reference keeps it
// (coat/activation/real_quantization/func_layernorm_noparam.py:93-113, func_layernorm_param.py:94-119).
// WMODE: dtype of w and b, or 3 = no affine parameters.
template <int KIND, int WMODE> struct LayerNormSource {
    static constexpr int kNW = WMODE == 3 ? 1 : (WMODE == kF32 ? 4 : 2);  // 16-byte pieces of 16 weights
    const uint8_t* q; const void* s; const void* w; const void* b; const float* mean; const float* rstd;
    int s_dt, qb; int64_t N;
    struct Raw { uint4 codes; uint32_t sc; float mean, rstd; };  // sc: the scale as loaded, converted in value()
    struct Col { uint4 w[kNW], b[kNW]; };
    __device__ __forceinline__ void load(int64_t m, int64_t n, Raw& r) const {
        r.codes = *(const uint4*)(q + m * N + n);
        r.sc = load_rt_raw(s, m * (N / qb) + n / qb, s_dt);
        r.mean = mean[m];
        r.rstd = rstd[m];
    }
    __device__ __forceinline__ void load_col(int64_t n, Col& c) const {
        if constexpr (WMODE != 3) {
            const uint4* wp = (const uint4*)((const uint8_t*)w + n * (WMODE == kF32 ? 4 : 2));
            const uint4* bp = (const uint4*)((const uint8_t*)b + n * (WMODE == kF32 ? 4 : 2));
#pragma unroll
            for (int i = 0; i < kNW; i++) { c.w[i] = wp[i]; c.b[i] = bp[i]; }
        }
    }
    static __device__ __forceinline__ void unpack16(const uint4* p, float* o) {
        if constexpr (WMODE == kF32) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                o[4 * i] = u2f(p[i].x); o[4 * i + 1] = u2f(p[i].y); o[4 * i + 2] = u2f(p[i].z); o[4 * i + 3] = u2f(p[i].w);
            }
        } else if constexpr (WMODE != 3) {
            const uint32_t u[8] = {p[0].x, p[0].y, p[0].z, p[0].w, p[1].x, p[1].y, p[1].z, p[1].w};
#pragma unroll
            for (int k = 0; k < 8; k++) {
                o[2 * k] = WMODE == kBF16 ? bf16lo(u[k]) : f16lo(u[k]);
                o[2 * k + 1] = WMODE == kBF16 ? bf16hi(u[k]) : f16hi(u[k]);
            }
        }
    }
    __device__ __forceinline__ void value(const Raw& r, const Col& col, float* v) const {
        const uint32_t c[4] = {r.codes.x, r.codes.y, r.codes.z, r.codes.w};
        const float sc = rt_raw_to_f32(r.sc, s_dt);
        float wv[16], bv[16];
        unpack16(col.w, wv);
        unpack16(col.b, bv);
#pragma unroll
        for (int k = 0; k < 4; k++) {
            float f[4];
            fp8x4_to_f32<KIND>(c[k], f);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float t = ((f[i] * sc) - r.mean) * r.rstd;
                if constexpr (WMODE != 3) t = t * wv[4 * k + i] + bv[4 * k + i];
                v[4 * k + i] = t;
            }
        }
    }
};

// bf16(dequant(a) * dequant(b)) of two per-group FP8 tensors: the product of k_silu_mul's forward
// (coat/activation/real_quantization/mul_fwd.py:136-150).  a is dense [M, N]; b may be a column slice of a wider tensor
// (row pitches in elements / scales).
template <int KIND> struct ProductSource {
    const uint8_t* a; const void* sa; const uint8_t* b; const void* sb;
    int sa_dt, sb_dt, qb; int64_t N, b_pitch, sb_pitch;
    struct Raw { uint4 ca, cb; uint32_t fa, fb; };  // fa, fb: the scales as loaded, converted in value()
    struct Col {};
    __device__ __forceinline__ void load_col(int64_t, Col&) const {}
    __device__ __forceinline__ void load(int64_t m, int64_t n, Raw& r) const {
        r.ca = *(const uint4*)(a + m * N + n);
        r.cb = *(const uint4*)(b + m * b_pitch + n);
        r.fa = load_rt_raw(sa, m * (N / qb) + n / qb, sa_dt);
        r.fb = load_rt_raw(sb, m * sb_pitch + n / qb, sb_dt);
    }
    __device__ __forceinline__ void value(const Raw& r, const Col&, float* v) const {
        const uint32_t ca[4] = {r.ca.x, r.ca.y, r.ca.z, r.ca.w}, cb[4] = {r.cb.x, r.cb.y, r.cb.z, r.cb.w};
        const float sfa = rt_raw_to_f32(r.fa, sa_dt), sfb = rt_raw_to_f32(r.fb, sb_dt);
#pragma unroll
        for (int k = 0; k < 4; k++) {
            float fa[4], fb[4];
            fp8x4_to_f32<KIND>(ca[k], fa);
            fp8x4_to_f32<KIND>(cb[k], fb);
#pragma unroll
            for (int i = 0; i < 4; i++) v[4 * k + i] = round_to<kBF16>((fa[i] * sfa) * (fb[i] * sfb));
        }
    }
};

// q = fp8(value / bf16(*s_max)) and its transpose; the rounded scale goes to s_out (bf16).  M % 16 == 0, N % 16 == 0.
// Launch with produced_division_grid(M, N) blocks.
static inline int64_t produced_division_grid(int64_t M, int64_t N) {
    const int64_t ntiles = ((M + 127) / 128) * ((N + kTileN - 1) / kTileN);
    return ((ntiles + 7) >> 3) << 3;
}
template <typename SRC, int KIND>
__global__ __launch_bounds__(kDivTThreads) void k_produced_division_transpose(SRC src, const float* __restrict__ s_max,
                                                                      void* __restrict__ s_out, void* __restrict__ q,
                                                                      void* __restrict__ qt, int64_t M, int64_t N) {
    constexpr int TM = 128;
    __shared__ uint32_t tile[TM * kPitchDw];
    enable_fp8_saturation();
    const int64_t tiles_n = (N + kTileN - 1) / kTileN;
    // Blocks go round-robin over the 8 XCDs, each with an L2 of its own.  A 128-byte line of group scales serves 8 tiles
    // that are neighbours along n: with tiles in plain block order those 8 tiles sit on 8 XCDs and every one of them
    // fetches the line (measured on [8192, 4096]: 67.6 MB fetched for 37.7 MB of inputs, 27.5 us against 22.9 us).  So XCD x takes the x-th contiguous eighth of
    // the row-major tile order and its blocks walk that band in launch order.
    const int64_t ntiles = ((M + TM - 1) / TM) * tiles_n, per_xcd = (ntiles + 7) >> 3;
    const int64_t in_band = per_xcd - 1 - (blockIdx.x >> 3);  // from the band's end, see block_from_end()
    const int64_t tile_id = (int64_t)(blockIdx.x & 7) * per_xcd + in_band;
    if (in_band < 0 || tile_id >= ntiles) return;  // grid = 8 * per_xcd
    const int64_t m0 = (tile_id / tiles_n) * TM, n0 = (tile_id % tiles_n) * kTileN;
    const float s = load_scale_or_max<kBF16>(s_max, s_out);
    const float r = 1.0f / s;
    const bool fast = s >= kMinFastDivScale && s < 0x1p100f;
    constexpr int NIT = TM * (kTileN / 16) / kDivTThreads;
    static_assert(kDivTThreads % (kTileN / 16) == 0, "all jobs of a thread lie in one 16-column strip");
    typename SRC::Raw raw[NIT];
    typename SRC::Col col;
    // all loads are unconditional (jobs outside the matrix re-read its last row / last 16 columns and are dropped):
    // under a condition the compiler makes the wave wait for each load before it issues the next
    {
        const int64_t n = n0 + (threadIdx.x % (kTileN / 16)) * 16;
        src.load_col(min(n, N - 16), col);
    }
#pragma unroll
    for (int it = 0; it < NIT; it++) {
        const int job = threadIdx.x + it * kDivTThreads;
        const int64_t m = m0 + job / (kTileN / 16), n = n0 + (job % (kTileN / 16)) * 16;
        src.load(min(m, M - 1), min(n, N - 16), raw[it]);
    }
#pragma unroll
    for (int it = 0; it < NIT; it++) {
        const int job = threadIdx.x + it * kDivTThreads;
        const int row = job / (kTileN / 16), c16 = job % (kTileN / 16);
        const int64_t m = m0 + row, n = n0 + c16 * 16;
        uint32_t c[4] = {0, 0, 0, 0};
        if (m < M && n < N) {
            float v[16];
            src.value(raw[it], col, v);
            if (fast) quantize_vec<KIND, 16>(v, s, r, c);
            else quantize_vec_slow<KIND, 16>(v, s, c);
            *(uint4*)((uint8_t*)q + m * N + n) = make_uint4(c[0], c[1], c[2], c[3]);
        }
#pragma unroll
        for (int k = 0; k < 4; k++) tile[row * kPitchDw + c16 * 4 + k] = c[k];
    }
    __syncthreads();
    store_tile_transposed<TM>(tile, qt, M, N, m0, n0);
}

// ------------------------------------------------------------------------------------------------
// K2: per-group quantize of x and of x^T in one pass over x.
// Tile = TM x TN fp32 values in LDS (pitch TN + 1 words; 64 x 128, or 128 x 128 for QB = 128).  Phase 1 does the row-direction groups exactly like
// k_quantize_pg and parks the fp32 values in LDS; phase 2 gives every lane a (column, 16-row chunk) job:
// amax over the chunk (and over QB/16 neighbouring lanes), quantize, one 16-byte store into qt.
template <int XDT, int SDT, int KIND, int QB, int TM, int TN>
__global__ __launch_bounds__(256) void k_quantize_transpose(const void* __restrict__ x, void* __restrict__ q,
                                                             void* __restrict__ s_out, void* __restrict__ qt,
                                                             void* __restrict__ st_out, int64_t M, int64_t N) {
    constexpr int VEC = VecOf<XDT>::kVec;
    constexpr int ESIZE = 16 / VEC;
    constexpr int LPG = QB / VEC;
    constexpr int PITCH = TN + 1;
    static_assert(QB <= TN && TM % QB == 0, "tile must hold whole groups in both directions");
    extern __shared__ float tile[];  // TM x PITCH fp32 (dynamic: 65 KiB for the 128 x 128 tile of QB = 128)
    enable_fp8_saturation();
    const int64_t tiles_n = (N + TN - 1) / TN;
    const int64_t SN = N / QB, SM = M / QB;
    // One tile per block, tiles taken in row-major order: the blocks resident at any time then read and write a few
    // whole bands of rows of x and q (long contiguous runs for the memory controllers) and the hardware balances the
    // rest.  Measured on bf16 [8192, 11008] against pairs of tiles walked down the columns per XCD with register
    // prefetch: 89 us instead of 118 us; more tiles per block were slower (4: 105 us, 8: 117 us).
    // tile rows are padded to a multiple of 8 blocks: blocks go round-robin over the 8 XCDs, so the tiles of one tile
    // column then share an XCD and the 8-byte pieces they write into the same line of the transposed scales meet in one
    // L2 (2 % on [8192, 11008], where a tile row has 86 tiles)
    const int64_t tn_pad = (tiles_n + 7) & ~(int64_t)7;
    const int64_t tm = (int64_t)blockIdx.x / tn_pad, tn = (int64_t)blockIdx.x % tn_pad;
    if (tn >= tiles_n) return;
    const int64_t m0 = tm * TM, n0 = tn * TN;

    // phase-1 jobs: VEC consecutive elements (16 bytes); a row of the tile is TN/VEC jobs (a multiple of LPG)
    constexpr int JPR = TN / VEC;
    constexpr int JOBS = TM * JPR;
    static_assert(JOBS % 256 == 0, "phase 1 keeps all lanes of a group in the same iteration");
    constexpr int NIT = JOBS / 256;
    uint4 raw[NIT];
#pragma unroll
    for (int it = 0; it < NIT; it++) {
        const int job = threadIdx.x + it * 256;
        const int64_t m = m0 + job / JPR, n = n0 + (job % JPR) * VEC;
        raw[it] = (m < M && n < N) ? *(const uint4*)((const uint8_t*)x + (m * N + n) * ESIZE) : make_uint4(0, 0, 0, 0);
    }
    {
#pragma unroll
        for (int it = 0; it < NIT; it++) {
            const int job = threadIdx.x + it * 256;
            const int row = job / JPR, cv = job % JPR;
            const int64_t m = m0 + row, n = n0 + cv * VEC;
            const bool ok = m < M && n < N;  // N % QB == 0: a group is inside or outside as a whole
            float v[VEC];
            unpack_vec<XDT>(raw[it], v);
            float amax = cluster_max<LPG>(vec_amax<VEC>(v));
            float s = group_scale<KIND>(amax);
            float r = 1.0f / s;
            uint32_t c[VEC / 4];
            quantize_vec<KIND, VEC>(v, s, r, c);
            if (ok) {
                store_codes<VEC>(q, m * N + n, c);
                if ((threadIdx.x % LPG) == 0) store_from_f32<SDT>(s_out, m * SN + n / QB, s);
            }
#pragma unroll
            for (int k = 0; k < VEC; k++) tile[row * PITCH + cv * VEC + k] = v[k];
        }
        __syncthreads();

        // phase 2: job = (column n, 16-row chunk mc), mc fastest so that neighbouring lanes write
        // neighbouring 16-byte pieces of one qt row; groups of QB rows are QB/16 neighbouring lanes.
        constexpr int MC = TM / 16;
        constexpr int LPG_T = QB / 16;
        constexpr int JOBS2 = MC * TN;
        static_assert(JOBS2 % 256 == 0, "phase 2 keeps all lanes of a group in the same iteration");
        for (int job = threadIdx.x; job < JOBS2; job += 256) {
            int mc = job % MC, col = job / MC;
            int64_t m = m0 + mc * 16, n = n0 + col;
            bool ok = m < M && n < N;  // M % QB == 0: whole groups again
            float v[16];
#pragma unroll
            for (int i = 0; i < 16; i++) v[i] = tile[(mc * 16 + i) * PITCH + col];
            float amax = cluster_max<LPG_T>(vec_amax<16>(v));
            float s = group_scale<KIND>(amax);
            float r = 1.0f / s;
            uint32_t c[4];
            quantize_vec<KIND, 16>(v, s, r, c);
            if (ok) {
                *(uint4*)((uint8_t*)qt + n * M + m) = make_uint4(c[0], c[1], c[2], c[3]);
                if ((mc % LPG_T) == 0) store_from_f32<SDT>(st_out, n * SM + m / QB, s);
            }
        }
    }
}

// K2 for 16-bit inputs (bf16 / fp16): the tile is parked in LDS as the raw 16-bit input (exact, half the footprint of
// fp32), which makes a 128 x 128 tile fit four times per CU: q, q^T and both scale tensors are then written in whole
// 128-byte lines / 16-byte scale pieces.  Phase 2 reads one dword = two neighbouring columns of one row, so a lane owns
// a column pair over a 16-row chunk (two 16-byte stores into neighbouring q^T rows); chunks vary fastest over the
// lanes, so 8 neighbouring lanes complete one 128-byte q^T line.
// NT threads per tile: 256 when the grid is about one round of resident blocks (17.6 against 19.5 us at [4096, 4096]),
// 512 = twice the waves per CU for larger tensors (78.9 against 82.4 us at [8192, 11008]).
template <int XDT, int SDT, int KIND, int QB, int NT>
__global__ __launch_bounds__(NT) void k_quantize_transpose16(const void* __restrict__ x, void* __restrict__ q,
                                                               void* __restrict__ s_out, void* __restrict__ qt,
                                                               void* __restrict__ st_out, int64_t M, int64_t N) {
    static_assert(XDT != kF32, "16-bit inputs only");
    constexpr int T = 128;            // tile edge
    constexpr int PDW = T / 2 + 1;    // row pitch in dwords (odd: column reads spread over the banks)
    constexpr int LPG = QB / 8;       // lanes per row-direction group (8 elements per lane)
    __shared__ uint32_t tile[T * PDW];
    enable_fp8_saturation();
    const int64_t tiles_n = (N + T - 1) / T;
    const int64_t SN = N / QB, SM = M / QB;
    const int64_t tn_pad = (tiles_n + 7) & ~(int64_t)7;  // see k_quantize_transpose
    const int64_t tm = (int64_t)blockIdx.x / tn_pad, tn = (int64_t)blockIdx.x % tn_pad;
    if (tn >= tiles_n) return;
    const int64_t m0 = tm * T, n0 = tn * T;

    // phase 1: 16 jobs of 8 elements per row, 8 jobs per thread; all loads first
    constexpr int JPR = T / 8, NIT = T * JPR / NT;
    uint4 raw[NIT];
#pragma unroll
    for (int it = 0; it < NIT; it++) {
        const int job = threadIdx.x + it * NT;
        const int64_t m = m0 + job / JPR, n = n0 + (job % JPR) * 8;
        // (conditional on purpose: all eight loads issued back to back were measured 11 % slower, 19.7 against 17.7 us)
        raw[it] = (m < M && n < N) ? *(const uint4*)((const uint16_t*)x + m * N + n) : make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int it = 0; it < NIT; it++) {
        const int job = threadIdx.x + it * NT;
        const int row = job / JPR, cv = job % JPR;
        const int64_t m = m0 + row, n = n0 + cv * 8;
        const bool ok = m < M && n < N;  // N % QB == 0: a group is inside or outside as a whole
        float v[8];
        unpack_vec<XDT>(raw[it], v);
        const float amax = cluster_max<LPG>(vec_amax<8>(v));
        const float s = group_scale<KIND>(amax);
        const float r = 1.0f / s;
        uint32_t c[2];
        quantize_vec<KIND, 8>(v, s, r, c);
        if (ok) {
            store_codes<8>(q, m * N + n, c);
            if ((threadIdx.x % LPG) == 0) store_from_f32<SDT>(s_out, m * SN + n / QB, s);
        }
        uint32_t* dst = tile + row * PDW + cv * 4;
        dst[0] = raw[it].x; dst[1] = raw[it].y; dst[2] = raw[it].z; dst[3] = raw[it].w;
    }
    __syncthreads();

    // phase 2: job = (column pair cp, 16-row chunk mc), mc fastest; groups of QB rows are QB/16 neighbouring lanes
    constexpr int MC = T / 16, LPG_T = QB / 16, JOBS2 = MC * (T / 2);
#pragma unroll
    for (int j0 = 0; j0 < JOBS2; j0 += NT) {
        const int job = j0 + threadIdx.x;
        const int mc = job % MC, cp = job / MC;
        const int64_t m = m0 + mc * 16, n = n0 + 2 * cp;
        const bool ok = m < M && n < N;  // M % QB == 0 and N even: whole groups, whole pairs
        float v0[16], v1[16];
#pragma unroll
        for (int i = 0; i < 16; i++) {
            const uint32_t w = tile[(mc * 16 + i) * PDW + cp];
            v0[i] = XDT == kBF16 ? bf16lo(w) : f16lo(w);
            v1[i] = XDT == kBF16 ? bf16hi(w) : f16hi(w);
        }
        const float s0 = group_scale<KIND>(cluster_max<LPG_T>(vec_amax<16>(v0)));
        const float s1 = group_scale<KIND>(cluster_max<LPG_T>(vec_amax<16>(v1)));
        uint32_t c0[4], c1[4];
        quantize_vec<KIND, 16>(v0, s0, 1.0f / s0, c0);
        quantize_vec<KIND, 16>(v1, s1, 1.0f / s1, c1);
        if (ok) {
            *(uint4*)((uint8_t*)qt + n * M + m) = make_uint4(c0[0], c0[1], c0[2], c0[3]);
            *(uint4*)((uint8_t*)qt + (n + 1) * M + m) = make_uint4(c1[0], c1[1], c1[2], c1[3]);
            if ((mc % LPG_T) == 0) {
                store_from_f32<SDT>(st_out, n * SM + m / QB, s0);
                store_from_f32<SDT>(st_out, (n + 1) * SM + m / QB, s1);
            }
        }
    }
}

}  // namespace coat

// ================================================================================================ C ABI
using namespace coat;

#define DISPATCH_XDT(XDT_VAR, ...)                                   \
    switch (XDT_VAR) {                                               \
        case COAT_F32: { constexpr int XDT = kF32; __VA_ARGS__; break; }   \
        case COAT_BF16: { constexpr int XDT = kBF16; __VA_ARGS__; break; } \
        case COAT_F16: { constexpr int XDT = kF16; __VA_ARGS__; break; }   \
        default: return COAT_EDTYPE;                                 \
    }
#define DISPATCH_SDT(SDT_VAR, ...)                                   \
    switch (SDT_VAR) {                                               \
        case COAT_F32: { constexpr int SDT = kF32; __VA_ARGS__; break; }   \
        case COAT_BF16: { constexpr int SDT = kBF16; __VA_ARGS__; break; } \
        case COAT_F16: { constexpr int SDT = kF16; __VA_ARGS__; break; }   \
        default: return COAT_EDTYPE;                                 \
    }
#define DISPATCH_KIND(KIND_VAR, ...)                                 \
    switch (KIND_VAR) {                                              \
        case COAT_E4M3: { constexpr int KIND = kE4M3; __VA_ARGS__; break; } \
        case COAT_E5M2: { constexpr int KIND = kE5M2; __VA_ARGS__; break; } \
        default: return COAT_EINVAL;                                 \
    }
/* QB 16 (the activation group size) is compiled in; 32 / 64 / 128 share one run-time variant (QB = 0). */
#define DISPATCH_QB(QB_VAR, ...)                                     \
    switch (QB_VAR) {                                                \
        case 16: { constexpr int QB = 16; const int QB_RT = 16; (void)QB_RT; __VA_ARGS__; break; } \
        case 32: case 64: case 128: { const int QB_RT = QB_VAR; constexpr int QB = 0; (void)QB_RT; __VA_ARGS__; break; } \
        default: return COAT_ESHAPE;                                 \
    }

static inline int check_mn(int64_t M, int64_t N, int QB) {
    if (M < 0 || N < 0) return COAT_EINVAL;
    if (QB <= 0 || N % QB != 0) return COAT_ESHAPE;
    return COAT_OK;
}

template <int XDT, int SDT, int KIND, int QB, bool WQ, bool WS, bool WMAX>
static int launch_quantize_pg(const void* x, void* q, void* s, float* s_max, int64_t numel, int qb, hipStream_t st) {
    constexpr int VEC = VecOf<XDT>::kVec;
    int64_t nvec = numel / VEC;
    if (nvec == 0) return COAT_OK;
    // two 16-byte loads per lane (bf16 [4096, 4096]: 11.1 us against 12.5 us with four; [8192, 11008]: 42.7 against 44.7 us)
    int64_t blocks = (nvec + 256 * 2 - 1) / (256 * 2);
    if (WMAX && blocks > 2048) blocks = 2048;  // fewer, longer blocks: one atomic per block
    hipLaunchKernelGGL((k_quantize_pg<XDT, SDT, KIND, QB, WQ, WS, WMAX, 2>), dim3((unsigned)blocks), dim3(256), 0, st, x, q, s, s_max, nvec, qb);
    return coat_launch_status();
}

extern "C" int coat_fp8_quantize(const void* x, int x_dtype, void* q, void* s, int s_dtype, int64_t M, int64_t N, int QB,
                                 int fp8, void* stream) {
    if (int e = check_mn(M, N, QB)) return e;
    if (M * N == 0) return COAT_OK;
    if (!x || !q || !s) return COAT_EINVAL;
    if (!coat_aligned16(x) || !coat_aligned16(q)) return COAT_EALIGN;
    hipStream_t st = (hipStream_t)stream;
    DISPATCH_XDT(x_dtype, DISPATCH_SDT(s_dtype, DISPATCH_KIND(fp8, DISPATCH_QB(QB,
        return launch_quantize_pg<XDT, SDT, KIND, QB, true, true, false>(x, q, s, nullptr, M * N, QB_RT, st)))));
    return COAT_EINVAL;
}

extern "C" int coat_fp8_group_scales(const void* x, int x_dtype, void* s_pg, int s_dtype, float* s_max, int64_t M,
                                     int64_t N, int QB, int fp8, void* stream) {
    if (int e = check_mn(M, N, QB)) return e;
    if (M * N == 0) return COAT_OK;
    if (!x || !s_max) return COAT_EINVAL;
    if (!coat_aligned16(x)) return COAT_EALIGN;
    hipStream_t st = (hipStream_t)stream;
    if (s_pg) {
        DISPATCH_XDT(x_dtype, DISPATCH_SDT(s_dtype, DISPATCH_KIND(fp8, DISPATCH_QB(QB,
            return launch_quantize_pg<XDT, SDT, KIND, QB, false, true, true>(x, nullptr, s_pg, s_max, M * N, QB_RT, st)))));
    } else {
        DISPATCH_XDT(x_dtype, DISPATCH_KIND(fp8, DISPATCH_QB(QB,
            return launch_quantize_pg<XDT, kF32, KIND, QB, false, false, true>(x, nullptr, nullptr, s_max, M * N, QB_RT, st))));
    }
    return COAT_EINVAL;
}

extern "C" int coat_absmax(const void* x, int x_dtype, float* amax, int64_t numel, void* stream) {
    if (numel < 0 || !amax) return COAT_EINVAL;
    if (numel == 0) return COAT_OK;
    if (!x) return COAT_EINVAL;
    if (!coat_aligned16(x)) return COAT_EALIGN;
    hipStream_t st = (hipStream_t)stream;
    DISPATCH_XDT(x_dtype, {
        constexpr int VEC = VecOf<XDT>::kVec;
        int64_t nvec = numel / VEC;
        int64_t blocks = (nvec + 256 * 4 - 1) / (256 * 4);
        if (blocks == 0) blocks = 1;
        if (blocks > 2048) blocks = 2048;
        hipLaunchKernelGGL((k_absmax<XDT, 4>), dim3((unsigned)blocks), dim3(256), 0, st, x, amax, nvec, numel);
        return coat_launch_status();
    });
    return COAT_EINVAL;
}

template <bool SR>
static int division_launch(const void* x, int x_dtype, const void* s, int s_dtype, void* q, void* qt, int64_t M, int64_t N,
                           int fp8, uint64_t seed, void* stream, void* s_out = nullptr) {
    if (M < 0 || N < 0) return COAT_EINVAL;
    if (M * N == 0) return COAT_OK;
    if (!x || !s || (!q && !qt)) return COAT_EINVAL;
    if (!coat_aligned16(x) || !coat_aligned16(q) || !coat_aligned16(qt)) return COAT_EALIGN;
    hipStream_t st = (hipStream_t)stream;
    const uint32_t k0 = (uint32_t)seed, k1 = (uint32_t)(seed >> 32);
    if (!qt) {
        DISPATCH_XDT(x_dtype, DISPATCH_SDT(s_dtype, DISPATCH_KIND(fp8, {
            constexpr int VEC = VecOf<XDT>::kVec;
            int64_t numel = M * N, nvec = numel / VEC;
            // two 16-byte loads per lane: 18.5 us on bf16 [8192, 4096] against 19.7 us with four and 20.5 us with one
            int64_t blocks = (nvec + 256 * 2 - 1) / (256 * 2);
            if (blocks == 0) blocks = 1;
            hipLaunchKernelGGL((k_division<XDT, SDT, KIND, 2, SR>), dim3((unsigned)blocks), dim3(256), 0, st, x, s, q, nvec, numel, k0, k1, s_out);
            return coat_launch_status();
        })));
        return COAT_EINVAL;
    }
    if (M % 16 != 0 || N % 16 != 0) return COAT_ESHAPE;
    constexpr int TM = 128;
    int64_t blocks = ((M + TM - 1) / TM) * ((N + kTileN - 1) / kTileN);
    if (q) {
        DISPATCH_XDT(x_dtype, DISPATCH_SDT(s_dtype, DISPATCH_KIND(fp8, {
            hipLaunchKernelGGL((k_division_transpose<XDT, SDT, KIND, false, true, TM, SR>), dim3((unsigned)blocks), dim3(kDivTThreads), 0, st, x, s, q, qt, M, N, k0, k1, s_out);
            return coat_launch_status();
        })));
    } else {
        DISPATCH_XDT(x_dtype, DISPATCH_SDT(s_dtype, DISPATCH_KIND(fp8, {
            hipLaunchKernelGGL((k_division_transpose<XDT, SDT, KIND, false, false, TM, SR>), dim3((unsigned)blocks), dim3(kDivTThreads), 0, st, x, s, q, qt, M, N, k0, k1, s_out);
            return coat_launch_status();
        })));
    }
    return COAT_EINVAL;
}

extern "C" int coat_fp8_division(const void* x, int x_dtype, const void* s, int s_dtype, void* q, void* qt, int64_t M,
                                 int64_t N, int fp8, void* stream) {
    return division_launch<false>(x, x_dtype, s, s_dtype, q, qt, M, N, fp8, 0, stream);
}

extern "C" int coat_fp8_division_from_max(const void* x, int x_dtype, const float* s_max, void* s_out, int s_dtype, void* q,
                                          void* qt, int64_t M, int64_t N, int fp8, void* stream) {
    if ((M > 0 && N > 0) && !s_out) return COAT_EINVAL;
    return division_launch<false>(x, x_dtype, s_max, s_dtype, q, qt, M, N, fp8, 0, stream, s_out);
}

extern "C" int coat_fp8_division_stochastic(const void* x, int x_dtype, const void* s, int s_dtype, void* q, void* qt,
                                            int64_t M, int64_t N, int fp8, uint64_t seed, void* stream) {
    // the noise counter is the 32-bit linear element index, as in the reference's int32 offset arithmetic
    if (M > 0 && N > 0 && M * N > ((int64_t)1 << 32)) return COAT_ESHAPE;
    return division_launch<true>(x, x_dtype, s, s_dtype, q, qt, M, N, fp8, seed, stream);
}

// The division (+ transpose) that follows coat_fp8_rmsnorm_forward, fed with that kernel's inputs instead of its bf16
// output (which the caller then need not store: y = NULL there).
extern "C" int coat_fp8_rmsnorm_division(const void* x, int fp8, const void* s_x, int s_dtype, const void* w, int w_dtype,
                                         const float* rstd, const float* s_max, void* s_out, void* q, void* qt, int64_t M,
                                         int64_t N, int QB, void* stream) {
    if (int e = check_mn(M, N, QB)) return e;
    if (M * N == 0) return COAT_OK;
    if (M % 16 != 0 || N % 16 != 0 || QB % 16 != 0) return COAT_ESHAPE;
    if (!x || !s_x || !w || !rstd || !s_max || !s_out || !q || !qt) return COAT_EINVAL;
    if (!coat_aligned16(x) || !coat_aligned16(w) || !coat_aligned16(q) || !coat_aligned16(qt)) return COAT_EALIGN;
    if (s_dtype < 0 || s_dtype > 2) return COAT_EDTYPE;
    const int64_t blocks = produced_division_grid(M, N);
    if (blocks >= ((int64_t)1 << 31)) return COAT_ESHAPE;
    hipStream_t st = (hipStream_t)stream;
#define RMS_DIV(KINDV, WDTV)                                                                                        \
    {                                                                                                               \
        RmsNormSource<KINDV, WDTV> src{(const uint8_t*)x, s_x, w, rstd, s_dtype, QB, N};                             \
        hipLaunchKernelGGL((k_produced_division_transpose<RmsNormSource<KINDV, WDTV>, KINDV>), dim3((unsigned)blocks), \
                           dim3(kDivTThreads), 0, st, src, s_max, s_out, q, qt, M, N);                                       \
        return coat_launch_status();                                                                                \
    }
    DISPATCH_KIND(fp8, {
        if (w_dtype == COAT_BF16) RMS_DIV(KIND, kBF16)
        if (w_dtype == COAT_F32) RMS_DIV(KIND, kF32)
        if (w_dtype == COAT_F16) RMS_DIV(KIND, kF16)
        return COAT_EDTYPE;
    });
#undef RMS_DIV
    return COAT_EINVAL;
}

// The same for coat_fp8_layernorm_forward (y = NULL there); w_dtype < 0: no affine parameters.
extern "C" int coat_fp8_layernorm_division(const void* x, int fp8, const void* s_x, int s_dtype, const void* w, const void* b,
                                           int w_dtype, const float* mean, const float* rstd, const float* s_max,
                                           void* s_out, void* q, void* qt, int64_t M, int64_t N, int QB, void* stream) {
    if (int e = check_mn(M, N, QB)) return e;
    if (M * N == 0) return COAT_OK;
    if (M % 16 != 0 || N % 16 != 0 || QB % 16 != 0) return COAT_ESHAPE;
    if (!x || !s_x || !mean || !rstd || !s_max || !s_out || !q || !qt) return COAT_EINVAL;
    if (w_dtype >= 0 && (!w || !b)) return COAT_EINVAL;
    if (w_dtype > 2) return COAT_EDTYPE;
    if (!coat_aligned16(x) || !coat_aligned16(w) || !coat_aligned16(b) || !coat_aligned16(q) || !coat_aligned16(qt))
        return COAT_EALIGN;
    if (s_dtype < 0 || s_dtype > 2) return COAT_EDTYPE;
    const int64_t blocks = produced_division_grid(M, N);
    if (blocks >= ((int64_t)1 << 31)) return COAT_ESHAPE;
    hipStream_t st = (hipStream_t)stream;
#define LN_DIV(KINDV, WM)                                                                                            \
    {                                                                                                                \
        LayerNormSource<KINDV, WM> src{(const uint8_t*)x, s_x, w, b, mean, rstd, s_dtype, QB, N};                    \
        hipLaunchKernelGGL((k_produced_division_transpose<LayerNormSource<KINDV, WM>, KINDV>), dim3((unsigned)blocks), \
                           dim3(kDivTThreads), 0, st, src, s_max, s_out, q, qt, M, N);                               \
        return coat_launch_status();                                                                                 \
    }
    DISPATCH_KIND(fp8, {
        if (w_dtype < 0) LN_DIV(KIND, 3)
        if (w_dtype == COAT_BF16) LN_DIV(KIND, kBF16)
        if (w_dtype == COAT_F32) LN_DIV(KIND, kF32)
        if (w_dtype == COAT_F16) LN_DIV(KIND, kF16)
        return COAT_EDTYPE;
    });
#undef LN_DIV
    return COAT_EINVAL;
}

// The division (+ transpose) of the product of two per-group FP8 tensors (what coat_fp8_silu_mul_forward and
// coat_fp8_mul_forward leave in their bf16 output), recomputed from the two factors.  a [M, N] dense with scales
// [M, N / QB]; b with row pitch b_pitch codes and sb_pitch scales (0 = dense).
extern "C" int coat_fp8_product_division(const void* a, const void* s_a, int sa_dtype, const void* b, const void* s_b,
                                         int sb_dtype, int fp8, const float* s_max, void* s_out, void* q, void* qt,
                                         int64_t M, int64_t N, int QB, int64_t b_pitch, int64_t sb_pitch, void* stream) {
    if (int e = check_mn(M, N, QB)) return e;
    if (M * N == 0) return COAT_OK;
    if (M % 16 != 0 || N % 16 != 0 || QB % 16 != 0) return COAT_ESHAPE;
    if (!a || !s_a || !b || !s_b || !s_max || !s_out || !q || !qt) return COAT_EINVAL;
    if (b_pitch == 0) b_pitch = N;
    if (sb_pitch == 0) sb_pitch = N / QB;
    if (b_pitch < N || b_pitch % 16 != 0 || sb_pitch < N / QB) return COAT_ESHAPE;
    if (!coat_aligned16(a) || !coat_aligned16(b) || !coat_aligned16(q) || !coat_aligned16(qt)) return COAT_EALIGN;
    if (sa_dtype < 0 || sa_dtype > 2 || sb_dtype < 0 || sb_dtype > 2) return COAT_EDTYPE;
    const int64_t blocks = produced_division_grid(M, N);
    if (blocks >= ((int64_t)1 << 31)) return COAT_ESHAPE;
    hipStream_t st = (hipStream_t)stream;
    DISPATCH_KIND(fp8, {
        ProductSource<KIND> src{(const uint8_t*)a, s_a, (const uint8_t*)b, s_b, sa_dtype, sb_dtype, QB, N, b_pitch, sb_pitch};
        hipLaunchKernelGGL((k_produced_division_transpose<ProductSource<KIND>, KIND>), dim3((unsigned)blocks), dim3(kDivTThreads), 0,
                           st, src, s_max, s_out, q, qt, M, N);
        return coat_launch_status();
    });
    return COAT_EINVAL;
}

extern "C" int coat_fp8_transpose(const void* x, void* y, int64_t M, int64_t N, void* stream) {
    if (M < 0 || N < 0) return COAT_EINVAL;
    if (M * N == 0) return COAT_OK;
    if (!x || !y) return COAT_EINVAL;
    if (M % 16 != 0 || N % 16 != 0) return COAT_ESHAPE;
    if (!coat_aligned16(x) || !coat_aligned16(y)) return COAT_EALIGN;
    constexpr int TM = 128;
    int64_t blocks = ((M + TM - 1) / TM) * ((N + kTileN - 1) / kTileN);
    hipLaunchKernelGGL((k_division_transpose<kBF16, kBF16, kE4M3, true, false, TM, false>), dim3((unsigned)blocks), dim3(kDivTThreads), 0,
                       (hipStream_t)stream, x, nullptr, nullptr, y, M, N, 0u, 0u, nullptr);
    return coat_launch_status();
}

extern "C" int coat_fp8_dequantize(const void* q, int fp8, const void* s, int s_dtype, void* y, int64_t M, int64_t N,
                                   int QB, void* stream) {
    if (int e = check_mn(M, N, QB)) return e;
    if (QB % 16 != 0) return COAT_ESHAPE;
    if (M * N == 0) return COAT_OK;
    if (!q || !s || !y) return COAT_EINVAL;
    if (!coat_aligned16(q) || !coat_aligned16(y)) return COAT_EALIGN;
    int64_t nchunk = M * N / 16;
    int64_t blocks = (nchunk + 255) / 256;
    hipStream_t st = (hipStream_t)stream;
    DISPATCH_SDT(s_dtype, DISPATCH_KIND(fp8, {
        hipLaunchKernelGGL((k_dequantize<SDT, KIND>), dim3((unsigned)blocks), dim3(256), 0, st, q, s, y, nchunk, QB);
        return coat_launch_status();
    }));
    return COAT_EINVAL;
}

extern "C" int coat_fp8_quantize_transpose(const void* x, int x_dtype, void* q, void* s, void* qt, void* st_out,
                                           int s_dtype, int64_t M, int64_t N, int QB, int fp8, void* stream) {
    if (int e = check_mn(M, N, QB)) return e;
    if (M % QB != 0) return COAT_ESHAPE;
    if (M * N == 0) return COAT_OK;
    if (!x || !q || !s || !qt || !st_out) return COAT_EINVAL;
    if (!coat_aligned16(x) || !coat_aligned16(q) || !coat_aligned16(qt)) return COAT_EALIGN;
    if (QB > 128) return COAT_ESHAPE;  // groups must fit the tile in both directions (the reference tunes 16..128)
    hipStream_t st = (hipStream_t)stream;
    // 64 x 128 tiles for QB <= 64 (33 KiB of LDS: four blocks per CU), 128 x 128 for QB = 128
    const int TMh = QB == 128 ? 128 : 64, TNh = 128;
    const int64_t blocks = ((M + TMh - 1) / TMh) * ((((N + TNh - 1) / TNh) + 7) & ~(int64_t)7);  // one tile per block, row-major
    if (blocks >= ((int64_t)1 << 31)) return COAT_ESHAPE;
#define LAUNCH_QT(QBV, TMV, TNV)                                                                                     \
    DISPATCH_XDT(x_dtype, DISPATCH_SDT(s_dtype, DISPATCH_KIND(fp8, {                                                 \
        constexpr int kLds = TMV * (TNV + 1) * 4;                                                                    \
        if (kLds > 65536) {                                                                                          \
            static coat_device_flags lds_ok;                                                                       \
            if (int e = coat_allow_lds(k_quantize_transpose<XDT, SDT, KIND, QBV, TMV, TNV>, kLds, lds_ok)) return e; \
        }                                                                                                            \
        hipLaunchKernelGGL((k_quantize_transpose<XDT, SDT, KIND, QBV, TMV, TNV>), dim3((unsigned)blocks), dim3(256), \
                           kLds, st, x, q, s, qt, st_out, M, N);                                                     \
        return coat_launch_status();                                                                                 \
    })))
    if (x_dtype != COAT_F32) {  // 16-bit inputs: 128 x 128 tiles parked in LDS as 16-bit values
        const int64_t tn16 = (N + 127) / 128;
        const int64_t blocks16 = ((M + 127) / 128) * ((tn16 + 7) & ~(int64_t)7);
        if (blocks16 >= ((int64_t)1 << 31)) return COAT_ESHAPE;
#define LAUNCH_QT16(XD, QBV)                                                                                          \
    DISPATCH_SDT(s_dtype, DISPATCH_KIND(fp8, {                                                                        \
        if (blocks16 > 2048)                                                                                          \
            hipLaunchKernelGGL((k_quantize_transpose16<XD, SDT, KIND, QBV, 512>), dim3((unsigned)blocks16), dim3(512), 0, st,  \
                               x, q, s, qt, st_out, M, N);                                                            \
        else                                                                                                          \
            hipLaunchKernelGGL((k_quantize_transpose16<XD, SDT, KIND, QBV, 256>), dim3((unsigned)blocks16), dim3(256), 0, st,  \
                               x, q, s, qt, st_out, M, N);                                                            \
        return coat_launch_status();                                                                                  \
    }))
#define LAUNCH_QT16_QB(XD)                                  \
    switch (QB) {                                           \
        case 16: LAUNCH_QT16(XD, 16); break;                \
        case 32: LAUNCH_QT16(XD, 32); break;                \
        case 64: LAUNCH_QT16(XD, 64); break;                \
        case 128: LAUNCH_QT16(XD, 128); break;              \
        default: return COAT_ESHAPE;                        \
    }
        if (x_dtype == COAT_BF16) { LAUNCH_QT16_QB(kBF16) } else if (x_dtype == COAT_F16) { LAUNCH_QT16_QB(kF16) }
#undef LAUNCH_QT16_QB
#undef LAUNCH_QT16
        return COAT_EDTYPE;
    }
    switch (QB) {
        case 16: LAUNCH_QT(16, 64, 128); break;
        case 32: LAUNCH_QT(32, 64, 128); break;
        case 64: LAUNCH_QT(64, 64, 128); break;
        case 128: LAUNCH_QT(128, 128, 128); break;
        default: return COAT_ESHAPE;
    }
#undef LAUNCH_QT
    return COAT_EINVAL;
}

// ------------------------------------------------------------------------------------------------
// Per-block quantize: one scale per QB x QB block, (max|x| + 1e-10) / fp8max, the block divided by the fp32 scale and the
// scale stored in the scale dtype (reference coat/activation/real_quantization/_quantize_perblock.py:33-104), optionally
// with the transposed codes and scales (_quantize_perblock_transpose.py:33-133, ONLY_TRANSPOSED = the plain outputs absent)
// and with a 1 x QB per-group quantization of the same input (_quantize_perblock_transpose_pergroup.py:140-172), which is
// what the DeepSeek-style linear consumes (coat/activation/deepseek/fp8linear.py:70-110).
// A block of 512 threads takes a 128 x 128 tile = (128 / QB)^2 quantization blocks: pass 1 leaves every block's maximum
// in LDS (row-group maximum by DPP, one LDS atomic per row group), pass 2 converts from the registers that still hold the
// tile, writes the codes and parks them in LDS for the transposed stores.
namespace coat {
__device__ __forceinline__ void store_scale_rt(void* p, int64_t i, float v, int dt) {
    if (dt == kF32) ((float*)p)[i] = v;
    else if (dt == kBF16) ((uint16_t*)p)[i] = (uint16_t)f2bf16(v);
    else ((uint16_t*)p)[i] = (uint16_t)f2f16(v);
}

template <int XDT, int KIND>
__global__ __launch_bounds__(kDivTThreads) void k_quantize_perblock(const void* __restrict__ x, void* __restrict__ q,
                                                                    void* __restrict__ s_out, void* __restrict__ qt,
                                                                    void* __restrict__ st_out, void* __restrict__ qpg,
                                                                    void* __restrict__ spg_out, int sdt, int64_t M, int64_t N,
                                                                    int QB) {
    constexpr int VEC = VecOf<XDT>::kVec, T = kTileN, JPR = T / VEC, NIT = T * JPR / kDivTThreads;
    static_assert(T * JPR % kDivTThreads == 0 && kDivTThreads % JPR == 0, "whole iterations, whole rows per iteration");
    __shared__ uint32_t tile[T * kPitchDw];
    __shared__ uint32_t bmax[64];  // (128 / 16)^2 block maxima at most, as bit patterns (non-negative floats order like integers)
    enable_fp8_saturation();
    const int64_t tiles_n = (N + T - 1) / T;
    const int64_t m0 = (blockIdx.x / tiles_n) * T, n0 = (blockIdx.x % tiles_n) * T;
    const int nb = T / QB;     // quantization blocks per tile edge
    const int lpg = QB / VEC;  // lanes that hold one row of a quantization block: aligned runs of consecutive lanes
    const int64_t SN = N / QB, SM = M / QB;
    if (threadIdx.x < 64) bmax[threadIdx.x] = 0;
    uint4 raw[NIT];
    float gmax[NIT];
#pragma unroll
    for (int it = 0; it < NIT; it++) {
        const int job = threadIdx.x + it * kDivTThreads;
        const int64_t m = m0 + job / JPR, n = n0 + (job % JPR) * VEC;
        raw[it] = (m < M && n < N) ? *(const uint4*)((const uint8_t*)x + (m * N + n) * (16 / VEC)) : make_uint4(0, 0, 0, 0);
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < NIT; it++) {
        const int job = threadIdx.x + it * kDivTThreads;
        const int row = job / JPR, cv = job % JPR;
        float v[VEC];
        unpack_vec<XDT>(raw[it], v);
        gmax[it] = cluster_max_rt(vec_amax<VEC>(v), lpg);
        if ((threadIdx.x % lpg) == 0) atomicMax(&bmax[(row / QB) * nb + (cv * VEC) / QB], f2u(gmax[it]));
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < NIT; it++) {
        const int job = threadIdx.x + it * kDivTThreads;
        const int row = job / JPR, cv = job % JPR;
        const int64_t m = m0 + row, n = n0 + cv * VEC;
        const bool ok = m < M && n < N;  // M % QB == 0 and N % QB == 0: a quantization block is inside or outside as a whole
        float v[VEC];
        unpack_vec<XDT>(raw[it], v);
        const float sb = group_scale<KIND>(u2f(bmax[(row / QB) * nb + (cv * VEC) / QB]));
        uint32_t c[VEC / 4];
        quantize_vec<KIND, VEC>(v, sb, 1.0f / sb, c);
        if (q && ok) store_codes<VEC>(q, m * N + n, c);
        if (qt) {
#pragma unroll
            for (int k = 0; k < VEC / 4; k++) tile[row * kPitchDw + cv * (VEC / 4) + k] = c[k];
        }
        if (ok && (row % QB) == 0 && ((cv * VEC) % QB) == 0) {
            if (s_out) store_scale_rt(s_out, (m / QB) * SN + n / QB, sb, sdt);
            if (st_out) store_scale_rt(st_out, (n / QB) * SM + m / QB, sb, sdt);
        }
        if (qpg) {
            const float sg = group_scale<KIND>(gmax[it]);
            uint32_t cg[VEC / 4];
            quantize_vec<KIND, VEC>(v, sg, 1.0f / sg, cg);
            if (ok) {
                store_codes<VEC>(qpg, m * N + n, cg);
                if ((threadIdx.x % lpg) == 0) store_scale_rt(spg_out, m * SN + n / QB, sg, sdt);
            }
        }
    }
    if (qt) {
        __syncthreads();
        store_tile_transposed<T>(tile, qt, M, N, m0, n0);
    }
}
}  // namespace coat

// x [M, N] (M % QB == 0, N % QB == 0, QB 16 / 32 / 64 / 128) -> any of: q [M, N] + s [M/QB, N/QB]; qt [N, M] + st [N/QB, M/QB];
// qpg [M, N] + spg [M, N/QB] (1 x QB groups).  A pair is produced when both of its pointers are given.
extern "C" int coat_fp8_quantize_perblock(const void* x, int x_dtype, void* q, void* s, void* qt, void* st_out, void* qpg,
                                          void* spg, int s_dtype, int64_t M, int64_t N, int QB, int fp8, void* stream) {
    if (M < 0 || N < 0) return COAT_EINVAL;
    if (QB != 16 && QB != 32 && QB != 64 && QB != 128) return COAT_ESHAPE;
    if (M % QB != 0 || N % QB != 0) return COAT_ESHAPE;
    if (s_dtype != COAT_F32 && s_dtype != COAT_BF16 && s_dtype != COAT_F16) return COAT_EDTYPE;
    if ((q == nullptr) != (s == nullptr) || (qt == nullptr) != (st_out == nullptr) || (qpg == nullptr) != (spg == nullptr)) return COAT_EINVAL;
    if (!q && !qt && !qpg) return COAT_EINVAL;
    if (M * N == 0) return COAT_OK;
    if (!x) return COAT_EINVAL;
    if (!coat_aligned16(x) || !coat_aligned16(q) || !coat_aligned16(qt) || !coat_aligned16(qpg)) return COAT_EALIGN;
    const int64_t blocks = ((M + kTileN - 1) / kTileN) * ((N + kTileN - 1) / kTileN);
    if (blocks >= ((int64_t)1 << 31)) return COAT_ESHAPE;
    hipStream_t st = (hipStream_t)stream;
    const int sdt = s_dtype == COAT_F32 ? kF32 : s_dtype == COAT_BF16 ? kBF16 : kF16;
    DISPATCH_XDT(x_dtype, DISPATCH_KIND(fp8, {
        hipLaunchKernelGGL((k_quantize_perblock<XDT, KIND>), dim3((unsigned)blocks), dim3(kDivTThreads), 0, st, x, q, s, qt, st_out,
                           qpg, spg, sdt, M, N, QB);
        return coat_launch_status();
    }));
    return COAT_EINVAL;
}
