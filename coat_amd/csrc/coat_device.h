// Device-side helpers shared by every gfx950 kernel of the FP8 hot path.
//
// Numeric contract (all kernels):
//   * the translation units are compiled with -ffp-contract=off, so every + - * written here is a
//     separately rounded IEEE fp32 operation and an FMA happens only where fmaf() is written;
//   * fp32 division by a scale is done as reciprocal + two FMAs (div_by_scale), which returns the
//     correctly rounded quotient whenever the scale is >= 2^-60 and the quotient is not below the
//     FP8 underflow threshold (validated exhaustively for bf16 inputs and on 6e8 random / adversarial
//     fp32 pairs on the CPU); callers fall back to plain division outside that domain;
//   * fp32 -> FP8 is the hardware OCP conversion (round to nearest even) with the wave's FP16_OVFL
//     mode bit set, i.e. saturate-to-finite for finite inputs; NaN is kept as NaN.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define COAT_WAVE 64

namespace coat {

enum Fp8Kind { kE4M3 = 0, kE5M2 = 1 };
enum DType { kF32 = 0, kBF16 = 1, kF16 = 2 };

template <int KIND> struct Fp8Traits;
template <> struct Fp8Traits<kE4M3> { static constexpr float kMax = 448.0f; };
template <> struct Fp8Traits<kE5M2> { static constexpr float kMax = 57344.0f; };

__device__ __forceinline__ float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }

// ------------------------------------------------------------------------------------------------ bf16 / f16
__device__ __forceinline__ float bf16lo(uint32_t w) { return u2f(w << 16); }
__device__ __forceinline__ float bf16hi(uint32_t w) { return u2f(w & 0xFFFF0000u); }

// fp32 -> bf16 bits, round to nearest even (same result as torch's): the gfx950 conversion instruction
// v_cvt_pk_bf16_f32, one VALU operation for two values instead of ten of integer arithmetic.
typedef float coat_f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 coat_bf16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    return __builtin_bit_cast(uint32_t, __builtin_convertvector((coat_f32x2){lo, hi}, coat_bf16x2));
}
__device__ __forceinline__ uint32_t f2bf16(float f) { return pack_bf16x2(f, 0.0f) & 0xFFFFu; }

__device__ __forceinline__ float f16lo(uint32_t w) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xFFFF)); }
__device__ __forceinline__ float f16hi(uint32_t w) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16)); }
__device__ __forceinline__ uint32_t f2f16(float f) { return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f); }

// Streaming (non-temporal) global loads for data that a kernel reads once and no later kernel reads again soon (the
// optimizer state, the logits of the loss): the caches treat such lines as first candidates for replacement.  On 1 GiB
// probes: read 7.1 instead of 6.5 TB/s, copy 6.2-6.6 instead of 5.8-6.2 TB/s; the AdamW step gains 8 %, the cross-entropy
// kernel 6 %.  Not used where a following kernel re-reads the tensor from the cache (the norms lose 16-26 % with it),
// nor for stores (the in-place AdamW update loses 9 % with streaming stores).
typedef uint32_t coat_u4v __attribute__((ext_vector_type(4)));
typedef uint32_t coat_u2v __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint4 ld_stream16(const void* p) {
    const coat_u4v v = __builtin_nontemporal_load((const coat_u4v*)p);
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 ld_stream8(const void* p) {
    const coat_u2v v = __builtin_nontemporal_load((const coat_u2v*)p);
    return make_uint2(v.x, v.y);
}
__device__ __forceinline__ uint32_t ld_stream4(const void* p) { return __builtin_nontemporal_load((const uint32_t*)p); }

// Typed scalar load / store used for scale tensors and ragged tails.
template <int DT> __device__ __forceinline__ float load_as_f32(const void* p, int64_t i) {
    if (DT == kF32) return ((const float*)p)[i];
    uint32_t h = ((const uint16_t*)p)[i];
    return DT == kBF16 ? u2f(h << 16) : f16lo(h);
}
template <int DT> __device__ __forceinline__ void store_from_f32(void* p, int64_t i, float v) {
    if (DT == kF32) ((float*)p)[i] = v;
    else if (DT == kBF16) ((uint16_t*)p)[i] = (uint16_t)f2bf16(v);
    else ((uint16_t*)p)[i] = (uint16_t)f2f16(v);
}
// Scalar load with a run-time dtype (scales, bias): wave-uniform branch.
__device__ __forceinline__ float load_rt_f32(const void* p, int64_t i, int dt) {
    if (dt == kBF16) return u2f((uint32_t)((const uint16_t*)p)[i] << 16);
    if (dt == kF32) return ((const float*)p)[i];
    return f16lo(((const uint16_t*)p)[i]);
}
// The same in two steps, for code that wants several loads in flight before the first conversion (a conversion right
// after its load makes the wave wait for that load before it can issue the next one).
__device__ __forceinline__ uint32_t load_rt_raw(const void* p, int64_t i, int dt) {
    if (dt == kF32) return ((const uint32_t*)p)[i];
    return ((const uint16_t*)p)[i];
}
__device__ __forceinline__ float rt_raw_to_f32(uint32_t raw, int dt) {
    if (dt == kBF16) return u2f(raw << 16);
    if (dt == kF32) return u2f(raw);
    return f16lo(raw);
}
// Round an fp32 value to dtype DT and back (what storing and re-loading would give).
template <int DT> __device__ __forceinline__ float round_to(float v) {
    if (DT == kF32) return v;
    if (DT == kBF16) return u2f(f2bf16(v) << 16);
    return (float)(_Float16)v;
}

// ------------------------------------------------------------------------------------------------ FP8
// The hardware conversion rounds to nearest even and, with MODE.FP16_OVFL = 1, saturates finite
// overflow to the largest finite code (e4m3 0x7E, e5m2 0x7B) instead of producing NaN / inf; NaN stays
// NaN.  (+-inf in gives NaN for e4m3 and +-inf for e5m2.)  Every kernel that emits FP8 calls this first.
__device__ __forceinline__ void enable_fp8_saturation() {
    // s_setreg_b32 hwreg(HW_REG_MODE, 23, 1), 1
    __builtin_amdgcn_s_setreg(1 | (23 << 6) | (0 << 11), 1);
}
// Two fp32 -> two FP8 codes packed into the low (hi=false) or high (hi=true) half of `old`.
template <int KIND> __device__ __forceinline__ uint32_t cvt_pk_fp8(float a, float b, uint32_t old, bool hi) {
    if (KIND == kE4M3) return hi ? __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, true) : __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, false);
    return hi ? __builtin_amdgcn_cvt_pk_bf8_f32(a, b, old, true) : __builtin_amdgcn_cvt_pk_bf8_f32(a, b, old, false);
}
template <int KIND> __device__ __forceinline__ uint32_t cvt4_fp8(float a, float b, float c, float d) {
    uint32_t w = cvt_pk_fp8<KIND>(a, b, 0u, false);
    return cvt_pk_fp8<KIND>(c, d, w, true);
}
// FP8 code (byte `sel` of w) -> fp32.
template <int KIND, int SEL> __device__ __forceinline__ float fp8_to_f32(uint32_t w) {
    if (KIND == kE4M3) return __builtin_amdgcn_cvt_f32_fp8(w, SEL);
    return __builtin_amdgcn_cvt_f32_bf8(w, SEL);
}
// four codes of one dword: two packed conversions (v_cvt_pk_f32_fp8 / _bf8 convert a 16-bit half each)
typedef float coat_f2v __attribute__((ext_vector_type(2)));
template <int KIND> __device__ __forceinline__ void fp8x4_to_f32(uint32_t w, float* o) {
    coat_f2v lo, hi;
    if (KIND == kE4M3) {
        lo = __builtin_amdgcn_cvt_pk_f32_fp8(w, false);
        hi = __builtin_amdgcn_cvt_pk_f32_fp8(w, true);
    } else {
        lo = __builtin_amdgcn_cvt_pk_f32_bf8(w, false);
        hi = __builtin_amdgcn_cvt_pk_f32_bf8(w, true);
    }
    o[0] = lo.x; o[1] = lo.y; o[2] = hi.x; o[3] = hi.y;
}

// ------------------------------------------------------------------------------------------------ exact division
// Correctly rounded t / C for the two FP8 maxima, C in {448, 57344}: reciprocal constant + two FMAs
// (exhaustively checked against IEEE division for every positive normal t with a normal quotient).
template <int KIND> __device__ __forceinline__ float div_by_fp8max(float t) {
    constexpr float C = Fp8Traits<KIND>::kMax;
    constexpr float rc = 1.0f / C;
    float q0 = t * rc;
    float e = fmaf(-q0, C, t);
    return fmaf(e, rc, q0);
}
// Group scale as the reference defines it: (amax + 1e-10) / fp8max, fp32.
template <int KIND> __device__ __forceinline__ float group_scale(float amax) { return div_by_fp8max<KIND>(amax + 1e-10f); }

// x / s given r = 1.0f / s (IEEE).  The sign is forced from x so that -0.0 / s stays -0.0.
__device__ __forceinline__ float div_by_scale(float x, float s, float r) {
    float q0 = x * r;
    float e = fmaf(-q0, s, x);
    float q = fmaf(e, r, q0);
    return u2f((f2u(q) & 0x7FFFFFFFu) | (f2u(x) & 0x80000000u));
}
constexpr float kMinFastDivScale = 0x1p-60f;

// ------------------------------------------------------------------------------------------------ stochastic rounding
// Philox-4x32, 10 rounds, counter (c0, 0, 0, 0), key (k0, k1): first output word.  This is the stream the
// reference draws with tl.rand(seed, offset) (coat/activation/real_quantization/_division.py:107-110):
// key = the 64-bit seed, c0 = the element's linear index.
__device__ __forceinline__ uint32_t philox4x32_10_word0(uint32_t c0, uint32_t k0, uint32_t k1) {
    uint32_t c1 = 0, c2 = 0, c3 = 0;
#pragma unroll
    for (int r = 0; r < 10; r++) {
        const uint64_t pb = (uint64_t)0xCD9E8D57u * c2, pa = (uint64_t)0xD2511F53u * c0;  // one 32x32->64 multiply each
        const uint32_t hi_b = (uint32_t)(pb >> 32), lo_b = (uint32_t)pb;
        const uint32_t hi_a = (uint32_t)(pa >> 32), lo_a = (uint32_t)pa;
        c0 = hi_b ^ c1 ^ k0;
        c2 = hi_a ^ c3 ^ k1;
        c1 = lo_b;
        c3 = lo_a;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    return c0;
}
// Random word -> fp32 in [0, 1) the way Triton's uint_to_uniform_float does: fold the negative half of the
// int32 range onto the non-negative one, convert (round to nearest even), scale by just under 2^-31.
__device__ __forceinline__ float uniform_from_word(uint32_t w) {
    int32_t x = (int32_t)w;
    x = x < 0 ? -x - 1 : x;
    return (float)x * 4.6566127342e-10f;
}
// The reference's _stochastic_rounding (coat/activation/real_quantization/_division.py:130-150): add
// noise * (one FP8 step of q's binade) to |q|, clamp to the binade, keep the sign; the caller then converts with
// round-to-nearest.  Below twice the smallest subnormal the step is the smallest subnormal itself and the
// ceiling 2^m_bit times it; the lower clamp lifts zeros to the smallest subnormal, as the reference does.
template <int KIND> __device__ __forceinline__ float stochastic_perturb(float q, float noise) {
    constexpr float kSubMin = KIND == kE4M3 ? 0x1p-9f : 0x1p-16f;
    constexpr float kSteps = KIND == kE4M3 ? 8.0f : 4.0f;  // 2^m_bit
    const float e = fmaxf(u2f(f2u(q) & 0x7F800000u), kSubMin);
    const bool sub = e == kSubMin;
    const float nz = (e * noise) * (sub ? 1.0f : 1.0f / kSteps);  // division by a power of two, exact either way
    float a = fabsf(q) + nz;
    a = fminf(fmaxf(a, e), (sub ? kSteps : 2.0f) * e);
    return u2f(f2u(a) | (f2u(q) & 0x80000000u));
}

// ------------------------------------------------------------------------------------------------ cross-lane
// DPP controls: quad_perm(1,0,3,2)=0xB1, quad_perm(2,3,0,1)=0x4E, row_half_mirror=0x141, row_mirror=0x140.
template <int CTRL> __device__ __forceinline__ float dpp_f32(float v) {
    return u2f((uint32_t)__builtin_amdgcn_update_dpp(0, (int)f2u(v), CTRL, 0xF, 0xF, true));
}
// lane ^ 16 / lane ^ 32 exchanges through ds_bpermute (no LDS memory is touched).
__device__ __forceinline__ float lane_xor_f32(float v, int mask) {
    int lane = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    return u2f((uint32_t)__builtin_amdgcn_ds_bpermute((lane ^ mask) << 2, (int)f2u(v)));
}
// max over aligned clusters of LANES consecutive lanes (LANES power of two <= 64); result in every lane.
template <int LANES> __device__ __forceinline__ float cluster_max(float v) {
    if (LANES >= 2) v = fmaxf(v, dpp_f32<0xB1>(v));
    if (LANES >= 4) v = fmaxf(v, dpp_f32<0x4E>(v));
    if (LANES >= 8) v = fmaxf(v, dpp_f32<0x141>(v));
    if (LANES >= 16) v = fmaxf(v, dpp_f32<0x140>(v));
    if (LANES >= 32) v = fmaxf(v, lane_xor_f32(v, 16));
    if (LANES >= 64) v = fmaxf(v, lane_xor_f32(v, 32));
    return v;
}
// Same with a run-time (wave-uniform) cluster width.
__device__ __forceinline__ float cluster_max_rt(float v, int lanes) {
    if (lanes >= 2) v = fmaxf(v, dpp_f32<0xB1>(v));
    if (lanes >= 4) v = fmaxf(v, dpp_f32<0x4E>(v));
    if (lanes >= 8) v = fmaxf(v, dpp_f32<0x141>(v));
    if (lanes >= 16) v = fmaxf(v, dpp_f32<0x140>(v));
    if (lanes >= 32) v = fmaxf(v, lane_xor_f32(v, 16));
    if (lanes >= 64) v = fmaxf(v, lane_xor_f32(v, 32));
    return v;
}
template <int LANES> __device__ __forceinline__ float cluster_sum(float v) {
    if (LANES >= 2) v = v + dpp_f32<0xB1>(v);
    if (LANES >= 4) v = v + dpp_f32<0x4E>(v);
    if (LANES >= 8) v = v + dpp_f32<0x141>(v);
    if (LANES >= 16) v = v + dpp_f32<0x140>(v);
    if (LANES >= 32) v = v + lane_xor_f32(v, 16);
    if (LANES >= 64) v = v + lane_xor_f32(v, 32);
    return v;
}

// Order-independent device-wide maximum of non-negative floats (bit pattern order == value order).
// Device-scope atomics on one 128-byte line are carried out one after the other, about 10 ns each on this part: 4096 waves
// that each merge one value into one word keep a 14 us kernel busy for 33 us.  So (i) callers reduce over a block first,
// (ii) the maximum lives in kMaxSlots words that are one line apart (COAT_MAX_WORDS floats in all, zero-initialised by the
// caller): block b merges into slot b % kMaxSlots and a consumer takes the maximum over the slots (measured on the RMSNorm
// statistics kernel, 1024 blocks: 17.9 us with 16 slots on 16 lines, 35 us with 16 slots inside one line, 14.1 us without
// any atomic), and (iii) the atomic is skipped when a read already shows a value that is not smaller: the stored maximum
// only grows, so a stale reading can only cause a redundant atomic, never a lost update.
constexpr int kMaxSlots = 16;
constexpr int kMaxSlotStride = 32;  // floats
__device__ __forceinline__ float* max_slot(float* base) { return base + (blockIdx.x & (kMaxSlots - 1)) * kMaxSlotStride; }
__device__ __forceinline__ float load_max(const float* base) {
    float m = 0.0f;
#pragma unroll
    for (int k = 0; k < kMaxSlots; k++) m = fmaxf(m, base[k * kMaxSlotStride]);
    return m;
}
__device__ __forceinline__ void atomic_max_nonneg(float* addr, float v) {
    const float cur = *(volatile float*)addr;
    if (!(v <= cur)) atomicMax((unsigned int*)addr, f2u(v));
}

// Block-wide (256 threads) version: one lazy atomic per block into the block's slot of `base`.  `smem` holds 4 floats;
// every thread must call.
__device__ __forceinline__ void block_atomic_max_nonneg(float* base, float v, float* smem) {
    v = cluster_max<64>(v);
    if ((threadIdx.x & 63) == 0) smem[threadIdx.x >> 6] = v;
    __syncthreads();
    if (threadIdx.x == 0) atomic_max_nonneg(max_slot(base), fmaxf(fmaxf(smem[0], smem[1]), fmaxf(smem[2], smem[3])));
}

}  // namespace coat
