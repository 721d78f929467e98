// FP8 AdamW step for gfx950: one fused streaming kernel per parameter tensor.
//
// Replaces fp8_adamw_cuda_expand_kernel (Dynamic Range Expansion) and fp8_adamw_cuda_kernel of the
// reference (one element per thread, 128-thread blocks, every thread recomputing the group constants).
//
// Layout: a wave owns 1024 consecutive elements = 8 quantization groups of 128.  Lane l works for group
// l/8; with lam = l%8 it holds, for j = 0..3, the 4 consecutive elements 32*j + 4*lam .. +3 of its group.
// A load instruction therefore reads, per group, one full 128-byte line of fp32 params / grads (16 bytes
// per lane) and one 32-byte piece of FP8 codes; all 16 elements a lane touches share one group, so group
// maxima / minima are 15 in-lane operations plus a 3-step DPP reduction over 8 lanes, and the group
// constants (centre c, exponent k, new scale) are computed once per lane for 16 elements.
//
// Numerics: in the plain (non-expand) step + - * / sqrt are the IEEE fp32 operations of the reference source
// in the same order without FMA contraction, so it is bit-exact against the CPU restatement.  The x^y of the
// expand step is exp2(y * log2(x)) on the hardware v_log_f32 / v_exp_f32 (about 1e-6 relative), with the IEEE
// special cases of powf (y = 0, y = inf, x = 0, x = 1) reproduced explicitly; see k_fp8_adamw_expand.
// The reference's order-dependent zero-skipping minimum is reproduced exactly: when a group holds an
// exact zero the kernel walks the reference's 32-lane shuffle tree, otherwise that tree equals a plain min.
#include <math.h>

#include "coat_device.h"
#include "coat_host.h"

namespace coat {

constexpr int kGroup = 128;
constexpr float kLog2RatioUpperBound = 16.61470984411521f;  // log2(448 * 448 / 2), rounded to fp32
constexpr float kFltMax = 3.402823466e+38f;

struct AdamArgs {
    float beta1, beta2, lr, wd, eps;
    float one_minus_beta1, one_minus_beta2;
    float correction1, correction2_sqrt;  // 1 - beta1^step, sqrt(1 - beta2^step), evaluated on the host
    float expand_min;
    float inv_expand_min;  // 1 / expand_min when expand_min is a power of two (the division is then a multiplication), else 0
};

__device__ __forceinline__ float log2_hw(float x) { return __builtin_amdgcn_logf(x); }
__device__ __forceinline__ float exp2_hw(float x) { return __builtin_amdgcn_exp2f(x); }

// x^y for x >= 0 in the common case 0 < y < inf (x = 0 -> 0 falls out of log2(0) = -inf).
__device__ __forceinline__ float pow_fast(float x, float y) { return exp2_hw(log2_hw(x) * y); }
// Same with the IEEE special cases: pow(x, 0) = 1, pow(1, y) = 1, pow(x, +inf) in {0, 1, inf}.
__device__ __forceinline__ float pow_full(float x, float y) {
    float t = log2_hw(x) * y;
    t = (y == 0.0f || x == 1.0f) ? 0.0f : t;
    return exp2_hw(t);
}

// The reference's combine step for the minimum: skip the partner when it is zero (NaN > 0 is false too).
__device__ __forceinline__ float min_skip_zero(float own, float partner) {
    float a = fabsf(partner);
    return (a > 0.0f) ? fminf(own, a) : own;
}

// Group minimum exactly as thread 0 of the reference block ends up holding it, for a[j][i] = |value| of
// reference thread 32*j + 4*lam + i (FLT_MAX where out of range).  Result valid in the lam == 0 lane.
__device__ __forceinline__ float reference_tree_min(const float (&a)[4][4]) {
    float w[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {  // reference warp j: shuffle offsets 16, 8, 4 move 4, 2, 1 lanes; 2 and 1 stay in-lane
        float s[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float x = a[j][i];
            x = min_skip_zero(x, dpp_f32<0x104>(x));  // row_shl:4  (lane reads lane+4)
            x = min_skip_zero(x, dpp_f32<0x102>(x));  // row_shl:2
            x = min_skip_zero(x, dpp_f32<0x101>(x));  // row_shl:1
            s[i] = x;
        }
        s[0] = min_skip_zero(s[0], s[2]);
        s[1] = min_skip_zero(s[1], s[3]);
        w[j] = min_skip_zero(s[0], s[1]);
    }
    // block level: threads 0..3 hold w[0..3], every other thread holds 1e9; offsets 16, 8, 4 meet only fillers
#pragma unroll
    for (int j = 0; j < 4; j++) w[j] = fminf(w[j], 1e9f);
    float t0 = min_skip_zero(w[0], w[2]);
    float t1 = min_skip_zero(w[1], w[3]);
    return min_skip_zero(t0, t1);
}

// Correctly rounded sqrtf for x = +0 or a normal x >= 2^-96 (also right for +inf and NaN): the hardware approximation is
// within one ulp; the residuals of its two neighbours, each one exact FMA, tell which of the three is the rounded root.
// (The same correction the compiler's sqrtf applies, without the rescaling that only denormal inputs need.)
__device__ __forceinline__ float sqrt_cr_normal(float x) {
    const float s = __builtin_amdgcn_sqrtf(x);
    const float s_dn = u2f(f2u(s) - 1u), s_up = u2f(f2u(s) + 1u);
    const float r_dn = fmaf(-s_dn, s, x), r_up = fmaf(-s_up, s, x);
    float r = r_dn <= 0.0f ? s_dn : s;
    r = r_up > 0.0f ? s_up : r;
    return r;
}

template <int PDT> struct PVec { static constexpr int kBytes = (PDT == kF32) ? 16 : 8; };

template <int PDT> __device__ __forceinline__ void load4(const void* base, int64_t e, int64_t numel, float* o) {
    if (e + 3 < numel) {
        if (PDT == kF32) {
            const uint4 t = ld_stream16((const float*)base + e);
            o[0] = u2f(t.x); o[1] = u2f(t.y); o[2] = u2f(t.z); o[3] = u2f(t.w);
        } else {
            const uint2 t = ld_stream8((const uint16_t*)base + e);
            o[0] = PDT == kBF16 ? bf16lo(t.x) : f16lo(t.x);
            o[1] = PDT == kBF16 ? bf16hi(t.x) : f16hi(t.x);
            o[2] = PDT == kBF16 ? bf16lo(t.y) : f16lo(t.y);
            o[3] = PDT == kBF16 ? bf16hi(t.y) : f16hi(t.y);
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; i++) o[i] = (e + i < numel) ? load_as_f32<PDT>(base, e + i) : 0.0f;
    }
}
template <int PDT> __device__ __forceinline__ void store4(void* base, int64_t e, int64_t numel, const float* v) {
    if (e + 3 < numel) {
        if (PDT == kF32) *(float4*)((float*)base + e) = make_float4(v[0], v[1], v[2], v[3]);
        else if (PDT == kBF16) *(uint2*)((uint16_t*)base + e) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
        else *(uint2*)((uint16_t*)base + e) = make_uint2(f2f16(v[0]) | (f2f16(v[1]) << 16), f2f16(v[2]) | (f2f16(v[3]) << 16));
    } else {
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (e + i < numel) store_from_f32<PDT>(base, e + i, v[i]);
    }
}
__device__ __forceinline__ uint32_t load_codes4(const uint8_t* base, int64_t e, int64_t numel) {
    if (e + 3 < numel) return ld_stream4(base + e);
    uint32_t w = 0;
#pragma unroll
    for (int i = 0; i < 4; i++)
        if (e + i < numel) w |= (uint32_t)base[e + i] << (8 * i);
    return w;
}
__device__ __forceinline__ void store_codes4(uint8_t* base, int64_t e, int64_t numel, uint32_t w) {
    if (e + 3 < numel) *(uint32_t*)(base + e) = w;
    else {
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (e + i < numel) base[e + i] = (uint8_t)(w >> (8 * i));
    }
}

// ------------------------------------------------------------------------------------------------
// Plain (no expansion) step: every operation is the IEEE operation of the reference, bit-exact.
// FULL: all eight groups of the wave are complete (no element or group masking anywhere).
template <int PDT, bool FULL>
__device__ __forceinline__ void adamw_plain_wave(void* __restrict__ params, const void* __restrict__ grads,
                                                 uint8_t* __restrict__ exp_avg, float* __restrict__ scale_m,
                                                 uint8_t* __restrict__ exp_avg_sq, float* __restrict__ scale_v,
                                                 const AdamArgs& A, int64_t numel_in, int64_t ngroups, int64_t wave, int lane) {
    const int lam = lane & 7;
    const int64_t gi = wave * 8 + (lane >> 3);
    const bool gvalid = FULL || gi < ngroups;
    const int64_t gidx = gvalid ? gi : ngroups - 1;  // lanes of absent groups redo the last group, stores masked
    const int64_t e0 = gidx * kGroup + lam * 4;
    const int64_t numel = FULL ? (int64_t)1 << 62 : numel_in;  // FULL: every bounds test folds away
    const int64_t lim = gvalid ? numel : 0;

    float p[4][4], g[4][4];
    uint32_t cm[4], cv[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        load4<PDT>(params, e0 + 32 * j, numel, p[j]);
        load4<PDT>(grads, e0 + 32 * j, numel, g[j]);
        cm[j] = load_codes4(exp_avg, e0 + 32 * j, numel);
        cv[j] = load_codes4(exp_avg_sq, e0 + 32 * j, numel);
    }
    const float sm = scale_m[gidx], sv = scale_v[gidx];
    float m[4][4], v[4][4];
    float mx_m = 0.0f, mx_v = 0.0f;
    uint32_t low_v = 0xFFFFFFFFu;  // smallest second moment other than +0, as bits - 1 (+0 wraps to the largest value)
#pragma unroll
    for (int j = 0; j < 4; j++) {
        float fm[4], fv[4];
        fp8x4_to_f32<kE4M3>(cm[j], fm);
        fp8x4_to_f32<kE4M3>(cv[j], fv);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const bool ok = FULL || e0 + 32 * j + i < lim;
            float em = fm[i] * sm, ev = fv[i] * sv;
            const float gr = g[j][i];
            em = A.beta1 * em + A.one_minus_beta1 * gr;
            ev = A.beta2 * ev + (A.one_minus_beta2 * gr) * gr;
            m[j][i] = em;
            v[j][i] = ev;
            low_v = min(low_v, f2u(ev) - 1u);
            mx_m = fmaxf(mx_m, ok ? fabsf(em) : 0.0f);
            mx_v = fmaxf(mx_v, ok ? fabsf(ev) : 0.0f);
        }
    }
    // sqrt(v) / c2: the correctly rounded square root from the hardware approximation and one correction step, and the
    // quotient through the reciprocal of the (wave-uniform) divisor with one correction step, which is the IEEE quotient
    // (div_by_scale; c2 = sqrt(1 - beta2^step) lies in (0, 1]).  Together they take a third of the instructions of the
    // compiler's sqrtf and division.  Anything outside their domain (denormal, infinite or NaN second moments, a
    // degenerate c2) takes the compiler's sequences, decided once per wave.
    const float c2 = A.correction2_sqrt;
    // every second moment is +0 or lies in [2^-96, inf): the domain of sqrt_cr_normal (negative values and NaNs have the
    // sign bit or an all-ones exponent, which also puts them above the upper bound)
    const bool plain_range = low_v >= f2u(0x1p-96f) - 1u && mx_v < INFINITY;
    const bool fast = __all(plain_range) && c2 >= 0x1p-20f && c2 <= 1.0f;
    if (fast) {
        const float rc2 = 1.0f / c2;
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float pr = p[j][i];
                const float sq = sqrt_cr_normal(v[j][i]);
                const float denom = (div_by_scale(sq, c2, rc2) + A.eps) * A.correction1;
                const float update = (m[j][i] / denom) + (A.wd * pr);
                p[j][i] = pr - (A.lr * update);
            }
    } else {
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const float pr = p[j][i];
                const float denom = (sqrtf(v[j][i]) / c2 + A.eps) * A.correction1;
                const float update = (m[j][i] / denom) + (A.wd * pr);
                p[j][i] = pr - (A.lr * update);
            }
    }
#pragma unroll
    for (int j = 0; j < 4; j++) store4<PDT>(params, e0 + 32 * j, lim, p[j]);
    mx_m = cluster_max<8>(mx_m);
    mx_v = cluster_max<8>(mx_v);
    // "+ 1e-20" is a double-precision add narrowed to float in the reference
    const float snew_m = (float)((double)mx_m + 1e-20) / 448.0f;
    const float snew_v = (float)((double)mx_v + 1e-20) / 448.0f;
    // m / s and v / s: through the reciprocal with one correction step, which gives the same FP8 code as the IEEE
    // quotient (every FP8 rounding boundary is a quotient the correction reproduces exactly); tiny scales, where the
    // reciprocal would overflow, take the plain division (wave-uniform choice)
    if (__all(snew_m >= kMinFastDivScale && snew_v >= kMinFastDivScale)) {
        const float rm = 1.0f / snew_m, rv = 1.0f / snew_v;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            store_codes4(exp_avg, e0 + 32 * j, lim,
                         cvt4_fp8<kE4M3>(div_by_scale(m[j][0], snew_m, rm), div_by_scale(m[j][1], snew_m, rm),
                                         div_by_scale(m[j][2], snew_m, rm), div_by_scale(m[j][3], snew_m, rm)));
            store_codes4(exp_avg_sq, e0 + 32 * j, lim,
                         cvt4_fp8<kE4M3>(div_by_scale(v[j][0], snew_v, rv), div_by_scale(v[j][1], snew_v, rv),
                                         div_by_scale(v[j][2], snew_v, rv), div_by_scale(v[j][3], snew_v, rv)));
        }
    } else {
#pragma unroll
        for (int j = 0; j < 4; j++) {
            store_codes4(exp_avg, e0 + 32 * j, lim,
                         cvt4_fp8<kE4M3>(m[j][0] / snew_m, m[j][1] / snew_m, m[j][2] / snew_m, m[j][3] / snew_m));
            store_codes4(exp_avg_sq, e0 + 32 * j, lim,
                         cvt4_fp8<kE4M3>(v[j][0] / snew_v, v[j][1] / snew_v, v[j][2] / snew_v, v[j][3] / snew_v));
        }
    }
    if (gvalid && lam == 0) {
        scale_m[gi] = snew_m;
        scale_v[gi] = snew_v;
    }
}

template <int PDT>
__global__ __launch_bounds__(256) void k_fp8_adamw_plain(void* __restrict__ params, const void* __restrict__ grads,
                                                          uint8_t* __restrict__ exp_avg, float* __restrict__ scale_m,
                                                          uint8_t* __restrict__ exp_avg_sq, float* __restrict__ scale_v,
                                                          AdamArgs A, int64_t numel, int64_t ngroups) {
    enable_fp8_saturation();
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (wave * 8 >= ngroups) return;  // whole wave out of range (wave-uniform)
    if ((wave * 8 + 8) * kGroup <= numel)
        adamw_plain_wave<PDT, true>(params, grads, exp_avg, scale_m, exp_avg_sq, scale_v, A, numel, ngroups, wave, lane);
    else
        adamw_plain_wave<PDT, false>(params, grads, exp_avg, scale_m, exp_avg_sq, scale_v, A, numel, ngroups, wave, lane);
}

// ------------------------------------------------------------------------------------------------
// Expand step.  x^y is exp2(y * log2 x) on the hardware units; the arguments of log2 are kept close to 1
// (code*s and |m|/c', both within [1/317, 317]) so that the absolute error of y*log2(x) stays ~1e-6 whatever
// the exponent, and the division by the new scale is folded into the exponent:
//   dequantize   m = sign * exp2(log2|code * s| * (1/k)) * c
//   requantize   m'/s' = sign * exp2(log2(|m| * (1/c')) * k' - log2(s'))
// sqrt and the reciprocal of the Adam denominator are the hardware approximations (1 ulp), FMAs are used
// freely; none of this is visible next to the 1e-6 of the hardware log2 / exp2.  Groups whose exponent is 0 or inf (all values
// equal, or an infinite max/min ratio) take the step-by-step path with the IEEE special cases of powf.
struct GroupIn {  // per-group constants of the incoming state
    float sm, sv, invk_m, invk_v, c_m, c_v;
};

template <int PDT, bool FULL>
__device__ __forceinline__ void adamw_expand_wave(void* __restrict__ params, const void* __restrict__ grads,
                                                  uint8_t* __restrict__ exp_avg, float* __restrict__ scale_m,
                                                  float* __restrict__ expand_m, float* __restrict__ sqrtmm_m,
                                                  uint8_t* __restrict__ exp_avg_sq, float* __restrict__ scale_v,
                                                  float* __restrict__ expand_v, float* __restrict__ sqrtmm_v,
                                                  const AdamArgs& A, int64_t numel, int64_t ngroups, int64_t wave,
                                                  int lane) {
    const int lam = lane & 7;
    const int64_t gi = wave * 8 + (lane >> 3);
    const bool gvalid = FULL || gi < ngroups;
    const int64_t gidx = gvalid ? gi : ngroups - 1;
    const int64_t e0 = gidx * kGroup + lam * 4;
    const int64_t lim = gvalid ? numel : 0;

    float p[4][4], g[4][4];
    uint32_t cm[4], cv[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
        load4<PDT>(params, e0 + 32 * j, FULL ? (int64_t)1 << 62 : numel, p[j]);
        load4<PDT>(grads, e0 + 32 * j, FULL ? (int64_t)1 << 62 : numel, g[j]);
        cm[j] = load_codes4(exp_avg, e0 + 32 * j, FULL ? (int64_t)1 << 62 : numel);
        cv[j] = load_codes4(exp_avg_sq, e0 + 32 * j, FULL ? (int64_t)1 << 62 : numel);
    }
    GroupIn G;
    G.sm = scale_m[gidx];
    G.sv = scale_v[gidx];
    G.invk_m = 1 / expand_m[gidx];
    G.invk_v = 1 / expand_v[gidx];
    G.c_m = sqrtmm_m[gidx];
    G.c_v = sqrtmm_v[gidx];
    // exponents outside (0, inf) need the special cases of powf; decided once per wave
    const bool odd_in = __builtin_amdgcn_ballot_w64(!(G.invk_m > 0.0f && G.invk_m < INFINITY) ||
                                                    !(G.invk_v > 0.0f && G.invk_v < INFINITY)) != 0;
    const float inv_c2 = 1.0f / A.correction2_sqrt;

    float m[4][4], v[4][4];
    float mx_m = 0.0f, mx_v = 0.0f, mn_m = kFltMax, mn_v = kFltMax;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        float fm[4], fv[4];
        fp8x4_to_f32<kE4M3>(cm[j], fm);
        fp8x4_to_f32<kE4M3>(cv[j], fv);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const bool ok = FULL || (e0 + 32 * j + i < lim);
            float em, ev;
            if (!odd_in) {
                em = copysignf(exp2_hw(log2_hw(fabsf(fm[i] * G.sm)) * G.invk_m) * G.c_m, fm[i]);
                ev = exp2_hw(log2_hw(fv[i] * G.sv) * G.invk_v) * G.c_v;
            } else {
                em = fm[i] * G.sm;
                ev = fv[i] * G.sv;
                em = copysignf(pow_full(fabsf(em), G.invk_m) * G.c_m, em);
                ev = pow_full(ev, G.invk_v) * G.c_v;
            }
            const float gr = g[j][i], pr = p[j][i];
            em = fmaf(A.beta1, em, A.one_minus_beta1 * gr);
            ev = fmaf(A.beta2, ev, (A.one_minus_beta2 * gr) * gr);
            const float denom = fmaf(__builtin_amdgcn_sqrtf(ev), inv_c2, A.eps) * A.correction1;
            const float update = fmaf(em, __builtin_amdgcn_rcpf(denom), A.wd * pr);
            p[j][i] = fmaf(-A.lr, update, pr);
            m[j][i] = em;
            v[j][i] = ev;
            const float am = fabsf(em), av = fabsf(ev);
            mx_m = fmaxf(mx_m, ok ? am : 0.0f);
            mx_v = fmaxf(mx_v, ok ? av : 0.0f);
            mn_m = fminf(mn_m, ok ? am : kFltMax);
            mn_v = fminf(mn_v, ok ? av : kFltMax);
        }
    }
#pragma unroll
    for (int j = 0; j < 4; j++) store4<PDT>(params, e0 + 32 * j, FULL ? (int64_t)1 << 62 : lim, p[j]);

    // ---- group statistics (8 lanes per group)
    mx_m = cluster_max<8>(mx_m);
    mx_v = cluster_max<8>(mx_v);
    mn_m = -cluster_max<8>(-mn_m);
    mn_v = -cluster_max<8>(-mn_v);
    // an exact zero (or a NaN, which fmin drops) anywhere in the wave: walk the reference's shuffle tree
    bool suspicious = !(mn_m > 0.0f) || !(mn_v > 0.0f) || !(mx_m == mx_m) || !(mx_v == mx_v);
    if (__builtin_amdgcn_ballot_w64(suspicious) != 0) {
        float a[4][4], b[4][4];
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const bool ok = FULL || (e0 + 32 * j + i < lim);
                a[j][i] = ok ? fabsf(m[j][i]) : kFltMax;
                b[j][i] = ok ? fabsf(v[j][i]) : kFltMax;
            }
        mn_m = reference_tree_min(a);
        mn_v = reference_tree_min(b);
        mn_m = u2f((uint32_t)__builtin_amdgcn_ds_bpermute((lane & ~7) << 2, (int)f2u(mn_m)));
        mn_v = u2f((uint32_t)__builtin_amdgcn_ds_bpermute((lane & ~7) << 2, (int)f2u(mn_v)));
    } else {
        // all values positive: the tree is a plain minimum, capped by the 1e9 filler of its block level
        mn_m = fminf(mn_m, 1e9f);
        mn_v = fminf(mn_v, 1e9f);
    }
    // "+ 1e-30" is a double-precision add narrowed to float in the reference
    const float Mx_m = (float)((double)mx_m + 1e-30), Mn_m = (float)((double)mn_m + 1e-30);
    const float Mx_v = (float)((double)mx_v + 1e-30), Mn_v = (float)((double)mn_v + 1e-30);
    const float ratio_m = Mx_m / Mn_m, ratio_v = Mx_v / Mn_v;
    // Group constants.  The same IEEE results with fewer instructions where the operands allow it (decided once per wave;
    // these constants are a quarter of the kernel's instructions, and every lane of a group computes them):
    //   sqrtf          hardware approximation + one correction step (sqrt_cr_normal: normal operands >= 2^-96)
    //   x / expand_min multiplication by the reciprocal when expand_min is a power of two (exact)
    //   x / 448        reciprocal constant + two FMAs (div_by_fp8max: finite x with a normal quotient)
    float cn_m, cn_v, k_m, k_v;
    const bool easy = __all(Mn_m >= 0x1p-96f && Mn_v >= 0x1p-96f && Mx_m < INFINITY && Mx_v < INFINITY) && A.inv_expand_min > 0.0f;
    if (easy) {
        cn_m = sqrt_cr_normal(Mx_m) * sqrt_cr_normal(Mn_m);
        cn_v = sqrt_cr_normal(Mx_v) * sqrt_cr_normal(Mn_v);
        k_m = floorf((kLog2RatioUpperBound / log2_hw(ratio_m)) * A.expand_min) * A.inv_expand_min;
        k_v = floorf((kLog2RatioUpperBound / log2_hw(ratio_v)) * A.expand_min) * A.inv_expand_min;
    } else {
        cn_m = sqrtf(Mx_m) * sqrtf(Mn_m);
        cn_v = sqrtf(Mx_v) * sqrtf(Mn_v);
        k_m = floorf((kLog2RatioUpperBound / log2_hw(ratio_m)) * A.expand_min) / A.expand_min;
        k_v = floorf((kLog2RatioUpperBound / log2_hw(ratio_v)) * A.expand_min) / A.expand_min;
    }
    const float pw_m = pow_full(Mx_m / cn_m, k_m), pw_v = pow_full(Mx_v / cn_v, k_v);
    float snew_m, snew_v;
    if (__all(pw_m >= 0x1p-100f && pw_m < INFINITY && pw_v >= 0x1p-100f && pw_v < INFINITY)) {
        snew_m = div_by_fp8max<kE4M3>(pw_m);
        snew_v = div_by_fp8max<kE4M3>(pw_v);
    } else {
        snew_m = pw_m / 448.0f;
        snew_v = pw_v / 448.0f;
    }
    const bool odd_out = __builtin_amdgcn_ballot_w64(!(k_m > 0.0f && k_m < INFINITY) || !(k_v > 0.0f && k_v < INFINITY) ||
                                                     !(snew_m > 0.0f && snew_m < INFINITY) ||
                                                     !(snew_v > 0.0f && snew_v < INFINITY)) != 0;
    const float rcn_m = 1.0f / cn_m, rcn_v = 1.0f / cn_v;
    const float qoff_m = -log2_hw(snew_m), qoff_v = -log2_hw(snew_v);

    // ---- requantize
#pragma unroll
    for (int j = 0; j < 4; j++) {
        float qm[4], qv[4];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float em = m[j][i], ev = v[j][i];
            if (!odd_out) {
                qm[i] = copysignf(exp2_hw(fmaf(log2_hw(fabsf(em) * rcn_m), k_m, qoff_m)), em);
                qv[i] = exp2_hw(fmaf(log2_hw(ev * rcn_v), k_v, qoff_v));
            } else {
                qm[i] = copysignf(pow_full(fabsf(em) / cn_m, k_m), em) / snew_m;
                qv[i] = pow_full(ev / cn_v, k_v) / snew_v;
            }
        }
        store_codes4(exp_avg, e0 + 32 * j, FULL ? (int64_t)1 << 62 : lim, cvt4_fp8<kE4M3>(qm[0], qm[1], qm[2], qm[3]));
        store_codes4(exp_avg_sq, e0 + 32 * j, FULL ? (int64_t)1 << 62 : lim, cvt4_fp8<kE4M3>(qv[0], qv[1], qv[2], qv[3]));
    }
    if (gvalid && lam == 0) {
        scale_m[gi] = snew_m;
        scale_v[gi] = snew_v;
        expand_m[gi] = k_m;
        expand_v[gi] = k_v;
        sqrtmm_m[gi] = cn_m;
        sqrtmm_v[gi] = cn_v;
    }
}

template <int PDT>
__global__ __launch_bounds__(256) void k_fp8_adamw_expand(void* __restrict__ params, const void* __restrict__ grads,
                                                           uint8_t* __restrict__ exp_avg, float* __restrict__ scale_m,
                                                           float* __restrict__ expand_m, float* __restrict__ sqrtmm_m,
                                                           uint8_t* __restrict__ exp_avg_sq, float* __restrict__ scale_v,
                                                           float* __restrict__ expand_v, float* __restrict__ sqrtmm_v,
                                                           AdamArgs A, int64_t numel, int64_t ngroups) {
    enable_fp8_saturation();
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (wave * 8 >= ngroups) return;  // whole wave out of range (wave-uniform)
    if ((wave * 8 + 8) * kGroup <= numel)
        adamw_expand_wave<PDT, true>(params, grads, exp_avg, scale_m, expand_m, sqrtmm_m, exp_avg_sq, scale_v, expand_v,
                                     sqrtmm_v, A, numel, ngroups, wave, lane);
    else
        adamw_expand_wave<PDT, false>(params, grads, exp_avg, scale_m, expand_m, sqrtmm_m, exp_avg_sq, scale_v, expand_v,
                                      sqrtmm_v, A, numel, ngroups, wave, lane);
}

// ------------------------------------------------------------------------------------------------
// Several tensors in one launch (the reference's optimizer loops over the parameters and launches once per parameter,
// coat/optimizer/fp8_adamw.py:419-515; a model's many small tensors, norm weights and biases, then cost a launch each for a
// few microseconds of work).  The records of up to kAdamMultiMax tensors travel in the kernel arguments; a block finds
// its tensor from the table of first block indices and then runs the very wave routine of the single-tensor kernels, so
// every tensor's result is bit-identical to its own launch.
constexpr int kAdamMultiMax = 32;
struct AdamMultiTensor {
    void* params;
    const void* grads;
    uint8_t* exp_avg;
    float *scale_m, *expand_m, *sqrtmm_m;
    uint8_t* exp_avg_sq;
    float *scale_v, *expand_v, *sqrtmm_v;
    int64_t numel;
};
struct AdamMultiArgs {
    AdamMultiTensor t[kAdamMultiMax];
    unsigned first_block[kAdamMultiMax + 1];  // first_block[count] = grid size
    int count;
};

template <int PDT, bool EXPAND>
__global__ __launch_bounds__(256) void k_fp8_adamw_multi(AdamMultiArgs M, AdamArgs A) {
    enable_fp8_saturation();
    int ti = 0;  // the last tensor whose first block is not after this one (block-uniform, scalar registers)
    for (int i = 1; i < M.count; i++)
        if (blockIdx.x >= M.first_block[i]) ti = i;
    const AdamMultiTensor& T = M.t[ti];
    const int64_t numel = T.numel, ngroups = (numel + kGroup - 1) / kGroup;
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)(blockIdx.x - M.first_block[ti]) * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    if (wave * 8 >= ngroups) return;
    const bool full = (wave * 8 + 8) * kGroup <= numel;
    if (EXPAND) {
        if (full)
            adamw_expand_wave<PDT, true>(T.params, T.grads, T.exp_avg, T.scale_m, T.expand_m, T.sqrtmm_m, T.exp_avg_sq, T.scale_v,
                                         T.expand_v, T.sqrtmm_v, A, numel, ngroups, wave, lane);
        else
            adamw_expand_wave<PDT, false>(T.params, T.grads, T.exp_avg, T.scale_m, T.expand_m, T.sqrtmm_m, T.exp_avg_sq, T.scale_v,
                                          T.expand_v, T.sqrtmm_v, A, numel, ngroups, wave, lane);
    } else {
        if (full)
            adamw_plain_wave<PDT, true>(T.params, T.grads, T.exp_avg, T.scale_m, T.exp_avg_sq, T.scale_v, A, numel, ngroups, wave, lane);
        else
            adamw_plain_wave<PDT, false>(T.params, T.grads, T.exp_avg, T.scale_m, T.exp_avg_sq, T.scale_v, A, numel, ngroups, wave, lane);
    }
}

}  // namespace coat

using namespace coat;

static AdamArgs adam_args(float beta1, float beta2, float lr, float wd, float eps, int step, int expand_min) {
    AdamArgs A;
    A.beta1 = beta1; A.beta2 = beta2; A.lr = lr; A.wd = wd; A.eps = eps;
    A.one_minus_beta1 = 1 - beta1;
    A.one_minus_beta2 = 1 - beta2;
    // correctly rounded powf(beta, step): double pow rounded once
    A.correction1 = 1.0f - (float)pow((double)beta1, (double)(float)step);
    A.correction2_sqrt = sqrtf(1.0f - (float)pow((double)beta2, (double)(float)step));
    A.expand_min = (float)expand_min;
    A.inv_expand_min = (expand_min > 0 && (expand_min & (expand_min - 1)) == 0) ? 1.0f / (float)expand_min : 0.0f;
    return A;
}

static int adamw_common(void* params, const void* grads, int p_dtype, void* exp_avg, float* scale_m, float* expand_m,
                        float* sqrtmm_m, void* exp_avg_sq, float* scale_v, float* expand_v, float* sqrtmm_v,
                        float beta1, float beta2, float lr, float wd, float eps, int step, int qgroup_size,
                        int expand_min, bool expand, int64_t numel, int64_t n_scale, void* stream) {
    if (qgroup_size != kGroup) return COAT_EQGROUP;  // "Only Support 128 per-group quantization currently"
    if (numel < 0) return COAT_EINVAL;
    const int64_t ngroups = (numel + kGroup - 1) / kGroup;
    if (n_scale != ngroups) return COAT_ESHAPE;  // AT_ASSERTM(grid_dim == scale_exp_avg.numel())
    if (numel == 0) return COAT_OK;
    if (!params || !grads || !exp_avg || !exp_avg_sq || !scale_m || !scale_v) return COAT_EINVAL;
    if (expand && (!expand_m || !expand_v || !sqrtmm_m || !sqrtmm_v)) return COAT_EINVAL;
    if (!coat_aligned16(params) || !coat_aligned16(grads) || !coat_aligned16(exp_avg) || !coat_aligned16(exp_avg_sq))
        return COAT_EALIGN;
    const AdamArgs A = adam_args(beta1, beta2, lr, wd, eps, step, expand_min);
    const int64_t waves = (ngroups + 7) / 8;
    const int64_t blocks = (waves + 3) / 4;
    hipStream_t st = (hipStream_t)stream;
#define LAUNCH(PDT)                                                                                                   \
    if (expand)                                                                                                       \
        hipLaunchKernelGGL((k_fp8_adamw_expand<PDT>), dim3((unsigned)blocks), dim3(256), 0, st, params, grads,        \
                           (uint8_t*)exp_avg, scale_m, expand_m, sqrtmm_m, (uint8_t*)exp_avg_sq, scale_v, expand_v,   \
                           sqrtmm_v, A, numel, ngroups);                                                              \
    else                                                                                                              \
        hipLaunchKernelGGL((k_fp8_adamw_plain<PDT>), dim3((unsigned)blocks), dim3(256), 0, st, params, grads,         \
                           (uint8_t*)exp_avg, scale_m, (uint8_t*)exp_avg_sq, scale_v, A, numel, ngroups);
    switch (p_dtype) {
        case COAT_F32: LAUNCH(kF32); break;
        case COAT_BF16: LAUNCH(kBF16); break;
        case COAT_F16: LAUNCH(kF16); break;
        default: return COAT_EDTYPE;
    }
#undef LAUNCH
    return coat_launch_status();
}

extern "C" int coat_fp8_adamw_expand_step(void* params, const void* grads, int p_dtype, void* exp_avg,
                                          float* scale_exp_avg, float* expand_exp_avg, float* sqrtminmax_exp_avg,
                                          void* exp_avg_sq, float* scale_exp_avg_sq, float* expand_exp_avg_sq,
                                          float* sqrtminmax_exp_avg_sq, float beta1, float beta2, float lr, float wd,
                                          float eps, int step, int qgroup_size, int expand_min, int64_t numel,
                                          int64_t n_scale, void* stream) {
    return adamw_common(params, grads, p_dtype, exp_avg, scale_exp_avg, expand_exp_avg, sqrtminmax_exp_avg, exp_avg_sq,
                        scale_exp_avg_sq, expand_exp_avg_sq, sqrtminmax_exp_avg_sq, beta1, beta2, lr, wd, eps, step,
                        qgroup_size, expand_min, true, numel, n_scale, stream);
}

extern "C" int coat_fp8_adamw_step(void* params, const void* grads, int p_dtype, void* exp_avg, float* scale_exp_avg,
                                   void* exp_avg_sq, float* scale_exp_avg_sq, float beta1, float beta2, float lr,
                                   float wd, float eps, int step, int qgroup_size, int64_t numel, int64_t n_scale,
                                   void* stream) {
    return adamw_common(params, grads, p_dtype, exp_avg, scale_exp_avg, nullptr, nullptr, exp_avg_sq, scale_exp_avg_sq,
                        nullptr, nullptr, beta1, beta2, lr, wd, eps, step, qgroup_size, 0, false, numel, n_scale, stream);
}

// Host side of the multi-tensor launches: validates every tensor like the single-tensor entry points, then launches the
// tensors in chunks of kAdamMultiMax (and of fewer than 2^31 blocks).
static int adamw_multi(int count, void* const* params, const void* const* grads, int p_dtype, void* const* exp_avg,
                       float* const* scale_m, float* const* expand_m, float* const* sqrtmm_m, void* const* exp_avg_sq,
                       float* const* scale_v, float* const* expand_v, float* const* sqrtmm_v, const int64_t* numel,
                       const int64_t* n_scale, float beta1, float beta2, float lr, float wd, float eps, int step,
                       int qgroup_size, int expand_min, bool expand, void* stream) {
    if (qgroup_size != kGroup) return COAT_EQGROUP;
    if (count < 0) return COAT_EINVAL;
    if (count == 0) return COAT_OK;
    if (!params || !grads || !exp_avg || !exp_avg_sq || !scale_m || !scale_v || !numel || !n_scale) return COAT_EINVAL;
    if (expand && (!expand_m || !expand_v || !sqrtmm_m || !sqrtmm_v)) return COAT_EINVAL;
    if (p_dtype != COAT_F32 && p_dtype != COAT_BF16 && p_dtype != COAT_F16) return COAT_EDTYPE;
    for (int i = 0; i < count; i++) {  // everything is checked before the first launch
        if (numel[i] < 0) return COAT_EINVAL;
        if (n_scale[i] != (numel[i] + kGroup - 1) / kGroup) return COAT_ESHAPE;
        if (numel[i] == 0) continue;
        if (!params[i] || !grads[i] || !exp_avg[i] || !exp_avg_sq[i] || !scale_m[i] || !scale_v[i]) return COAT_EINVAL;
        if (expand && (!expand_m[i] || !expand_v[i] || !sqrtmm_m[i] || !sqrtmm_v[i])) return COAT_EINVAL;
        if (!coat_aligned16(params[i]) || !coat_aligned16(grads[i]) || !coat_aligned16(exp_avg[i]) || !coat_aligned16(exp_avg_sq[i]))
            return COAT_EALIGN;
    }
    const AdamArgs A = adam_args(beta1, beta2, lr, wd, eps, step, expand_min);
    hipStream_t st = (hipStream_t)stream;
    AdamMultiArgs M;
    int i = 0;
    while (i < count) {
        M.count = 0;
        uint64_t blocks = 0;
        for (; i < count && M.count < kAdamMultiMax; i++) {
            if (numel[i] == 0) continue;
            const int64_t ngroups = (numel[i] + kGroup - 1) / kGroup;
            const uint64_t b = (uint64_t)((ngroups + 31) / 32);  // 4 waves of 8 groups per block
            if (blocks + b > 0x7fffffffull) {
                if (M.count == 0) return COAT_ESHAPE;  // one tensor beyond 2^31 blocks (2^43 elements)
                break;
            }
            AdamMultiTensor& T = M.t[M.count];
            T.params = params[i]; T.grads = grads[i]; T.exp_avg = (uint8_t*)exp_avg[i]; T.scale_m = scale_m[i];
            T.expand_m = expand ? expand_m[i] : nullptr; T.sqrtmm_m = expand ? sqrtmm_m[i] : nullptr;
            T.exp_avg_sq = (uint8_t*)exp_avg_sq[i]; T.scale_v = scale_v[i];
            T.expand_v = expand ? expand_v[i] : nullptr; T.sqrtmm_v = expand ? sqrtmm_v[i] : nullptr;
            T.numel = numel[i];
            M.first_block[M.count++] = (unsigned)blocks;
            blocks += b;
        }
        if (M.count == 0) break;  // only empty tensors were left
        M.first_block[M.count] = (unsigned)blocks;
#define LAUNCH_MULTI(PDT)                                                                                             \
    if (expand) hipLaunchKernelGGL((k_fp8_adamw_multi<PDT, true>), dim3((unsigned)blocks), dim3(256), 0, st, M, A);   \
    else hipLaunchKernelGGL((k_fp8_adamw_multi<PDT, false>), dim3((unsigned)blocks), dim3(256), 0, st, M, A);
        switch (p_dtype) {
            case COAT_F32: LAUNCH_MULTI(kF32); break;
            case COAT_BF16: LAUNCH_MULTI(kBF16); break;
            default: LAUNCH_MULTI(kF16); break;
        }
#undef LAUNCH_MULTI
        const int rc = coat_launch_status();
        if (rc != COAT_OK) return rc;
    }
    return COAT_OK;
}

extern "C" int coat_fp8_adamw_expand_step_multi(int count, void* const* params, const void* const* grads, int p_dtype,
                                                void* const* exp_avg, float* const* scale_exp_avg,
                                                float* const* expand_exp_avg, float* const* sqrtminmax_exp_avg,
                                                void* const* exp_avg_sq, float* const* scale_exp_avg_sq,
                                                float* const* expand_exp_avg_sq, float* const* sqrtminmax_exp_avg_sq,
                                                const int64_t* numel, const int64_t* n_scale, float beta1, float beta2,
                                                float lr, float wd, float eps, int step, int qgroup_size, int expand_min,
                                                void* stream) {
    return adamw_multi(count, params, grads, p_dtype, exp_avg, scale_exp_avg, expand_exp_avg, sqrtminmax_exp_avg, exp_avg_sq,
                       scale_exp_avg_sq, expand_exp_avg_sq, sqrtminmax_exp_avg_sq, numel, n_scale, beta1, beta2, lr, wd, eps,
                       step, qgroup_size, expand_min, true, stream);
}

extern "C" int coat_fp8_adamw_step_multi(int count, void* const* params, const void* const* grads, int p_dtype,
                                         void* const* exp_avg, float* const* scale_exp_avg, void* const* exp_avg_sq,
                                         float* const* scale_exp_avg_sq, const int64_t* numel, const int64_t* n_scale,
                                         float beta1, float beta2, float lr, float wd, float eps, int step, int qgroup_size,
                                         void* stream) {
    return adamw_multi(count, params, grads, p_dtype, exp_avg, scale_exp_avg, nullptr, nullptr, exp_avg_sq, scale_exp_avg_sq,
                       nullptr, nullptr, numel, n_scale, beta1, beta2, lr, wd, eps, step, qgroup_size, 0, false, stream);
}
