/* Plain-C restatement of the reference's two FP8 AdamW CUDA kernels.  TEST INFRASTRUCTURE ONLY.
 *
 * Follows, statement by statement,
 *   coat/optimizer/kernels/fp8_adamw_expand_cuda_kernel.cu:20-203   (Dynamic Range Expansion)
 *   coat/optimizer/kernels/fp8_adamw_cuda_kernel.cu:20-125          (plain per-group FP8 state)
 * One CUDA block of 128 threads (= one quantization group, :222-223) becomes one iteration of
 * the group loop below; the two-level __shfl_down reduction is emulated lane by lane so that the
 * order-dependent "skip zeros" minimum (:95-101, :130-136) gives the value thread 0 would hold.
 *
 * Arithmetic conventions (where the CUDA source leaves the bits to the compiler/library):
 *   - every + - * / is a separately rounded IEEE fp32 operation (no FMA contraction; nvcc may
 *     contract, which is one reason the reference's own test tolerance is rtol 1e-4);
 *   - powf / log2f are the correctly rounded functions, evaluated as the double-precision libm
 *     function rounded once to float (CUDA documents powf <= 4 ulp, log2f <= 1 ulp);
 *   - sqrtf and / are correctly rounded (nvcc defaults -prec-sqrt=true -prec-div=true);
 *   - "x + 1e-30" / "x + 1e-20" add a double literal, so the sum is formed in double and then
 *     narrowed to float (QUANT_MIN_VAL, :15 and :154-157);
 *   - float -> e4m3 is round-to-nearest-even with saturation to +-448, NaN -> 0x7F
 *     (cuda_fp8.h: __nv_fp8_e4m3(float) converts with __NV_SATFINITE).
 *
 * Pins: tests/test_oracle_adamw.py (closed-form AdamW from tests/test_fp8_adamw_expand.py:111-131
 * and nvcc_qoptim.cu:39-58; the reference test's search definition of the exponent k, :146-148;
 * DRE invariants; k=1,c=1 reduces to the plain kernel; fresh state step 1 == torch.optim.AdamW; the plain
 * step's parameters, codes and scales bit-identical over six steps to the same kernel written with whole-tensor
 * torch operations and torch's own float -> e4m3 cast).
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off -shared -fPIC).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#define QGROUP 128
#define WARP 32

/* ---------------------------------------------------------------- e4m3fn codec (integer arithmetic) */
static float e4m3_decode(uint8_t c) {
    int e = (c >> 3) & 0xF, m = c & 7;
    float v;
    if ((c & 0x7F) == 0x7F) return NAN;
    v = e == 0 ? ldexpf((float)m / 8.0f, -6) : ldexpf(1.0f + (float)m / 8.0f, e - 7);
    return (c & 0x80) ? -v : v;
}

static uint8_t e4m3_encode(float x) {
    uint32_t bits;
    memcpy(&bits, &x, 4);
    uint32_t sign = (bits >> 24) & 0x80, mag = bits & 0x7FFFFFFFu;
    if (mag > 0x7F800000u) return (uint8_t)(sign | 0x7F);
    int e32 = (int)(mag >> 23);
    uint32_t sig = e32 == 0 ? (mag & 0x7FFFFF) : ((mag & 0x7FFFFF) | 0x800000);
    int e_t = (e32 == 0 ? 1 : e32) - 127 + 7;
    int shift = e_t >= 1 ? 20 : 20 + (1 - e_t);
    if (shift > 31) return (uint8_t)sign; /* below half of the smallest subnormal */
    uint32_t q = sig >> shift, rem = sig & ((1u << shift) - 1), half = 1u << (shift - 1);
    if (rem > half || (rem == half && (q & 1))) q++;
    uint32_t code = e_t >= 1 ? (((uint32_t)(e_t - 1)) << 3) + q : q;
    if (code > 0x7E) code = 0x7E;
    return (uint8_t)(sign | code);
}

uint8_t coat_oracle_e4m3_encode(float x) { return e4m3_encode(x); }
float coat_oracle_e4m3_decode(uint8_t c) { return e4m3_decode(c); }

/* ---------------------------------------------------------------- bf16 helpers (param dtype bf16) */
static float bf16_to_f32(uint16_t h) {
    uint32_t b = (uint32_t)h << 16;
    float f;
    memcpy(&f, &b, 4);
    return f;
}
static uint16_t f32_to_bf16(float f) {
    uint32_t b;
    memcpy(&b, &f, 4);
    if ((b & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((b >> 16) | 0x40);
    b += 0x7FFF + ((b >> 16) & 1);
    return (uint16_t)(b >> 16);
}

/* ---------------------------------------------------------------- library functions as stated above */
static float powf_cr(float x, float y) { return (float)pow((double)x, (double)y); }
static float log2f_cr(float x) { return (float)log2((double)x); }

/* One level set of the reference's shuffle tree over 32 lanes (:89-103 and :124-137).
 * with_min == 0 reproduces the plain kernel's max-only tree (fp8_adamw_cuda_kernel.cu:71-77). */
static void shfl_tree(float *mx, float *mn, int with_min) {
    for (int off = WARP / 2; off > 0; off /= 2) {
        for (int lane = 0; lane < WARP; lane++) { /* ascending: lane+off still holds its pre-level value */
            int src = lane + off < WARP ? lane + off : lane;
            float rmx = mx[src];
            mx[lane] = fmaxf(mx[lane], fabsf(rmx));
            if (with_min) {
                float a = fabsf(mn[src]);
                mn[lane] = (a > 0) ? fminf(mn[lane], a) : mn[lane];
            }
        }
    }
}

/* Block-level max / zero-skipping min of |val[0..127]| exactly as thread 0 ends up holding them.
 * valid = number of in-range threads of this block. */
static void block_minmax(const float *val, int valid, int with_min, float *out_max, float *out_min) {
    float smx[WARP], smn[WARP];
    for (int w = 0; w < QGROUP / WARP; w++) {
        float mx[WARP], mn[WARP];
        for (int l = 0; l < WARP; l++) {
            int t = w * WARP + l;
            float a = t < valid ? fabsf(val[t]) : 0.0f; /* :66-67, :79-82 */
            mx[l] = a;
            mn[l] = t < valid ? a : 3.402823466e+38f; /* :84-87 (0x7f7fffff) */
        }
        shfl_tree(mx, mn, with_min);
        smx[w] = mx[0];
        smn[w] = mn[0];
    }
    float mx[WARP], mn[WARP];
    for (int l = 0; l < WARP; l++) { /* :119-122: threads >= blockDim/warpSize get 0 / 1e9 */
        mx[l] = l < QGROUP / WARP ? smx[l] : 0.0f;
        mn[l] = l < QGROUP / WARP ? smn[l] : 1e9f;
    }
    shfl_tree(mx, mn, with_min);
    *out_max = mx[0];
    if (with_min) *out_min = mn[0];
}

/* Adam update of one element; returns the new parameter (fp32), updates *m, *v.  (:52-64) */
static float adam_update(float p, float g, float *m, float *v, float beta1, float beta2, float lr, float wd,
                         float eps, int step) {
    *m = beta1 * *m + (1 - beta1) * g;
    *v = beta2 * *v + ((1 - beta2) * g) * g;
    float correction1 = 1.0f - powf_cr(beta1, (float)step);
    float correction2_sqrt = sqrtf(1.0f - powf_cr(beta2, (float)step));
    float denom = (sqrtf(*v) / correction2_sqrt + eps) * correction1;
    float update = (*m / denom) + (wd * p);
    return p - (lr * update);
}

#define LOAD_P(i) (p_is_bf16 ? bf16_to_f32(((const uint16_t *)params)[i]) : ((const float *)params)[i])
#define LOAD_G(i) (p_is_bf16 ? bf16_to_f32(((const uint16_t *)grads)[i]) : ((const float *)grads)[i])
#define STORE_P(i, x)                                                  \
    do {                                                               \
        if (p_is_bf16) ((uint16_t *)params)[i] = f32_to_bf16(x);       \
        else ((float *)params)[i] = (x);                               \
    } while (0)

/* fp8_adamw_expand_cuda_kernel.cu:20-203.  All state is updated in place. */
void coat_oracle_adamw_expand(void *params, const void *grads, int p_is_bf16, uint8_t *exp_avg, float *scale_exp_avg,
                              float *expand_exp_avg, float *sqrtminmax_exp_avg, uint8_t *exp_avg_sq,
                              float *scale_exp_avg_sq, float *expand_exp_avg_sq, float *sqrtminmax_exp_avg_sq,
                              float beta1, float beta2, float lr, float wd, float eps, int step, int expand_min,
                              int64_t total_elements) {
    int64_t ngroups = (total_elements + QGROUP - 1) / QGROUP;
    for (int64_t gi = 0; gi < ngroups; gi++) {
        int64_t base = gi * QGROUP;
        int valid = (int)(total_elements - base < QGROUP ? total_elements - base : QGROUP);
        float m[QGROUP], v[QGROUP];
        for (int t = 0; t < valid; t++) {
            int64_t idx = base + t;
            /* dequantize (:44-49) */
            float fm = e4m3_decode(exp_avg[idx]) * scale_exp_avg[gi];
            int sgn = 1 - 2 * (signbit(fm) ? 1 : 0);
            fm = sgn * powf_cr(fabsf(fm), 1 / expand_exp_avg[gi]) * sqrtminmax_exp_avg[gi];
            float fv = e4m3_decode(exp_avg_sq[idx]) * scale_exp_avg_sq[gi];
            fv = powf_cr(fv, 1 / expand_exp_avg_sq[gi]) * sqrtminmax_exp_avg_sq[gi];
            float p = LOAD_P(idx), g = LOAD_G(idx);
            float pn = adam_update(p, g, &fm, &fv, beta1, beta2, lr, wd, eps, step);
            STORE_P(idx, pn);
            m[t] = fm;
            v[t] = fv;
        }
        float mx1, mn1, mx2, mn2;
        block_minmax(m, valid, 1, &mx1, &mn1);
        block_minmax(v, valid, 1, &mx2, &mn2);

        float fp8MaxVal = 448; /* :151 */
        float firstMaxVal = (float)((double)mx1 + 1e-30), firstMinVal = (float)((double)mn1 + 1e-30);
        float secondMaxVal = (float)((double)mx2 + 1e-30), secondMinVal = (float)((double)mn2 + 1e-30);
        float firstRatio = firstMaxVal / firstMinVal, secondRatio = secondMaxVal / secondMinVal; /* :162-163 */
        float firstSqrtMinMax = sqrtf(firstMaxVal) * sqrtf(firstMinVal);                         /* :164 */
        float secondSqrtMinMax = sqrtf(secondMaxVal) * sqrtf(secondMinVal);
        float ratioUpperBound = fp8MaxVal * fp8MaxVal / 2; /* :170 */
        float firstExp = floorf((log2f_cr(ratioUpperBound) / log2f_cr(firstRatio)) * expand_min) / expand_min;
        float secondExp = floorf((log2f_cr(ratioUpperBound) / log2f_cr(secondRatio)) * expand_min) / expand_min;
        float new_scale_exp_avg = powf_cr(firstMaxVal / firstSqrtMinMax, firstExp) / fp8MaxVal; /* :180-181 */
        float new_scale_exp_avg_sq = powf_cr(secondMaxVal / secondSqrtMinMax, secondExp) / fp8MaxVal;
        for (int t = 0; t < valid; t++) {
            int64_t idx = base + t;
            int sgn = 1 - 2 * (signbit(m[t]) ? 1 : 0);
            float em = sgn * powf_cr(fabsf(m[t]) / firstSqrtMinMax, firstExp); /* :175-177 */
            float ev = powf_cr(v[t] / secondSqrtMinMax, secondExp);
            exp_avg[idx] = e4m3_encode(em / new_scale_exp_avg); /* :186-187 */
            exp_avg_sq[idx] = e4m3_encode(ev / new_scale_exp_avg_sq);
        }
        scale_exp_avg[gi] = new_scale_exp_avg; /* :196-201 */
        scale_exp_avg_sq[gi] = new_scale_exp_avg_sq;
        expand_exp_avg[gi] = firstExp;
        expand_exp_avg_sq[gi] = secondExp;
        sqrtminmax_exp_avg[gi] = firstSqrtMinMax;
        sqrtminmax_exp_avg_sq[gi] = secondSqrtMinMax;
    }
}

/* fp8_adamw_cuda_kernel.cu:20-125. */
void coat_oracle_adamw(void *params, const void *grads, int p_is_bf16, uint8_t *exp_avg, float *scale_exp_avg,
                       uint8_t *exp_avg_sq, float *scale_exp_avg_sq, float beta1, float beta2, float lr, float wd,
                       float eps, int step, int64_t total_elements) {
    int64_t ngroups = (total_elements + QGROUP - 1) / QGROUP;
    for (int64_t gi = 0; gi < ngroups; gi++) {
        int64_t base = gi * QGROUP;
        int valid = (int)(total_elements - base < QGROUP ? total_elements - base : QGROUP);
        float m[QGROUP], v[QGROUP];
        for (int t = 0; t < valid; t++) {
            int64_t idx = base + t;
            float fm = e4m3_decode(exp_avg[idx]) * scale_exp_avg[gi]; /* :40-41 */
            float fv = e4m3_decode(exp_avg_sq[idx]) * scale_exp_avg_sq[gi];
            float p = LOAD_P(idx), g = LOAD_G(idx);
            float pn = adam_update(p, g, &fm, &fv, beta1, beta2, lr, wd, eps, step);
            STORE_P(idx, pn);
            m[t] = fm;
            v[t] = fv;
        }
        float mx1, mx2, unused;
        block_minmax(m, valid, 0, &mx1, &unused);
        block_minmax(v, valid, 0, &mx2, &unused);
        float fp8MaxVal = 448;
        /* :105-106: the CUDA source adds into the __shared__ variable from every thread (a benign
         * race that can add 1e-20 more than once); the single add is the intended value. */
        float a1 = (float)((double)mx1 + 1e-20), a2 = (float)((double)mx2 + 1e-20);
        float new_scale_exp_avg = a1 / fp8MaxVal, new_scale_exp_avg_sq = a2 / fp8MaxVal; /* :108-109 */
        for (int t = 0; t < valid; t++) {
            int64_t idx = base + t;
            exp_avg[idx] = e4m3_encode(m[t] / new_scale_exp_avg); /* :112-113 */
            exp_avg_sq[idx] = e4m3_encode(v[t] / new_scale_exp_avg_sq);
        }
        scale_exp_avg[gi] = new_scale_exp_avg;
        scale_exp_avg_sq[gi] = new_scale_exp_avg_sq;
    }
}

/* Exact-division check used by tests of the device's reciprocal+FMA division:
 * returns the number of (x, s) pairs for which the three-operation sequence differs from x / s. */
int64_t coat_oracle_count_recip_div_mismatch(const float *x, int64_t nx, const float *s, int64_t ns) {
    int64_t bad = 0;
    for (int64_t j = 0; j < ns; j++) {
        float sv = s[j], r = 1.0f / sv;
        for (int64_t i = 0; i < nx; i++) {
            float xv = x[i];
            float q0 = xv * r;
            float e = fmaf(-q0, sv, xv);
            float q = copysignf(fmaf(e, r, q0), xv);
            float ref = xv / sv;
            uint32_t a, b;
            memcpy(&a, &q, 4);
            memcpy(&b, &ref, 4);
            bad += (a != b) && !(isnan(q) && isnan(ref));
        }
    }
    return bad;
}

/* Check of the device's square-root correction (sqrt_cr_normal in coat_amd/csrc/adamw.hip): starting from the correctly
 * rounded root moved by -1, 0 and +1 ulp (the hardware approximation is within one ulp), the two-residual correction must
 * return the correctly rounded root, for x = +0, x = +inf and normal x >= 2^-96 (smaller inputs are outside the domain
 * of the device function and are skipped).  Returns the number of (x, start) pairs for which it does not. */
int64_t coat_oracle_count_sqrt_correction_mismatch(const float *x, int64_t nx) {
    int64_t bad = 0;
    for (int64_t i = 0; i < nx; i++) {
        const float xv = x[i], ref = sqrtf(xv);
        if (!(xv == 0.0f || xv >= 0x1p-96f)) continue;
        uint32_t rb;
        memcpy(&rb, &ref, 4);
        const int exact_only = xv == 0.0f || isinf(xv);  /* the hardware returns these two exactly */
        for (int d = exact_only ? 0 : -1; d <= (exact_only ? 0 : 1); d++) {
            uint32_t sb = rb + (uint32_t)d, dn = sb - 1u, up = sb + 1u;
            float s, s_dn, s_up;
            memcpy(&s, &sb, 4);
            memcpy(&s_dn, &dn, 4);
            memcpy(&s_up, &up, 4);
            const float r_dn = fmaf(-s_dn, s, xv), r_up = fmaf(-s_up, s, xv);
            float r = r_dn <= 0.0f ? s_dn : s;
            r = r_up > 0.0f ? s_up : r;
            uint32_t a;
            memcpy(&a, &r, 4);
            bad += a != rb;
        }
    }
    return bad;
}

