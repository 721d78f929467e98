// Fused FP8 element-wise kernels for gfx950: SiLU, GELU, mul, residual add (forward and backward).
//
// Reference kernels (coat/activation/real_quantization/): silu_fwd.py:47, silu_bwd.py:47, mul_fwd.py:51,
// mul_bwd.py:49, gelu_fwd.py:47, gelu_bwd.py:47, add_fwd.py:46, add_bwd.py:48.  All of them dequantize
// per-group FP8 inputs (or read bf16), compute in fp32, and emit either per-group FP8 (+ scales) or a
// bf16 value with per-group scales whose maximum becomes the per-tensor scale of a following division.
//
// Layout: one lane owns 16 consecutive elements: one 16-byte load of FP8 codes, two 16-byte loads of bf16,
// one scale.  With QB = 16 a quantization group never leaves the lane; larger groups are QB/16 neighbouring
// lanes (DPP max).  Outputs are written the same way (16 B of codes, 2 x 16 B of bf16, one scale per group).
// The maximum of the fp32 group scales of the whole tensor is accumulated with an order-independent atomic
// max on the bit pattern, so the per-tensor scale needs no separate reduction pass.
#include <math.h>

#include "coat_device.h"
#include "coat_host.h"

namespace coat {

enum EwOp { kSiluFwd = 0, kSiluBwd, kMulFwd, kMulBwd, kGeluFwd, kGeluBwd, kAddFwd, kAddBwd };

struct EwArgs {
    const void* x1;   // fp8 codes (or bf16 for add)
    const void* s1;   // per-group scales of x1
    const void* x2;   // second fp8 input (mul) or second bf16 input (add)
    const void* s2;
    const void* g;    // bf16 gradient
    void* y;          // bf16 output (value that a later division quantizes) or nullptr
    void* y1;         // mul backward: bf16 g * x2
    void* q;          // per-group FP8 output
    void* s_out;      // per-group scales of the output (bf16) or nullptr
    float* s_max;     // device scalar receiving max of fp32 group scales, or nullptr
    int64_t nchunk;   // number of 16-element chunks
    int qb;           // group size (multiple of 16)
    int s_in_dtype;   // dtype of s1 / s2 (COAT_BF16 or COAT_F32 / COAT_F16)
    int s_out_dtype;  // dtype of s_out: bf16 (0-initialised default below is overwritten) except for the SiLU forward,
                      // whose scales take the dtype of the input scales (silu_fwd.py:166-167)
};

// Dequantizes 16 loaded codes.  The 16 bytes of codes and the raw scale word are loaded first (load_rt_raw) and
// converted here, after every load of the iteration has been issued; a scale converted right where it is loaded costs
// a run-time dtype branch and a wait for that one load before the next is issued.
template <int KIND> __device__ __forceinline__ void dequant_chunk(uint4 c, float scale, float* v) {
    uint32_t w[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
    for (int k = 0; k < 4; k++) {
        float f[4];
        fp8x4_to_f32<KIND>(w[k], f);
#pragma unroll
        for (int i = 0; i < 4; i++) v[4 * k + i] = f[i] * scale;  // dequantize: float(q) * float(s)
    }
}
__device__ __forceinline__ uint4 load_codes16(const void* p, int64_t chunk) { return *(const uint4*)((const uint8_t*)p + chunk * 16); }
__device__ __forceinline__ void load_bf16x16(const void* p, int64_t chunk, float* v) {
    const uint4* src = (const uint4*)((const uint16_t*)p + chunk * 16);
    uint4 a = src[0], b = src[1];
    uint32_t w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
    for (int k = 0; k < 8; k++) {
        v[2 * k] = bf16lo(w[k]);
        v[2 * k + 1] = bf16hi(w[k]);
    }
}
__device__ __forceinline__ void store_bf16x16(void* p, int64_t chunk, const float* v) {
    uint32_t w[8];
#pragma unroll
    for (int k = 0; k < 8; k++) w[k] = pack_bf16x2(v[2 * k], v[2 * k + 1]);
    uint4* dst = (uint4*)((uint16_t*)p + chunk * 16);
    dst[0] = make_uint4(w[0], w[1], w[2], w[3]);
    dst[1] = make_uint4(w[4], w[5], w[6], w[7]);
}

// 1 / (1 + exp(-x)) on the hardware transcendental units: exp(-x) = 2^n * v_exp_f32(f) with t = -x log2(e) split into
// n = rint(t) and f = fma(x, -log2(e), -n) (so the exponent argument keeps full precision for large |x|), then
// v_rcp_f32.  About 2 ulp against the correctly rounded value; overflow of 2^t gives 1 / inf = 0 like the libm form.
__device__ __forceinline__ float sigmoid_f32(float x) {
    constexpr float kNegLog2e = -1.44269504088896340736f;
    const float n = __builtin_rintf(fminf(fmaxf(x * kNegLog2e, -150.0f), 150.0f));
    const float f = fmaf(x, kNegLog2e, -n);
    const float e = __builtin_amdgcn_ldexpf(__builtin_amdgcn_exp2f(f), (int)n);
    return __builtin_amdgcn_rcpf(1.0f + e);
}

template <int OP, int KIND_IN, int KIND_OUT>
__global__ __launch_bounds__(256) void k_elementwise(EwArgs A) {
    constexpr bool kBf16In = (OP == kAddFwd || OP == kAddBwd);
    constexpr bool kTwoIn = (OP == kMulFwd || OP == kMulBwd || kBf16In);
    constexpr bool kHasG = (OP == kSiluBwd || OP == kMulBwd || OP == kGeluBwd);
    constexpr bool kQuantPg = (OP == kSiluFwd || OP == kAddFwd);         // emit per-group FP8 + scales
    constexpr bool kWriteY = !(OP == kSiluFwd);                          // emit the bf16 value
    __shared__ float smem_max[4];
    enable_fp8_saturation();
    const int lpg = A.qb >> 4;  // lanes per group
    const int gshift = 27 - __builtin_clz(A.qb);  // chunk index -> group index (qb is a power of two >= 16)
    float tensor_max = 0.0f;
    // grid-stride over 256-chunk slabs: the trip count is block-uniform, so the lanes of a group stay together
    for (int64_t base = (int64_t)blockIdx.x * 256; base < A.nchunk; base += (int64_t)gridDim.x * 256) {
    const int64_t chunk = base + threadIdx.x;
    const bool ok = chunk < A.nchunk;
    const int64_t c = ok ? chunk : 0;

    float a[16], b[16], g[16], v[16];
    if (kBf16In) {
        load_bf16x16(A.x1, c, a);
        load_bf16x16(A.x2, c, b);
    } else {
        const int64_t gidx = c >> gshift;
        const uint32_t rs1 = load_rt_raw(A.s1, gidx, A.s_in_dtype);
        const uint32_t rs2 = kTwoIn ? load_rt_raw(A.s2, gidx, A.s_in_dtype) : 0u;
        const uint4 c1 = load_codes16(A.x1, c);
        const uint4 c2 = kTwoIn ? load_codes16(A.x2, c) : make_uint4(0, 0, 0, 0);
        if (kHasG) load_bf16x16(A.g, c, g);
        dequant_chunk<KIND_IN>(c1, rt_raw_to_f32(rs1, A.s_in_dtype), a);
        if (kTwoIn) dequant_chunk<KIND_IN>(c2, rt_raw_to_f32(rs2, A.s_in_dtype), b);
    }

#pragma unroll
    for (int i = 0; i < 16; i++) {
        const float x = a[i];
        if (OP == kSiluFwd) {
            v[i] = sigmoid_f32(x) * x;
        } else if (OP == kSiluBwd) {
            const float sig = sigmoid_f32(x);
            v[i] = (sig + (x * sig) * (1 - sig)) * g[i];
        } else if (OP == kMulFwd) {
            v[i] = x * b[i];
        } else if (OP == kMulBwd) {
            v[i] = g[i] * x;         // grad of the second input: g * x1
            b[i] = g[i] * b[i];      // grad of the first input:  g * x2 (bf16 output y1)
        } else if (OP == kGeluFwd) {
            const float cdf = (1.0f + erff(x / 1.41421356237309515f)) / 2;
            v[i] = cdf * x;
        } else if (OP == kGeluBwd) {
            const float cdf = (1.0f + erff(x / 1.41421356237309515f)) / 2;
            const float pdf_term = x * expf(-(x * x) / 2) / 2.50662827463100024f;  // sqrt(2*pi) in fp32
            v[i] = (cdf + pdf_term) * g[i];
        } else {
            v[i] = x + b[i];
        }
    }
    if (OP == kMulBwd && ok) store_bf16x16(A.y1, c, b);
    if (kWriteY && ok) store_bf16x16(A.y, c, v);

    float amax = fmaxf(fabsf(v[0]), fabsf(v[1]));
#pragma unroll
    for (int i = 2; i < 16; i++) amax = fmaxf(amax, fabsf(v[i]));
    amax = cluster_max_rt(amax, lpg);
    float s;
    if (kQuantPg) s = group_scale<KIND_OUT>(amax);
    else s = A.s_max || A.s_out ? group_scale<KIND_OUT>(amax) : 0.0f;
    if (kQuantPg) {
        const float r = 1.0f / s;
        uint32_t w[4];
#pragma unroll
        for (int k = 0; k < 4; k++)
            w[k] = cvt4_fp8<KIND_OUT>(div_by_scale(v[4 * k], s, r), div_by_scale(v[4 * k + 1], s, r),
                                      div_by_scale(v[4 * k + 2], s, r), div_by_scale(v[4 * k + 3], s, r));
        if (ok) *(uint4*)((uint8_t*)A.q + c * 16) = make_uint4(w[0], w[1], w[2], w[3]);
    }
    if (A.s_out && ok && (threadIdx.x % lpg) == 0) {
        const int64_t si = c >> gshift;
        if (A.s_out_dtype == kBF16) ((uint16_t*)A.s_out)[si] = (uint16_t)f2bf16(s);
        else if (A.s_out_dtype == kF32) ((float*)A.s_out)[si] = s;
        else ((uint16_t*)A.s_out)[si] = (uint16_t)f2f16(s);
    }
    if (A.s_max) tensor_max = fmaxf(tensor_max, ok ? s : 0.0f);
    }
    if (A.s_max) block_atomic_max_nonneg(A.s_max, tensor_max, smem_max);
}

// ---- SiLU(gate) * up in one pass, forward and backward -------------------------------------------------------------
// The reference runs SiLU and the product as separate kernels (silu_fwd.py:152 then mul_fwd.py:191; mul_bwd.py:221 then
// silu_bwd.py:170), re-reading the FP8 SiLU output and writing / re-reading the bf16 gradient of the product in between.
// These kernels produce bit-identical tensors in one pass: every rounding the chain performs (SiLU -> per-group FP8 with
// a bf16 scale -> dequantize; g * up -> bf16) is performed in registers.
struct SiluMulArgs {
    const void *gate, *s_gate, *up, *s_up, *silu, *s_silu;  // per-group FP8 inputs (silu: backward only) and their scales
    const void* g;                                          // backward: bf16 gradient of the product
    void *q_silu, *s_silu_out;                              // forward: per-group FP8 SiLU output + bf16 scales (saved for backward)
    void* y;                                                // forward: bf16 product;  backward: bf16 gradient of gate
    void* y2;                                               // backward: bf16 gradient of up
    float *s_max, *s_max2;                                  // max of the fp32 group scales of y / y2
    void *q_gate_out, *s_gate_out, *q_up_out, *s_up_out;    // forward from bf16 gate / up: their per-group FP8 codes and bf16 scales
    int64_t nchunk;
    int qb, s_dtype;
    // Row pitches, for gate / up taken as column slices of a wider tensor and y / y2 written into one (strided != 0):
    // chunks of 16 elements per logical row, per row of gate / up, per row of y / y2; scales per row of s_gate / s_up.
    int strided;
    int64_t cpr, in_cpr, in_spr, y_cpr;
};

template <int KIND> __device__ __forceinline__ void dequant_words(const uint32_t* w, float scale, float* v) {
#pragma unroll
    for (int k = 0; k < 4; k++) {
        float f[4];
        fp8x4_to_f32<KIND>(w[k], f);
#pragma unroll
        for (int i = 0; i < 4; i++) v[4 * k + i] = f[i] * scale;
    }
}
__device__ __forceinline__ float round_bf16(float x) { return u2f((uint32_t)f2bf16(x) << 16); }
__device__ __forceinline__ float amax16(const float* v) {
    float a = fmaxf(fabsf(v[0]), fabsf(v[1]));
#pragma unroll
    for (int i = 2; i < 16; i++) a = fmaxf(a, fabsf(v[i]));
    return a;
}

// FROM16 (forward only): gate / up are bf16 tensors; they are quantized per group here exactly as k_quantize_pg would
// (codes and bf16 scales stored for the backward) and the rest of the kernel works on the dequantized values.
template <bool BWD, int KIND_IN, int KIND_OUT, bool FROM16 = false>
__global__ __launch_bounds__(256) void k_silu_mul(SiluMulArgs A) {
    __shared__ float smem_max[4];
    enable_fp8_saturation();
    const int lpg = A.qb >> 4;
    const int gshift = 27 - __builtin_clz(A.qb);  // chunk index -> group index (qb is a power of two >= 16)
    float tmax = 0.0f, tmax2 = 0.0f;
    for (int64_t base = (int64_t)blockIdx.x * 256; base < A.nchunk; base += (int64_t)gridDim.x * 256) {
        const int64_t chunk = base + threadIdx.x;
        const bool ok = chunk < A.nchunk;
        const int64_t c = ok ? chunk : 0;
        const int64_t gidx = c >> gshift;
        int64_t cin = c, gin = gidx, cy = c;
        if (A.strided) {  // uniform
            const int64_t row = c / A.cpr, col = c - row * A.cpr;
            cin = row * A.in_cpr + col;
            gin = row * A.in_spr + (col >> gshift);
            cy = row * A.y_cpr + col;
        }
        float a[16], b[16], sl[16], g[16];
        if (FROM16) {
            float raw[2][16];
            load_bf16x16(A.gate, c, raw[0]);
            load_bf16x16(A.up, c, raw[1]);
#pragma unroll
            for (int t = 0; t < 2; t++) {
                const float s = group_scale<KIND_IN>(cluster_max_rt(amax16(raw[t]), lpg));
                const float r = 1.0f / s;
                uint32_t w[4];
#pragma unroll
                for (int k = 0; k < 4; k++)
                    w[k] = cvt4_fp8<KIND_IN>(div_by_scale(raw[t][4 * k], s, r), div_by_scale(raw[t][4 * k + 1], s, r),
                                             div_by_scale(raw[t][4 * k + 2], s, r), div_by_scale(raw[t][4 * k + 3], s, r));
                if (ok) {
                    *(uint4*)((uint8_t*)(t ? A.q_up_out : A.q_gate_out) + c * 16) = make_uint4(w[0], w[1], w[2], w[3]);
                    if ((threadIdx.x % lpg) == 0) ((uint16_t*)(t ? A.s_up_out : A.s_gate_out))[gidx] = (uint16_t)f2bf16(s);
                }
                dequant_words<KIND_IN>(w, round_bf16(s), t ? b : a);  // as the saved activation is read back
            }
        } else {
            // every load of the iteration is issued before the first conversion
            const uint32_t rs_a = load_rt_raw(A.s_gate, gin, A.s_dtype), rs_b = load_rt_raw(A.s_up, gin, A.s_dtype);
            const uint32_t rs_l = BWD ? load_rt_raw(A.s_silu, gidx, A.s_dtype) : 0u;
            const uint4 ca = load_codes16(A.gate, cin), cb = load_codes16(A.up, cin);
            if (BWD) {
                const uint4 cl = load_codes16(A.silu, c);
                load_bf16x16(A.g, c, g);
                dequant_chunk<KIND_IN>(cl, rt_raw_to_f32(rs_l, A.s_dtype), sl);
            }
            dequant_chunk<KIND_IN>(ca, rt_raw_to_f32(rs_a, A.s_dtype), a);
            dequant_chunk<KIND_IN>(cb, rt_raw_to_f32(rs_b, A.s_dtype), b);
        }
        if (!BWD) {
            float sv[16];
#pragma unroll
            for (int i = 0; i < 16; i++) sv[i] = sigmoid_f32(a[i]) * a[i];
            const float s = group_scale<KIND_IN>(cluster_max_rt(amax16(sv), lpg));
            const float r = 1.0f / s;
            uint32_t w[4];
#pragma unroll
            for (int k = 0; k < 4; k++)
                w[k] = cvt4_fp8<KIND_IN>(div_by_scale(sv[4 * k], s, r), div_by_scale(sv[4 * k + 1], s, r),
                                         div_by_scale(sv[4 * k + 2], s, r), div_by_scale(sv[4 * k + 3], s, r));
            if (ok) {
                *(uint4*)((uint8_t*)A.q_silu + c * 16) = make_uint4(w[0], w[1], w[2], w[3]);
                if ((threadIdx.x % lpg) == 0) ((uint16_t*)A.s_silu_out)[gidx] = (uint16_t)f2bf16(s);
            }
            // what the product kernel would read back: the codes times the bf16-rounded scale
            float d[16], v[16];
            dequant_words<KIND_IN>(w, round_bf16(s), d);
#pragma unroll
            for (int i = 0; i < 16; i++) v[i] = d[i] * b[i];
            if (ok && A.y) store_bf16x16(A.y, c, v);  // NULL: maximum only (the division recomputes the product)
            const float s2 = group_scale<KIND_IN>(cluster_max_rt(amax16(v), lpg));
            tmax = fmaxf(tmax, ok ? s2 : 0.0f);
        } else {
            float v[16], v2[16];
#pragma unroll
            for (int i = 0; i < 16; i++) {
                v2[i] = g[i] * sl[i];                       // gradient of up
                const float g1 = round_bf16(g[i] * b[i]);   // gradient of SiLU's output as the chain stores it (bf16)
                const float sig = sigmoid_f32(a[i]);
                v[i] = (sig + (a[i] * sig) * (1 - sig)) * g1;
            }
            if (ok) {
                store_bf16x16(A.y, cy, v);
                store_bf16x16(A.y2, cy, v2);
            }
            const float s1 = group_scale<KIND_OUT>(cluster_max_rt(amax16(v), lpg));
            const float s2 = group_scale<KIND_OUT>(cluster_max_rt(amax16(v2), lpg));
            tmax = fmaxf(tmax, ok ? s1 : 0.0f);
            tmax2 = fmaxf(tmax2, ok ? s2 : 0.0f);
        }
    }
    block_atomic_max_nonneg(A.s_max, tmax, smem_max);
    if (BWD) {
        __syncthreads();
        block_atomic_max_nonneg(A.s_max2, tmax2, smem_max);
    }
}

}  // namespace coat

using namespace coat;

template <int OP> static int launch_ew(const EwArgs& A, int kind_in, int kind_out, hipStream_t st) {
    int64_t blocks = (A.nchunk + 255) / 256;
    if (blocks > 2048) blocks = 2048;  // 8 blocks per CU; the kernel strides over the rest (8192 blocks or no cap: slower)
#define EW_LAUNCH(KI, KO)                                                                                   \
    hipLaunchKernelGGL((k_elementwise<OP, KI, KO>), dim3((unsigned)blocks), dim3(256), 0, st, A); \
    return coat_launch_status();
    if (kind_in == COAT_E4M3 && kind_out == COAT_E4M3) { EW_LAUNCH(kE4M3, kE4M3) }
    if (kind_in == COAT_E4M3 && kind_out == COAT_E5M2) { EW_LAUNCH(kE4M3, kE5M2) }
    if (kind_in == COAT_E5M2 && kind_out == COAT_E4M3) { EW_LAUNCH(kE5M2, kE4M3) }
    if (kind_in == COAT_E5M2 && kind_out == COAT_E5M2) { EW_LAUNCH(kE5M2, kE5M2) }
#undef EW_LAUNCH
    return COAT_EINVAL;
}

static int ew_common(EwArgs& A, int64_t M, int64_t N, int QB, int s_in_dtype) {
    if (M < 0 || N < 0) return COAT_EINVAL;
    if (QB < 16 || QB > 1024 || (QB & (QB - 1)) || N % QB != 0) return COAT_ESHAPE;
    if (s_in_dtype != COAT_BF16 && s_in_dtype != COAT_F32 && s_in_dtype != COAT_F16) return COAT_EDTYPE;
    const void* ptrs[] = {A.x1, A.x2, A.g, A.y, A.y1, A.q};
    for (const void* p : ptrs)
        if (!coat_aligned16(p)) return COAT_EALIGN;
    A.nchunk = M * N / 16;
    A.qb = QB;
    A.s_in_dtype = s_in_dtype;
    return COAT_OK;
}

extern "C" int coat_fp8_silu_forward(const void* x, int fp8, const void* s_x, int s_dtype, void* y, void* s_y,
                                     int64_t M, int64_t N, int QB, void* stream) {
    EwArgs A = {x, s_x, nullptr, nullptr, nullptr, nullptr, nullptr, y, s_y, nullptr, 0, 0, 0, kBF16};
    if (int e = ew_common(A, M, N, QB, s_dtype)) return e;
    A.s_out_dtype = s_dtype;  // the output scales are stored in the dtype of the input scales
    if (M * N == 0) return COAT_OK;
    if (!x || !s_x || !y || !s_y) return COAT_EINVAL;
    return launch_ew<kSiluFwd>(A, fp8, fp8, (hipStream_t)stream);
}

extern "C" int coat_fp8_silu_backward(const void* x, int fp8_in, const void* s_x, int s_dtype, const void* g, void* y,
                                      void* s_y, float* s_max, int fp8_out, int64_t M, int64_t N, int QB, void* stream) {
    EwArgs A = {x, s_x, nullptr, nullptr, g, y, nullptr, nullptr, s_y, s_max, 0, 0, 0, kBF16};
    if (int e = ew_common(A, M, N, QB, s_dtype)) return e;
    if (M * N == 0) return COAT_OK;
    if (!x || !s_x || !g || !y) return COAT_EINVAL;
    return launch_ew<kSiluBwd>(A, fp8_in, fp8_out, (hipStream_t)stream);
}

extern "C" int coat_fp8_mul_forward(const void* x1, const void* s_x1, const void* x2, const void* s_x2, int fp8_in,
                                    int s_dtype, void* y, void* s_y, float* s_max, int64_t M, int64_t N, int QB,
                                    void* stream) {
    EwArgs A = {x1, s_x1, x2, s_x2, nullptr, y, nullptr, nullptr, s_y, s_max, 0, 0, 0, kBF16};
    if (int e = ew_common(A, M, N, QB, s_dtype)) return e;
    if (M * N == 0) return COAT_OK;
    if (!x1 || !s_x1 || !x2 || !s_x2 || !y) return COAT_EINVAL;
    return launch_ew<kMulFwd>(A, fp8_in, fp8_in, (hipStream_t)stream);
}

extern "C" int coat_fp8_mul_backward(const void* x1, const void* s_x1, const void* x2, const void* s_x2, int fp8_in,
                                     int s_dtype, const void* g, void* y1, void* y2, void* s_y2, float* s_max,
                                     int fp8_out, int64_t M, int64_t N, int QB, void* stream) {
    EwArgs A = {x1, s_x1, x2, s_x2, g, y2, y1, nullptr, s_y2, s_max, 0, 0, 0, kBF16};
    if (int e = ew_common(A, M, N, QB, s_dtype)) return e;
    if (M * N == 0) return COAT_OK;
    if (!x1 || !s_x1 || !x2 || !s_x2 || !g || !y1 || !y2) return COAT_EINVAL;
    return launch_ew<kMulBwd>(A, fp8_in, fp8_out, (hipStream_t)stream);
}

extern "C" int coat_fp8_gelu_forward(const void* x, int fp8, const void* s_x, int s_dtype, void* y, void* s_y,
                                     float* s_max, int64_t M, int64_t N, int QB, void* stream) {
    EwArgs A = {x, s_x, nullptr, nullptr, nullptr, y, nullptr, nullptr, s_y, s_max, 0, 0, 0, kBF16};
    if (int e = ew_common(A, M, N, QB, s_dtype)) return e;
    if (M * N == 0) return COAT_OK;
    if (!x || !s_x || !y) return COAT_EINVAL;
    return launch_ew<kGeluFwd>(A, fp8, fp8, (hipStream_t)stream);
}

extern "C" int coat_fp8_gelu_backward(const void* x, int fp8_in, const void* s_x, int s_dtype, const void* g, void* y,
                                      void* s_y, float* s_max, int fp8_out, int64_t M, int64_t N, int QB, void* stream) {
    EwArgs A = {x, s_x, nullptr, nullptr, g, y, nullptr, nullptr, s_y, s_max, 0, 0, 0, kBF16};
    if (int e = ew_common(A, M, N, QB, s_dtype)) return e;
    if (M * N == 0) return COAT_OK;
    if (!x || !s_x || !g || !y) return COAT_EINVAL;
    return launch_ew<kGeluBwd>(A, fp8_in, fp8_out, (hipStream_t)stream);
}

extern "C" int coat_fp8_add_fwd(const void* x1, const void* x2, void* y, void* q, void* s_q, int fp8_out, int64_t M,
                                int64_t N, int QB, void* stream) {
    EwArgs A = {x1, nullptr, x2, nullptr, nullptr, y, nullptr, q, s_q, nullptr, 0, 0, 0, kBF16};
    if (int e = ew_common(A, M, N, QB, COAT_BF16)) return e;
    if (M * N == 0) return COAT_OK;
    if (!x1 || !x2 || !y || !q || !s_q) return COAT_EINVAL;
    return launch_ew<kAddFwd>(A, COAT_E4M3, fp8_out, (hipStream_t)stream);
}

extern "C" int coat_fp8_add_bwd(const void* x1, const void* x2, void* y, void* s_y, float* s_max, int fp8_out,
                                int64_t M, int64_t N, int QB, void* stream) {
    EwArgs A = {x1, nullptr, x2, nullptr, nullptr, y, nullptr, nullptr, s_y, s_max, 0, 0, 0, kBF16};
    if (int e = ew_common(A, M, N, QB, COAT_BF16)) return e;
    if (M * N == 0) return COAT_OK;
    if (!x1 || !x2 || !y) return COAT_EINVAL;
    return launch_ew<kAddBwd>(A, COAT_E4M3, fp8_out, (hipStream_t)stream);
}

static int silu_mul_launch(SiluMulArgs& A, bool bwd, int fp8_in, int fp8_out, int64_t M, int64_t N, int QB, int s_dtype,
                           int64_t in_pitch, int64_t s_pitch, int64_t y_pitch, hipStream_t st) {
    if (M < 0 || N < 0) return COAT_EINVAL;
    // pitches in elements (0 = contiguous rows); a slice must keep rows 16-byte aligned and whole groups
    if (in_pitch == 0) in_pitch = N;
    if (y_pitch == 0) y_pitch = N;
    if (QB > 0 && s_pitch == 0) s_pitch = N / QB;
    if (in_pitch < N || y_pitch < N || in_pitch % 16 != 0 || y_pitch % 16 != 0 || (!bwd && y_pitch != N)) return COAT_ESHAPE;
    if (QB < 16 || QB > 1024 || (QB & (QB - 1)) || N % QB != 0) return COAT_ESHAPE;
    if (s_dtype != COAT_BF16 && s_dtype != COAT_F32 && s_dtype != COAT_F16) return COAT_EDTYPE;
    if (fp8_in != COAT_E4M3 && fp8_in != COAT_E5M2) return COAT_EINVAL;
    if (bwd && fp8_out != COAT_E4M3 && fp8_out != COAT_E5M2) return COAT_EINVAL;
    if (M * N == 0) return COAT_OK;
    const void* ptrs[] = {A.gate, A.up, A.silu, A.g, A.q_silu, A.y, A.y2, A.q_gate_out, A.q_up_out};
    for (const void* p : ptrs)
        if (!coat_aligned16(p)) return COAT_EALIGN;
    if (s_pitch < N / QB) return COAT_ESHAPE;
    A.nchunk = M * N / 16;
    A.qb = QB;
    A.s_dtype = s_dtype;
    A.strided = in_pitch != N || y_pitch != N || s_pitch != N / QB;
    A.cpr = N / 16;
    A.in_cpr = in_pitch / 16;
    A.in_spr = s_pitch;
    A.y_cpr = y_pitch / 16;
    int64_t blocks = (A.nchunk + 255) / 256;
    if (blocks > 2048) blocks = 2048;
#define SM_LAUNCH(B, KI, KO) hipLaunchKernelGGL((k_silu_mul<B, KI, KO>), dim3((unsigned)blocks), dim3(256), 0, st, A)
    if (!bwd && A.q_gate_out) {
        if (fp8_in == COAT_E4M3) hipLaunchKernelGGL((k_silu_mul<false, kE4M3, kE4M3, true>), dim3((unsigned)blocks), dim3(256), 0, st, A);
        else hipLaunchKernelGGL((k_silu_mul<false, kE5M2, kE5M2, true>), dim3((unsigned)blocks), dim3(256), 0, st, A);
    } else if (!bwd) {
        if (fp8_in == COAT_E4M3) SM_LAUNCH(false, kE4M3, kE4M3); else SM_LAUNCH(false, kE5M2, kE5M2);
    } else if (fp8_in == COAT_E4M3) {
        if (fp8_out == COAT_E4M3) SM_LAUNCH(true, kE4M3, kE4M3); else SM_LAUNCH(true, kE4M3, kE5M2);
    } else {
        if (fp8_out == COAT_E4M3) SM_LAUNCH(true, kE5M2, kE4M3); else SM_LAUNCH(true, kE5M2, kE5M2);
    }
#undef SM_LAUNCH
    return coat_launch_status();
}

extern "C" int coat_fp8_silu_mul_forward(const void* gate, const void* s_gate, const void* up, const void* s_up, int fp8,
                                         int s_dtype, void* q_silu, void* s_silu, void* y, float* s_max, int64_t M,
                                         int64_t N, int QB, int64_t in_pitch, int64_t s_pitch, void* stream) {
    if ((M > 0 && N > 0) && (!gate || !s_gate || !up || !s_up || !q_silu || !s_silu || !s_max)) return COAT_EINVAL;  // y may be NULL
    SiluMulArgs A = {gate, s_gate, up, s_up, nullptr, nullptr, nullptr, q_silu, s_silu, y, nullptr, s_max, nullptr,
                     nullptr, nullptr, nullptr, nullptr};
    return silu_mul_launch(A, false, fp8, fp8, M, N, QB, s_dtype, in_pitch, s_pitch, 0, (hipStream_t)stream);
}

// The forward from bf16 gate / up [M, N] (dense): additionally writes their per-group FP8 codes and bf16 scales (what
// coat_fp8_quantize would give), so the three saved activations and the product's maximum come out of one pass.
extern "C" int coat_fp8_silu_mul_forward_bf16(const void* gate, const void* up, int fp8, void* q_gate, void* s_gate,
                                              void* q_up, void* s_up, void* q_silu, void* s_silu, void* y, float* s_max,
                                              int64_t M, int64_t N, int QB, void* stream) {
    if ((M > 0 && N > 0) && (!gate || !up || !q_gate || !s_gate || !q_up || !s_up || !q_silu || !s_silu || !s_max))
        return COAT_EINVAL;  // y may be NULL
    SiluMulArgs A = {gate, nullptr, up, nullptr, nullptr, nullptr, nullptr, q_silu, s_silu, y, nullptr, s_max, nullptr,
                     q_gate, s_gate, q_up, s_up};
    return silu_mul_launch(A, false, fp8, fp8, M, N, QB, COAT_BF16, 0, 0, 0, (hipStream_t)stream);
}

extern "C" int coat_fp8_silu_mul_backward(const void* gate, const void* s_gate, const void* up, const void* s_up,
                                          const void* silu, const void* s_silu, int fp8_in, int s_dtype, const void* g,
                                          void* y_gate, float* s_max_gate, void* y_up, float* s_max_up, int fp8_out,
                                          int64_t M, int64_t N, int QB, int64_t in_pitch, int64_t s_pitch,
                                          int64_t y_pitch, void* stream) {
    if ((M > 0 && N > 0) && (!gate || !s_gate || !up || !s_up || !silu || !s_silu || !g || !y_gate || !s_max_gate || !y_up || !s_max_up))
        return COAT_EINVAL;
    SiluMulArgs A = {gate, s_gate, up, s_up, silu, s_silu, g, nullptr, nullptr, y_gate, y_up, s_max_gate, s_max_up,
                     nullptr, nullptr, nullptr, nullptr};
    return silu_mul_launch(A, true, fp8_in, fp8_out, M, N, QB, s_dtype, in_pitch, s_pitch, y_pitch, (hipStream_t)stream);
}
