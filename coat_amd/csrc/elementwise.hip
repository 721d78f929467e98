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
};

__device__ __forceinline__ float load_scale_rt(const void* p, int64_t i, int dt) {
    if (dt == kBF16) return u2f((uint32_t)((const uint16_t*)p)[i] << 16);
    if (dt == kF32) return ((const float*)p)[i];
    return f16lo(((const uint16_t*)p)[i]);
}

template <int KIND> __device__ __forceinline__ void load_fp8x16(const void* p, int64_t chunk, float scale, float* v) {
    uint4 c = *(const uint4*)((const uint8_t*)p + chunk * 16);
    uint32_t w[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
    for (int k = 0; k < 4; k++) {
        float f[4];
        fp8x4_to_f32<KIND>(w[k], f);
#pragma unroll
        for (int i = 0; i < 4; i++) v[4 * k + i] = f[i] * scale;  // dequantize: float(q) * float(s)
    }
}
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
        const int64_t gidx = (c * 16) / A.qb;
        load_fp8x16<KIND_IN>(A.x1, c, load_scale_rt(A.s1, gidx, A.s_in_dtype), a);
        if (kTwoIn) load_fp8x16<KIND_IN>(A.x2, c, load_scale_rt(A.s2, gidx, A.s_in_dtype), b);
    }
    if (kHasG) load_bf16x16(A.g, c, g);

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
    if (A.s_out && ok && (threadIdx.x % lpg) == 0) ((uint16_t*)A.s_out)[(c * 16) / A.qb] = (uint16_t)f2bf16(s);
    if (A.s_max) tensor_max = fmaxf(tensor_max, ok ? s : 0.0f);
    }
    if (A.s_max) block_atomic_max_nonneg(A.s_max, tensor_max, smem_max);
}

}  // namespace coat

using namespace coat;

template <int OP> static int launch_ew(const EwArgs& A, int kind_in, int kind_out, hipStream_t st) {
    int64_t blocks = (A.nchunk + 255) / 256;
    if (blocks > 2048) blocks = 2048;  // 8 blocks per CU; the kernel strides over the rest
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
    EwArgs A = {x, s_x, nullptr, nullptr, nullptr, nullptr, nullptr, y, s_y, nullptr, 0, 0, 0};
    if (int e = ew_common(A, M, N, QB, s_dtype)) return e;
    if (M * N == 0) return COAT_OK;
    if (!x || !s_x || !y || !s_y) return COAT_EINVAL;
    return launch_ew<kSiluFwd>(A, fp8, fp8, (hipStream_t)stream);
}

extern "C" int coat_fp8_silu_backward(const void* x, int fp8_in, const void* s_x, int s_dtype, const void* g, void* y,
                                      void* s_y, float* s_max, int fp8_out, int64_t M, int64_t N, int QB, void* stream) {
    EwArgs A = {x, s_x, nullptr, nullptr, g, y, nullptr, nullptr, s_y, s_max, 0, 0, 0};
    if (int e = ew_common(A, M, N, QB, s_dtype)) return e;
    if (M * N == 0) return COAT_OK;
    if (!x || !s_x || !g || !y) return COAT_EINVAL;
    return launch_ew<kSiluBwd>(A, fp8_in, fp8_out, (hipStream_t)stream);
}

extern "C" int coat_fp8_mul_forward(const void* x1, const void* s_x1, const void* x2, const void* s_x2, int fp8_in,
                                    int s_dtype, void* y, void* s_y, float* s_max, int64_t M, int64_t N, int QB,
                                    void* stream) {
    EwArgs A = {x1, s_x1, x2, s_x2, nullptr, y, nullptr, nullptr, s_y, s_max, 0, 0, 0};
    if (int e = ew_common(A, M, N, QB, s_dtype)) return e;
    if (M * N == 0) return COAT_OK;
    if (!x1 || !s_x1 || !x2 || !s_x2 || !y) return COAT_EINVAL;
    return launch_ew<kMulFwd>(A, fp8_in, fp8_in, (hipStream_t)stream);
}

extern "C" int coat_fp8_mul_backward(const void* x1, const void* s_x1, const void* x2, const void* s_x2, int fp8_in,
                                     int s_dtype, const void* g, void* y1, void* y2, void* s_y2, float* s_max,
                                     int fp8_out, int64_t M, int64_t N, int QB, void* stream) {
    EwArgs A = {x1, s_x1, x2, s_x2, g, y2, y1, nullptr, s_y2, s_max, 0, 0, 0};
    if (int e = ew_common(A, M, N, QB, s_dtype)) return e;
    if (M * N == 0) return COAT_OK;
    if (!x1 || !s_x1 || !x2 || !s_x2 || !g || !y1 || !y2) return COAT_EINVAL;
    return launch_ew<kMulBwd>(A, fp8_in, fp8_out, (hipStream_t)stream);
}

extern "C" int coat_fp8_gelu_forward(const void* x, int fp8, const void* s_x, int s_dtype, void* y, void* s_y,
                                     float* s_max, int64_t M, int64_t N, int QB, void* stream) {
    EwArgs A = {x, s_x, nullptr, nullptr, nullptr, y, nullptr, nullptr, s_y, s_max, 0, 0, 0};
    if (int e = ew_common(A, M, N, QB, s_dtype)) return e;
    if (M * N == 0) return COAT_OK;
    if (!x || !s_x || !y) return COAT_EINVAL;
    return launch_ew<kGeluFwd>(A, fp8, fp8, (hipStream_t)stream);
}

extern "C" int coat_fp8_gelu_backward(const void* x, int fp8_in, const void* s_x, int s_dtype, const void* g, void* y,
                                      void* s_y, float* s_max, int fp8_out, int64_t M, int64_t N, int QB, void* stream) {
    EwArgs A = {x, s_x, nullptr, nullptr, g, y, nullptr, nullptr, s_y, s_max, 0, 0, 0};
    if (int e = ew_common(A, M, N, QB, s_dtype)) return e;
    if (M * N == 0) return COAT_OK;
    if (!x || !s_x || !g || !y) return COAT_EINVAL;
    return launch_ew<kGeluBwd>(A, fp8_in, fp8_out, (hipStream_t)stream);
}

extern "C" int coat_fp8_add_fwd(const void* x1, const void* x2, void* y, void* q, void* s_q, int fp8_out, int64_t M,
                                int64_t N, int QB, void* stream) {
    EwArgs A = {x1, nullptr, x2, nullptr, nullptr, y, nullptr, q, s_q, nullptr, 0, 0, 0};
    if (int e = ew_common(A, M, N, QB, COAT_BF16)) return e;
    if (M * N == 0) return COAT_OK;
    if (!x1 || !x2 || !y || !q || !s_q) return COAT_EINVAL;
    return launch_ew<kAddFwd>(A, COAT_E4M3, fp8_out, (hipStream_t)stream);
}

extern "C" int coat_fp8_add_bwd(const void* x1, const void* x2, void* y, void* s_y, float* s_max, int fp8_out,
                                int64_t M, int64_t N, int QB, void* stream) {
    EwArgs A = {x1, nullptr, x2, nullptr, nullptr, y, nullptr, nullptr, s_y, s_max, 0, 0, 0};
    if (int e = ew_common(A, M, N, QB, COAT_BF16)) return e;
    if (M * N == 0) return COAT_OK;
    if (!x1 || !x2 || !y) return COAT_EINVAL;
    return launch_ew<kAddBwd>(A, COAT_E4M3, fp8_out, (hipStream_t)stream);
}
