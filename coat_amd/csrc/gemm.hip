// Per-tensor-scaled FP8 GEMM on CDNA4 MFMA:  C[M,N] = (A[M,K] . B[N,K]^T) * (sA * sB) (+ bias), fp32 accumulate.
//
// Replaces _fp8matmul_kernel (coat/activation/real_quantization/linear.py:61-169).  Both operands are
// K-contiguous ("A row-major times the transpose of a row-major B"), which is the only form the reference uses:
// every tensor is kept in both orientations so that forward, dgrad and wgrad are all of this form
// (linear.py:253-302).  Operand formats are independent (e4m3 or e5m2 each: gradients are e5m2).
//
// Tiling: 256 x 256 x 128 per 256-thread block, 2 x 2 waves, each wave 128 x 128 as 4 x 4 tiles of
// v_mfma_f32_32x32x64_f8f6f4 (two K-steps per 128-byte K-slab).  LDS holds two stages of A and B slabs
// (2 x 64 KiB); 16-byte chunks are XOR-swizzled with the row (chunk ^ (row & 7)) so that the 32-byte-per-lane
// fragment reads (32 consecutive rows) and the 16-byte-per-lane global->LDS writes are both conflict-free.
// Global loads for slab k+1 are issued before the MFMAs of slab k and stored to the other LDS stage afterwards:
// one barrier per slab.  The MFMA takes the B tile as its first operand, so a lane ends up holding 4 consecutive
// n for one m per accumulator quad: bf16 rows are packed 4 at a time, and a 1 x 16 quantization group is two
// quads in each of the lanes l and l^32.
// Block ids are remapped so that the 8 XCDs (round-robin block dispatch) each work on a contiguous band of
// tiles, ordered in panels of 8 tile-rows, which keeps A / B slabs hot in that XCD's L2.
#include "coat_device.h"
#include "coat_host.h"

namespace coat {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int BM = 256, BN = 256, BK = 128;
constexpr int kStageBytes = (BM + BN) * BK;  // 64 KiB

enum Epilogue { kEpiBf16 = 0, kEpiQuantE4M3 = 1, kEpiQuantE5M2 = 2 };

struct GemmArgs {
    const uint8_t* A;   // [M, K]
    const uint8_t* B;   // [N, K]
    void* C;            // bf16 [M, N] or fp8 [M, N]
    void* Cs;           // bf16 [M, N/16] (quantize epilogue)
    const void* sa;     // per-tensor scales, one element each
    const void* sb;
    const void* bias;   // [N] or nullptr
    int s_dt, bias_dt;
    int M, N, K;
    int tiles_m, tiles_n;
};

__device__ __forceinline__ int swz(int row, int chunk) { return row * BK + ((chunk ^ (row & 7)) << 4); }

// 16-byte global load of chunk c of row `row` of a [rows, K] matrix, zero outside.
__device__ __forceinline__ uint4 gload(const uint8_t* base, int row, int rows, int kbyte, int K) {
    uint4 z = make_uint4(0, 0, 0, 0);
    if (row < rows && kbyte < K) z = *(const uint4*)(base + (int64_t)row * K + kbyte);
    return z;
}

template <int FMT_A, int FMT_B, int EPI>
__global__ __launch_bounds__(256) void k_fp8_gemm(GemmArgs G) {
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    // ---- XCD-aware tile mapping
    const int ntiles = G.tiles_m * G.tiles_n;
    const int per_xcd = (ntiles + 7) / 8;
    int tile = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (tile >= ntiles) return;
    constexpr int GROUP_M = 8;
    const int width = GROUP_M * G.tiles_n;
    const int group = tile / width;
    const int gsize = min(G.tiles_m - group * GROUP_M, GROUP_M);
    const int tm = group * GROUP_M + (tile % width) % gsize;
    const int tn = (tile % width) / gsize;
    const int m0 = tm * BM, n0 = tn * BN;

    // ---- global -> register staging: thread owns chunk (row = id/8, c = id%8) for id = tid + 256*i
    uint4 ra[8], rb[8];
    auto load_slab = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int id = tid + 256 * i, row = id >> 3, c = id & 7;
            ra[i] = gload(G.A, m0 + row, G.M, k0 + c * 16, G.K);
            rb[i] = gload(G.B, n0 + row, G.N, k0 + c * 16, G.K);
        }
    };
    auto store_slab = [&](int stage) {
        uint8_t* sA = lds + stage * kStageBytes;
        uint8_t* sB = sA + BM * BK;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const int id = tid + 256 * i, row = id >> 3, c = id & 7;
            *(uint4*)(sA + swz(row, c)) = ra[i];
            *(uint4*)(sB + swz(row, c)) = rb[i];
        }
    };

    v16f acc[4][4];  // [n-tile j][m-tile i]
#pragma unroll
    for (int j = 0; j < 4; j++)
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[j][i][r] = 0.0f;

    const int nslab = (G.K + BK - 1) / BK;
    load_slab(0);
    store_slab(0);
    __syncthreads();
    for (int kt = 0; kt < nslab; kt++) {
        if (kt + 1 < nslab) load_slab((kt + 1) * BK);
        const uint8_t* sA = lds + (kt & 1) * kStageBytes;
        const uint8_t* sB = sA + BM * BK;
#pragma unroll
        for (int ks = 0; ks < 2; ks++) {
            const int kb = ks * 2 + (lane >> 5);  // 32-byte block of the 128-byte slab row
            v8i fa[4], fb[4];
#pragma unroll
            for (int t = 0; t < 4; t++) {
                const int rowa = wm * 128 + t * 32 + (lane & 31);
                const int rowb = wn * 128 + t * 32 + (lane & 31);
                const uint4 a0 = *(const uint4*)(sA + swz(rowa, 2 * kb)), a1 = *(const uint4*)(sA + swz(rowa, 2 * kb + 1));
                const uint4 b0 = *(const uint4*)(sB + swz(rowb, 2 * kb)), b1 = *(const uint4*)(sB + swz(rowb, 2 * kb + 1));
                fa[t] = (v8i){(int)a0.x, (int)a0.y, (int)a0.z, (int)a0.w, (int)a1.x, (int)a1.y, (int)a1.z, (int)a1.w};
                fb[t] = (v8i){(int)b0.x, (int)b0.y, (int)b0.z, (int)b0.w, (int)b1.x, (int)b1.y, (int)b1.z, (int)b1.w};
            }
#pragma unroll
            for (int j = 0; j < 4; j++)
#pragma unroll
                for (int i = 0; i < 4; i++)
                    acc[j][i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[j], fa[i], acc[j][i], FMT_B, FMT_A, 0, 0, 0, 0);
        }
        if (kt + 1 < nslab) store_slab((kt + 1) & 1);
        __syncthreads();
    }

    // ---- epilogue
    const float scale = load_rt_f32(G.sa, 0, G.s_dt) * load_rt_f32(G.sb, 0, G.s_dt);
    if (EPI != kEpiBf16) enable_fp8_saturation();
    const int half = lane >> 5;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int m = m0 + wm * 128 + i * 32 + (lane & 31);
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int nb = n0 + wn * 128 + j * 32 + 4 * half;  // + 8*q + {0..3}
            float v[16];
#pragma unroll
            for (int r = 0; r < 16; r++) v[r] = acc[j][i][r] * scale;
            if (G.bias) {
#pragma unroll
                for (int q = 0; q < 4; q++)
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int n = nb + 8 * q + e;
                        if (n < G.N) v[4 * q + e] += load_rt_f32(G.bias, n, G.bias_dt);
                    }
            }
            if (EPI == kEpiBf16) {
                if (m < G.M) {
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const int n = nb + 8 * q;
                        if (n + 3 < G.N) {
                            *(uint2*)((uint16_t*)G.C + (int64_t)m * G.N + n) =
                                make_uint2(pack_bf16x2(v[4 * q], v[4 * q + 1]), pack_bf16x2(v[4 * q + 2], v[4 * q + 3]));
                        } else {
                            for (int e = 0; e < 4; e++)
                                if (n + e < G.N) ((uint16_t*)G.C)[(int64_t)m * G.N + n + e] = (uint16_t)f2bf16(v[4 * q + e]);
                        }
                    }
                }
            } else {
                constexpr int KIND = EPI == kEpiQuantE4M3 ? kE4M3 : kE5M2;
                // group g2 of 16 consecutive n = quads 2*g2, 2*g2+1 of this lane and of lane ^ 32
#pragma unroll
                for (int g2 = 0; g2 < 2; g2++) {
                    float amax = 0.0f;
#pragma unroll
                    for (int e = 0; e < 8; e++) amax = fmaxf(amax, fabsf(v[8 * g2 + e]));
                    amax = fmaxf(amax, lane_xor_f32(amax, 32));
                    const float s = group_scale<KIND>(amax);
                    const float r = 1.0f / s;
                    const int ng = n0 + wn * 128 + j * 32 + 16 * g2;  // first n of the group
                    if (m < G.M && ng < G.N) {
#pragma unroll
                        for (int qq = 0; qq < 2; qq++) {
                            const int q = 2 * g2 + qq;
                            const uint32_t w = cvt4_fp8<KIND>(div_by_scale(v[4 * q], s, r), div_by_scale(v[4 * q + 1], s, r),
                                                              div_by_scale(v[4 * q + 2], s, r), div_by_scale(v[4 * q + 3], s, r));
                            *(uint32_t*)((uint8_t*)G.C + (int64_t)m * G.N + nb + 8 * q) = w;
                        }
                        if (half == 0) ((uint16_t*)G.Cs)[(int64_t)m * (G.N >> 4) + (ng >> 4)] = (uint16_t)f2bf16(s);
                    }
                }
            }
        }
    }
}

}  // namespace coat

using namespace coat;

extern "C" int coat_fp8_gemm(const void* a, int fmt_a, const void* b, int fmt_b, void* c, void* c_scale, int out_kind,
                             const void* scale_a, const void* scale_b, int s_dtype, const void* bias, int bias_dtype,
                             int64_t M, int64_t N, int64_t K, int QB, void* stream) {
    if (M < 0 || N < 0 || K < 0) return COAT_EINVAL;
    if (M * N == 0) return COAT_OK;
    if (!a || !b || !c || !scale_a || !scale_b) return COAT_EINVAL;
    if (M >= (1 << 30) || N >= (1 << 30) || K >= (1 << 30)) return COAT_ESHAPE;
    if (K % 16 != 0) return COAT_ESHAPE;
    if (!coat_aligned16(a) || !coat_aligned16(b) || !coat_aligned16(c)) return COAT_EALIGN;
    if ((fmt_a != COAT_E4M3 && fmt_a != COAT_E5M2) || (fmt_b != COAT_E4M3 && fmt_b != COAT_E5M2)) return COAT_EINVAL;
    if (out_kind < 0 || out_kind > 2) return COAT_EINVAL;
    if (out_kind != 0 && (QB != 16 || N % 16 != 0 || !c_scale)) return COAT_ESHAPE;
    if (s_dtype < 0 || s_dtype > 2 || (bias && (bias_dtype < 0 || bias_dtype > 2))) return COAT_EDTYPE;
    GemmArgs G;
    G.A = (const uint8_t*)a; G.B = (const uint8_t*)b; G.C = c; G.Cs = c_scale;
    G.sa = scale_a; G.sb = scale_b; G.bias = bias; G.s_dt = s_dtype; G.bias_dt = bias_dtype;
    G.M = (int)M; G.N = (int)N; G.K = (int)K;
    G.tiles_m = (int)((M + BM - 1) / BM);
    G.tiles_n = (int)((N + BN - 1) / BN);
    const int ntiles = G.tiles_m * G.tiles_n;
    const int grid = ((ntiles + 7) / 8) * 8;
    const size_t lds_bytes = 2 * kStageBytes;
    hipStream_t st = (hipStream_t)stream;
#define GEMM_LAUNCH(FA, FB, EP)                                                                                    \
    {                                                                                                              \
        static bool attr_set = false;                                                                              \
        if (!attr_set) {                                                                                           \
            hipError_t e = hipFuncSetAttribute((const void*)k_fp8_gemm<FA, FB, EP>,                                \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);        \
            if (e != hipSuccess) return (int)e;                                                                    \
            attr_set = true;                                                                                       \
        }                                                                                                          \
        hipLaunchKernelGGL((k_fp8_gemm<FA, FB, EP>), dim3(grid), dim3(256), lds_bytes, st, G);                     \
        return coat_launch_status();                                                                               \
    }
#define GEMM_FMT(EP)                                                             \
    if (fmt_a == COAT_E4M3 && fmt_b == COAT_E4M3) GEMM_LAUNCH(0, 0, EP)          \
    if (fmt_a == COAT_E5M2 && fmt_b == COAT_E4M3) GEMM_LAUNCH(1, 0, EP)          \
    if (fmt_a == COAT_E4M3 && fmt_b == COAT_E5M2) GEMM_LAUNCH(0, 1, EP)          \
    if (fmt_a == COAT_E5M2 && fmt_b == COAT_E5M2) GEMM_LAUNCH(1, 1, EP)
    if (out_kind == 0) { GEMM_FMT(kEpiBf16) }
    if (out_kind == 1) { GEMM_FMT(kEpiQuantE4M3) }
    if (out_kind == 2) { GEMM_FMT(kEpiQuantE5M2) }
    return COAT_EINVAL;
}
