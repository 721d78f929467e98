// Per-tensor-scaled FP8 GEMM on CDNA4 MFMA:  C[M,N] = (A[M,K] . B[N,K]^T) * (sA * sB) (+ bias), fp32 accumulate.
//
// Replaces _fp8matmul_kernel (coat/activation/real_quantization/linear.py:61-169).  Both operands are
// K-contiguous ("A row-major times the transpose of a row-major B"), which is the only form the reference uses:
// every tensor is kept in both orientations so that forward, dgrad and wgrad are all of this form
// (linear.py:253-302).  Operand formats are independent (e4m3 or e5m2 each: gradients are e5m2).
//
// Tiling: 256 x 256 per 256-thread block, 2 x 2 waves, each wave 128 x 128 as 4 x 4 tiles of
// v_mfma_f32_32x32x64_f8f6f4; K advances in 64-byte slabs (one MFMA K-step).  LDS is a ring of four slabs
// (4 x 32 KiB) filled straight from global memory (buffer_load ... lds, no register staging) three slabs ahead of
// the one being multiplied; 16-byte chunks are XOR-swizzled with the row so that the 32-byte-per-lane fragment reads
// are conflict-free.  Fragments are double-buffered in registers: those of slab k+1 are read while the 16 MFMAs of
// slab k issue.  One barrier per slab.  The MFMA takes the B tile as its first operand, so a lane ends up holding
// 4 consecutive n for one m per accumulator quad: bf16 rows are packed 4 at a time, and a 1 x 16 quantization group
// is two quads in each of the lanes l and l^32.
// Block ids are remapped so that the 8 XCDs (round-robin block dispatch) each work on a contiguous band of
// tiles, ordered in panels of 8 tile-rows, which keeps A / B slabs hot in that XCD's L2.
#include <stdlib.h>

#include "coat_device.h"
#include "coat_host.h"

namespace coat {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int NSTAGE = 5;                      // LDS ring of K-slabs (5 x 32 KiB = the whole 160 KiB LDS)
constexpr int PREFETCH = 4;                    // slabs in flight ahead of the one being multiplied
constexpr int kStageBytes = (BM + BN) * BK;    // 32 KiB
constexpr int kLdsBytes = NSTAGE * kStageBytes;

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
    int remap;  // 1: XCD-aware block -> tile mapping
};

// A slab row is 64 bytes = four 16-byte chunks.  A 16-byte-per-lane LDS read is served 16 lanes (256 bytes, 64
// banks) per cycle, so 16 consecutive rows reading the same chunk must land in 16 different 16-byte slots modulo 256:
// row & 3 already selects the 64-byte quarter, and placing chunk c of row r at position c ^ ((r >> 2) & 3) makes the
// four rows that share a quarter use four different slots.  (SQ_LDS_BANK_CONFLICT: 0 with this layout, 50 % of the
// LDS cycles with c ^ ((r >> 1) & 3), 75 % with c ^ (r & 3).)
__device__ __forceinline__ int swz_chunk(int row, int chunk) { return chunk ^ ((row >> 2) & 3); }

typedef __attribute__((address_space(3))) void* lds_ptr_t;

// s_waitcnt vmcnt(N) only (expcnt / lgkmcnt left at their maxima), gfx9 encoding.
#define COAT_WAIT_VMCNT(N) __builtin_amdgcn_s_waitcnt(((N) & 0xF) | (0x7 << 4) | (0xF << 8) | ((((N) >> 4) & 0x3) << 14))

// NWN = waves along N (2: four waves of 128 x 128, one per SIMD; 4: eight waves of 128 x 64, two per SIMD).
template <int FMT_A, int FMT_B, int EPI, int NWN>
__global__ __launch_bounds__(128 * NWN) void k_fp8_gemm(GemmArgs G) {
    constexpr int NW = 2 * NWN;               // waves per block
    constexpr int TJ = BN / (NWN * 32);       // n-tiles per wave (4 or 2); m-tiles per wave is always 4
    constexpr int LROWS = BM / NW;            // slab rows each wave fetches per matrix (64 or 32)
    constexpr int LI = LROWS / 16;            // load instructions per wave per matrix per slab
    constexpr int LOADS = 2 * LI;             // buffer loads per wave per slab
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / NWN, wn = wave % NWN;

    // ---- XCD-aware tile mapping
    const int ntiles = G.tiles_m * G.tiles_n;
    const int per_xcd = (ntiles + 7) / 8;
    int tile = G.remap ? (blockIdx.x % 8) * per_xcd + blockIdx.x / 8 : blockIdx.x;
    if (tile >= ntiles) return;
    constexpr int GROUP_M = 8;
    const int width = GROUP_M * G.tiles_n;
    const int group = tile / width;
    const int gsize = min(G.tiles_m - group * GROUP_M, GROUP_M);
    const int tm = group * GROUP_M + (tile % width) % gsize;
    const int tn = (tile % width) / gsize;
    const int m0 = tm * BM, n0 = tn * BN;

    // ---- global -> LDS without passing through registers: buffer_load_dwordx4 ... lds.
    // One wave instruction fills 1 KiB of LDS contiguously (lane i at +16 i) = 16 slab rows; the lane picks the global
    // chunk that belongs at its position under the swizzle.  Out-of-range rows / K-tail chunks use an offset beyond
    // num_records, for which the buffer load returns zeros.
    const __amdgpu_buffer_rsrc_t rsrcA = __builtin_amdgcn_make_buffer_rsrc((void*)G.A, 0, G.M * G.K, 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrcB = __builtin_amdgcn_make_buffer_rsrc((void*)G.B, 0, G.N * G.K, 0x00020000);
    int offA[LI], offB[LI], kc[LI];
#pragma unroll
    for (int i = 0; i < LI; i++) {
        const int row = wave * LROWS + i * 16 + (lane >> 2);
        const int c = swz_chunk(row, lane & 3);
        kc[i] = c * 16;
        offA[i] = (m0 + row < G.M) ? (m0 + row) * G.K + c * 16 : -1;
        offB[i] = (n0 + row < G.N) ? (n0 + row) * G.K + c * 16 : -1;
    }
    auto issue_slab = [&](int kt) {
        const int stage = kt % NSTAGE;
        const int k0 = kt * BK;
        uint8_t* sA = lds + stage * kStageBytes + wave * LROWS * BK;
        uint8_t* sB = sA + BM * BK;
#pragma unroll
        for (int i = 0; i < LI; i++) {
            const bool kin = k0 + kc[i] < G.K;
            const int oa = (kin && offA[i] >= 0) ? offA[i] + k0 : 0x7FFFFFFF;
            const int ob = (kin && offB[i] >= 0) ? offB[i] + k0 : 0x7FFFFFFF;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrcA, (lds_ptr_t)(sA + i * 16 * BK), 16, oa, 0, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrcB, (lds_ptr_t)(sB + i * 16 * BK), 16, ob, 0, 0, 0);
        }
    };
    // fragment addresses (bytes inside a stage) for this lane: row = tile base + lane%32, 32-byte half = lane/32
    int fa_off[4][2], fb_off[TJ][2];
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const int c = 2 * (lane >> 5) + h;
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const int rowa = wm * 128 + t * 32 + (lane & 31);
            fa_off[t][h] = rowa * BK + (swz_chunk(rowa, c) << 4);
        }
#pragma unroll
        for (int t = 0; t < TJ; t++) {
            const int rowb = wn * (TJ * 32) + t * 32 + (lane & 31);
            fb_off[t][h] = BM * BK + rowb * BK + (swz_chunk(rowb, c) << 4);
        }
    }

    v16f acc[TJ][4];  // [n-tile j][m-tile i]
#pragma unroll
    for (int j = 0; j < TJ; j++)
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[j][i][r] = 0.0f;

    const int nslab = (G.K + BK - 1) / BK;
    auto load_frags = [&](int kt, v8i* fa, v8i* fb) {
        const uint8_t* st = lds + (kt % NSTAGE) * kStageBytes;
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const uint4 a0 = *(const uint4*)(st + fa_off[t][0]), a1 = *(const uint4*)(st + fa_off[t][1]);
            fa[t] = (v8i){(int)a0.x, (int)a0.y, (int)a0.z, (int)a0.w, (int)a1.x, (int)a1.y, (int)a1.z, (int)a1.w};
        }
#pragma unroll
        for (int t = 0; t < TJ; t++) {
            const uint4 b0 = *(const uint4*)(st + fb_off[t][0]), b1 = *(const uint4*)(st + fb_off[t][1]);
            fb[t] = (v8i){(int)b0.x, (int)b0.y, (int)b0.z, (int)b0.w, (int)b1.x, (int)b1.y, (int)b1.z, (int)b1.w};
        }
    };
    // prologue: PREFETCH slabs in flight (slabs past the end are all-zero fills, which keeps the counts uniform)
#pragma unroll
    for (int p = 0; p < PREFETCH; p++) issue_slab(p);
    COAT_WAIT_VMCNT(LOADS * (PREFETCH - 1));  // slab 0 has landed (this wave's part)
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    v8i fa0[4], fb0[TJ], fa1[4], fb1[TJ];
    load_frags(0, fa0, fb0);
    // One step: wait for this wave's part of slab kt+1, barrier (slab kt+1 is now complete and visible, and every wave
    // has issued the MFMAs of slab kt-1, i.e. finished reading that stage), refill that stage with slab kt+PREFETCH,
    // fetch the fragments of slab kt+1 and issue the MFMAs of slab kt while they arrive.
    auto step = [&](int kt, v8i* fc_a, v8i* fc_b, v8i* fn_a, v8i* fn_b) {
        COAT_WAIT_VMCNT(LOADS * (PREFETCH - 2));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        issue_slab(kt + PREFETCH);
        load_frags(kt + 1, fn_a, fn_b);
#pragma unroll
        for (int j = 0; j < TJ; j++)
#pragma unroll
            for (int i = 0; i < 4; i++)
                acc[j][i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fc_b[j], fc_a[i], acc[j][i], FMT_B, FMT_A, 0, 0, 0, 0);
    };
    for (int kt = 0; kt < nslab; kt += 2) {
        step(kt, fa0, fb0, fa1, fb1);
        if (kt + 1 < nslab) step(kt + 1, fa1, fb1, fa0, fb0);
    }
    COAT_WAIT_VMCNT(0);  // drain the zero-fill slabs before the block may exit

    // ---- epilogue
    const float scale = load_rt_f32(G.sa, 0, G.s_dt) * load_rt_f32(G.sb, 0, G.s_dt);
    if (EPI != kEpiBf16) enable_fp8_saturation();
    const int half = lane >> 5;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int m = m0 + wm * 128 + i * 32 + (lane & 31);
#pragma unroll
        for (int j = 0; j < TJ; j++) {
            const int nb = n0 + wn * (TJ * 32) + j * 32 + 4 * half;  // + 8*q + {0..3}
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
                    const int ng = n0 + wn * (TJ * 32) + j * 32 + 16 * g2;  // first n of the group
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

#ifndef COAT_GEMM_NWN
#define COAT_GEMM_NWN 4
#endif

extern "C" int coat_fp8_gemm(const void* a, int fmt_a, const void* b, int fmt_b, void* c, void* c_scale, int out_kind,
                             const void* scale_a, const void* scale_b, int s_dtype, const void* bias, int bias_dtype,
                             int64_t M, int64_t N, int64_t K, int QB, void* stream) {
    if (M < 0 || N < 0 || K < 0) return COAT_EINVAL;
    if (M * N == 0) return COAT_OK;
    if (!a || !b || !c || !scale_a || !scale_b) return COAT_EINVAL;
    if (M >= (1 << 30) || N >= (1 << 30) || K >= (1 << 30)) return COAT_ESHAPE;
    if (K % 16 != 0) return COAT_ESHAPE;
    if (M * K >= ((int64_t)1 << 31) - 64 || N * K >= ((int64_t)1 << 31) - 64) return COAT_ESHAPE;  // 32-bit buffer offsets
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
    G.remap = getenv("COAT_GEMM_NOREMAP") ? 0 : 1;
    const int ntiles = G.tiles_m * G.tiles_n;
    const int grid = ((ntiles + 7) / 8) * 8;
    const size_t lds_bytes = kLdsBytes;
    hipStream_t st = (hipStream_t)stream;
#define GEMM_LAUNCH(FA, FB, EP)                                                                                    \
    {                                                                                                              \
        static bool attr_set = false;                                                                              \
        if (!attr_set) {                                                                                           \
            hipError_t e = hipFuncSetAttribute((const void*)k_fp8_gemm<FA, FB, EP, COAT_GEMM_NWN>,                 \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes);        \
            if (e != hipSuccess) return (int)e;                                                                    \
            attr_set = true;                                                                                       \
        }                                                                                                          \
        hipLaunchKernelGGL((k_fp8_gemm<FA, FB, EP, COAT_GEMM_NWN>), dim3(grid), dim3(128 * COAT_GEMM_NWN), lds_bytes, st, G); \
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
