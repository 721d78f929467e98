// Per-tensor-scaled FP8 GEMM: argument checks and the choice of kernel instance.  The kernel is gemm_kernel.h; its
// instances are compiled in gemm_bf16.hip, gemm_quant_e4m3.hip, gemm_quant_e5m2.hip and gemm_residual.hip.
#include "gemm_kernel.h"

using namespace coat;

// Validates and launches `count` problems of one shape (count = 1: the plain GEMM).
// `residual` != NULL selects the product + residual epilogues (count 1 only): c is the bf16 sum, c_q / c_scale[0] the
// codes and scales of the sum for out_kind 1 / 2.
static int gemm_launch(int count, const void* const* a, int fmt_a, const void* const* b, int fmt_b, void* const* c,
                       void* const* c_scale, int out_kind, const void* const* scale_a, int sa_dtype,
                       const void* const* scale_b, int sb_dtype, const void* const* bias, int bias_dtype, int64_t M,
                       int64_t N, int64_t K, int QB, void* stream, const void* residual = nullptr, void* c_q = nullptr) {
    if (count < 1 || count > kMaxGroup) return COAT_EINVAL;
    if (M < 0 || N < 0 || K < 0) return COAT_EINVAL;
    if (M * N == 0) return COAT_OK;
    if (!a || !b || !c || !scale_a || !scale_b) return COAT_EINVAL;
    if (M >= (1 << 30) || N >= (1 << 30) || K >= (1 << 30)) return COAT_ESHAPE;
    if (K % 16 != 0) return COAT_ESHAPE;
    if (M * K >= ((int64_t)1 << 31) - 64 || N * K >= ((int64_t)1 << 31) - 64) return COAT_ESHAPE;  // 32-bit buffer offsets
    if ((fmt_a != COAT_E4M3 && fmt_a != COAT_E5M2) || (fmt_b != COAT_E4M3 && fmt_b != COAT_E5M2)) return COAT_EINVAL;
    if (out_kind < 0 || out_kind > 2) return COAT_EINVAL;
    if (out_kind != 0 && ((QB != 16 && QB != 32 && QB != 64) || N % QB != 0 || !c_scale)) return COAT_ESHAPE;
    if (residual) {
        if (count != 1) return COAT_EINVAL;
        if (N % 8 != 0 || N >= (1 << 22) || (out_kind != 0 && (QB != 16 || !c_q))) return COAT_ESHAPE;
        if (!coat_aligned16(residual) || (c_q && !coat_aligned16(c_q))) return COAT_EALIGN;
    }
    if (sa_dtype < 0 || sa_dtype > 2 || sb_dtype < 0 || sb_dtype > 2) return COAT_EDTYPE;
    GemmArgs G = {};
    G.nprob = count;
    bool any_bias = false;
    for (int p = 0; p < count; p++) {
        if (!a[p] || !b[p] || !c[p] || !scale_a[p] || !scale_b[p]) return COAT_EINVAL;
        if (out_kind != 0 && !c_scale[p]) return COAT_ESHAPE;
        if (!coat_aligned16(a[p]) || !coat_aligned16(b[p]) || !coat_aligned16(c[p])) return COAT_EALIGN;
        G.P[p].A = (const uint8_t*)a[p]; G.P[p].B = (const uint8_t*)b[p]; G.P[p].C = c[p];
        G.P[p].Cs = out_kind != 0 ? c_scale[p] : nullptr;
        G.P[p].sa = scale_a[p]; G.P[p].sb = scale_b[p];
        G.P[p].bias = bias ? bias[p] : nullptr;
        any_bias = any_bias || G.P[p].bias;
    }
    if (any_bias && (bias_dtype < 0 || bias_dtype > 2)) return COAT_EDTYPE;
    G.res = residual;
    G.Cq = c_q;
    G.sa_dt = sa_dtype; G.sb_dt = sb_dtype; G.bias_dt = bias_dtype;
    G.M = (int)M; G.N = (int)N; G.K = (int)K;
    G.tiles_m = (int)((M + BM - 1) / BM);
    G.tiles_n = (int)((N + BN - 1) / BN);
    const int ntiles = G.nprob * G.tiles_m * G.tiles_n;
    // persistent grid: one block per CU (the block's LDS ring takes a whole CU's LDS); CU count cached per device
    static std::atomic<int> n_cu_dev[kCoatMaxDevices];
    const int dev = coat_device_index();
    if (dev < 0) return COAT_EINVAL;
    int n_cu = n_cu_dev[dev].load(std::memory_order_relaxed);
    if (n_cu == 0) {
        int v = 0;
        if (hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || v < 8) return COAT_EINVAL;
        n_cu = v & ~7;
        n_cu_dev[dev].store(n_cu, std::memory_order_relaxed);
    }
    const int grid = min(((ntiles + 7) / 8) * 8, n_cu);
    hipStream_t st = (hipStream_t)stream;
    if (residual) return gemm_dispatch_residual(G, fmt_a, fmt_b, out_kind, grid, st);
    if (out_kind == 0) return gemm_dispatch_bf16(G, fmt_a, fmt_b, grid, st);
    if (out_kind == 1) return gemm_dispatch_quant_e4m3(G, fmt_a, fmt_b, QB, grid, st);
    if (out_kind == 2) return gemm_dispatch_quant_e5m2(G, fmt_a, fmt_b, QB, grid, st);
    return COAT_EINVAL;
}

extern "C" int coat_fp8_gemm(const void* a, int fmt_a, const void* b, int fmt_b, void* c, void* c_scale, int out_kind,
                             const void* scale_a, int sa_dtype, const void* scale_b, int sb_dtype, const void* bias,
                             int bias_dtype, int64_t M, int64_t N, int64_t K, int QB, void* stream) {
    return gemm_launch(1, &a, fmt_a, &b, fmt_b, &c, &c_scale, out_kind, &scale_a, sa_dtype, &scale_b, sb_dtype, &bias,
                       bias_dtype, M, N, K, QB, stream);
}

extern "C" int coat_fp8_gemm_residual(const void* a, int fmt_a, const void* b, int fmt_b, const void* residual, void* c,
                                      void* c_q, void* c_scale, int out_kind, const void* scale_a, int sa_dtype,
                                      const void* scale_b, int sb_dtype, const void* bias, int bias_dtype, int64_t M,
                                      int64_t N, int64_t K, void* stream) {
    if (!residual) return COAT_EINVAL;
    return gemm_launch(1, &a, fmt_a, &b, fmt_b, &c, &c_scale, out_kind, &scale_a, sa_dtype, &scale_b, sb_dtype, &bias,
                       bias_dtype, M, N, K, 16, stream, residual, c_q);
}

extern "C" int coat_fp8_gemm_grouped(int count, const void* const* a, int fmt_a, const void* const* b, int fmt_b,
                                     void* const* c, void* const* c_scale, int out_kind, const void* const* scale_a,
                                     int sa_dtype, const void* const* scale_b, int sb_dtype, const void* const* bias,
                                     int bias_dtype, int64_t M, int64_t N, int64_t K, int QB, void* stream) {
    return gemm_launch(count, a, fmt_a, b, fmt_b, c, c_scale, out_kind, scale_a, sa_dtype, scale_b, sb_dtype, bias,
                       bias_dtype, M, N, K, QB, stream);
}
