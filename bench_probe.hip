// Measurement kernels of bench.py: built into libcoat_bench_probe.so beside bench.py, never part of libcoat_hip.so.
//
//   bench_hbm_probe   what this GPU's memory delivers to the simplest kernels (copy / read / fill), quoted next to the
//                     nominal 8 TB/s in the benchmark records
//   bench_pattern_probe  the access patterns of the quantizing kernels without their arithmetic: 2-byte elements in, 1-byte
//                     elements out, streaming or as 128 x 128 tiles written in both orientations
//   bench_gemm_clock  the library's FP8 GEMM kernel (coat_amd/csrc/gemm_kernel.h, bf16 epilogue) instantiated with its
//                     PROBE switch: every block records its duration in shader clocks and in ticks of the constant
//                     100 MHz counter, whose ratio is the clock the kernel really runs at
#include "coat_amd/csrc/gemm_kernel.h"

namespace coat {
// One 16-byte access per lane and array, many small blocks (more work per thread was slower for these on gfx950).
// KIND 0: copy (streaming loads), 1: read only (streaming loads; the OR of the data keeps the loads alive), 2: fill.
template <int KIND>
__global__ __launch_bounds__(256) void k_hbm_probe(const uint4* __restrict__ src, uint4* __restrict__ dst, int64_t n16,
                                                   uint32_t* __restrict__ sink) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n16) return;
    if (KIND == 0) dst[i] = ld_stream16(src + i);
    if (KIND == 1) {
        const uint4 v = ld_stream16(src + i);
        if ((v.x | v.y | v.z | v.w) == 0x9E3779B9u) sink[0] = 1;  // practically never true; sink is never read
    }
    if (KIND == 2) dst[i] = make_uint4(0x01010101u, 0x01010101u, 0x01010101u, 0x01010101u);
}

// The memory accesses of a per-tensor division (k_division: one 16-byte load and one 8-byte store per lane and job, two jobs
// per thread) with the arithmetic replaced by two shifts: what the memory system gives that pattern.
__global__ __launch_bounds__(256) void k_narrow_probe(const uint4* __restrict__ src, uint2* __restrict__ dst, int64_t n16) {
    const int64_t base = (int64_t)blockIdx.x * 512 + threadIdx.x;
    uint4 a[2];
#pragma unroll
    for (int u = 0; u < 2; u++) a[u] = src[min(base + u * 256, n16 - 1)];
#pragma unroll
    for (int u = 0; u < 2; u++)
        if (base + u * 256 < n16) dst[base + u * 256] = make_uint2(a[u].x ^ (a[u].y << 3), a[u].z ^ (a[u].w << 5));
}
// The memory accesses of k_division_transpose on 2-byte input: a block of 512 threads takes a 128 x 128 tile, a thread two
// jobs of 16 elements (32 bytes of one row in), and writes 16 bytes of the same row of q [M, N] and 16 bytes of a row of
// q^T [N, M] per job, all loads before the first store; no LDS, no conversion (the bytes written are not a transpose).
__global__ __launch_bounds__(512) void k_tile_probe(const uint8_t* __restrict__ x, uint8_t* __restrict__ q,
                                                    uint8_t* __restrict__ qt, int64_t M, int64_t N) {
    const int64_t tiles_n = N / 128;
    const int64_t m0 = (blockIdx.x / tiles_n) * 128, n0 = (blockIdx.x % tiles_n) * 128;
    uint4 a[2][2];
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int job = j * 512 + threadIdx.x, r = job >> 3, c = job & 7;
        const uint4* p = (const uint4*)(x + ((m0 + r) * N + n0 + c * 16) * 2);
        a[j][0] = p[0];
        a[j][1] = p[1];
    }
#pragma unroll
    for (int j = 0; j < 2; j++) {
        const int job = j * 512 + threadIdx.x, r = job >> 3, c = job & 7;
        const uint4 o = make_uint4(a[j][0].x ^ a[j][1].x, a[j][0].y ^ a[j][1].y, a[j][0].z ^ a[j][1].z, a[j][0].w ^ a[j][1].w);
        *(uint4*)(q + (m0 + r) * N + n0 + c * 16) = o;
        *(uint4*)(qt + (n0 + r) * M + m0 + c * 16) = o;
    }
}
}  // namespace coat

using namespace coat;

// kind 0: `src` holds M x N 2-byte elements, `dst` receives M x N bytes, streaming (M * N % 8 == 0).
// kind 1: the same input as 128 x 128 tiles, `dst` receives M x N bytes in row-major and `dst_t` N x M bytes in the transposed
// tile positions (M % 128 == 0, N % 128 == 0).
extern "C" int bench_pattern_probe(int kind, const void* src, void* dst, void* dst_t, int64_t M, int64_t N, void* stream) {
    if (kind < 0 || kind > 1 || !src || !dst || M <= 0 || N <= 0) return COAT_EINVAL;
    if (!coat_aligned16(src) || !coat_aligned16(dst)) return COAT_EALIGN;
    hipStream_t st = (hipStream_t)stream;
    if (kind == 0) {
        if (M * N % 8 != 0) return COAT_ESHAPE;
        const int64_t n16 = M * N / 8, blocks = (n16 + 511) / 512;
        if (blocks >= ((int64_t)1 << 31)) return COAT_ESHAPE;
        hipLaunchKernelGGL(k_narrow_probe, dim3((unsigned)blocks), dim3(256), 0, st, (const uint4*)src, (uint2*)dst, n16);
    } else {
        if (!dst_t || !coat_aligned16(dst_t)) return COAT_EINVAL;
        if (M % 128 != 0 || N % 128 != 0 || (M / 128) * (N / 128) >= ((int64_t)1 << 31)) return COAT_ESHAPE;
        hipLaunchKernelGGL(k_tile_probe, dim3((unsigned)((M / 128) * (N / 128))), dim3(512), 0, st, (const uint8_t*)src,
                           (uint8_t*)dst, (uint8_t*)dst_t, M, N);
    }
    return coat_launch_status();
}

// kind 0 copies `bytes` from src to dst, 1 reads src (dst: 4 bytes that are practically never written), 2 fills dst.
extern "C" int bench_hbm_probe(int kind, const void* src, void* dst, int64_t bytes, void* stream) {
    if (kind < 0 || kind > 2 || bytes < 0 || bytes % 16 != 0) return COAT_EINVAL;
    if (bytes == 0) return COAT_OK;
    if ((kind != 2 && !src) || !dst) return COAT_EINVAL;
    if (!coat_aligned16(src) || !coat_aligned16(dst)) return COAT_EALIGN;
    const int64_t n16 = bytes / 16, blocks = (n16 + 255) / 256;
    if (blocks >= ((int64_t)1 << 31)) return COAT_ESHAPE;
    hipStream_t st = (hipStream_t)stream;
    if (kind == 0) hipLaunchKernelGGL((k_hbm_probe<0>), dim3((unsigned)blocks), dim3(256), 0, st, (const uint4*)src, (uint4*)dst, n16, nullptr);
    if (kind == 1) hipLaunchKernelGGL((k_hbm_probe<1>), dim3((unsigned)blocks), dim3(256), 0, st, (const uint4*)src, nullptr, n16, (uint32_t*)dst);
    if (kind == 2) hipLaunchKernelGGL((k_hbm_probe<2>), dim3((unsigned)blocks), dim3(256), 0, st, nullptr, (uint4*)dst, n16, nullptr);
    return coat_launch_status();
}

// C bf16 [M, N] = A[M, K] (fmt_a: coat_fp8) . B[N, K]^T (e4m3) * sa * sb (bf16 scalars); N % 8 == 0, K % 16 == 0.
// `probe`: 2 x 256 uint64 in device memory; block b leaves (shader clocks, 100 MHz ticks) in probe[2b], probe[2b + 1].
extern "C" int bench_gemm_clock(const void* a, int fmt_a, const void* b, void* c, const void* sa, const void* sb, int64_t M,
                                int64_t N, int64_t K, unsigned long long* probe, void* stream) {
    if (!a || !b || !c || !sa || !sb || !probe || M <= 0 || N <= 0 || K <= 0 || N % 8 != 0 || K % 16 != 0) return COAT_EINVAL;
    if (M * K >= ((int64_t)1 << 31) - 64 || N * K >= ((int64_t)1 << 31) - 64) return COAT_ESHAPE;
    GemmArgs G = {};
    G.nprob = 1;
    G.P[0].A = (const uint8_t*)a; G.P[0].B = (const uint8_t*)b; G.P[0].C = c;
    G.P[0].sa = sa; G.P[0].sb = sb;
    G.sa_dt = kBF16; G.sb_dt = kBF16;
    G.M = (int)M; G.N = (int)N; G.K = (int)K;
    G.tiles_m = (int)((M + BM - 1) / BM);
    G.tiles_n = (int)((N + BN - 1) / BN);
    G.probe = probe;
    int dev = 0, n_cu = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n_cu, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return COAT_EINVAL;
    n_cu &= ~7;
    if (n_cu < 8 || n_cu > 256) return COAT_EINVAL;
    const int grid = min(((G.tiles_m * G.tiles_n + 7) / 8) * 8, n_cu);
    hipStream_t st = (hipStream_t)stream;
    if (fmt_a == COAT_E4M3) return gemm_launch_instance<0, 0, kEpiBf16, true, 16, false, true>(G, grid, st);
    if (fmt_a == COAT_E5M2) return gemm_launch_instance<1, 0, kEpiBf16, true, 16, false, true>(G, grid, st);
    return COAT_EINVAL;
}
