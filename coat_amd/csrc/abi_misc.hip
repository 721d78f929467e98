// Version and error strings of the C ABI, and the memory-bandwidth probe the benchmarks quote next to the nominal peak.
#include "coat_device.h"
#include "coat_host.h"

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
}  // namespace coat

extern "C" int coat_hbm_probe(int kind, const void* src, void* dst, int64_t bytes, void* stream) {
    if (kind < 0 || kind > 2 || bytes < 0 || bytes % 16 != 0) return COAT_EINVAL;
    if (bytes == 0) return COAT_OK;
    if ((kind != 2 && !src) || !dst) return COAT_EINVAL;  // kind 1 writes at most 4 bytes to dst
    if (!coat_aligned16(src) || !coat_aligned16(dst)) return COAT_EALIGN;
    const int64_t n16 = bytes / 16, blocks = (n16 + 255) / 256;
    if (blocks >= ((int64_t)1 << 31)) return COAT_ESHAPE;
    hipStream_t st = (hipStream_t)stream;
    if (kind == 0) hipLaunchKernelGGL((coat::k_hbm_probe<0>), dim3((unsigned)blocks), dim3(256), 0, st, (const uint4*)src, (uint4*)dst, n16, nullptr);
    if (kind == 1) hipLaunchKernelGGL((coat::k_hbm_probe<1>), dim3((unsigned)blocks), dim3(256), 0, st, (const uint4*)src, nullptr, n16, (uint32_t*)dst);
    if (kind == 2) hipLaunchKernelGGL((coat::k_hbm_probe<2>), dim3((unsigned)blocks), dim3(256), 0, st, nullptr, (uint4*)dst, n16, nullptr);
    return coat_launch_status();
}

extern "C" const char* coat_version(void) { return "coat_amd 0.1 (gfx950)"; }

extern "C" const char* coat_status_string(int status) {
    switch (status) {
        case COAT_OK: return "ok";
        case COAT_EINVAL: return "invalid argument (null pointer, negative size or unknown enum)";
        case COAT_ESHAPE: return "shape contract violated (group / tile divisibility or scale length)";
        case COAT_EDTYPE: return "unsupported dtype combination";
        case COAT_EQGROUP: return "Only Support 128 per-group quantization currently";
        case COAT_EALIGN: return "tensor base address must be 16-byte aligned";
        default: return status > 0 ? hipGetErrorString((hipError_t)status) : "unknown coat status";
    }
}
