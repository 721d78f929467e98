// Instances of k_fp8_gemm whose epilogue quantizes the product per 1 x QB group to e4m3 (QB 16, 32 or 64).
#include "gemm_kernel.h"

namespace coat {
template <int QE> static int by_group(const GemmArgs& G, int fmt_a, int fmt_b, int grid, hipStream_t st) {
    if (G.nprob > 1) return gemm_launch_formats<kEpiQuantE4M3, false, QE, true>(G, fmt_a, fmt_b, grid, st);
    return gemm_launch_formats<kEpiQuantE4M3, false, QE, false>(G, fmt_a, fmt_b, grid, st);
}
int gemm_dispatch_quant_e4m3(const GemmArgs& G, int fmt_a, int fmt_b, int QB, int grid, hipStream_t st) {
    if (QB == 16) return by_group<16>(G, fmt_a, fmt_b, grid, st);
    if (QB == 32) return by_group<32>(G, fmt_a, fmt_b, grid, st);
    if (QB == 64) return by_group<64>(G, fmt_a, fmt_b, grid, st);
    return COAT_ESHAPE;
}
}  // namespace coat
