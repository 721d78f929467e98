// Instances of k_fp8_gemm with the bf16 epilogue (16-byte stores when rows of C start 16-byte aligned).
#include "gemm_kernel.h"

namespace coat {
int gemm_dispatch_bf16(const GemmArgs& G, int fmt_a, int fmt_b, int grid, hipStream_t st) {
    const bool v16 = (G.N & 7) == 0, grouped = G.nprob > 1;
    if (v16 && grouped) return gemm_launch_formats<kEpiBf16, true, 16, true>(G, fmt_a, fmt_b, grid, st);
    if (v16) return gemm_launch_formats<kEpiBf16, true, 16, false>(G, fmt_a, fmt_b, grid, st);
    if (grouped) return gemm_launch_formats<kEpiBf16, false, 16, true>(G, fmt_a, fmt_b, grid, st);
    return gemm_launch_formats<kEpiBf16, false, 16, false>(G, fmt_a, fmt_b, grid, st);
}
}  // namespace coat
