// Instances of k_fp8_gemm whose epilogue adds a bf16 tensor to the rounded product (and quantizes the sum per 1 x 16 group).
#include "gemm_kernel.h"

namespace coat {
int gemm_dispatch_residual(const GemmArgs& G, int fmt_a, int fmt_b, int out_kind, int grid, hipStream_t st) {
    if (out_kind == 0) return gemm_launch_formats<kEpiResBf16, true, 16, false>(G, fmt_a, fmt_b, grid, st);
    if (out_kind == 1) return gemm_launch_formats<kEpiResQuantE4M3, true, 16, false>(G, fmt_a, fmt_b, grid, st);
    if (out_kind == 2) return gemm_launch_formats<kEpiResQuantE5M2, true, 16, false>(G, fmt_a, fmt_b, grid, st);
    return COAT_EINVAL;
}
}  // namespace coat
