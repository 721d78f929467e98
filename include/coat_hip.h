/* C ABI of libcoat_hip.so: the MI355X (gfx950) kernels of COAT's FP8 hot path.
 *
 * Every entry point
 *   - takes raw device pointers, sizes, small enums and the HIP stream to launch on
 *     (`stream` is a hipStream_t passed as void*; NULL is the default stream);
 *   - allocates nothing, frees nothing and never synchronises the host; the only state kept between calls is per-device
 *     and idempotent (atomic flags "this kernel's LDS limit has been raised", the cached CU count, the address of the
 *     static scratch array of coat_fp8_rmsnorm_backward_static), so entry points may be called from several host threads;
 *   - returns COAT_OK (0), a negative COAT_E* code for a rejected argument, or the positive
 *     hipError_t of a failed launch.
 * Tensors are row-major and contiguous.  "pg" = per-group scales, one per 1 x QB group along the
 * last dimension; "pt" = per-tensor scale, a single element in device memory.
 *
 * Citations name the reference interface each entry point replaces (paths relative to the
 * NVlabs/COAT repository; rq/ = coat/activation/real_quantization/).
 */
#ifndef COAT_HIP_H
#define COAT_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum coat_status {
    COAT_OK = 0,
    COAT_EINVAL = -1,   /* null pointer, negative size, unknown enum */
    COAT_ESHAPE = -2,   /* divisibility / shape contract violated (N % QB, M % QB for transposes, ...) */
    COAT_EDTYPE = -3,   /* dtype combination not supported */
    COAT_EQGROUP = -4,  /* optimizer group size other than 128 (fp8_adamw_expand_cuda_kernel.cu:221) */
    COAT_EALIGN = -5    /* a tensor base address is not 16-byte aligned */
};

enum coat_dtype { COAT_F32 = 0, COAT_BF16 = 1, COAT_F16 = 2 };
enum coat_fp8 { COAT_E4M3 = 0, COAT_E5M2 = 1 }; /* torch.float8_e4m3fn / torch.float8_e5m2 (rq/common.py:22-27) */

/* The device-wide maximum that links a producer kernel to the per-tensor division after it ("s_max", "amax" below) is not
 * one word but COAT_MAX_WORDS fp32 words: COAT_MAX_SLOTS slots, one 128-byte line apart (atomics on one line are carried
 * out one at a time; spreading the blocks of a launch over 16 lines takes their serialisation out of the kernel's
 * duration).  The caller zero-fills the buffer (or leaves a previous partial maximum in it); block b of a producer merges
 * into word COAT_MAX_SLOT_STRIDE * (b % COAT_MAX_SLOTS); the maximum is the largest of those COAT_MAX_SLOTS words, which
 * is what the consuming entry points (coat_fp8_division_from_max, coat_fp8_*_division) compute for themselves. */
#define COAT_MAX_SLOTS 16
#define COAT_MAX_SLOT_STRIDE 32
#define COAT_MAX_WORDS (COAT_MAX_SLOTS * COAT_MAX_SLOT_STRIDE)

/* Bumped whenever an entry point's argument list or the size of a buffer it writes changes (2: every s_max / amax
 * argument became COAT_MAX_WORDS words; 3: coat_fp8_gemm_residual, coat_fp8_rmsnorm_backward_add and coat_attention_forward_bf16 added,
 * coat_hbm_probe removed; 4: coat_rope_bf16 and coat_attention_forward_bf16 take a maximum buffer, the multi-tensor optimizer
 * steps and coat_fp8_layernorm_backward_add added; 5: coat_fp8_quantize_perblock added).  A caller compiled against this header checks coat_abi_version() == COAT_ABI_VERSION when it
 * loads the library. */
#define COAT_ABI_VERSION 5
int coat_abi_version(void);
const char* coat_version(void);
const char* coat_status_string(int status);

/* ---- quantize family -------------------------------------------------------------------------- */

/* rq/_quantize.py:120 fp8_quantize (kernel :37-113): q = fp8(x / s32), s = (amax_g + 1e-10) / fp8max.
 * x [M,N] x_dtype -> q [M,N] fp8, s [M,N/QB] s_dtype.  QB in {16,32,64,128}, N % QB == 0. */
int coat_fp8_quantize(const void* x, int x_dtype, void* q, void* s, int s_dtype, int64_t M, int64_t N, int QB,
                      int fp8, void* stream);

/* rq/_quantize_transpose.py:175 fp8_quantize_transpose (kernel :39-167): the above for x and for x^T
 * (groups of QB along M).  qt [N,M], st [N,M/QB].  Also M % QB == 0. */
int coat_fp8_quantize_transpose(const void* x, int x_dtype, void* q, void* s, void* qt, void* st, int s_dtype,
                                int64_t M, int64_t N, int QB, int fp8, void* stream);

/* rq/_quantize_perblock.py:107 fp8_quantize_perblock (kernel :33-104), rq/_quantize_perblock_transpose.py:136
 * fp8_quantize_perblock_transpose (kernel :33-133) and rq/_quantize_perblock_transpose_pergroup.py:175
 * fp8_quantize_perblock_transpose_pergroup (kernel :33-172): one scale per QB x QB block, s = (amax_block + 1e-10) / fp8max,
 * q = fp8(x / s32); optionally the transposed codes and scales, and the 1 x QB per-group quantization of the same input.
 * x [M,N] x_dtype; outputs in pairs, a pair is produced when both pointers are given (at least one pair):
 *   q [M,N] fp8 + s [M/QB, N/QB];  qt [N,M] fp8 + st [N/QB, M/QB];  qpg [M,N] fp8 + spg [M, N/QB]   (scales: s_dtype).
 * QB in {16,32,64,128}, M % QB == 0, N % QB == 0. */
int coat_fp8_quantize_perblock(const void* x, int x_dtype, void* q, void* s, void* qt, void* st, void* qpg, void* spg,
                               int s_dtype, int64_t M, int64_t N, int QB, int fp8, void* stream);

/* rq/_quantize_pertensor.py:46-103 (+ the `s_y.max()` at :139): per-group scales and their maximum.
 * s_pg [M,N/QB] s_dtype (may be NULL when only the maximum is wanted); s_max: COAT_MAX_WORDS fp32 in device
 * memory that must hold 0.0f (or a previous partial maximum) on entry and receive max(s32) by
 * atomic max; the largest of the slots, rounded to s_dtype, is the reference's `s_y.max()`. */
int coat_fp8_group_scales(const void* x, int x_dtype, void* s_pg, int s_dtype, float* s_max, int64_t M, int64_t N,
                          int QB, int fp8, void* stream);

/* rq/_division.py:178-179: s = (x.abs().max() + 1e-10) / fp8max evaluated in x's dtype.
 * amax: COAT_MAX_WORDS fp32 in device memory holding 0.0f on entry; the slots receive max|x| by atomic max. */
int coat_absmax(const void* x, int x_dtype, float* amax, int64_t numel, void* stream);

/* rq/_division.py:153 fp8_division (kernel :45-126, non-stochastic) and
 * rq/_division_transpose.py:147 fp8_division_transpose (kernel :48-144): q = fp8(x / float(*s)).
 * s: one element of s_dtype in device memory.  q [M,N] and/or qt [N,M]; either may be NULL
 * (qt NULL = fp8_division; q NULL = only_transposed=True). */
int coat_fp8_division(const void* x, int x_dtype, const void* s, int s_dtype, void* q, void* qt, int64_t M,
                      int64_t N, int fp8, void* stream);

/* The same division fed with the producer kernel's fp32 maximum of the group scales (the COAT_MAX_WORDS buffer that
 * coat_fp8_group_scales and the fused kernels merge their atomics into): the kernel rounds the maximum to s_dtype, divides by
 * that value and stores it to s_out (one element of s_dtype) for the consumers.  Replaces "convert the maximum to bf16 on
 * the host side, then divide" (the reference's s_y.max() at rq/_quantize_pertensor.py:139 and the like) by one launch. */
int coat_fp8_division_from_max(const void* x, int x_dtype, const float* s_max, void* s_out, int s_dtype, void* q, void* qt,
                               int64_t M, int64_t N, int fp8, void* stream);

/* The same two entry points with stochastic=True (rq/_division.py:96-112 and :130-150 _stochastic_rounding;
 * rq/_division_transpose.py:103-119): the quotient of element i (linear index in x) is moved up by
 * noise_i * (one FP8 step of its binade), clamped to the binade, then rounded to nearest.  noise_i is Triton's
 * tl.rand(seed, i): Philox-4x32-10, key = seed, counter = (i, 0, 0, 0), first word mapped to [0, 1).  The reference
 * hard-codes seed 0.  M * N <= 2^32 (the counter is the 32-bit index). */
int coat_fp8_division_stochastic(const void* x, int x_dtype, const void* s, int s_dtype, void* q, void* qt, int64_t M,
                                 int64_t N, int fp8, uint64_t seed, void* stream);

/* rq/_transpose.py:85 fp8_transpose (kernel :39-82): byte transpose, x [M,N] -> y [N,M]. */
int coat_fp8_transpose(const void* x, void* y, int64_t M, int64_t N, void* stream);

/* rq/_dequantize.py:119 fp8_dequantize (kernel :44-116): y = bf16(float(q) * float(s_pg)). */
int coat_fp8_dequantize(const void* q, int fp8, const void* s, int s_dtype, void* y, int64_t M, int64_t N, int QB,
                        void* stream);

/* ---- fused element-wise kernels -----------------------------------------------------------------
 * Inputs x* are per-group FP8 ([M,N] codes + [M,N/QB] scales of s_dtype); g is a bf16 gradient.
 * "value" outputs y are bf16 [M,N]; s_y (optional, may be NULL) receives the bf16 per-group scales
 * (amax_g + 1e-10) / fp8max(fp8_out) of the fp32 value; s_max (optional) is a zero-initialised buffer of COAT_MAX_WORDS
 * fp32 that receives their maximum (the per-tensor scale of the division that follows in the reference). */

/* rq/silu_fwd.py:152 fp8_silu_forward (kernel :47-149): y = per-group fp8(silu(x)), same fp8 type as x; s_y in s_dtype,
 * the dtype of the input scales (:166-167), unlike the bf16 s_y of the other kernels of this block. */
int coat_fp8_silu_forward(const void* x, int fp8, const void* s_x, int s_dtype, void* y, void* s_y, int64_t M,
                          int64_t N, int QB, void* stream);
/* rq/silu_bwd.py:170 fp8_silu_backward (kernel :47-167): y = bf16((sig + x*sig*(1-sig)) * g). */
int coat_fp8_silu_backward(const void* x, int fp8_in, const void* s_x, int s_dtype, const void* g, void* y, void* s_y,
                           float* s_max, int fp8_out, int64_t M, int64_t N, int QB, void* stream);
/* rq/mul_fwd.py:191 fp8_mul_forward (kernel :51-188): y = bf16(x1 * x2). */
int coat_fp8_mul_forward(const void* x1, const void* s_x1, const void* x2, const void* s_x2, int fp8_in, int s_dtype,
                         void* y, void* s_y, float* s_max, int64_t M, int64_t N, int QB, void* stream);
/* rq/mul_bwd.py:221 fp8_mul_backward (kernel :49-218): y1 = bf16(g * x2); y2 = bf16(g * x1) with scales. */
int coat_fp8_mul_backward(const void* x1, const void* s_x1, const void* x2, const void* s_x2, int fp8_in, int s_dtype,
                          const void* g, void* y1, void* y2, void* s_y2, float* s_max, int fp8_out, int64_t M,
                          int64_t N, int QB, void* stream);
/* rq/gelu_fwd.py:152 fp8_gelu_forward (kernel :47-149): y = bf16(x * (1 + erf(x / sqrt 2)) / 2). */
int coat_fp8_gelu_forward(const void* x, int fp8, const void* s_x, int s_dtype, void* y, void* s_y, float* s_max,
                          int64_t M, int64_t N, int QB, void* stream);
/* rq/gelu_bwd.py:173 fp8_gelu_backward (kernel :47-170): y = bf16((cdf + x * exp(-x^2/2) / sqrt(2 pi)) * g). */
int coat_fp8_gelu_backward(const void* x, int fp8_in, const void* s_x, int s_dtype, const void* g, void* y, void* s_y,
                           float* s_max, int fp8_out, int64_t M, int64_t N, int QB, void* stream);
/* rq/add_fwd.py:162 fp8_add_Ifp_Ifp_Ofp_Og16 (kernel :46-159): bf16 x1, x2 -> y = bf16(x1 + x2) and the
 * per-group FP8 (q, s_q) of the fp32 sum. */
int coat_fp8_add_fwd(const void* x1, const void* x2, void* y, void* q, void* s_q, int fp8_out, int64_t M, int64_t N,
                     int QB, void* stream);
/* rq/add_bwd.py:147 fp8_add_Ifp_Ifp_Ofp_Opt (kernel :48-144): y = bf16(x1 + x2), scales of the fp32 sum. */
int coat_fp8_add_bwd(const void* x1, const void* x2, void* y, void* s_y, float* s_max, int fp8_out, int64_t M,
                     int64_t N, int QB, void* stream);

/* SiLU(gate) * up in one pass; bit-identical to the reference's two-kernel chains, which re-read the FP8 SiLU output
 * (forward: rq/silu_fwd.py:152 then rq/mul_fwd.py:191) and round-trip the bf16 gradient of the product (backward:
 * rq/mul_bwd.py:221 then rq/silu_bwd.py:170).  No single counterpart in the reference; used by the MLP module.
 * forward: q_silu / s_silu = per-group FP8 SiLU(gate) with bf16 scales (saved for backward), y = bf16 product of the
 * dequantized SiLU and up (may be NULL: the maximum alone, for coat_fp8_product_division), s_max (COAT_MAX_WORDS words,
 * as above) receives the max of the product's fp32 group scales (fp8 = format of gate / up / silu). */
int coat_fp8_silu_mul_forward(const void* gate, const void* s_gate, const void* up, const void* s_up, int fp8,
                              int s_dtype, void* q_silu, void* s_silu, void* y, float* s_max, int64_t M, int64_t N,
                              int QB, int64_t in_pitch, int64_t s_pitch, void* stream);
/* The same forward from bf16 gate / up [M, N] (dense): also writes their per-group FP8 codes and bf16 scales, bit for bit
 * what coat_fp8_quantize gives (rq/_quantize.py:120), so that "quantize gate, quantize up, SiLU, multiply" is one pass over
 * the two bf16 tensors.  No counterpart in the reference (its MLP receives gate / up quantized by the GEMM epilogue). */
int coat_fp8_silu_mul_forward_bf16(const void* gate, const void* up, int fp8, void* q_gate, void* s_gate, void* q_up,
                                   void* s_up, void* q_silu, void* s_silu, void* y, float* s_max, int64_t M, int64_t N,
                                   int QB, void* stream);
/* backward: y_up = bf16(g * silu), y_gate = bf16(silu'(gate) * bf16(g * up)); s_max_gate / s_max_up (COAT_MAX_WORDS
 * words each) receive the max of their fp32 group scales for the format fp8_out (the per-tensor division that follows is
 * coat_fp8_division_from_max).
 * Row pitches in elements, 0 = contiguous: in_pitch / s_pitch for gate, up and their scales when they are the two column
 * halves of a fused projection's output (coat/models/coat_olmo.py:520-523 chunks and copies them), y_pitch (backward
 * only) for y_gate / y_up written side by side into one [M, 2N] tensor (coat_olmo.py:600 concatenates them). */
int coat_fp8_silu_mul_backward(const void* gate, const void* s_gate, const void* up, const void* s_up, const void* silu,
                               const void* s_silu, int fp8_in, int s_dtype, const void* g, void* y_gate,
                               float* s_max_gate, void* y_up, float* s_max_up, int fp8_out, int64_t M, int64_t N,
                               int QB, int64_t in_pitch, int64_t s_pitch, int64_t y_pitch, void* stream);

/* rq/func_rmsnorm.py:223 fp8_rmsnorm_forward (kernel :54-111): y = bf16(x * rstd * w); s_row [M] bf16 row scales
 * (max|y| + 1e-10) / fp8max; rstd [M] fp32; s_max as above.  N <= 16384, N % 16 == 0.  y may be NULL (statistics
 * only, for coat_fp8_rmsnorm_division). */
int coat_fp8_rmsnorm_forward(const void* x, int fp8, const void* s_x, int s_dtype, const void* w, int w_dtype, void* y,
                             void* s_row, float* rstd, float* s_max, int64_t M, int64_t N, int QB, float eps,
                             void* stream);
/* The per-tensor division + transpose that ends rq/func_rmsnorm.py:223 (its fp8_division_transpose call at :269),
 * fed with the norm's inputs: every tile of y = bf16(x * rstd * w) is recomputed in registers with the forward kernel's
 * expressions, so q / qt equal those of coat_fp8_division_from_max on the stored y, and y is never written or read.
 * s_max: the COAT_MAX_WORDS buffer filled by coat_fp8_rmsnorm_forward; s_out: one bf16 element, the rounded scale.
 * M % 16 == 0, N % 16 == 0, QB % 16 == 0; q / qt in the format of x. */
int coat_fp8_rmsnorm_division(const void* x, int fp8, const void* s_x, int s_dtype, const void* w, int w_dtype,
                              const float* rstd, const float* s_max, void* s_out, void* q, void* qt, int64_t M, int64_t N,
                              int QB, void* stream);
/* The same for coat_fp8_layernorm_forward (rq/func_layernorm_noparam.py:188, rq/func_layernorm_param.py:243; y = NULL
 * there): y = (x - mean) * rstd (* w + b) in fp32, as the reference keeps it, recomputed per tile.  w_dtype < 0: no affine
 * parameters (w, b NULL). */
int coat_fp8_layernorm_division(const void* x, int fp8, const void* s_x, int s_dtype, const void* w, const void* b,
                                int w_dtype, const float* mean, const float* rstd, const float* s_max, void* s_out, void* q,
                                void* qt, int64_t M, int64_t N, int QB, void* stream);
/* The same for the product of two per-group FP8 tensors, y = bf16(dequant(a) * dequant(b)) (kernel rq/mul_fwd.py:136-150;
 * the division is its fp8_division_transpose call at :243): a [M, N] dense (the SiLU output that
 * coat_fp8_silu_mul_forward just wrote, or x1 of fp8_mul_forward), b with row pitches b_pitch codes / sb_pitch scales
 * (0 = dense). */
int coat_fp8_product_division(const void* a, const void* s_a, int sa_dtype, const void* b, const void* s_b, int sb_dtype,
                              int fp8, const float* s_max, void* s_out, void* q, void* qt, int64_t M, int64_t N, int QB,
                              int64_t b_pitch, int64_t sb_pitch, void* stream);
/* rq/func_rmsnorm.py:281 fp8_rmsnorm_backward (kernels :121-196, :200-220): dx bf16 [M,N], dw [N] in w's dtype.
 * dw_partial: caller-provided fp32 workspace [n_partial, N]; the kernel uses min(n_partial, M) blocks and sums their
 * partial rows in block order (deterministic, unlike the reference's lock-ordered accumulation).
 * dy2 / dy3 (NULL or bf16 [M,N]): further gradients of the same tensor; the kernel uses bf16(bf16(dy + dy2) + dy3), which
 * is what the reference's callers compute with tensor additions before the call (coat/models/coat_llama.py:328, :742). */
int coat_fp8_rmsnorm_backward(const void* x, int fp8, const void* s_x, int s_dtype, const void* dy, const void* dy2,
                              const void* dy3, const void* w, int w_dtype, const float* rstd, void* dx, void* dw,
                              float* dw_partial, int n_partial, int64_t M, int64_t N, int QB, void* stream);
/* coat_fp8_rmsnorm_backward followed by the residual-gradient addition rq/add_bwd.py:147 fp8_add_Ifp_Ifp_Ofp_Opt (kernel
 * :107-135), as one kernel (the reference runs the two one after the other, coat/models/coat_llama.py:331-339, :745-754):
 * dx is rounded to bf16 as coat_fp8_rmsnorm_backward stores it, v = float(residual_grad) + float(dx) in fp32,
 * y = bf16(v) [M,N]; s_pg = bf16 scales (amax + 1e-10) / fp8max(fp8_out) of the 1 x QB groups of v [M, N/QB]; the largest
 * fp32 group scale is merged into s_max (COAT_MAX_WORDS, zero-filled by the caller), from which
 * coat_fp8_division_from_max of y gives the per-tensor codes.  Bit-identical to the two entry points.  N <= 8192. */
int coat_fp8_rmsnorm_backward_add(const void* x, int fp8, const void* s_x, int s_dtype, const void* dy, const void* dy2,
                                  const void* dy3, const void* w, int w_dtype, const float* rstd,
                                  const void* residual_grad, void* y, void* s_pg, float* s_max, int fp8_out, void* dw,
                                  float* dw_partial, int n_partial, int64_t M, int64_t N, int QB, void* stream);

/* No counterpart in the reference.  For callers that cannot allocate (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc): coat_fp8_rmsnorm_backward without the workspace argument.  The partial rows live in a
 * device array inside the library, COAT_RMSNORM_STATIC_PARTIALS x COAT_RMSNORM_STATIC_FULL_N floats (16 MiB per GPU, held
 * until the process ends); the call allocates and frees nothing.  It uses coat_rmsnorm_static_partials(N) partial rows
 * (512 up to N = 8192, 256 beyond), so dx and dw equal those of coat_fp8_rmsnorm_backward called with that n_partial.
 * N > 16384 is rejected with COAT_ESHAPE, as everywhere.  All calls on one GPU share the array: calls that overlap on one
 * GPU (two streams, two threads) race on it; calls on one stream are ordered and need no clearing in between.  The first
 * call on a device looks up the array's address (hipGetSymbolAddress): make one call on that device before capturing a
 * graph that contains this entry point. */
#define COAT_RMSNORM_STATIC_PARTIALS 512
#define COAT_RMSNORM_STATIC_FULL_N 8192
static inline int coat_rmsnorm_static_partials(int64_t N) {
    const int64_t rows = N > 0 ? ((int64_t)COAT_RMSNORM_STATIC_PARTIALS * COAT_RMSNORM_STATIC_FULL_N) / N : 0;
    return (int)(rows < COAT_RMSNORM_STATIC_PARTIALS ? rows : COAT_RMSNORM_STATIC_PARTIALS);
}
int coat_fp8_rmsnorm_backward_static(const void* x, int fp8, const void* s_x, int s_dtype, const void* dy, const void* dy2,
                                     const void* dy3, const void* w, int w_dtype, const float* rstd, void* dx, void* dw,
                                     int64_t M, int64_t N, int QB, void* stream);

/* rq/func_layernorm_noparam.py:188 fp8_layernorm_noparam_forward (kernel :53-115) and rq/func_layernorm_param.py:243
 * fp8_layernorm_param_forward (kernel :52-119): y fp32 [M,N] = (x - mean) * rstd (* w + b); mean, rstd [M] fp32;
 * s_row [M] bf16 row scales (max|y| + 1e-10) / fp8max; s_max as above.  w_dtype < 0: no affine parameters (w, b
 * ignored); otherwise w and b share that dtype.  N <= 16384, N % 16 == 0. */
int coat_fp8_layernorm_forward(const void* x, int fp8, const void* s_x, int s_dtype, const void* w, const void* b,
                               int w_dtype, float* y, void* s_row, float* mean, float* rstd, float* s_max, int64_t M,
                               int64_t N, int QB, float eps, void* stream);
/* rq/func_layernorm_noparam.py:248 fp8_layernorm_noparam_backward (kernel :122-185) and
 * rq/func_layernorm_param.py:305 fp8_layernorm_param_backward (kernels :128-209, :214-240): dx bf16 [M,N]; with
 * parameters also dw, db [N] in w's dtype through the caller-provided fp32 workspaces dw_partial, db_partial
 * [n_partial, N] (summed in block order; the reference accumulates under a spin lock in w's dtype). */
int coat_fp8_layernorm_backward(const void* x, int fp8, const void* s_x, int s_dtype, const void* dy, const void* w,
                                int w_dtype, const float* mean, const float* rstd, void* dx, void* dw, void* db,
                                float* dw_partial, float* db_partial, int n_partial, int64_t M, int64_t N, int QB,
                                void* stream);

/* coat_fp8_layernorm_backward followed by the value pass of fp8_add_Ifp_Ifp_Ofp_Opt (rq/add_bwd.py:147; the sequence at
 * coat/models/coat_olmo.py:318-339) in one kernel, like coat_fp8_rmsnorm_backward_add: dx is rounded to bf16 as it would be
 * stored, residual_grad (bf16 [M, N]) is added in fp32; y receives bf16 of the sum, s_pg [M, N / QB] the bf16 scales
 * (amax + 1e-10) / fp8max of its 1 x QB groups for format fp8_out, s_max (COAT_MAX_WORDS) their maximum;
 * coat_fp8_division_from_max of y gives the per-tensor codes.  Bit-identical to the two entry points. */
int coat_fp8_layernorm_backward_add(const void* x, int fp8, const void* s_x, int s_dtype, const void* dy, const void* w,
                                    int w_dtype, const float* mean, const float* rstd, const void* residual_grad, void* y,
                                    void* s_pg, float* s_max, int fp8_out, void* dw, void* db, float* dw_partial,
                                    float* db_partial, int n_partial, int64_t M, int64_t N, int QB, void* stream);

/* Rotary position embedding of the bf16 attention (no single counterpart in the reference, which applies it with
 * several torch kernels: transformers' apply_rotary_pos_emb as called at coat/models/coat_llama.py:1029-1030, olmo's
 * RotaryEmbedding at coat/models/coat_olmo.py:860-861).  x, y bf16 [rows, heads, head_dim], rows = batch * seq;
 * cos_tab / sin_tab fp32 [n_pos, head_dim / 2] holding cos / sin of p * theta^(-2d / head_dim); pos int64 [rows] or NULL
 * (position = row % seq_len, seq_len <= n_pos); a pos[row] outside [0, n_pos) is never used as a table index: the kernel
 * computes that row's angles from theta itself;
 * y1 = x1 cos - x2 sin, y2 = x2 cos + x1 sin on the (d, d + head_dim/2) pairs; inverse != 0 negates the angle, which
 * is the backward pass.  head_dim % 16 == 0.  x_pitch / y_pitch: row pitches in elements, 0 = contiguous; a multiple
 * of 8 (16-byte rows), for x or y that is a column slice of a fused q/k/v tensor (coat/models/coat_olmo.py:1003-1006).
 * s_max (may be NULL): a COAT_MAX_WORDS buffer as above; the kernel merges (max|y| + 1e-10) / fp8max of format fp8_max
 * into it, which is what coat_fp8_group_scales would merge for y with any group size, so a caller that quantizes the
 * rotated tensor per tensor (the gradients at coat/models/coat_llama.py:318-326) skips that pass.  inverse == 2 (needs s_max):
 * no rotation, y = x with the maximum merged, for the v part of a fused q / k / v gradient (coat/models/coat_olmo.py:1003-1006),
 * whose three parts are quantized as one tensor. */
int coat_rope_bf16(const void* x, void* y, const float* cos_tab, const float* sin_tab, int64_t n_pos, float theta,
                   const int64_t* pos, int64_t rows, int seq_len, int heads, int head_dim, int inverse, int64_t x_pitch,
                   int64_t y_pitch, float* s_max, int fp8_max, void* stream);

/* ---- bf16 attention (forward) ------------------------------------------------------------------------
 * The attention between the FP8 projections: the reference calls the flash-attn library here
 * (coat/models/coat_llama.py:960-971, used by LlamaAttentionWithoutLinear :981-1074).
 * out = softmax(q k^T * scale (+ causal mask)) v per (batch, head); q, k, v, out bf16 [batch, seq, heads, 128] addressed
 * through element strides (batch, token, head; the head dimension is contiguous; all strides multiples of 8), so the
 * projections' outputs are used where they lie.  k and v have kv_heads heads (heads % kv_heads == 0).  lse (may be
 * NULL): fp32 [batch, heads, seq], natural logarithm of each query's sum of exponentials, as backward kernels expect it.
 * head_dim must be 128. s_max (may be NULL): a COAT_MAX_WORDS buffer; the kernel merges (max|out| + 1e-10) / fp8max of
 * format fp8_max into it, what coat_fp8_group_scales would merge for out, so the per-tensor quantization of the attention
 * output (coat/models/coat_llama.py:434, fp8_quantize_pertensor) goes straight to its division pass. */
int coat_attention_forward_bf16(const void* q, const void* k, const void* v, void* out, float* lse, int64_t batch,
                                int64_t heads, int64_t kv_heads, int64_t seq, int64_t head_dim, int64_t q_sb, int64_t q_ss,
                                int64_t q_sh, int64_t k_sb, int64_t k_ss, int64_t k_sh, int64_t v_sb, int64_t v_ss,
                                int64_t v_sh, int64_t o_sb, int64_t o_ss, int64_t o_sh, float scale, int causal,
                                float* s_max, int fp8_max, void* stream);

/* ---- GEMM -------------------------------------------------------------------------------------------
 * rq/linear.py:172 fp8matmul (kernel :61-169): C[M,N] = (A[M,K] . B[N,K]^T) * (float(*scale_a) * float(*scale_b))
 * (+ bias[N]), fp32 accumulation on FP8 MFMA.  A and B are row-major with K contiguous (the reference passes B as
 * the .t() view of such a matrix, linear.py:253-302); fmt_a / fmt_b are coat_fp8 values and may differ.
 * out_kind 0: C is bf16 [M,N] (:166-169).  out_kind 1 / 2: C is e4m3 / e5m2 [M,N], quantized per 1 x QB group along
 * N with scale (amax + 1e-10) / fp8max, and c_scale is bf16 [M, N/QB] (:139-164); QB 16, 32 or 64, N % QB == 0.
 * scale_a / scale_b: one element each in device memory, of sa_dtype / sb_dtype (each is loaded in its own dtype and the
 * two are multiplied in fp32, :123-125: an fp32 weight scale next to a bf16 activation scale keeps all its bits).
 * K % 16 == 0. */
int coat_fp8_gemm(const void* a, int fmt_a, const void* b, int fmt_b, void* c, void* c_scale, int out_kind,
                  const void* scale_a, int sa_dtype, const void* scale_b, int sb_dtype, const void* bias, int bias_dtype,
                  int64_t M, int64_t N, int64_t K, int QB, void* stream);

/* The same product followed by the addition of a bf16 tensor, as one kernel (no counterpart function in the reference,
 * which runs fp8matmul, rq/linear.py:172, and then a tensor addition: rq/add_fwd.py:162 fp8_add_Ifp_Ifp_Ofp_Og16 after the
 * output and down projections, coat/models/coat_llama.py:440-441, :673-674; plain bf16 `+` for the gradients that reach one
 * tensor, :328, :742).  t = bf16 of the product as coat_fp8_gemm stores it; v = float(t) + float(residual) in fp32;
 * c = bf16(v).  out_kind 1 / 2: also c_q = e4m3 / e5m2 codes of v per 1 x 16 group with scale (amax + 1e-10) / fp8max and
 * c_scale = the bf16 scales [M, N/16] (add_fwd.py:107-137), bit-identical to running the two kernels.  residual bf16 [M,N]
 * may be c itself (accumulation in place).  N % 8 == 0 (N % 16 == 0 with out_kind 1 / 2), N < 2^22. */
int coat_fp8_gemm_residual(const void* a, int fmt_a, const void* b, int fmt_b, const void* residual, void* c, void* c_q,
                           void* c_scale, int out_kind, const void* scale_a, int sa_dtype, const void* scale_b,
                           int sb_dtype, const void* bias, int bias_dtype, int64_t M, int64_t N, int64_t K, void* stream);

/* `count` (1 .. 4) such products of one shape and one pair of formats in one launch: problem i is
 * (a[i], b[i], c[i], c_scale[i], scale_a[i], scale_b[i], bias[i]); the seven arrays are host arrays of `count` device
 * pointers, read before the call returns (c_scale may be NULL for out_kind 0, bias may be NULL or hold NULLs).  Every
 * result is bit-identical to coat_fp8_gemm on the same problem.  The reference calls fp8matmul once per projection
 * (coat/models/coat_llama.py:267-269 q / k / v, :647-648 gate / up, and their backward :318-326, :735-740); on a persistent grid of
 * 256 x 256 tiles the problems' tiles are taken as one sequence, so the partial last round of tiles is paid once per
 * group. */
int coat_fp8_gemm_grouped(int count, const void* const* a, int fmt_a, const void* const* b, int fmt_b, void* const* c,
                          void* const* c_scale, int out_kind, const void* const* scale_a, int sa_dtype,
                          const void* const* scale_b, int sb_dtype, const void* const* bias, int bias_dtype, int64_t M,
                          int64_t N, int64_t K, int QB, void* stream);

/* ---- optimizer -------------------------------------------------------------------------------- */

/* qoptim_cuda.fp8_adamw_expand_step (coat/optimizer/kernels/bindings.cpp:7,
 * include/fp8_adamw_expand.h:6-17, fp8_adamw_expand_cuda_kernel.cu:205-245).
 * params/grads: p_dtype (F32, BF16 or F16), numel elements, updated in place.
 * exp_avg / exp_avg_sq: e4m3 codes; scale_*, expand_*, sqrtminmax_*: fp32, ceil(numel/128) each.
 * Unlike the reference launcher the kernel runs on `stream`, not on the legacy default stream. */
int coat_fp8_adamw_expand_step(void* params, const void* grads, int p_dtype, void* exp_avg, float* scale_exp_avg,
                               float* expand_exp_avg, float* sqrtminmax_exp_avg, void* exp_avg_sq,
                               float* scale_exp_avg_sq, float* expand_exp_avg_sq, float* sqrtminmax_exp_avg_sq,
                               float beta1, float beta2, float lr, float wd, float eps, int step, int qgroup_size,
                               int expand_min, int64_t numel, int64_t n_scale, void* stream);

/* qoptim_cuda.fp8_adamw_step (bindings.cpp:6, include/fp8_adamw.h:6-13, fp8_adamw_cuda_kernel.cu:127-159). */
int coat_fp8_adamw_step(void* params, const void* grads, int p_dtype, void* exp_avg, float* scale_exp_avg,
                        void* exp_avg_sq, float* scale_exp_avg_sq, float beta1, float beta2, float lr, float wd,
                        float eps, int step, int qgroup_size, int64_t numel, int64_t n_scale, void* stream);

/* The two steps above for several tensors in one launch (no single counterpart: the reference's optimizer launches once
 * per parameter, coat/optimizer/fp8_adamw.py:419-515).  Every argument that is a device pointer above is a host array of
 * `count` such pointers here, numel / n_scale host arrays of `count` sizes; dtype, hyperparameters and step are common to
 * the tensors of a call.  The arrays are read before the call returns.  Tensors are launched 32 to a kernel; every
 * tensor's result is bit-identical to its own coat_fp8_adamw_expand_step / coat_fp8_adamw_step call; empty tensors are
 * skipped; all tensors are validated before the first launch. */
int coat_fp8_adamw_expand_step_multi(int count, void* const* params, const void* const* grads, int p_dtype,
                                     void* const* exp_avg, float* const* scale_exp_avg, float* const* expand_exp_avg,
                                     float* const* sqrtminmax_exp_avg, void* const* exp_avg_sq,
                                     float* const* scale_exp_avg_sq, float* const* expand_exp_avg_sq,
                                     float* const* sqrtminmax_exp_avg_sq, const int64_t* numel, const int64_t* n_scale,
                                     float beta1, float beta2, float lr, float wd, float eps, int step, int qgroup_size,
                                     int expand_min, void* stream);
int coat_fp8_adamw_step_multi(int count, void* const* params, const void* const* grads, int p_dtype, void* const* exp_avg,
                              float* const* scale_exp_avg, void* const* exp_avg_sq, float* const* scale_exp_avg_sq,
                              const int64_t* numel, const int64_t* n_scale, float beta1, float beta2, float lr, float wd,
                              float eps, int step, int qgroup_size, void* stream);

/* coat/activation/liger/cross_entropy.py:24-198 liger_cross_entropy_kernel as launched by cross_entropy_forward
 * (:212-278): softmax cross-entropy over x [n_rows, n_cols] (row pitch x_stride elements, fp32 / bf16 / fp16).
 * On return x holds the gradient of the reduced loss w.r.t. the logits, loss[row] (and z_loss[row] when z_loss is
 * not NULL) the row's contribution, both in x's dtype; rows whose target equals ignore_index get zeros.
 * target: int64 [n_rows].  reduction: 0 "none", 1 "mean", 2 "sum"; for "mean" the divisor is read from
 * *n_non_ignore (one int64 in device memory: the number of targets != ignore_index), so the host never waits for it
 * (the reference calls .item(), :240).  has_softcap != 0: logits pass through softcap * tanh(x / softcap) first. */
int coat_cross_entropy_forward(void* x, int x_dtype, int64_t x_stride, const int64_t* target, void* loss, void* z_loss,
                               const int64_t* n_non_ignore, int64_t n_rows, int64_t n_cols, int64_t ignore_index,
                               float lse_square_scale, float label_smoothing, int reduction, float softcap,
                               int has_softcap, void* stream);

/* coat/activation/liger/cross_entropy.py:281-302 cross_entropy_backward (element_mul_kernel, liger/utils.py):
 * x *= *grad_output in place; grad_output is one element of g_dtype in device memory.  The kernel itself returns
 * without touching x when the factor is 1 (the reference compares on the host with torch.equal, a synchronisation). */
int coat_cross_entropy_scale_grad(void* x, int x_dtype, int64_t x_stride, const void* grad_output, int g_dtype,
                                  int64_t n_rows, int64_t n_cols, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* COAT_HIP_H */
