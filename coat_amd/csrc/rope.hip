// Rotary position embedding for the bf16 attention of the decoder layers, forward and backward in one pass each.
//
// The reference applies RoPE with separate torch kernels (transformers' apply_rotary_pos_emb as called from
// coat/models/coat_llama.py:1029-1030; olmo's RotaryEmbedding from coat/models/coat_olmo.py:860-861): two multiplies, a
// negate, a concatenation and an add per tensor and direction, each a full pass over q and k.  Here one streaming
// kernel reads x once and writes the rotated tensor once; the backward pass is the same kernel with the angle negated.
//   x, y: bf16 [rows, heads, head_dim] (rows = batch * seq, contiguous), "half" layout: element d pairs with d + head_dim/2
//   cos_tab, sin_tab: fp32 [n_pos, head_dim/2];  position of a row = pos[row] if pos is given, else row % seq_len;
//   a position outside the tables (only possible with pos) gets its angle p * theta^(-2d/head_dim) computed in the kernel
//   y1 = x1 cos - x2 sin,  y2 = x2 cos + x1 sin   (inverse: sin -> -sin), computed in fp32, rounded once to bf16.
// With s_max the kernel also merges (max|y| + 1e-10) / fp8max, the largest 1 x QB group scale of y for any QB (dividing
// and rounding are monotone), into the maximum buffer: what the scale pass of fp8_quantize_pertensor(_transpose)
// (coat/activation/real_quantization/_quantize_pertensor_transpose.py:123-139) would find on y, so a caller that quantizes
// the rotated gradient per tensor goes straight to the division pass.
#include "coat_device.h"
#include "coat_host.h"

namespace coat {

// MAXKIND: -1 no maximum; kE4M3 / kE5M2: merge the largest group scale of y for that format into s_max.
// COPY: no rotation, y = x (for the part of a fused q / k / v gradient that has no rotary embedding but shares the maximum)
template <int MAXKIND, bool COPY>
__global__ __launch_bounds__(256) void k_rope_bf16(const uint16_t* __restrict__ x, uint16_t* __restrict__ y,
                                                    const float* __restrict__ cos_tab, const float* __restrict__ sin_tab,
                                                    int64_t n_pos, float theta, const int64_t* __restrict__ pos,
                                                    int64_t rows, int seq_len, int heads, int head_dim, float sign,
                                                    int64_t x_pitch, int64_t y_pitch, float* __restrict__ s_max) {
    __shared__ float smem[4];
    float amax = 0.0f;
    const int half = head_dim >> 1;
    const int cpr = half >> 3;                      // 16-byte chunks per half row
    const int64_t total = rows * heads * cpr;       // one job = 8 pairs
    for (int64_t job = (int64_t)blockIdx.x * 256 + threadIdx.x; job < total; job += (int64_t)gridDim.x * 256) {
        const int c = (int)(job % cpr);
        const int64_t rh = job / cpr;               // row * heads + head
        const int64_t row = rh / heads;
        const int64_t p = pos ? pos[row] : row % seq_len;
        const int head = (int)(rh - row * heads);
        const uint16_t* src = x + row * x_pitch + head * head_dim + c * 8;
        const uint4 a = *(const uint4*)src, b = *(const uint4*)(src + half);
        float cs[8], sn[8];
        if (COPY) {
            // nothing to look up
        } else if (p >= 0 && p < n_pos) {
            const float4* ct = (const float4*)(cos_tab + p * half + c * 8);
            const float4* st = (const float4*)(sin_tab + p * half + c * 8);
            const float4 c0 = ct[0], c1 = ct[1], s0 = st[0], s1 = st[1];
            cs[0] = c0.x; cs[1] = c0.y; cs[2] = c0.z; cs[3] = c0.w; cs[4] = c1.x; cs[5] = c1.y; cs[6] = c1.z; cs[7] = c1.w;
            sn[0] = s0.x; sn[1] = s0.y; sn[2] = s0.z; sn[3] = s0.w; sn[4] = s1.x; sn[5] = s1.y; sn[6] = s1.z; sn[7] = s1.w;
        } else {
            // off the tables: the table's own formula, angle = float(p) * (1 / theta^(2d / head_dim)), never an out-of-bounds read
#pragma unroll
            for (int k = 0; k < 8; k++) {
                const float inv_freq = 1.0f / powf(theta, (float)(2 * (c * 8 + k)) / (float)head_dim);
                const float ang = (float)p * inv_freq;
                cs[k] = cosf(ang);
                sn[k] = sinf(ang);
            }
        }
        const uint32_t aw[4] = {a.x, a.y, a.z, a.w}, bw[4] = {b.x, b.y, b.z, b.w};
        uint32_t o1[4], o2[4];
#pragma unroll
        for (int k = 0; k < 4; k++) {
            if (COPY) {
                o1[k] = aw[k];
                o2[k] = bw[k];
                continue;
            }
            const float x1l = bf16lo(aw[k]), x1h = bf16hi(aw[k]), x2l = bf16lo(bw[k]), x2h = bf16hi(bw[k]);
            const float sl = sign * sn[2 * k], sh = sign * sn[2 * k + 1];
            o1[k] = pack_bf16x2(x1l * cs[2 * k] - x2l * sl, x1h * cs[2 * k + 1] - x2h * sh);
            o2[k] = pack_bf16x2(x2l * cs[2 * k] + x1l * sl, x2h * cs[2 * k + 1] + x1h * sh);
        }
        uint16_t* dst = y + row * y_pitch + head * head_dim + c * 8;
        *(uint4*)dst = make_uint4(o1[0], o1[1], o1[2], o1[3]);
        *(uint4*)(dst + half) = make_uint4(o2[0], o2[1], o2[2], o2[3]);
        if (MAXKIND >= 0) {
#pragma unroll
            for (int k = 0; k < 4; k++) {  // of the values as stored
                amax = fmaxf(amax, fmaxf(fmaxf(fabsf(bf16lo(o1[k])), fabsf(bf16hi(o1[k]))),
                                         fmaxf(fabsf(bf16lo(o2[k])), fabsf(bf16hi(o2[k])))));
            }
        }
    }
    constexpr int KIND = MAXKIND < 0 ? (int)kE4M3 : MAXKIND;
    if (MAXKIND >= 0) block_atomic_max_nonneg(s_max, group_scale<KIND>(amax), smem);
}

}  // namespace coat

using namespace coat;

extern "C" int coat_rope_bf16(const void* x, void* y, const float* cos_tab, const float* sin_tab, int64_t n_pos, float theta,
                              const int64_t* pos, int64_t rows, int seq_len, int heads, int head_dim, int inverse,
                              int64_t x_pitch, int64_t y_pitch, float* s_max, int fp8_max, void* stream) {
    if (s_max && fp8_max != kE4M3 && fp8_max != kE5M2) return COAT_EINVAL;
    if (inverse < 0 || inverse > 2) return COAT_EINVAL;
    if (rows < 0 || heads <= 0 || head_dim <= 0 || seq_len <= 0 || n_pos <= 0 || !(theta > 0.0f)) return COAT_EINVAL;
    if (!pos && seq_len > n_pos) return COAT_ESHAPE;  // positions 0 .. seq_len-1 must all be in the tables
    if (head_dim % 16 != 0) return COAT_ESHAPE;  // 8 pairs per lane
    // row pitches in elements (0 = contiguous): x or y may be a column slice of a wider tensor (a fused q/k/v projection)
    const int64_t width = (int64_t)heads * head_dim;
    if (x_pitch == 0) x_pitch = width;
    if (y_pitch == 0) y_pitch = width;
    if (x_pitch < width || y_pitch < width || x_pitch % 8 != 0 || y_pitch % 8 != 0) return COAT_ESHAPE;
    if (rows == 0) return COAT_OK;
    if (!x || !y || !cos_tab || !sin_tab) return COAT_EINVAL;
    if (!coat_aligned16(x) || !coat_aligned16(y) || !coat_aligned16(cos_tab) || !coat_aligned16(sin_tab)) return COAT_EALIGN;
    const int64_t total = rows * heads * (head_dim / 16);
    int64_t blocks = (total + 255) / 256;
    if (blocks > 16384) blocks = 16384;
    if (s_max && blocks > 2048) blocks = 2048;  // one atomic per block: fewer, longer blocks
    auto* kern = !s_max ? k_rope_bf16<-1, false> : fp8_max == kE4M3 ? k_rope_bf16<kE4M3, false> : k_rope_bf16<kE5M2, false>;
    if (inverse == 2) {  // plain copy with the maximum
        if (!s_max) return COAT_EINVAL;
        kern = fp8_max == kE4M3 ? k_rope_bf16<kE4M3, true> : k_rope_bf16<kE5M2, true>;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, (const uint16_t*)x, (uint16_t*)y,
                       cos_tab, sin_tab, n_pos, theta, pos, rows, seq_len, heads, head_dim, inverse == 1 ? -1.0f : 1.0f, x_pitch,
                       y_pitch, s_max);
    return coat_launch_status();
}
