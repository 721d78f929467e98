// Causal bf16 attention forward for the decoder layers, head dimension 128, on CDNA4 MFMA
// (v_mfma_f32_32x32x16_bf16), with online softmax: O = softmax(Q K^T * scale) V and the row-wise log-sum-exp.
//
// The reference hands this step to the flash-attn library (coat/models/coat_llama.py:960-971 through transformers'
// attention classes, used by LlamaAttentionWithoutLinear :981-1074); the projections around it are the FP8 modules.
//
// Layout.  q, k, v and the output are bf16 [batch, seq, heads, 128] as the projections leave them (strides are
// arguments).  A block of four waves owns 128 consecutive queries of one (batch, head): wave w the 32 queries
// 32 w .. 32 w + 31, all 128 dimensions.  Keys are walked in tiles of 64.  Both products are computed transposed, so that
// the accumulator layout of the first is the operand layout of the second:
//   S^T[key, query] = K Q^T      A = K tile rows (a lane reads 16 contiguous bytes of a key's row), B = Q (registers)
//   O^T[dim, query] = V^T P^T    A = V^T tile rows (16 contiguous bytes of a dimension's row of keys), B = P^T
// In both results a lane holds one query (column lane % 32), so the running maximum, the running sum and the rescaling
// of O are per-lane scalars; the only cross-lane step of the softmax is one swap between lane l and lane l + 32, which
// hold the two halves of a query's keys.  P^T needs no layout change either: the contraction over keys may run in any
// order as long as both operands agree, and one v_permlane32_swap per two packed registers puts keys 16 j + 8 h .. + 7 into
// half-wave h, which is what a 16-byte read of a V^T row delivers.
// V^T (keys contiguous) does not exist in the projections' output: k_attn_transpose_v writes it once per call,
// [batch, kv_heads, 128, seq padded to 64].
// K and V^T tiles go from global memory into a two-stage LDS ring without passing through registers
// (buffer_load_dwordx4 ... lds); 16-byte chunks are XOR-swizzled with the row so that the fragment reads are free of
// bank conflicts.  Blocks are ordered so that the blocks of one (batch, head) run on one XCD (one L2) one after the other,
// longest first (under the causal mask a block's work grows with its position).
#include <math.h>

#include "coat_device.h"
#include "coat_host.h"

namespace coat {

typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef int v4i_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_ptr3_t;

constexpr int kHeadDim = 128;
constexpr int kBlockQ = 128, kTileK = 64;
constexpr int kKTileBytes = kTileK * kHeadDim * 2;   // 64 keys x 256 bytes
constexpr int kVTileBytes = kHeadDim * kTileK * 2;   // 128 dims x 128 bytes
constexpr int kStageBytes = kKTileBytes + kVTileBytes;
constexpr int kAttnLdsBytes = 2 * kStageBytes;       // 64 KiB: two blocks per CU

struct AttnArgs {
    const uint16_t* q;
    const uint16_t* k;
    const uint16_t* vt;   // [batch, kv_heads, 128, s_pad]
    uint16_t* out;
    float* lse;           // [batch, heads, seq], natural logarithm
    int64_t q_sb, q_ss, q_sh, k_sb, k_ss, k_sh, o_sb, o_ss, o_sh;  // element strides: batch, token, head
    int batch, heads, kv_heads, seq, s_pad;
    float scale_log2e;    // softmax scale * log2(e)
};

__device__ __forceinline__ void attn_lds_dma16(v4i_t rsrc, uint32_t lds_addr, int voff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(rsrc)
                 : "memory", "m0");
}
__device__ __forceinline__ v4i_t attn_rsrc(const void* p, uint32_t bytes) {
    const uint64_t a = (uint64_t)p;
    return (v4i_t){(int)(uint32_t)a, (int)(uint32_t)(a >> 32) & 0xFFFF, (int)bytes, 0x00020000};
}
#define ATTN_WAIT_VMCNT0() __builtin_amdgcn_s_waitcnt(0 | (0x7 << 4) | (0xF << 8))

template <bool CAUSAL>
__global__ __launch_bounds__(256, 2) void k_attn_fwd(AttnArgs A) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63, h32 = lane >> 5, l32 = lane & 31;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int nqb = (A.seq + kBlockQ - 1) / kBlockQ;
    // blocks are dispatched round-robin over the 8 XCDs: XCD x takes the (batch, head) pairs x, x + 8, ..., each with all
    // its query blocks one after the other, last (longest under the causal mask) first
    const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
    const int bh = (idx / nqb) * 8 + xcd;
    if (bh >= A.batch * A.heads) return;
    const int qb = nqb - 1 - idx % nqb;
    const int b = bh / A.heads, head = bh % A.heads;
    const int kvh = head / (A.heads / A.kv_heads);
    const int q0 = qb * kBlockQ;
    const int nkt_all = (A.seq + kTileK - 1) / kTileK;
    const int nsteps = CAUSAL ? min((q0 + kBlockQ + kTileK - 1) / kTileK, nkt_all) : nkt_all;

    // ---- the wave's Q fragments: B operand of S^T = K Q^T, 8 chunks of 16 dimensions
    const int my_q = q0 + wave * 32 + l32;
    v8bf qf[8];
    {
        const uint16_t* qrow = A.q + b * A.q_sb + (int64_t)min(my_q, A.seq - 1) * A.q_ss + head * A.q_sh;
#pragma unroll
        for (int c = 0; c < 8; c++) qf[c] = *(const v8bf*)(qrow + 16 * c + 8 * h32);
    }

    // ---- tile loads (global -> LDS)
    const uint16_t* kbase = A.k + b * A.k_sb + kvh * A.k_sh;
    const uint16_t* vbase = A.vt + ((int64_t)(b * A.kv_heads + kvh) * kHeadDim) * A.s_pad;
    const v4i_t k_rsrc = attn_rsrc(kbase, (uint32_t)(((int64_t)(A.seq - 1) * A.k_ss + kHeadDim) * 2));
    const v4i_t v_rsrc = attn_rsrc(vbase, (uint32_t)((int64_t)kHeadDim * A.s_pad * 2));
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr3_t)lds;
    // K: one instruction = 4 rows of 256 bytes; lane i fills position i % 16 of row i / 16 with the chunk that belongs there
    // V^T: one instruction = 8 rows of 128 bytes; lane i fills position i % 8 of row i / 8
    int k_off[4], v_off[4];
#pragma unroll
    for (int x = 0; x < 4; x++) {
        const int krow = 4 * (4 * wave + x) + (lane >> 4);
        k_off[x] = krow * (int)(A.k_ss * 2) + (((lane & 15) ^ (krow & 15)) << 4);
        const int vrow = 8 * (4 * wave + x) + (lane >> 3);
        v_off[x] = vrow * (A.s_pad * 2) + (((lane & 7) ^ ((vrow >> 1) & 7)) << 4);
    }
    auto issue_tile = [&](int t, int stage) {
        const uint32_t kdst = lds_base + stage * kStageBytes + (4 * wave) * 1024;
        const uint32_t vdst = kdst + kKTileBytes;
        const int kt_off = t * kTileK * (int)(A.k_ss * 2), vt_off = t * kTileK * 2;
#pragma unroll
        for (int x = 0; x < 4; x++) attn_lds_dma16(k_rsrc, kdst + x * 1024, k_off[x] + kt_off);
#pragma unroll
        for (int x = 0; x < 4; x++) attn_lds_dma16(v_rsrc, vdst + x * 1024, v_off[x] + vt_off);
    };
    // fragment addresses inside a stage: K row l32 (+ 32 kt), chunk 2 c + h32; V^T row l32 (+ 32 dt), chunk 2 j + h32
    auto k_frag = [&](int stage, int kt, int c) -> v8bf {
        const int row = 32 * kt + l32;
        return *(const v8bf*)(lds + stage * kStageBytes + row * 256 + (((2 * c + h32) ^ (row & 15)) << 4));
    };
    auto v_frag = [&](int stage, int dt, int j) -> v8bf {
        const int row = 32 * dt + l32;
        return *(const v8bf*)(lds + stage * kStageBytes + kKTileBytes + row * 128 + (((2 * j + h32) ^ ((row >> 1) & 7)) << 4));
    };

    v16f o_acc[4];
#pragma unroll
    for (int dt = 0; dt < 4; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) o_acc[dt][r] = 0.0f;
    float m_run = -INFINITY, l_run = 0.0f;  // running maximum (log2 domain) and this lane's part of the running sum

    issue_tile(0, 0);
    for (int t = 0; t < nsteps; t++) {
        const int stage = t & 1;
        ATTN_WAIT_VMCNT0();               // this wave's part of tile t has landed
        __builtin_amdgcn_s_barrier();     // ... and everybody's; everybody is also done reading tile t - 1
        asm volatile("" ::: "memory");
        if (t + 1 < nsteps) issue_tile(t + 1, stage ^ 1);
        const int key0 = t * kTileK;
        // waves whose queries all lie before this tile have nothing to add (causal); they still take part in the loads
        if (CAUSAL && key0 > q0 + wave * 32 + 31) continue;

        // ---- S^T = K Q^T for the tile's 64 keys
        v16f s_acc[2];
#pragma unroll
        for (int kt = 0; kt < 2; kt++) {
#pragma unroll
            for (int r = 0; r < 16; r++) s_acc[kt][r] = 0.0f;
#pragma unroll
            for (int c = 0; c < 8; c++)
                s_acc[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(k_frag(stage, kt, c), qf[c], s_acc[kt], 0, 0, 0);
        }
        // ---- scale, mask, running maximum
        const bool edge = (CAUSAL && key0 + kTileK - 1 > q0 + wave * 32) || key0 + kTileK > A.seq;  // wave-uniform
        float mx = -INFINITY;
#pragma unroll
        for (int kt = 0; kt < 2; kt++)
#pragma unroll
            for (int r = 0; r < 16; r++) {
                float s = s_acc[kt][r] * A.scale_log2e;
                if (edge) {
                    const int key = key0 + 32 * kt + 8 * (r >> 2) + 4 * h32 + (r & 3);
                    if ((CAUSAL && key > my_q) || key >= A.seq) s = -INFINITY;
                }
                s_acc[kt][r] = s;
                mx = fmaxf(mx, s);
            }
        {
            const auto sw = __builtin_amdgcn_permlane32_swap(f2u(mx), f2u(mx), false, false);
            mx = fmaxf(u2f(sw[0]), u2f(sw[1]));
        }
        const float m_new = fmaxf(m_run, mx);  // finite: key 0 is visible to every query
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
        m_run = m_new;
        // ---- P = exp2(S - m), packed to bf16 as the B operand of O^T = V^T P^T
        float psum = 0.0f;
        uint32_t pk[2][8];
#pragma unroll
        for (int kt = 0; kt < 2; kt++)
#pragma unroll
            for (int r = 0; r < 16; r += 2) {
                const float p0 = __builtin_amdgcn_exp2f(s_acc[kt][r] - m_new), p1 = __builtin_amdgcn_exp2f(s_acc[kt][r + 1] - m_new);
                psum += p0 + p1;
                pk[kt][r >> 1] = pack_bf16x2(p0, p1);
            }
        l_run = l_run * alpha + psum;
        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
            for (int dt = 0; dt < 4; dt++)
#pragma unroll
                for (int r = 0; r < 16; r++) o_acc[dt][r] *= alpha;
        }
        // ---- O^T += V^T P^T, 16 keys per instruction: chunk j = 2 kt + u takes accumulator registers 8 u .. 8 u + 7
#pragma unroll
        for (int kt = 0; kt < 2; kt++)
#pragma unroll
            for (int u = 0; u < 2; u++) {
                // packed registers 4 u, 4 u + 1 hold keys 16 u + 4 h .. + 3, registers 4 u + 2, 4 u + 3 keys 16 u + 8 + 4 h .. + 3
                const auto s0 = __builtin_amdgcn_permlane32_swap(pk[kt][4 * u], pk[kt][4 * u + 2], false, false);
                const auto s1 = __builtin_amdgcn_permlane32_swap(pk[kt][4 * u + 1], pk[kt][4 * u + 3], false, false);
                // half-wave h now holds keys 16 u + 8 h .. + 7 in slot order
                const v4i_t pw = (v4i_t){(int)s0[0], (int)s1[0], (int)s0[1], (int)s1[1]};
                const v8bf pfrag = __builtin_bit_cast(v8bf, pw);
#pragma unroll
                for (int dt = 0; dt < 4; dt++)
                    o_acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v_frag(stage, dt, 2 * kt + u), pfrag, o_acc[dt], 0, 0, 0);
            }
    }

    // ---- normalise and store: the two half-waves hold the two parts of each query's sum
    {
        const auto sw = __builtin_amdgcn_permlane32_swap(f2u(l_run), f2u(l_run), false, false);
        l_run = u2f(sw[0]) + u2f(sw[1]);
    }
    const float inv_l = 1.0f / l_run;
    if (my_q < A.seq) {
        uint16_t* orow = A.out + b * A.o_sb + (int64_t)my_q * A.o_ss + head * A.o_sh;
#pragma unroll
        for (int dt = 0; dt < 4; dt++)
#pragma unroll
            for (int g = 0; g < 4; g++) {  // accumulator registers 4 g .. 4 g + 3: dimensions 32 dt + 8 g + 4 h .. + 3
                const v16f& o = o_acc[dt];
                *(uint2*)(orow + 32 * dt + 8 * g + 4 * h32) =
                    make_uint2(pack_bf16x2(o[4 * g] * inv_l, o[4 * g + 1] * inv_l), pack_bf16x2(o[4 * g + 2] * inv_l, o[4 * g + 3] * inv_l));
            }
        if (h32 == 0 && A.lse)
            A.lse[((int64_t)b * A.heads + head) * A.seq + my_q] = (m_run + __builtin_amdgcn_logf(l_run)) * 0.6931471805599453f;
    }
}

// v [batch, seq, kv_heads, 128] (strides given) -> vt [batch, kv_heads, 128, s_pad], columns seq .. s_pad - 1 zero.
// One block = 64 keys x 128 dimensions of one (batch, head), through LDS.
__global__ __launch_bounds__(256) void k_attn_transpose_v(const uint16_t* __restrict__ v, uint16_t* __restrict__ vt, int64_t v_sb,
                                                          int64_t v_ss, int64_t v_sh, int kv_heads, int seq, int s_pad) {
    __shared__ uint16_t tile[kTileK][kHeadDim + 2];
    const int t = blockIdx.x, bh = blockIdx.y;
    const int b = bh / kv_heads, hd = bh % kv_heads;
    const uint16_t* src = v + b * v_sb + hd * v_sh;
    // 64 rows x 16 chunks of 16 bytes: four per thread
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const int job = threadIdx.x + 256 * it, row = job >> 4, ch = job & 15;
        const int key = t * kTileK + row;
        uint4 val = make_uint4(0, 0, 0, 0);
        if (key < seq) val = *(const uint4*)(src + (int64_t)key * v_ss + ch * 8);
        uint32_t* dst = (uint32_t*)&tile[row][ch * 8];  // rows are 260 bytes apart: 4-byte aligned
        dst[0] = val.x; dst[1] = val.y; dst[2] = val.z; dst[3] = val.w;
    }
    __syncthreads();
    // 128 dims x 8 chunks of 8 keys: four per thread
    uint16_t* dstb = vt + ((int64_t)bh * kHeadDim) * s_pad + t * kTileK;
#pragma unroll
    for (int it = 0; it < 4; it++) {
        const int job = threadIdx.x + 256 * it, dim = job >> 3, kc = job & 7;
        uint32_t w[4];
#pragma unroll
        for (int e = 0; e < 4; e++) w[e] = (uint32_t)tile[kc * 8 + 2 * e][dim] | ((uint32_t)tile[kc * 8 + 2 * e + 1][dim] << 16);
        *(uint4*)(dstb + (int64_t)dim * s_pad + kc * 8) = make_uint4(w[0], w[1], w[2], w[3]);
    }
}

}  // namespace coat

using namespace coat;

extern "C" int coat_attention_transpose_v(const void* v, void* vt, int64_t batch, int64_t seq, int64_t kv_heads, int64_t head_dim,
                                          int64_t v_sb, int64_t v_ss, int64_t v_sh, int64_t s_pad, void* stream) {
    if (batch < 0 || seq < 0 || kv_heads <= 0) return COAT_EINVAL;
    if (head_dim != kHeadDim || s_pad % kTileK != 0 || s_pad < seq) return COAT_ESHAPE;
    if (batch * seq == 0) return COAT_OK;
    if (!v || !vt) return COAT_EINVAL;
    if (!coat_aligned16(v) || !coat_aligned16(vt) || v_ss % 8 != 0 || v_sh % 8 != 0 || v_sb % 8 != 0) return COAT_EALIGN;
    if (batch * kv_heads >= 65536 || s_pad / kTileK >= ((int64_t)1 << 31)) return COAT_ESHAPE;
    hipLaunchKernelGGL(k_attn_transpose_v, dim3((unsigned)(s_pad / kTileK), (unsigned)(batch * kv_heads)), dim3(256), 0,
                       (hipStream_t)stream, (const uint16_t*)v, (uint16_t*)vt, v_sb, v_ss, v_sh, (int)kv_heads, (int)seq, (int)s_pad);
    return coat_launch_status();
}

extern "C" int coat_attention_forward_bf16(const void* q, const void* k, const void* vt, void* out, float* lse, int64_t batch,
                                           int64_t heads, int64_t kv_heads, int64_t seq, int64_t head_dim, int64_t q_sb,
                                           int64_t q_ss, int64_t q_sh, int64_t k_sb, int64_t k_ss, int64_t k_sh, int64_t o_sb,
                                           int64_t o_ss, int64_t o_sh, int64_t s_pad, float scale, int causal, void* stream) {
    if (batch < 0 || seq < 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0) return COAT_EINVAL;
    if (head_dim != kHeadDim || s_pad % kTileK != 0 || s_pad < seq) return COAT_ESHAPE;
    if (batch * seq == 0) return COAT_OK;
    if (!q || !k || !vt || !out) return COAT_EINVAL;
    if (!coat_aligned16(q) || !coat_aligned16(k) || !coat_aligned16(vt) || !coat_aligned16(out)) return COAT_EALIGN;
    for (int64_t s : {q_sb, q_ss, q_sh, k_sb, k_ss, k_sh, o_sb, o_ss, o_sh})
        if (s % 8 != 0 || s < 0) return COAT_EALIGN;
    // 32-bit byte offsets inside one (batch, head) of k and of vt
    if (seq * k_ss * 2 >= ((int64_t)1 << 31) || (int64_t)kHeadDim * s_pad * 2 >= ((int64_t)1 << 31)) return COAT_ESHAPE;
    AttnArgs A;
    A.q = (const uint16_t*)q; A.k = (const uint16_t*)k; A.vt = (const uint16_t*)vt; A.out = (uint16_t*)out; A.lse = lse;
    A.q_sb = q_sb; A.q_ss = q_ss; A.q_sh = q_sh; A.k_sb = k_sb; A.k_ss = k_ss; A.k_sh = k_sh;
    A.o_sb = o_sb; A.o_ss = o_ss; A.o_sh = o_sh;
    A.batch = (int)batch; A.heads = (int)heads; A.kv_heads = (int)kv_heads; A.seq = (int)seq; A.s_pad = (int)s_pad;
    A.scale_log2e = scale * 1.4426950408889634f;
    const int64_t nqb = (seq + kBlockQ - 1) / kBlockQ;
    const int64_t grid = ((batch * heads + 7) / 8) * 8 * nqb;
    if (grid >= ((int64_t)1 << 31)) return COAT_ESHAPE;
    hipStream_t st = (hipStream_t)stream;
    if (causal) {
        static coat_device_flags ok;
        if (int e = coat_allow_lds(k_attn_fwd<true>, kAttnLdsBytes, ok)) return e;
        hipLaunchKernelGGL((k_attn_fwd<true>), dim3((unsigned)grid), dim3(256), kAttnLdsBytes, st, A);
    } else {
        static coat_device_flags ok;
        if (int e = coat_allow_lds(k_attn_fwd<false>, kAttnLdsBytes, ok)) return e;
        hipLaunchKernelGGL((k_attn_fwd<false>), dim3((unsigned)grid), dim3(256), kAttnLdsBytes, st, A);
    }
    return coat_launch_status();
}
