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
//   O^T[dim, query] = V^T P^T    A = V^T fragments (8 keys of one dimension per lane), B = P^T
// In both results a lane holds one query (column lane % 32), so the running maximum, the running sum and the rescaling
// of O are per-lane scalars; the only cross-lane step of the softmax is one swap between lane l and lane l + 32, which
// hold the two halves of a query's keys.  P^T needs no layout change either: the contraction over keys may run in any
// order as long as both operands agree, and one v_permlane32_swap per two packed registers puts keys 16 j + 8 h .. + 7 into
// half-wave h, which is what two transposing reads of the V tile deliver.
// V^T (keys contiguous) does not exist in memory, and is never formed: the V tile lies in LDS as it lies in memory
// (a key's 128 dimensions per row) and its fragments are read with ds_read_b64_tr_b16, the transposing LDS read of
// gfx950: 16 lanes point at 4 keys x 16 dimensions (lane i at key i / 4, dimensions 4 (i % 4) .. + 3) and lane j receives the
// 4 keys of dimension j.
// K and V tiles go from global memory into a two-stage LDS ring without passing through registers
// (buffer_load_dwordx4 ... lds); 16-byte chunks (K) and 32-byte pieces (V) are XOR-swizzled with the row so that the
// fragment reads are free of bank conflicts.  Blocks are ordered so that the blocks of one (batch, head) run on one XCD (one L2) one after the other,
// longest first (under the causal mask a block's work grows with its position).
#include <math.h>

#include <type_traits>

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
constexpr int kVTileBytes = kTileK * kHeadDim * 2;   // 64 keys x 256 bytes
constexpr int kStageBytes = kKTileBytes + kVTileBytes;
constexpr int kAttnLdsBytes = 2 * kStageBytes;       // 64 KiB: two blocks per CU

struct AttnArgs {
    const uint16_t* q;
    const uint16_t* k;
    const uint16_t* v;
    uint16_t* out;
    float* lse;           // [batch, heads, seq], natural logarithm
    int64_t q_sb, q_ss, q_sh, k_sb, k_ss, k_sh, v_sb, v_ss, v_sh, o_sb, o_ss, o_sh;  // element strides: batch, token, head
    int batch, heads, kv_heads, seq;
    float scale_log2e;    // softmax scale * log2(e)
    float* s_max;         // COAT_MAX_WORDS buffer or NULL: receives the largest group scale of the output
    int fp8_max;          // ... for this FP8 format
};

__device__ __forceinline__ void attn_lds_dma16(v4i_t rsrc, uint32_t lds_addr, int voff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(rsrc)
                 : "memory", "m0");
}
// Four such loads into four consecutive KiB of LDS with one M0 write: the instruction's immediate offset moves both the
// LDS and the memory address on by 1024 per load, so the per-lane memory offsets are passed less that amount; `soff`
// (the tile's offset) is added to the memory address only and takes no part in the range check.
__device__ __forceinline__ void attn_lds_dma16x4(v4i_t rsrc, uint32_t lds_addr, int v0, int v1, int v2, int v3, int soff) {
    asm volatile(
        "s_mov_b32 m0, %0\n\ts_nop 0\n\t"
        "buffer_load_dwordx4 %1, %5, %6 offen lds\n\t"
        "buffer_load_dwordx4 %2, %5, %6 offen offset:1024 lds\n\t"
        "buffer_load_dwordx4 %3, %5, %6 offen offset:2048 lds\n\t"
        "buffer_load_dwordx4 %4, %5, %6 offen offset:3072 lds"
        :
        : "s"(lds_addr), "v"(v0), "v"(v1), "v"(v2), "v"(v3), "s"(rsrc), "s"(soff)
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
    const uint16_t* vbase = A.v + b * A.v_sb + kvh * A.v_sh;
    const v4i_t k_rsrc = attn_rsrc(kbase, (uint32_t)(((int64_t)(A.seq - 1) * A.k_ss + kHeadDim) * 2));
    const v4i_t v_rsrc = attn_rsrc(vbase, (uint32_t)(((int64_t)(A.seq - 1) * A.v_ss + kHeadDim) * 2));
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr3_t)lds;
    // one instruction = 4 rows (keys) of 256 bytes; lane i fills position i % 16 of row i / 16 with the chunk that belongs
    // there: K position p holds chunk p ^ (row & 15); V position p holds chunk ((p / 2) ^ 2 (row & 3)) * 2 + p % 2 (32-byte
    // pieces stay whole: a transposing read takes 32 contiguous bytes of each of 4 keys; the two 16-lane groups that are
    // served together read an even and an odd piece of the same 4 keys, and the swizzle by twice the key keeps the four even
    // and the four odd pieces apart: all 64 banks once).  Keys past the end read zeros.
    int k_off[4], v_off[4];
#pragma unroll
    for (int x = 0; x < 4; x++) {
        const int row = 4 * (4 * wave + x) + (lane >> 4), p = lane & 15;
        k_off[x] = row * (int)(A.k_ss * 2) + ((p ^ (row & 15)) << 4);
        v_off[x] = row * (int)(A.v_ss * 2) + ((((((p >> 1) ^ ((row & 3) << 1)) << 1) | (p & 1))) << 4);
    }
    // per-lane offsets for the four-load form (less the immediate offsets; a row is at least 256 bytes, so none is negative)
    int k_off4[4], v_off4[4];
#pragma unroll
    for (int x = 0; x < 4; x++) {
        k_off4[x] = k_off[x] - 1024 * x;
        v_off4[x] = v_off[x] - 1024 * x;
    }
    auto issue_tile = [&](int t, int stage) {
        const uint32_t kdst = lds_base + stage * kStageBytes + (4 * wave) * 1024;
        const uint32_t vdst = kdst + kKTileBytes;
        const int kt_off = t * kTileK * (int)(A.k_ss * 2), vt_off = t * kTileK * (int)(A.v_ss * 2);
        if ((t + 1) * kTileK <= A.seq) {
            // every key of the tile exists: the tile's offset travels in the scalar offset, outside the range check
            attn_lds_dma16x4(k_rsrc, kdst, k_off4[0], k_off4[1], k_off4[2], k_off4[3], kt_off);
            attn_lds_dma16x4(v_rsrc, vdst, v_off4[0], v_off4[1], v_off4[2], v_off4[3], vt_off);
        } else {
            // the last, partial tile: the whole offset per lane, so that keys past the end fall outside the buffer and read zeros
#pragma unroll
            for (int x = 0; x < 4; x++) attn_lds_dma16(k_rsrc, kdst + x * 1024, k_off[x] + kt_off);
#pragma unroll
            for (int x = 0; x < 4; x++) attn_lds_dma16(v_rsrc, vdst + x * 1024, v_off[x] + vt_off);
        }
    };
    // K fragment (A operand of S^T): row l32 (+ 32 kt), chunk 2 c + h32.  The lane's byte offset inside a K tile is kept
    // per chunk (the swizzle is not linear in c); stage and key half are compile-time constants and end up in the
    // instruction's offset field, so a fragment read costs no address arithmetic.
    uint32_t k_base[8];
#pragma unroll
    for (int c = 0; c < 8; c++) k_base[c] = l32 * 256 + (((2 * c + h32) ^ (l32 & 15)) << 4);
    auto k_frag = [&](auto stage_c, int kt, int c) -> v8bf {
        constexpr int stage = decltype(stage_c)::value;
        return *(const v8bf*)(lds + k_base[c] + (stage * kStageBytes + kt * 32 * 256));
    };
    // V^T fragment (A operand of O^T): dimension 32 dt + l32; the 8 slots of half-wave h hold keys 16 j + 4 h .. + 3 and
    // 16 j + 8 + 4 h .. + 3, the order in which the score accumulators hold them, through two transposing reads.
    // Within a group of 16 lanes, lane i points at key (16 j + 4 h32) + i / 4 (+ 8 for the second read), dimensions
    // d0 + 4 (i % 4) .. + 3 with d0 = 32 dt + 16 * (group % 2); lane i then receives dimension d0 + i of 4 consecutive keys.
    typedef short v4s __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) v4s* lds_v4s_ptr;
    const int tr_i = lane & 15, tr_dim = 16 * ((lane >> 4) & 1) + 4 * (tr_i & 3), tr_key = 4 * h32 + (tr_i >> 2);
    uint32_t v_base[4];  // the lane's byte offset inside a V tile for dimension block dt, key block 0 (the swizzle is not linear in dt)
#pragma unroll
    for (int dt = 0; dt < 4; dt++) {
        const int dim = 32 * dt + tr_dim;
        v_base[dt] = ((dim & 15) << 1) + tr_key * 256 + (((dim >> 4) ^ ((tr_key & 3) << 1)) << 5);
    }
    auto v_frag = [&](auto stage_c, int dt, int j) -> v8bf {
        constexpr int stage = decltype(stage_c)::value;
        const uint8_t* a0 = lds + v_base[dt] + (stage * kStageBytes + kKTileBytes + j * 16 * 256);  // key 16 j + tr_key: same key & 3
        const uint8_t* a1 = a0 + 8 * 256;  // key + 8: the same piece
        const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_ptr)a0);
        const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_ptr)a1);
        typedef short v8s __attribute__((ext_vector_type(8)));
        const v8s both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        return __builtin_bit_cast(v8bf, both);
    };

    v16f o_acc[4];
#pragma unroll
    for (int dt = 0; dt < 4; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) o_acc[dt][r] = 0.0f;
    // Softmax state.  m_ref: the reference maximum of this lane's query, in raw score units; every exponent is taken
    // relative to it, and it is raised (and the accumulators rescaled, for the whole wave) when a tile's maximum exceeds it
    // by more than kLazy log2 units after scaling.  With kLazy = 0 the largest probability of a row is exactly 1, as in the
    // textbook recurrence; a threshold of 8 rescales a few times per block instead of once per tile and was 4 % faster at
    // 4 x 32 x 2048, but then the largest probabilities are rounded to bf16 like all the others and rows with few keys lose
    // a bit (max |out - ref| 1.7e-2 instead of 0.8e-2 on unit-variance values), so it is not used.
    constexpr float kLazy = 0.0f;
    auto max3 = [](float a, float b, float c) {
        float r;
        asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
        return r;
    };
    float m_ref = -INFINITY, l_run = 0.0f;
    const float c2 = A.scale_log2e;

    // One 64-key step; the ring stage is a compile-time constant (the loop below alternates two instances of this code).
    auto step = [&](int t, auto stage_c) {
        constexpr int stage = decltype(stage_c)::value;
        ATTN_WAIT_VMCNT0();               // this wave's part of tile t has landed
        __builtin_amdgcn_s_barrier();     // ... and everybody's; everybody is also done reading tile t - 1
        asm volatile("" ::: "memory");
        // the next tile's loads go out first: issued behind this tile's score products instead (so that the four waves do
        // not queue 32 KiB at the address unit together) they land too late, 196 us against 182 us
        if (t + 1 < nsteps) issue_tile(t + 1, stage ^ 1);
        const int key0 = t * kTileK;
        // waves whose queries all lie before this tile have nothing to add (causal); they still take part in the loads
        if (CAUSAL && key0 > q0 + wave * 32 + 31) return;

        // ---- S^T = K Q^T for the tile's 64 keys
        // The 16 K fragments are read four at a time, each batch while the previous one is multiplied: left to itself the
        // compiler reads one fragment, waits for it and multiplies, 16 LDS round trips in a row.
        v16f s_acc[2];
        v8bf kf[2][4];
#pragma unroll
        for (int c = 0; c < 4; c++) kf[0][c] = k_frag(stage_c, 0, c);
#pragma unroll
        for (int b = 0; b < 4; b++) {          // batch b: key half b / 2, dimension chunks 4 (b % 2) .. + 3
            if (b < 3) {
#pragma unroll
                for (int c = 0; c < 4; c++) kf[(b + 1) & 1][c] = k_frag(stage_c, (b + 1) >> 1, 4 * ((b + 1) & 1) + c);
            }
            __builtin_amdgcn_sched_barrier(0);
            const int kt = b >> 1;
            if ((b & 1) == 0) {
#pragma unroll
                for (int r = 0; r < 16; r++) s_acc[kt][r] = 0.0f;
            }
#pragma unroll
            for (int c = 0; c < 4; c++)
                s_acc[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[b & 1][c], qf[4 * (b & 1) + c], s_acc[kt], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
        // ---- mask (edge tiles only) and the tile's maximum per query, on the raw scores (the scale is positive)
        const bool edge = (CAUSAL && key0 + kTileK - 1 > q0 + wave * 32) || key0 + kTileK > A.seq;  // wave-uniform
        if (edge) {
#pragma unroll
            for (int kt = 0; kt < 2; kt++)
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const int key = key0 + 32 * kt + 8 * (r >> 2) + 4 * h32 + (r & 3);
                    if ((CAUSAL && key > my_q) || key >= A.seq) s_acc[kt][r] = -INFINITY;
                }
        }
        // v_max3_f32 written out: through fmaxf the compiler first canonicalises every accumulator register (a v_max_f32
        // of the value with itself), 59 instructions for these 32 values instead of 18.  No score is a NaN.
        float mx;
        {
            float ma = max3(s_acc[0][0], s_acc[0][1], s_acc[0][2]), mb = max3(s_acc[1][0], s_acc[1][1], s_acc[1][2]);
#pragma unroll
            for (int r = 3; r < 15; r += 2) {
                ma = max3(ma, s_acc[0][r], s_acc[0][r + 1]);
                mb = max3(mb, s_acc[1][r], s_acc[1][r + 1]);
            }
            ma = max3(ma, s_acc[0][15], s_acc[1][15]);
            mx = max3(ma, mb, mb);
            const auto sw = __builtin_amdgcn_permlane32_swap(f2u(mx), f2u(mx), false, false);  // the other 32 keys of this query
            mx = max3(u2f(sw[0]), u2f(sw[1]), u2f(sw[1]));
        }
        // raise the reference where the tile exceeds it by more than kLazy (always on the first tile, from -inf)
        if (__builtin_amdgcn_ballot_w64((mx - m_ref) * c2 > kLazy) != 0) {
            const float m_new = fmaxf(m_ref, mx);  // finite: key 0 is visible to every query
            const float alpha = __builtin_amdgcn_exp2f((m_ref - m_new) * c2);
            m_ref = m_new;
            l_run *= alpha;
#pragma unroll
            for (int dt = 0; dt < 4; dt++)
#pragma unroll
                for (int r = 0; r < 16; r++) o_acc[dt][r] *= alpha;
        }
        // ---- P = exp2(S c - m c), packed to bf16 as the B operand of O^T = V^T P^T
        const float mc = -m_ref * c2;
        uint32_t pk[2][8];
        float ps0 = 0.0f, ps1 = 0.0f;
#pragma unroll
        for (int kt = 0; kt < 2; kt++)
#pragma unroll
            for (int r = 0; r < 16; r += 2) {
                const float p0 = __builtin_amdgcn_exp2f(fmaf(s_acc[kt][r], c2, mc)), p1 = __builtin_amdgcn_exp2f(fmaf(s_acc[kt][r + 1], c2, mc));
                ps0 += p0;
                ps1 += p1;
                pk[kt][r >> 1] = pack_bf16x2(p0, p1);
            }
        l_run += ps0 + ps1;
        // ---- O^T += V^T P^T, 16 keys per instruction: chunk j = 2 kt + u takes accumulator registers 8 u .. 8 u + 7
#pragma unroll
        for (int kt = 0; kt < 2; kt++)
#pragma unroll
            for (int u = 0; u < 2; u++) {
                // The 16 keys of chunk j = 2 kt + u are summed over, so their order inside the product is free as long as P and V
                // agree: the lane's packed registers 4 u .. 4 u + 3 (keys 16 j + 4 h .. + 3 and 16 j + 8 + 4 h .. + 3) are taken as
                // its 8 slots as they are, and the V^T fragment reads those keys into the same slots: no lane exchange.
                const v4i_t pw = (v4i_t){(int)pk[kt][4 * u], (int)pk[kt][4 * u + 1], (int)pk[kt][4 * u + 2], (int)pk[kt][4 * u + 3]};
                const v8bf pfrag = __builtin_bit_cast(v8bf, pw);
#pragma unroll
                for (int dt = 0; dt < 4; dt++)
                    o_acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(v_frag(stage_c, dt, 2 * kt + u), pfrag, o_acc[dt], 0, 0, 0);
            }
    };
    issue_tile(0, 0);
    for (int t = 0; t < nsteps; t += 2) {
        step(t, std::integral_constant<int, 0>{});
        if (t + 1 < nsteps) step(t + 1, std::integral_constant<int, 1>{});
    }

    // ---- normalise and store: the two half-waves hold the two parts of each query's sum
    {
        const auto sw = __builtin_amdgcn_permlane32_swap(f2u(l_run), f2u(l_run), false, false);
        l_run = u2f(sw[0]) + u2f(sw[1]);
    }
    const float inv_l = 1.0f / l_run;
    float amax = 0.0f;  // of the values as stored (rows beyond the sequence excluded)
    if (my_q < A.seq) {
        uint16_t* orow = A.out + b * A.o_sb + (int64_t)my_q * A.o_ss + head * A.o_sh;
#pragma unroll
        for (int dt = 0; dt < 4; dt++)
#pragma unroll
            for (int g = 0; g < 4; g++) {  // accumulator registers 4 g .. 4 g + 3: dimensions 32 dt + 8 g + 4 h .. + 3
                const v16f& o = o_acc[dt];
                const uint32_t w0 = pack_bf16x2(o[4 * g] * inv_l, o[4 * g + 1] * inv_l), w1 = pack_bf16x2(o[4 * g + 2] * inv_l, o[4 * g + 3] * inv_l);
                *(uint2*)(orow + 32 * dt + 8 * g + 4 * h32) = make_uint2(w0, w1);
                if (A.s_max) amax = fmaxf(amax, fmaxf(fmaxf(fabsf(bf16lo(w0)), fabsf(bf16hi(w0))), fmaxf(fabsf(bf16lo(w1)), fabsf(bf16hi(w1)))));
            }
        if (h32 == 0 && A.lse)
            A.lse[((int64_t)b * A.heads + head) * A.seq + my_q] = (m_ref * c2 + __builtin_amdgcn_logf(l_run)) * 0.6931471805599453f;
    }
    // the largest 1 x QB group scale of the output, for a consumer that quantizes it per tensor: one lazy atomic per wave
    if (A.s_max) {
        amax = cluster_max<64>(amax);
        const float sc = A.fp8_max == kE4M3 ? group_scale<kE4M3>(amax) : group_scale<kE5M2>(amax);
        if (lane == 0) atomic_max_nonneg(max_slot(A.s_max), sc);
    }
}

}  // namespace coat

using namespace coat;

extern "C" int coat_attention_forward_bf16(const void* q, const void* k, const void* v, void* out, float* lse, int64_t batch,
                                           int64_t heads, int64_t kv_heads, int64_t seq, int64_t head_dim, int64_t q_sb,
                                           int64_t q_ss, int64_t q_sh, int64_t k_sb, int64_t k_ss, int64_t k_sh, int64_t v_sb,
                                           int64_t v_ss, int64_t v_sh, int64_t o_sb, int64_t o_ss, int64_t o_sh, float scale,
                                           int causal, float* s_max, int fp8_max, void* stream) {
    if (s_max && fp8_max != kE4M3 && fp8_max != kE5M2) return COAT_EINVAL;
    if (batch < 0 || seq < 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0) return COAT_EINVAL;
    if (head_dim != kHeadDim) return COAT_ESHAPE;
    if (batch * seq == 0) return COAT_OK;
    if (!q || !k || !v || !out) return COAT_EINVAL;
    if (!coat_aligned16(q) || !coat_aligned16(k) || !coat_aligned16(v) || !coat_aligned16(out)) return COAT_EALIGN;
    for (int64_t s : {q_sb, q_ss, q_sh, k_sb, k_ss, k_sh, v_sb, v_ss, v_sh, o_sb, o_ss, o_sh})
        if (s % 8 != 0 || s < 0) return COAT_EALIGN;
    // 32-bit byte offsets inside one (batch, head) of k and of v
    if ((seq + kTileK) * k_ss * 2 >= ((int64_t)1 << 31) || (seq + kTileK) * v_ss * 2 >= ((int64_t)1 << 31)) return COAT_ESHAPE;
    AttnArgs A;
    A.q = (const uint16_t*)q; A.k = (const uint16_t*)k; A.v = (const uint16_t*)v; A.out = (uint16_t*)out; A.lse = lse; A.s_max = s_max; A.fp8_max = fp8_max;
    A.q_sb = q_sb; A.q_ss = q_ss; A.q_sh = q_sh; A.k_sb = k_sb; A.k_ss = k_ss; A.k_sh = k_sh;
    A.v_sb = v_sb; A.v_ss = v_ss; A.v_sh = v_sh; A.o_sb = o_sb; A.o_ss = o_ss; A.o_sh = o_sh;
    A.batch = (int)batch; A.heads = (int)heads; A.kv_heads = (int)kv_heads; A.seq = (int)seq;
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
