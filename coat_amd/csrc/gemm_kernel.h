// Per-tensor-scaled FP8 GEMM on CDNA4 MFMA:  C[M,N] = (A[M,K] . B[N,K]^T) * (sA * sB) (+ bias), fp32 accumulate.
//
// Replaces _fp8matmul_kernel (coat/activation/real_quantization/linear.py:61-169).  Both operands are
// K-contiguous ("A row-major times the transpose of a row-major B"), which is the only form the reference uses:
// every tensor is kept in both orientations so that forward, dgrad and wgrad are all of this form
// (linear.py:253-302).  Operand formats are independent (e4m3 or e5m2 each: gradients are e5m2).
//
// Tiling: one 256 x 256 output tile per 512-thread block at a time, 2 x 4 waves, each wave 128 x 64 as 4 x 2 tiles of
// v_mfma_f32_32x32x64_f8f6f4 (two waves per SIMD).  The grid is persistent, one block per CU (the LDS ring takes the
// whole 160 KiB), and every block walks its share of the tiles; block ids map to tiles so that the 8 XCDs
// (round-robin block dispatch) each work on a contiguous band of tiles, ordered in panels of 8 tile-rows, which keeps
// A / B slabs hot in that XCD's L2.
// K advances in steps of 128 bytes (two MFMA K-substeps).  LDS is a ring of five 32 KiB slabs (256 rows x 128 bytes of
// one matrix), alternately A and B, filled straight from global memory (buffer_load_dwordx4 ... lds, no register
// staging); the ring runs across tile boundaries, so the next tile's first slabs are in flight during the epilogue.
// 16-byte chunks are XOR-swizzled with the row so that the 32-byte-per-lane fragment reads are conflict-free.
// Fragments of both substeps are double-buffered in registers; there is one barrier per K-step, placed where every
// wave holds the rest of the step in registers, which frees the step's two slabs for refilling.
// The MFMA takes the B tile as its first operand, so a lane ends up holding 4 consecutive n for one m per accumulator
// quad: bf16 rows are packed 4 at a time, and a 1 x 16 quantization group is two quads in each of the lanes l, l^32.
#pragma once
#include <type_traits>
#include "coat_device.h"
#include "coat_host.h"

namespace coat {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int BM = 256, BN = 256, BK = 128;
constexpr int NUNIT = 5;                       // LDS ring of slabs (5 x 32 KiB = the whole 160 KiB LDS)
constexpr int kUnitBytes = BM * BK;            // one matrix's 256 rows x 128 bytes of K = 32 KiB
constexpr int kLdsBytes = NUNIT * kUnitBytes;
static_assert(BM == BN, "A and B slabs share one unit size");

// kEpiRes*: the product is rounded to bf16 as kEpiBf16 would store it, a bf16 tensor R of C's shape is added in fp32, and
// the sum goes out as bf16 (the residual additions that follow a projection, and the sums of the gradients that reach one
// tensor); the Quant variants also emit the 1 x 16 per-group FP8 codes and bf16 scales of the fp32 sum.
enum Epilogue { kEpiBf16 = 0, kEpiQuantE4M3 = 1, kEpiQuantE5M2 = 2, kEpiResBf16 = 3, kEpiResQuantE4M3 = 4, kEpiResQuantE5M2 = 5 };

// One launch multiplies up to kMaxGroup independent problems of one shape (the q / k / v or gate / up projections of a
// layer): their tiles form one sequence for the persistent grid, so a partial last round of tiles is paid once per
// group instead of once per problem, and the LDS ring runs on from one problem into the next.
constexpr int kMaxGroup = 4;
struct GemmProblem {
    const uint8_t* A;   // [M, K]
    const uint8_t* B;   // [N, K]
    void* C;            // bf16 [M, N] or fp8 [M, N]
    void* Cs;           // bf16 [M, N/16] (quantize epilogue)
    const void* sa;     // per-tensor scales, one element each
    const void* sb;
    const void* bias;   // [N] or nullptr
};
// The shape and the first problem come first: a wave fetches its kernel arguments when it starts (the host writes them per
// launch, so they are not in any cache), and the plain GEMM then touches two 64-byte lines of them as it would without the
// group (with the seven pointers laid out as arrays of four the same kernel ran 1.3 % slower on config 3).
struct GemmArgs {
    int sa_dt, sb_dt, bias_dt;
    int M, N, K;
    int tiles_m, tiles_n;
    int nprob;                     // problems in this launch (1 .. kMaxGroup)
    const void* res;               // kEpiRes*: bf16 [M, N] added to the rounded product (may be the tensor C itself)
    void* Cq;                      // kEpiResQuant*: fp8 [M, N] codes of the sum (P[0].C: its bf16, P[0].Cs: the scales)
    GemmProblem P[kMaxGroup];
    unsigned long long* probe;     // PROBE instances only (never part of the library): 2 x gridDim.x durations
};

// A slab row is 128 bytes = eight 16-byte chunks (one full cache line per row and load instruction: fetching rows as
// two 64-byte halves was measured at 0.6 x the LDS-DMA throughput).  A 16-byte-per-lane LDS read is served 16 lanes
// (256 bytes, 64 banks) per cycle, so 16 consecutive rows reading the same chunk must land in 16 different 16-byte
// slots modulo 256: row & 1 selects the 128-byte half, and placing chunk c of row r at position c ^ ((r >> 1) & 7)
// spreads the eight row pairs over the eight slots of a half.
__device__ __forceinline__ int swz_chunk(int row, int chunk) { return chunk ^ ((row >> 1) & 7); }

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef __attribute__((address_space(1))) void* global_ptr_t;
typedef int v4i __attribute__((ext_vector_type(4)));

// buffer_load_dwordx4 ... lds: every lane fetches 16 bytes at byte offset `voff` of the buffer and the wave's 1 KiB
// lands in LDS at lds_addr + 16 * lane without passing through registers; offsets beyond the buffer's extent fill
// zeros.  Issued as inline assembly so that the compiler does not order later LDS reads behind it with a full
// vmcnt(0) wait (it cannot tell which ring stage a read touches); completion is tracked by hand with s_waitcnt vmcnt.
// `soff` is a wave-uniform byte offset added to every lane's address; it takes no part in the range check, which is on
// `voff` alone.
__device__ __forceinline__ void lds_dma16(v4i rsrc, uint32_t lds_addr, int voff, int soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(rsrc), "s"(soff)
                 : "memory", "m0");
}
__device__ __forceinline__ v4i make_rsrc(const void* p, uint32_t bytes) {
    const uint64_t a = (uint64_t)p;
    return (v4i){(int)(uint32_t)a, (int)(uint32_t)(a >> 32) & 0xFFFF, (int)bytes, 0x00020000};
}

// v_writelane with a constant lane: lane LANE of `t` becomes the wave-uniform value v.
template <int LANE> __device__ __forceinline__ void write_lane(uint32_t& t, uint32_t v) {
    asm volatile("v_writelane_b32 %0, %1, %2" : "+v"(t) : "s"(v), "n"(LANE));
}
template <int LANE> __device__ __forceinline__ void write_lane_ptr(uint32_t& t, const void* p) {
    write_lane<LANE>(t, (uint32_t)(uintptr_t)p);
    write_lane<LANE + 1>(t, (uint32_t)((uintptr_t)p >> 32));
}
// Problems P .. kMaxGroup - 1 into the table: lanes 14 P .. 14 P + 13 = the seven pointers, lane 14 kMaxGroup + P = the
// product of the two scales.
template <int P> __device__ __forceinline__ void fill_table(uint32_t& t, const GemmArgs& G) {
    if constexpr (P < kMaxGroup) {
        if (P < G.nprob) {  // (the arguments of unused problems are not even fetched)
            write_lane_ptr<14 * P + 0>(t, G.P[P].A);
            write_lane_ptr<14 * P + 2>(t, G.P[P].B);
            write_lane_ptr<14 * P + 4>(t, G.P[P].C);
            write_lane_ptr<14 * P + 6>(t, G.P[P].Cs);
            write_lane_ptr<14 * P + 8>(t, G.P[P].sa);
            write_lane_ptr<14 * P + 10>(t, G.P[P].sb);
            write_lane_ptr<14 * P + 12>(t, G.P[P].bias);
            const float sc = load_rt_f32(G.P[P].sa, 0, G.sa_dt) * load_rt_f32(G.P[P].sb, 0, G.sb_dt);
            write_lane<14 * kMaxGroup + P>(t, __builtin_amdgcn_readfirstlane(f2u(sc)));
            fill_table<P + 1>(t, G);
        }
    }
}

// s_waitcnt vmcnt(N) only (expcnt / lgkmcnt left at their maxima), gfx9 encoding.
#define COAT_WAIT_VMCNT(N) __builtin_amdgcn_s_waitcnt(((N) & 0xF) | (0x7 << 4) | (0xF << 8) | ((((N) >> 4) & 0x3) << 14))
// lgkmcnt(0) only: all LDS reads issued so far have returned
#define COAT_WAIT_LGKM0() __builtin_amdgcn_s_waitcnt(0xC07F)

// Eight waves (2 along M x 4 along N), each 128 x 64 of the 256 x 256 tile as 4 x 2 tiles of
// v_mfma_f32_32x32x64_f8f6f4, two waves per SIMD.
// Persistent: the grid is one block per CU; a block walks its share of the output tiles and the LDS ring runs straight
// across tile boundaries, so the first slabs of the next tile are already in flight while the epilogue stores drain.
// PROBE: every block also leaves its duration in shader clocks (s_memtime) and in ticks of the constant 100 MHz counter
// (s_memrealtime) in G.probe, which gives the clock the kernel really runs at.  The library instantiates PROBE = false
// only; the benchmark builds its own instances.
template <int FMT_A, int FMT_B, int EPI, bool VEC16, int QBE, bool GROUPED, bool PROBE = false>
__global__ __launch_bounds__(512) void k_fp8_gemm(GemmArgs G) {
    static_assert(QBE == 16 || ((EPI == kEpiQuantE4M3 || EPI == kEpiQuantE5M2) && (QBE == 32 || QBE == 64)), "group size of the quantizing epilogue");
    static_assert(EPI < kEpiResBf16 || (VEC16 && !GROUPED), "the residual epilogues are single problems with 16-byte rows");
    constexpr int NWN = 4, NW = 2 * NWN;      // waves along N, waves per block
    constexpr int TJ = BN / (NWN * 32);       // n-tiles per wave (2); m-tiles per wave is 4
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / NWN, wn = wave % NWN;

    // ---- XCD-aware tile schedule.  Blocks are dispatched round-robin over the 8 XCDs, so block b runs on XCD b % 8.
    // XCD x owns the contiguous band [x * per_xcd, (x + 1) * per_xcd) of the tile order below, and its blocks take the
    // band's tiles in rounds of gridDim.x / 8: at any time one XCD works on neighbouring tiles, whose A / B slabs are
    // shared through that XCD's L2.  The tile order runs down panels of GROUP_M tile-rows.
    const int ntiles1 = G.tiles_m * G.tiles_n;  // tiles of one problem; the problems' tiles follow one another
    const int ntiles = GROUPED ? G.nprob * ntiles1 : ntiles1;
    const int per_xcd = (ntiles + 7) / 8;
    const int xcd = blockIdx.x & 7, my = blockIdx.x >> 3, stride = gridDim.x >> 3;
    const int band = min(max(ntiles - xcd * per_xcd, 0), per_xcd);
    const int my_ntiles = my < band ? (band - my + stride - 1) / stride : 0;
    if (my_ntiles == 0) return;
    uint64_t probe_t0 = 0, probe_r0 = 0;
    if constexpr (PROBE) {
        probe_t0 = __builtin_amdgcn_s_memtime();
        probe_r0 = __builtin_amdgcn_s_memrealtime();
    }
    // Grouped launch: the problems' pointers and scales are kept across the lanes of one VGPR (lane 14 p + 2 f and the
    // next: pointer f of problem p as two dwords; lane 56 + p: its combined scale) and fetched with v_readlane when a
    // tile begins: scalar registers for four problems are not to be had, and reading the kernel arguments at that point
    // would put a scalar load and its wait into the loading role's path once per tile.
    uint32_t ptab = 0;
    if (GROUPED) {
        static_assert(sizeof(GemmProblem) == 56 && kMaxGroup * 14 + kMaxGroup <= 64, "table fits the lanes of one register");
        // the kernel arguments arrive through scalar loads (one fetch per scalar cache, not one per wave)
        fill_table<0>(ptab, G);
    }
    auto tab_ptr = [&](int prob, int field) -> const void* {
        const uint32_t lo = __builtin_amdgcn_readlane(ptab, prob * 14 + 2 * field);
        const uint32_t hi = __builtin_amdgcn_readlane(ptab, prob * 14 + 2 * field + 1);
        // known to be global memory: a generic pointer would turn the epilogue's stores into flat stores, which count
        // as LDS operations too, and the next tile's first wait for its fragment reads would then wait for them
        return (const void*)(global_ptr_t)(((uint64_t)hi << 32) | lo);
    };
    constexpr int GROUP_M = 4;  // 4 x 8 tiles per XCD round; measured against 2, 8, 16: 0.3-0.7 % per GEMM, 0.6 % on the 7B layer
    auto tile_origin = [&](int it, int& m0, int& n0, int& prob) {
        int tile = xcd * per_xcd + my + it * stride;
        prob = 0;
        if (GROUPED) {
            prob = __builtin_amdgcn_readfirstlane(tile / ntiles1);
            tile -= prob * ntiles1;
        }
        const int width = GROUP_M * G.tiles_n;
        const int group = tile / width;
        const int gsize = min(G.tiles_m - group * GROUP_M, GROUP_M);
        m0 = (group * GROUP_M + (tile % width) % gsize) * BM;
        n0 = ((tile % width) / gsize) * BN;
    };

    // ---- global -> LDS without passing through registers.  The ring holds 5 slabs; slab u of this block's slab
    // sequence is the A slab (u even) or the B slab (u odd) of K-step u / 2 and lives in slot u % 5.  One wave
    // instruction fills 1 KiB of LDS contiguously (lane i at +16 i) = 8 slab rows; the lane picks the global chunk
    // that belongs at its position under the swizzle.  Out-of-range rows / K-tail chunks use an offset beyond the
    // buffer's extent, which fills zeros.
    //
    // Ping-pong schedule.  The two waves of a SIMD work half a K-step apart: waves 0-3 (role 0) and waves 4-7 (role 1)
    // alternate between a memory phase (read the 24 fragments of a K-step from LDS into registers, issue 8 loads of a
    // later slab) and a compute phase (16 MFMAs back to back, nothing else in the instruction stream), separated by
    // block-wide barriers; role 1 starts one phase late.  In every phase each SIMD has one wave feeding the matrix
    // pipe and one wave doing memory work, so a load or LDS read that waits for its unit never delays an MFMA.
    //   phase 2j-1: role 0 mem(j)  [reads slabs A(j) B(j); loads B(j+1)]   role 1 MFMA(j-1)
    //   phase 2j  : role 0 MFMA(j)                                          role 1 mem(j) [reads A(j) B(j); loads A(j+2)]
    // Slots: B(j+1) replaces A(j-1) and A(j+2) replaces B(j-1), both last read in phase 2j-2; a wave waits for its own
    // loads at the end of its compute phase (a whole phase after issuing them), before the barrier that publishes them.
    const int role = wave >> 2;                     // 0: loads B slabs, 1: loads A slabs
    const uint32_t rsrc_bytes = role ? (uint32_t)(G.M * G.K) : (uint32_t)(G.N * G.K);
    v4i rsrc = make_rsrc(role ? G.P[0].A : G.P[0].B, rsrc_bytes);  // of the problem whose slabs are being loaded
    const int R = role ? G.M : G.N;                 // rows of the matrix this wave loads
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_ptr_t)lds;
    const int nstep = (G.K + BK - 1) / BK;
    constexpr int kOob = 0x7FFFFFFF;
    constexpr int LI = 8;                           // load instructions per wave per slab (8 rows each; 4 waves per slab)
    const int lrow = (wave & 3) * (LI * 8) + (lane >> 3);  // + 8 i
    // rows 8 i apart alternate between two swizzle patterns, and two instructions of the same parity differ by a
    // multiple of 16 rows, which goes into the scalar offset: two per-lane offsets suffice
    int kc[2], off[2];
    kc[0] = swz_chunk(lrow, lane & 7) * 16;
    kc[1] = swz_chunk(lrow + 8, lane & 7) * 16;
    // load cursor: tile iteration lt, K-step lstep of that tile, global K-step counter lg (gives the ring slot)
    int lt = 0, lstep = 0, lslot = role ? 0 : 1;    // A(g) lives in slot 2g % 5, B(g) in (2g + 1) % 5
    int lr0 = 0;                                    // first row (of the loaded matrix) of the tile being loaded
    bool ledge = false;                             // its rows run past the end of the matrix (or there is no such tile)
    auto set_load_tile = [&](int it) {
        const bool live = it < my_ntiles;
        int m0 = 0, n0 = 0, prob = 0;
        if (live) {
            tile_origin(it, m0, n0, prob);
            if (GROUPED) rsrc = make_rsrc(tab_ptr(prob, role ? 0 : 1), rsrc_bytes);
        }
        lr0 = live ? (role ? m0 : n0) : R;
        ledge = lr0 + BM > R;
#pragma unroll
        for (int p = 0; p < 2; p++) off[p] = live ? (lr0 + lrow + 8 * p) * G.K + kc[p] : 0;
    };
    set_load_tile(0);
    // The K-step offset and the 16-row multiple go into the scalar offset, which takes no part in the range check:
    // rows past the matrix end and chunks past K (edge tiles / a last partial K-step only) are masked by hand.
    auto issue_slab = [&]() {
        const int k0 = lstep * BK;
        const uint32_t dst = lds_base + lslot * kUnitBytes + (wave & 3) * (LI * 8 * BK);
        const bool check = ledge || k0 + BK > G.K;
#pragma unroll
        for (int i = 0; i < LI; i++) {
            int v = off[i & 1];
            if (check) {
                if (lr0 + lrow + 8 * i >= R || k0 + kc[i & 1] >= G.K) v = kOob;
            }
            lds_dma16(rsrc, dst + i * (8 * BK), v, k0 + (i >> 1) * 16 * G.K);
        }
        lslot = lslot + 2 >= NUNIT ? lslot + 2 - NUNIT : lslot + 2;
        if (++lstep == nstep) {
            lstep = 0;
            set_load_tile(++lt);  // past the last tile: zero fills
        }
    };
    // fragment addresses (bytes inside a slab) for this lane and K-substep 0: row = tile base + lane % 32, 16-byte
    // chunks 2 * (lane / 32) + h; the chunks of substep 1 are those + 4, i.e. the address with bit 6 flipped.
    int fa_off[2], fb_off[2];  // + t * 32 * BK per 32-row tile
#pragma unroll
    for (int h = 0; h < 2; h++) {
        const int c = 2 * (lane >> 5) + h;
        const int rowa = wm * 128 + (lane & 31), rowb = wn * (TJ * 32) + (lane & 31);
        fa_off[h] = rowa * BK + (swz_chunk(rowa, c) << 4);
        fb_off[h] = rowb * BK + (swz_chunk(rowb, c) << 4);
    }
    int sl_frag = 0;  // ring slot of the A slab of the K-step whose fragments are read next (its B slab: next slot)
    auto load_fa = [&](int slot_a, int sub, int t) -> v8i {
        const uint8_t* sa = lds + slot_a * kUnitBytes + t * 32 * BK;
        const int x = sub * 64;
        const uint4 a0 = *(const uint4*)(sa + (fa_off[0] ^ x)), a1 = *(const uint4*)(sa + (fa_off[1] ^ x));
        return (v8i){(int)a0.x, (int)a0.y, (int)a0.z, (int)a0.w, (int)a1.x, (int)a1.y, (int)a1.z, (int)a1.w};
    };
    auto load_fb = [&](int slot_a, int sub, int t) -> v8i {
        const uint8_t* sb = lds + (slot_a + 1 == NUNIT ? 0 : slot_a + 1) * kUnitBytes + t * 32 * BK;
        const int x = sub * 64;
        const uint4 b0 = *(const uint4*)(sb + (fb_off[0] ^ x)), b1 = *(const uint4*)(sb + (fb_off[1] ^ x));
        return (v8i){(int)b0.x, (int)b0.y, (int)b0.z, (int)b0.w, (int)b1.x, (int)b1.y, (int)b1.z, (int)b1.w};
    };

    v16f acc[TJ][4];  // [n-tile j][m-tile i]
    v8i fax[4], fbx[TJ], fay[4], fby[TJ];  // fragments of K-substep 0 (x) and 1 (y)
    // prologue: A(0) B(0) A(1) in flight (role 1: two A slabs, role 0: one B slab), all landed and published
    issue_slab();
    if (role) issue_slab();
    COAT_WAIT_VMCNT(0);
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    if (role) __builtin_amdgcn_s_barrier();  // role 1 runs one phase behind
#define COAT_MFMA(FB_, FA_, J, I) \
    acc[J][I] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(FB_[J], FA_[I], acc[J][I], FMT_B, FMT_A, 0, 0, 0, 0)
    static_assert(TJ == 2 && NW == 8, "the schedule is written for eight waves of 128 x 64");
    // The four groups of fragment reads are kept in this order (scheduling barriers): left to itself the compiler
    // hoisted the address additions and issued the reads in another order in one instantiation of this kernel, whose
    // K loop then ran 3 % slower with otherwise the same instructions (the loop sits at the LDS limit).
    auto mem_phase = [&]() {
#pragma unroll
        for (int t = 0; t < 4; t++) fax[t] = load_fa(sl_frag, 0, t);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < TJ; t++) fbx[t] = load_fb(sl_frag, 0, t);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 4; t++) fay[t] = load_fa(sl_frag, 1, t);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < TJ; t++) fby[t] = load_fb(sl_frag, 1, t);
        __builtin_amdgcn_sched_barrier(0);
        sl_frag = sl_frag + 2 >= NUNIT ? sl_frag + 2 - NUNIT : sl_frag + 2;
        issue_slab();
        // every fragment has arrived before the barrier: the compute phase has nothing to wait for, and the slabs
        // just read may be overwritten by loads issued after the barrier that follows the compute phase
        COAT_WAIT_LGKM0();
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };
    auto compute_phase = [&]() {
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < TJ; j++)
#pragma unroll
            for (int i = 0; i < 4; i++) COAT_MFMA(fbx, fax, j, i);
#pragma unroll
        for (int j = 0; j < TJ; j++)
#pragma unroll
            for (int i = 0; i < 4; i++) COAT_MFMA(fby, fay, j, i);
        __builtin_amdgcn_sched_barrier(0);
        COAT_WAIT_VMCNT(0);  // this wave's loads (issued a phase ago) and, once per tile, its epilogue stores
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };
    const float scale0 = load_rt_f32(G.P[0].sa, 0, G.sa_dt) * load_rt_f32(G.P[0].sb, 0, G.sb_dt);
    if (EPI != kEpiBf16 && EPI != kEpiResBf16) enable_fp8_saturation();
    const int half = lane >> 5;
    constexpr bool vec16 = VEC16;  // rows of C start 16-byte aligned (N % 8 == 0): 16-byte stores

    // Tile loop.  The epilogue of tile it-1 opens the first memory phase of tile it (the other role computes
    // meanwhile); after the last tile it runs on its own.
    for (int it = 0; it <= my_ntiles; it++) {
    if (it > 0) {
    int m0, n0, prob;
    tile_origin(it - 1, m0, n0, prob);
    float scale = scale0;
    void* Cp = G.P[0].C;
    void* Csp = G.P[0].Cs;
    const void* biasp = G.P[0].bias;
    if (GROUPED) {
        scale = u2f(__builtin_amdgcn_readlane(ptab, kMaxGroup * 14 + prob));
        Cp = (void*)tab_ptr(prob, 2);
        Csp = (void*)tab_ptr(prob, 3);
        biasp = tab_ptr(prob, 6);
    }

    // ---- epilogue (stores are not waited for: they drain while the next tile is multiplied)
    uint8_t* const c_tile = (uint8_t*)Cp + ((int64_t)m0 * G.N + n0) * 2;  // bf16 output: origin of this tile
    const uint32_t c_lane_off = (uint32_t)((wm * 128 + (lane & 31)) * G.N + wn * (TJ * 32) + 8 * half) * 2;
    const int m_lim = G.M - m0 - wm * 128 - (lane & 31);   // row i * 32 of this lane exists iff i * 32 < m_lim
    const int n_lim = G.N - n0 - wn * (TJ * 32) - 8 * half;  // column offset c of this lane exists iff c < n_lim
    // quantized output: fp8 codes [M, N] and bf16 scales [M, N / 16] (N % 16 == 0), same addressing scheme
    uint8_t* const q_tile = (uint8_t*)Cp + ((int64_t)m0 * G.N + n0);
    uint8_t* const s_tile = (uint8_t*)Csp + ((int64_t)m0 * (G.N >> 4) + (n0 >> 4)) * 2;
    const uint32_t q_lane_off = (uint32_t)((wm * 128 + (lane & 31)) * G.N + wn * (TJ * 32) + 8 * half);
    const uint32_t s_lane_off = (uint32_t)((wm * 128 + (lane & 31)) * (G.N >> 4) + wn * (TJ * 2)) * 2;
    const int q_n_lim = G.N - n0 - wn * (TJ * 32);          // a 16-column group at offset c exists iff c < q_n_lim
    const bool pack_scales = (G.N & 63) == 0 && q_n_lim >= TJ * 32 && ((uintptr_t)Csp & 7) == 0;  // wave-uniform
    if constexpr (EPI >= kEpiResBf16) {
        // Product + residual.  t = bf16(acc * scale (+ bias)) is what kEpiBf16 stores; after the same lane swap a lane
        // holds one 16-byte run of t (8 consecutive columns of one row), loads the same run of R, adds in fp32 and
        // stores bf16 of the sum: bit for bit what a bf16 tensor addition of the stored product and R gives
        // (reference add_fwd.py:107-137 after linear.py:166-169).  kEpiResQuant*: the run is also half of a 1 x 16 group
        // (the other half sits in lane ^ 32), so the group's scale (amax + 1e-10) / fp8max of the fp32 sum, its codes and
        // the bf16 scale come out of the same registers.
        constexpr bool QUANT = EPI != kEpiResBf16;
        constexpr int KIND = EPI == kEpiResQuantE5M2 ? kE5M2 : kE4M3;
        const uint8_t* const r_tile = (const uint8_t*)G.res + ((int64_t)m0 * G.N + n0) * 2;
        uint8_t* const cq_tile = (uint8_t*)G.Cq + ((int64_t)m0 * G.N + n0);
        // FULL (wave-uniform): the wave's 128 x 64 lie inside the matrix and there is no bias, so no load, store or
        // addition is conditional; edge tiles take the guarded instance of the same code.
        auto residual_epilogue = [&](auto full_c) {
        constexpr bool FULL = decltype(full_c)::value;
        constexpr int RD = 2;
        uint4 rres[RD][TJ][2];  // the residual runs of accumulator row-block i (slot i % RD); the next blocks' are in flight
        auto load_res = [&](int i) {
#pragma unroll
            for (int j = 0; j < TJ; j++)
#pragma unroll
                for (int qp = 0; qp < 2; qp++) {
                    // unconditional load (a load under a branch is waited for on the spot); lanes outside read the tile's origin
                    const bool in = FULL || (i * 32 < m_lim && j * 32 + 16 * qp < n_lim);
                    const uint32_t off = (uint32_t)(((i * 32) * G.N + j * 32 + 16 * qp) * 2) + c_lane_off;
                    rres[i % RD][j][qp] = *(const uint4*)(r_tile + (in ? off : 0u));
                }
        };
#pragma unroll
        for (int i = 0; i < RD - 1; i++) load_res(i);
#pragma unroll
        for (int i = 0; i < 4; i++) {
            if (i + RD - 1 < 4) load_res(i + RD - 1);
            uint32_t spack[TJ] = {};
#pragma unroll
            for (int j = 0; j < TJ; j++) {
                const int nb = n0 + wn * (TJ * 32) + j * 32 + 4 * half;
                float v[16];
#pragma unroll
                for (int r = 0; r < 16; r++) v[r] = acc[j][i][r] * scale;
                if (!FULL && biasp) {
#pragma unroll
                    for (int q = 0; q < 4; q++)
#pragma unroll
                        for (int e = 0; e < 4; e++) {
                            const int n = nb + 8 * q + e;
                            if (n < G.N) v[4 * q + e] += load_rt_f32(biasp, n, G.bias_dt);
                        }
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int qp = 0; qp < 2; qp++) {
                    const uint32_t a0 = pack_bf16x2(v[8 * qp], v[8 * qp + 1]), a1 = pack_bf16x2(v[8 * qp + 2], v[8 * qp + 3]);
                    const uint32_t b0 = pack_bf16x2(v[8 * qp + 4], v[8 * qp + 5]), b1 = pack_bf16x2(v[8 * qp + 6], v[8 * qp + 7]);
                    const auto s0 = __builtin_amdgcn_permlane32_swap(a0, b0, false, false);
                    const auto s1 = __builtin_amdgcn_permlane32_swap(a1, b1, false, false);
                    const uint32_t t[4] = {s0[0], s1[0], s0[1], s1[1]};  // columns j*32 + 16*qp + 8*half .. + 7 of the row
                    const uint4 rv = rres[i % RD][j][qp];
                    const uint32_t ru[4] = {rv.x, rv.y, rv.z, rv.w};
                    float f[8];
#pragma unroll
                    for (int k = 0; k < 4; k++) {
                        f[2 * k] = bf16lo(t[k]) + bf16lo(ru[k]);
                        f[2 * k + 1] = bf16hi(t[k]) + bf16hi(ru[k]);
                    }
                    const bool in = FULL || (i * 32 < m_lim && j * 32 + 16 * qp < n_lim);
                    if (in) {
                        uint8_t* base = c_tile + ((int64_t)(i * 32) * G.N + j * 32 + 16 * qp) * 2;
                        *(uint4*)(base + c_lane_off) = make_uint4(pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]),
                                                                  pack_bf16x2(f[4], f[5]), pack_bf16x2(f[6], f[7]));
                    }
                    if constexpr (QUANT) {
                        float amax = 0.0f;
#pragma unroll
                        for (int e = 0; e < 8; e++) amax = fmaxf(amax, fabsf(f[e]));
                        const auto am = __builtin_amdgcn_permlane32_swap(f2u(amax), f2u(amax), false, false);
                        amax = fmaxf(u2f(am[0]), u2f(am[1]));
                        const float sg = group_scale<KIND>(amax);
                        const float rg = 1.0f / sg;
                        const uint32_t w0 = cvt4_fp8<KIND>(div_by_scale(f[0], sg, rg), div_by_scale(f[1], sg, rg),
                                                           div_by_scale(f[2], sg, rg), div_by_scale(f[3], sg, rg));
                        const uint32_t w1 = cvt4_fp8<KIND>(div_by_scale(f[4], sg, rg), div_by_scale(f[5], sg, rg),
                                                           div_by_scale(f[6], sg, rg), div_by_scale(f[7], sg, rg));
                        if (in) {  // N % 16 == 0: a group is inside or outside as a whole
                            uint8_t* base = cq_tile + ((int64_t)(i * 32) * G.N + j * 32 + 16 * qp);
                            *(uint2*)(base + q_lane_off) = make_uint2(w0, w1);
                            if (half == 0 && !(FULL || pack_scales)) {
                                uint8_t* sbase = s_tile + ((int64_t)(i * 32) * (G.N >> 4) + j * 2 + qp) * 2;
                                *(uint16_t*)(sbase + s_lane_off) = (uint16_t)f2bf16(sg);
                            }
                        }
                        spack[j] |= f2bf16(sg) << (16 * qp);
                    }
                }
            }
            if (QUANT && (FULL || pack_scales) && half == 0 && (FULL || i * 32 < m_lim)) {
                uint8_t* sbase = s_tile + (int64_t)(i * 32) * (G.N >> 4) * 2;
                *(uint2*)(sbase + s_lane_off) = make_uint2(spack[0], spack[1]);
            }
        }
        };
        // uniform over the wave: every row and column of its sub-tile exists, rows of the scale tensor can take 8-byte stores
        const bool full = m0 + wm * 128 + 128 <= G.M && n0 + wn * (TJ * 32) + TJ * 32 <= G.N && !biasp &&
                          (!QUANT || pack_scales);
        if (full) residual_epilogue(std::true_type{});
        else residual_epilogue(std::false_type{});
    } else if constexpr (EPI != kEpiBf16 && QBE > 16) {
        // Groups of 32 or 64 columns (reference linear.py:139-164 is generic in the group size): a row's 32 columns of
        // one accumulator tile sit in lanes l and l ^ 32, its 64 columns of the wave in the two tiles of those lanes, so
        // the group maximum is an in-lane maximum plus one lane swap.  Both tiles of a row are scaled before the first
        // code is formed (32 live values instead of 16; this path is off the shipped configurations, which use 16).
        constexpr int KIND = EPI == kEpiQuantE4M3 ? kE4M3 : kE5M2;
        const int sn = G.N / QBE;  // scales per row
        uint8_t* const sw_tile = (uint8_t*)Csp + ((int64_t)m0 * sn + (n0 + wn * (TJ * 32)) / QBE) * 2;
        const uint32_t sw_lane_off = (uint32_t)((wm * 128 + (lane & 31)) * sn) * 2;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            float v[TJ][16], am[TJ];
#pragma unroll
            for (int j = 0; j < TJ; j++) {
                const int nb = n0 + wn * (TJ * 32) + j * 32 + 4 * half;
                float a = 0.0f;
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    float t = acc[j][i][r] * scale;
                    if (biasp) {
                        const int n = nb + 8 * (r >> 2) + (r & 3);
                        if (n < G.N) t += load_rt_f32(biasp, n, G.bias_dt);
                    }
                    v[j][r] = t;
                    a = fmaxf(a, fabsf(t));
                }
                const auto sw2 = __builtin_amdgcn_permlane32_swap(f2u(a), f2u(a), false, false);
                am[j] = fmaxf(u2f(sw2[0]), u2f(sw2[1]));
            }
            if (QBE == 64) am[0] = am[1] = fmaxf(am[0], am[1]);
#pragma unroll
            for (int j = 0; j < TJ; j++) {
                const float s = group_scale<KIND>(am[j]);
                const float r = 1.0f / s;
                const bool inside = i * 32 < m_lim && j * 32 < q_n_lim;  // N % QBE == 0: a group is inside or outside as a whole
#pragma unroll
                for (int g2 = 0; g2 < 2; g2++) {
                    const uint32_t w0 = cvt4_fp8<KIND>(div_by_scale(v[j][8 * g2], s, r), div_by_scale(v[j][8 * g2 + 1], s, r),
                                                       div_by_scale(v[j][8 * g2 + 2], s, r), div_by_scale(v[j][8 * g2 + 3], s, r));
                    const uint32_t w1 = cvt4_fp8<KIND>(div_by_scale(v[j][8 * g2 + 4], s, r), div_by_scale(v[j][8 * g2 + 5], s, r),
                                                       div_by_scale(v[j][8 * g2 + 6], s, r), div_by_scale(v[j][8 * g2 + 7], s, r));
                    const auto sw = __builtin_amdgcn_permlane32_swap(w0, w1, false, false);
                    if (inside) {
                        uint8_t* base = q_tile + ((int64_t)(i * 32) * G.N + j * 32 + 16 * g2);
                        *(uint2*)(base + q_lane_off) = make_uint2(sw[0], sw[1]);
                    }
                }
                if (inside && half == 0 && (QBE == 32 || j == 0)) {
                    uint8_t* sbase = sw_tile + ((int64_t)(i * 32) * sn + (QBE == 32 ? j : 0)) * 2;
                    *(uint16_t*)(sbase + sw_lane_off) = (uint16_t)f2bf16(s);
                }
            }
        }
    } else {
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int m = m0 + wm * 128 + i * 32 + (lane & 31);
        uint32_t spack[TJ] = {};
#pragma unroll
        for (int j = 0; j < TJ; j++) {
            const int nb = n0 + wn * (TJ * 32) + j * 32 + 4 * half;  // + 8*q + {0..3}
            float v[16];
#pragma unroll
            for (int r = 0; r < 16; r++) v[r] = acc[j][i][r] * scale;
            if (biasp) {
#pragma unroll
                for (int q = 0; q < 4; q++)
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        const int n = nb + 8 * q + e;
                        if (n < G.N) v[4 * q + e] += load_rt_f32(biasp, n, G.bias_dt);
                    }
            }
            __builtin_amdgcn_sched_barrier(0);  // one accumulator tile at a time: keeps the epilogue's live ranges short
            if (EPI == kEpiBf16 && vec16) {
                // lanes l and l + 32 hold the two 8-byte halves of a 16-byte run of row m for each quad; swapping the
                // halves of two neighbouring quads between them (v_permlane32_swap) leaves every lane with one whole
                // 16-byte run: half as many store instructions, each covering 32 rows x 32 bytes
#pragma unroll
                for (int qp = 0; qp < 2; qp++) {
                    uint32_t a0 = pack_bf16x2(v[8 * qp], v[8 * qp + 1]), a1 = pack_bf16x2(v[8 * qp + 2], v[8 * qp + 3]);
                    uint32_t b0 = pack_bf16x2(v[8 * qp + 4], v[8 * qp + 5]), b1 = pack_bf16x2(v[8 * qp + 6], v[8 * qp + 7]);
                    const auto s0 = __builtin_amdgcn_permlane32_swap(a0, b0, false, false);
                    const auto s1 = __builtin_amdgcn_permlane32_swap(a1, b1, false, false);
                    // lanes < 32 now hold quad 2 qp whole (n = 16 qp .. + 7 of this 32-column tile), lanes >= 32 quad
                    // 2 qp + 1.  Address = uniform tile / sub-tile base (scalar) + one 32-bit per-lane offset.
                    uint8_t* base = c_tile + ((int64_t)(i * 32) * G.N + j * 32 + 16 * qp) * 2;
                    if (i * 32 < m_lim && j * 32 + 16 * qp < n_lim)  // N % 8 == 0: a 16-byte run is inside or outside as a whole
                        *(uint4*)(base + c_lane_off) = make_uint4(s0[0], s1[0], s0[1], s1[1]);
                }
            } else if (EPI == kEpiBf16) {
                if (m < G.M) {
#pragma unroll
                    for (int q = 0; q < 4; q++) {
                        const int n = nb + 8 * q;
                        if (n + 3 < G.N) {
                            *(uint2*)((uint16_t*)Cp + (int64_t)m * G.N + n) =
                                make_uint2(pack_bf16x2(v[4 * q], v[4 * q + 1]), pack_bf16x2(v[4 * q + 2], v[4 * q + 3]));
                        } else {
                            for (int e = 0; e < 4; e++)
                                if (n + e < G.N) ((uint16_t*)Cp)[(int64_t)m * G.N + n + e] = (uint16_t)f2bf16(v[4 * q + e]);
                        }
                    }
                }
            } else {
                constexpr int KIND = EPI == kEpiQuantE4M3 ? kE4M3 : kE5M2;
                // group g2 of 16 consecutive n = quads 2*g2, 2*g2+1 of this lane and of lane ^ 32; after the swap a
                // lane holds 8 consecutive codes (lanes < 32 the group's first half, lanes >= 32 its second half)
#pragma unroll
                for (int g2 = 0; g2 < 2; g2++) {
                    float amax = 0.0f;
#pragma unroll
                    for (int e = 0; e < 8; e++) amax = fmaxf(amax, fabsf(v[8 * g2 + e]));
                    // the other half of the group sits in lane ^ 32: a swap of the value with itself leaves [lo, lo] and
                    // [hi, hi] in the two results
                    const auto am = __builtin_amdgcn_permlane32_swap(f2u(amax), f2u(amax), false, false);
                    amax = fmaxf(u2f(am[0]), u2f(am[1]));
                    const float s = group_scale<KIND>(amax);
                    const float r = 1.0f / s;
                    const uint32_t w0 = cvt4_fp8<KIND>(div_by_scale(v[8 * g2], s, r), div_by_scale(v[8 * g2 + 1], s, r),
                                                       div_by_scale(v[8 * g2 + 2], s, r), div_by_scale(v[8 * g2 + 3], s, r));
                    const uint32_t w1 = cvt4_fp8<KIND>(div_by_scale(v[8 * g2 + 4], s, r), div_by_scale(v[8 * g2 + 5], s, r),
                                                       div_by_scale(v[8 * g2 + 6], s, r), div_by_scale(v[8 * g2 + 7], s, r));
                    const auto sw = __builtin_amdgcn_permlane32_swap(w0, w1, false, false);
                    if (i * 32 < m_lim && j * 32 + 16 * g2 < q_n_lim) {
                        uint8_t* base = q_tile + ((int64_t)(i * 32) * G.N + j * 32 + 16 * g2);
                        *(uint2*)(base + q_lane_off) = make_uint2(sw[0], sw[1]);
                        if (half == 0 && !pack_scales) {
                            uint8_t* sbase = s_tile + ((int64_t)(i * 32) * (G.N >> 4) + j * 2 + g2) * 2;
                            *(uint16_t*)(sbase + s_lane_off) = (uint16_t)f2bf16(s);
                        }
                    }
                    spack[j] |= f2bf16(s) << (16 * g2);
                }
            }
        }
        // the wave's four group scales of a row (64 columns) are 8 contiguous bytes: one store when they are all inside
        // the matrix and the row's scales start 8-byte aligned
        if (EPI != kEpiBf16 && pack_scales && half == 0 && i * 32 < m_lim) {
            uint8_t* sbase = s_tile + (int64_t)(i * 32) * (G.N >> 4) * 2;
            *(uint2*)(sbase + s_lane_off) = make_uint2(spack[0], spack[1]);
        }
    }
    }  // group size 16 / bf16 output
    }  // epilogue of tile it - 1
    if (it == my_ntiles) break;
#pragma unroll
    for (int j = 0; j < TJ; j++)
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[j][i][r] = 0.0f;
    // the rest of the tile's first memory phase: fragments of K-step 0 and this phase's loads
#pragma unroll
    for (int t = 0; t < 4; t++) fax[t] = load_fa(sl_frag, 0, t);
#pragma unroll
    for (int t = 0; t < TJ; t++) fbx[t] = load_fb(sl_frag, 0, t);
#pragma unroll
    for (int t = 0; t < 4; t++) fay[t] = load_fa(sl_frag, 1, t);
#pragma unroll
    for (int t = 0; t < TJ; t++) fby[t] = load_fb(sl_frag, 1, t);
    sl_frag = sl_frag + 2 >= NUNIT ? sl_frag + 2 - NUNIT : sl_frag + 2;
    issue_slab();
    COAT_WAIT_LGKM0();
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    compute_phase();
    for (int ks = 1; ks < nstep; ks++) {
        mem_phase();
        compute_phase();
    }
    }  // tiles
    if (!role) __builtin_amdgcn_s_barrier();  // role 0 started a phase early: its last barrier pairs with role 1's
    COAT_WAIT_VMCNT(0);  // drain the trailing zero-fill slabs before the block may exit
    if constexpr (PROBE) {
        if (tid == 0 && G.probe) {
            G.probe[2 * blockIdx.x] = __builtin_amdgcn_s_memtime() - probe_t0;
            G.probe[2 * blockIdx.x + 1] = __builtin_amdgcn_s_memrealtime() - probe_r0;
        }
    }
}


// One instance on the persistent grid (one block per CU; the block's LDS ring takes the whole CU's LDS).
template <int FA, int FB, int EP, bool V16, int QE, bool GR, bool PROBE = false>
static int gemm_launch_instance(const GemmArgs& G, int grid, hipStream_t st) {
    static coat_device_flags lds_ok;
    if (int e = coat_allow_lds(k_fp8_gemm<FA, FB, EP, V16, QE, GR, PROBE>, kLdsBytes, lds_ok)) return e;
    hipLaunchKernelGGL((k_fp8_gemm<FA, FB, EP, V16, QE, GR, PROBE>), dim3(grid), dim3(512), kLdsBytes, st, G);
    return coat_launch_status();
}
// Operand formats (coat_fp8 values) -> instance of epilogue EP.
template <int EP, bool V16, int QE, bool GR>
static int gemm_launch_formats(const GemmArgs& G, int fmt_a, int fmt_b, int grid, hipStream_t st) {
    if (fmt_a == COAT_E4M3 && fmt_b == COAT_E4M3) return gemm_launch_instance<0, 0, EP, V16, QE, GR>(G, grid, st);
    if (fmt_a == COAT_E5M2 && fmt_b == COAT_E4M3) return gemm_launch_instance<1, 0, EP, V16, QE, GR>(G, grid, st);
    if (fmt_a == COAT_E4M3 && fmt_b == COAT_E5M2) return gemm_launch_instance<0, 1, EP, V16, QE, GR>(G, grid, st);
    if (fmt_a == COAT_E5M2 && fmt_b == COAT_E5M2) return gemm_launch_instance<1, 1, EP, V16, QE, GR>(G, grid, st);
    return COAT_EINVAL;
}
// The instances are compiled in four translation units (gemm_bf16.hip, gemm_quant_e4m3.hip, gemm_quant_e5m2.hip,
// gemm_residual.hip), one per family of epilogues; gemm.hip validates the arguments and picks the family.
int gemm_dispatch_bf16(const GemmArgs& G, int fmt_a, int fmt_b, int grid, hipStream_t st);
int gemm_dispatch_quant_e4m3(const GemmArgs& G, int fmt_a, int fmt_b, int QB, int grid, hipStream_t st);
int gemm_dispatch_quant_e5m2(const GemmArgs& G, int fmt_a, int fmt_b, int QB, int grid, hipStream_t st);
int gemm_dispatch_residual(const GemmArgs& G, int fmt_a, int fmt_b, int out_kind, int grid, hipStream_t st);

}  // namespace coat
