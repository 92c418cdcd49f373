// Core of the MXFP8 NT GEMM kernels for gfx950: tile shape, LDS layout, the K-stage body on
// v_mfma_scale_f32_16x16x128_f8f6f4 and the persistent tile loop.  Dense, grouped and
// expert kernels plug a "problem" policy (tile iterator, operand addressing, epilogue)
// into persistent_gemm().
//
// Shape of the kernel
//   * workgroup tile BM x BN x 128, 64-lane waves arranged WGM x WGN, each wave owning a
//     (BM/WGM) x (BN/WGN) sub-tile as 16x16 MFMA accumulators;
//   * one workgroup per CU, persistent: it walks a strided list of tiles and issues the
//     first operand stage (and scales) of the next tile before the epilogue of the current
//     one, so HBM latency, the epilogue and workgroup dispatch never sit between two tiles;
//   * operand tiles travel HBM -> LDS with the direct global-to-LDS load (16 bytes per lane,
//     each lane supplying its own global address, which is what makes row gathers free),
//     double buffered, one workgroup barrier per 128-wide K stage;
//   * operand layout of the scaled 16x16x128 MFMA (measured on gfx950): lane (r = l%16,
//     g = l/16) holds row r; its first 16 bytes belong to MX block g>>1 and its last 16 bytes
//     to MX block 2 + (g>>1) of the 128-wide K step, and the scale of (row r, block b) is read
//     from lane r + 16 b.  So a lane loads K bytes [16g,16g+16) and [64+16g,64+16g+16) and
//     supplies the scale byte of block g;
//   * LDS rows are 128 bytes with the 16-byte chunks XOR-swizzled so that the 16 lanes of
//     an MFMA row group read 16 different bank quads;
//   * scales are fetched once per 512 of K (16 bytes per row), byte-transposed 4x4 and
//     parked in LDS so a lane reads ONE dword per sub-tile per 4 stages and the stage picks
//     its byte with the instruction's op_sel: no VALU work on scales in the main loop;
//   * the MFMA is issued "A rows x B rows": a lane owns 4 consecutive rows (m = 4 (lane / 16) + v)
//     at one N per sub-tile (n = lane % 16), and the B tile is gathered so that LDS row 16 j + r
//     of a wave's slice holds B row NT r + j, which makes the NT = 8 sub-tiles of a lane 8
//     consecutive N: one 16-byte store, and 16 neighbouring lanes write 256 contiguous bytes of
//     one output row.  The CU's store path coalesces neighbouring lanes only: measured 65-74
//     B/clk per CU for this layout against 20 B/clk for one that puts neighbouring lanes on
//     different rows;
//   * A is held in registers for the stage (MT fragments), B streams through two fragment
//     buffers, the read of sub-tile j+1 in flight under the MFMAs of sub-tile j.
#pragma once

#include <atomic>
#include <type_traits>
#include <utility>

#include "mx_common.h"

namespace mx {

typedef __attribute__((address_space(1))) const void gptr_t;
typedef __attribute__((address_space(3))) void lptr_t;

// Direct global-to-LDS copy of 16 bytes per lane.  `base` (wave-uniform, in scalar registers)
// plus the lane's 32-bit byte offset is the global address; the wave's 64 x 16 bytes land
// contiguously in LDS at byte address `lds` (wave-uniform, goes through M0).
// Written as inline asm on purpose: the kernel orders these copies against LDS reads itself,
// with explicit vmcnt waits and workgroup barriers, and lets chosen younger operations (the
// epilogue's stores) stay in flight across a barrier; the compiler's own accounting would
// insert a full vmcnt(0) before every LDS read that follows a copy it can see.
__device__ __forceinline__ void dma16(const uint8_t *base, uint32_t voff, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :
                 : "v"(voff), "s"(base), "s"(lds)
                 : "memory");
}

// Runs of copies behind ONE write of M0.  The instruction's immediate offset is added to the LDS address as well
// as to the global one, so the copies of a run land P0, P0 + 1, ... KB behind the run's LDS base when each lane's
// offset register holds its global offset minus the same immediate.  The immediate is 13 bits, signed, and the offset
// register is unsigned: copies are numbered inside groups of COPY_GROUP = 4 (immediates 0 .. 3 KB), the scalar base
// is pre-decremented by COPY_BIAS = 3 KB and copy q carries copy_bias(q) = 3 KB - (q % 4) KB in its offset register
// (the problem policies add it when they build a tile's offsets), so no offset register ever goes negative.
// What this saves is issue time: every write of M0 costs the wave the move, the wait state behind it and a scalar
// dependency in front of the copy, 64 times per stage and CU when every copy brings its own.
constexpr int COPY_GROUP = 4;
constexpr uint32_t COPY_BIAS = (COPY_GROUP - 1) * 1024;
__host__ __device__ constexpr uint32_t copy_bias(int q) { return COPY_BIAS - (uint32_t)(q % COPY_GROUP) * 1024; }

template <int P0>
__device__ __forceinline__ void dma16_run2(const uint8_t *biased_base, uint32_t v0, uint32_t v1, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\t"
                 "global_load_lds_dwordx4 %0, %2 offset:%4\n\t"
                 "global_load_lds_dwordx4 %1, %2 offset:%5"
                 :
                 : "v"(v0), "v"(v1), "s"(biased_base), "s"(lds), "n"(P0 * 1024), "n"((P0 + 1) * 1024)
                 : "memory");
}

// The same run with both halves of the execution mask set to `mask` around it (all ones, or zero: the copies are issued
// and move nothing).  A wave-uniform "whether", without a branch in the stage body.
template <int P0>
__device__ __forceinline__ void dma16_run2_masked(const uint8_t *biased_base, uint32_t v0, uint32_t v1, uint32_t lds, uint32_t mask) {
    uint64_t saved;
    asm volatile("s_mov_b64 %0, exec\n\t"
                 "s_mov_b32 exec_lo, %5\n\t"
                 "s_mov_b32 exec_hi, %5\n\t"
                 "s_mov_b32 m0, %4\n\ts_nop 0\n\t"
                 "global_load_lds_dwordx4 %1, %3 offset:%6\n\t"
                 "global_load_lds_dwordx4 %2, %3 offset:%7\n\t"
                 "s_mov_b64 exec, %0"
                 : "=&s"(saved)
                 : "v"(v0), "v"(v1), "s"(biased_base), "s"(lds), "s"(mask), "n"(P0 * 1024), "n"((P0 + 1) * 1024)
                 : "memory");
}

__device__ __forceinline__ void dma16_run4(const uint8_t *biased_base, uint32_t v0, uint32_t v1, uint32_t v2, uint32_t v3,
                                           uint32_t lds) {
    asm volatile("s_mov_b32 m0, %5\n\ts_nop 0\n\t"
                 "global_load_lds_dwordx4 %0, %4\n\t"
                 "global_load_lds_dwordx4 %1, %4 offset:1024\n\t"
                 "global_load_lds_dwordx4 %2, %4 offset:2048\n\t"
                 "global_load_lds_dwordx4 %3, %4 offset:3072"
                 :
                 : "v"(v0), "v"(v1), "v"(v2), "v"(v3), "s"(biased_base), "s"(lds)
                 : "memory");
}

__device__ __forceinline__ uint32_t lds_addr(const void *p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)p;
}

// A workgroup-wide event counter in LDS for the look-ahead of the A operand (see persistent_gemm): lane 0 of a wave adds
// one once the wave's A fragments of a stage are in registers; a wave about to overwrite that stage's A rows waits until
// all waves have.  Both are single asm statements -- no control flow the compiler can see, so the stage body stays one
// basic block -- and both wait on lgkmcnt(0) first: LDS operations return in order.
__device__ __forceinline__ void lds_count_up(uint32_t counter) {
    uint64_t saved;
    uint32_t one = 1;
    asm volatile("s_waitcnt lgkmcnt(0)\n\t"
                 "s_mov_b64 %0, exec\n\t"
                 "s_mov_b64 exec, 1\n\t"
                 "ds_add_u32 %1, %2\n\t"
                 "s_mov_b64 exec, %0"
                 : "=&s"(saved)
                 : "v"(counter), "v"(one)
                 : "memory");
}
__device__ __forceinline__ void lds_count_wait(uint32_t counter, uint32_t target) {
    uint32_t v, sv;
    asm volatile("lds_count_wait_%=:\n\t"
                 "ds_read_b32 %0, %2\n\t"
                 "s_waitcnt lgkmcnt(0)\n\t"
                 "v_readfirstlane_b32 %1, %0\n\t"
                 "s_cmp_lt_u32 %1, %3\n\t"
                 "s_cbranch_scc1 lds_count_wait_%="
                 : "=&v"(v), "=&s"(sv)
                 : "v"(counter), "s"(target)
                 : "memory", "scc");
}

__device__ __forceinline__ const uint8_t *uniform_ptr(const uint8_t *p) {
    uint64_t u = (uint64_t)p;
    uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)u);
    uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(u >> 32));
    return (const uint8_t *)(((uint64_t)hi << 32) | lo);
}

template <int BM_, int BN_, int WGM_, int WGN_>
struct GemmShape {
    static constexpr int BM = BM_, BN = BN_, WGM = WGM_, WGN = WGN_;
    static constexpr int BK = 128;
    static constexpr int NW = WGM * WGN;
    static constexpr int NTHR = NW * 64;
    static constexpr int WTM = BM / WGM, WTN = BN / WGN;
    static constexpr int MT = WTM / 16, NT = WTN / 16;
    static constexpr int QA = BM / 8 / NW, QB = BN / 8 / NW;  // DMA instructions per wave per stage
    static constexpr int DATA_A = BM * BK, DATA_B = BN * BK;  // bytes per stage
    // Scale planes [buffer][g][row] of dwords; the plane pitch is padded so the 64 lanes of
    // a wave (16 rows x 4 planes) read 64 different banks.
    static constexpr int PA = BM + 16, PB = BN + 16;
    static constexpr int SC_A = 4 * PA * 4, SC_B = 4 * PB * 4;  // bytes per super-step
    static constexpr int LDS_BYTES = 2 * (DATA_A + DATA_B + SC_A + SC_B);
    // + the staging area of SCALES_COPY (16 bytes per row of A and B) and the event counter of the A look-ahead
    static constexpr int LDS_BYTES_STAGED = LDS_BYTES + 16 * (BM + BN);  // SCALES_COPY without the look-ahead
    static constexpr int LDS_BYTES_AHEAD = LDS_BYTES_STAGED + 64;
    static constexpr bool TWO_ROWS = BM + BN > NTHR;
    static_assert(NT == 8 || NT == 4, "a lane's NT sub-tiles are NT consecutive N: one 16-byte (or 8-byte) store");
    static_assert(WTM % 16 == 0, "a wave's M extent must be a multiple of 16");
    static_assert((BM / 8) % NW == 0 && (BN / 8) % NW == 0, "DMA rows must divide over the waves");
    static_assert(BM + BN <= 2 * NTHR, "scale loader assumes at most two rows per thread");
};

// chunk swizzle: position of logical 16-byte chunk c of LDS row r (A or B tile) is c ^ swz_a(r)
__device__ __forceinline__ int swz_a(int r) { return (r >> 1) & 7; }

// 4x4 byte transpose: in d[s] = bytes {4s+0..4s+3}; out t[g] = bytes {g, 4+g, 8+g, 12+g}.
__device__ __forceinline__ void transpose4x4(const uint32_t (&d)[4], uint32_t (&t)[4]) {
    // v_perm_b32(a, b, sel): byte i of the result is byte sel[i] of the 8-byte {a:b} (b = bytes 0-3).
    uint32_t p01l = __builtin_amdgcn_perm(d[1], d[0], 0x05010400u);  // d0.b0 d1.b0 d0.b1 d1.b1
    uint32_t p01h = __builtin_amdgcn_perm(d[1], d[0], 0x07030602u);  // d0.b2 d1.b2 d0.b3 d1.b3
    uint32_t p23l = __builtin_amdgcn_perm(d[3], d[2], 0x05010400u);
    uint32_t p23h = __builtin_amdgcn_perm(d[3], d[2], 0x07030602u);
    t[0] = __builtin_amdgcn_perm(p23l, p01l, 0x05040100u);  // lo16(p01l) lo16(p23l)
    t[1] = __builtin_amdgcn_perm(p23l, p01l, 0x07060302u);  // hi16(p01l) hi16(p23l)
    t[2] = __builtin_amdgcn_perm(p23h, p01h, 0x05040100u);
    t[3] = __builtin_amdgcn_perm(p23h, p01h, 0x07060302u);
}

// Where the lane sits: which wave, and its (row-in-16, K-group) role in the MFMA operands.
struct Lane {
    int tid, lane, wave, wm, wn, r16, g;
};

template <typename S>
__device__ __forceinline__ Lane lane_of() {
    Lane L;
    L.tid = threadIdx.x;
    L.lane = L.tid & 63;
    L.wave = __builtin_amdgcn_readfirstlane(L.tid >> 6);
    L.wm = L.wave / S::WGN;
    L.wn = L.wave % S::WGN;
    L.r16 = L.lane & 15;
    L.g = L.lane >> 4;
    return L;
}

// B row (0..BN-1, relative to the tile) kept in LDS row `r` of the B tile.
template <typename S>
__device__ __forceinline__ int b_row_of_lds(int r) {
    const int in = r % S::WTN;
    return r - in + (in % 16) * S::NT + in / 16;
}

// Everything the copy engine needs for one tile: where A and B rows come from and where
// this thread's scale rows live.  `a_voff`/`b_voff` are byte offsets of this lane's 16-byte
// chunk of each DMA instruction relative to the (wave-uniform) bases, for K = 0.
template <typename S>
struct IssueCtx {
    static constexpr int NA = S::QA, NB = S::QB;  // copies of A rows / B rows this wave issues per stage
    const uint8_t *a_base, *b_base;
    int64_t a_ks = 128, b_ks = 128;  // bytes from one K stage of an operand to the next (128: row-major)
    // per copy q: byte offset of this lane's chunk from the base, plus copy_bias(q) (see dma16_run2)
    uint32_t a_voff[S::QA], b_voff[S::QB];
    const uint8_t *srow0, *srow1;  // scale rows tid and tid + NTHR of the [A rows; B rows] list
    // SCALES_COPY: the scale matrices and this lane's byte offset to the start of scale row tid of the list
    const uint8_t *sa_base, *sb_base;
    uint32_t s_voff;
    int kt0, kt1;                  // K range in 128-byte stages (absolute)
    // K % 128 != 0: stage tail_kt holds only tail_bytes of K.  Its copies re-read the stage's first
    // chunk in place of chunks past the end of the row (never past the matrix), and those
    // chunks' MX blocks carry scale byte 0, so they add nothing.  tail_kt = -1: no such stage.
    int tail_kt, tail_bytes;
};

// Byte offset correction of a copy's lane for stage `kt`: 0, or minus the lane's chunk offset when
// that chunk lies past the end of K.
template <typename C>
__device__ __forceinline__ uint32_t tail_fix_row(const C &c, const Lane &L, int kt, int row) {
    if (kt != c.tail_kt) return 0;
    const int chunk = (L.lane & 7) ^ ((row >> 1) & 7);
    return chunk * 16 >= c.tail_bytes ? (uint32_t)(chunk * 16) : 0u;
}

// LDS row (of the A tile, of the B tile) of this lane's 16-byte chunk of copy q.  A wave's copies of an operand land
// contiguously: wave w owns rows [w Q 8, (w + 1) Q 8) of the tile's LDS image, copy q the 8 rows from (w Q + q) 8, so a
// run of copies needs one LDS base.
template <typename S>
__device__ __forceinline__ int dma_row(const Lane &L, int q) {
    static_assert(S::QA == S::QB, "one row map for both operands");
    return (L.wave * S::QA + q) * 8 + (L.lane >> 3);
}

template <typename S>
__device__ __forceinline__ uint32_t tail_fix(const IssueCtx<S> &c, const Lane &L, int kt, int q) {
    return tail_fix_row(c, L, kt, dma_row<S>(L, q));
}

// Compile-time loop: f(std::integral_constant<int, 0>{}), ..., f(std::integral_constant<int, N - 1>{}).
template <typename F, int... I>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, I...>) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// Copies per write of M0 (2 or 4).
#ifndef MX_COPY_RUN
#define MX_COPY_RUN 2
#endif

// The stage's copies as runs: the runs of A first, then those of B.  `ga`/`gb` are the stage's bases minus COPY_BIAS,
// `wa`/`wb` the LDS addresses of this wave's rows of the two tile images.
template <typename S>
struct CopyRuns {
    static constexpr int RUN = MX_COPY_RUN;
    static_assert(S::QA % RUN == 0 && S::QB % RUN == 0 && COPY_GROUP % RUN == 0, "whole runs inside a group of four");
    static constexpr int RA = S::QA / RUN, RB = S::QB / RUN, N = RA + RB;
    template <int R, bool MASKED = false>
    static __device__ __forceinline__ void issue(const IssueCtx<S> &c, const Lane &L, int kt, const uint8_t *ga,
                                                 const uint8_t *gb, uint32_t wa, uint32_t wb, uint32_t mask = ~0u) {
        constexpr bool B = R >= RA;
        constexpr int q0 = (B ? R - RA : R) * RUN;
        const uint8_t *g = B ? gb : ga;
        const uint32_t lds = (B ? wb : wa) + (q0 / COPY_GROUP) * (COPY_GROUP * 1024);
        const uint32_t *voff = B ? c.b_voff : c.a_voff;
        static_assert(!MASKED || RUN == 2, "masked copies come in runs of two");
        if constexpr (MASKED)
            dma16_run2_masked<q0 % COPY_GROUP>(g, voff[q0] - tail_fix<S>(c, L, kt, q0), voff[q0 + 1] - tail_fix<S>(c, L, kt, q0 + 1), lds,
                                               mask);
        else if constexpr (RUN == 2)
            dma16_run2<q0 % COPY_GROUP>(g, voff[q0] - tail_fix<S>(c, L, kt, q0), voff[q0 + 1] - tail_fix<S>(c, L, kt, q0 + 1), lds);
        else
            dma16_run4(g, voff[q0] - tail_fix<S>(c, L, kt, q0), voff[q0 + 1] - tail_fix<S>(c, L, kt, q0 + 1),
                       voff[q0 + 2] - tail_fix<S>(c, L, kt, q0 + 2), voff[q0 + 3] - tail_fix<S>(c, L, kt, q0 + 3), lds);
    }
};

// A copy of the lane descriptor the optimiser cannot see through: address arithmetic done on
// it inside the per-tile setup is recomputed once per tile instead of being hoisted out of
// the tile loop and kept in (spilled) registers across the K loop.
__device__ __forceinline__ Lane opaque(const Lane &L) {
    Lane R = L;
    asm volatile("" : "+v"(R.tid), "+v"(R.lane));
    return R;
}

// The whole descriptor rebuilt from such a copy: for an epilogue whose per-lane addresses would otherwise be invariants of
// the tile loop, computed once in front of it and spilled across the K loop.  (A spill in front of the loop costs more
// than its two instructions: every write inside the loop to a register the pending scratch store reads gets a full
// vector-memory wait in front of it, which also waits for the stage's copies.)  Only for policies that run under
// lane_of's wave -> sub-tile mapping: a schedule that deals the waves differently hands its epilogue its own descriptor.
template <typename S>
__device__ __forceinline__ Lane rebuilt(const Lane &L) {
    Lane R = opaque(L);
    R.wave = __builtin_amdgcn_readfirstlane(R.tid >> 6);
    R.wm = R.wave / S::WGN;
    R.wn = R.wave % S::WGN;
    R.r16 = R.lane & 15;
    R.g = R.lane >> 4;
    return R;
}

template <typename S>
__device__ __forceinline__ void issue_stage(const IssueCtx<S> &c, const Lane &L, int kt, uint8_t *ldsA, uint8_t *ldsB,
                                            int buf) {
    // The stage's base address is forced into SGPRs so each load is "scalar base + 32-bit
    // lane offset" and costs no 64-bit vector address arithmetic.
    const uint8_t *ga = uniform_ptr(c.a_base + (int64_t)kt * c.a_ks - COPY_BIAS);
    const uint8_t *gb = uniform_ptr(c.b_base + (int64_t)kt * c.b_ks - COPY_BIAS);
    const uint32_t la = __builtin_amdgcn_readfirstlane(lds_addr(ldsA) + buf * S::DATA_A + L.wave * S::QA * 1024);
    const uint32_t lb = __builtin_amdgcn_readfirstlane(lds_addr(ldsB) + buf * S::DATA_B + L.wave * S::QB * 1024);
    static_for<CopyRuns<S>::N>([&](auto r) { CopyRuns<S>::template issue<r.value>(c, L, kt, ga, gb, la, lb); });
}

// The A rows of stage `kt` alone (the look-ahead's second stage in a kernel's prologue).
template <typename S>
__device__ __forceinline__ void issue_a(const IssueCtx<S> &c, const Lane &L, int kt, uint8_t *ldsA, int buf) {
    const uint8_t *ga = uniform_ptr(c.a_base + (int64_t)kt * c.a_ks - COPY_BIAS);
    const uint32_t la = __builtin_amdgcn_readfirstlane(lds_addr(ldsA) + buf * S::DATA_A + L.wave * S::QA * 1024);
    static_for<CopyRuns<S>::RA>([&](auto r) { CopyRuns<S>::template issue<r.value>(c, L, kt, ga, ga, la, la); });
}

// How a row's scale bytes are fetched: one 16-byte load per 512 of K (K % 512 == 0, 16-byte
// aligned rows), one dword per stage (K % 128 == 0, 4-byte aligned rows), or byte by byte (any
// K % 32 == 0 and any pitch; blocks past the end of K read as scale byte 0).  SCALES_QUAD: one
// 16-byte load per 4 stages from a 4-byte aligned address, for K ranges that start on any stage
// (the token ranges of experts); it reads up to 12 bytes past the last stage's bytes, which the
// caller guarantees to lie inside the row's pitch.  Against SCALES_DWORD it asks the L2 for a
// row's line once per four stages instead of once per stage: 512 rows x 4 bytes a stage is half
// as many lines again as the stage's codes.
// SCALES_COPY: the rows' 16 scale bytes per 512 of K go from memory to LDS through the copy engine, like the codes (one
// copy per wave and four stages, into a staging area of 16 bytes per row), and the thread that would have loaded a row
// takes it from there when it transposes it into the planes.  No registers hold scale bytes in flight, and -- what it
// is for -- the K loop holds no vector load the compiler can see: in front of such a load's use it puts a full
// vector-memory wait, which under the A look-ahead waits for copies that are meant to stay in flight.  A row is staged
// and transposed by the same wave, so the wave's own vector-memory waits order the two.  Needs what SCALES_VEC16 needs
// and scale matrices under 4 GB; a policy fills IssueCtx::s_voff / sa_base / sb_base for it.
enum { SCALES_VEC16 = 0, SCALES_DWORD = 1, SCALES_BYTES = 2, SCALES_QUAD = 3, SCALES_COPY = 4 };

// 16 scale bytes (4 stages x 4 blocks) of one row starting at scale column kb0.
template <int MODE>
__device__ __forceinline__ void load_scales(const uint8_t *row, int kb0, int kb_end, uint32_t (&d)[4]) {
    const uint8_t *p = row + kb0;
    if (MODE == SCALES_VEC16) {
        v4i t = *(const v4i *)p;
        d[0] = t[0], d[1] = t[1], d[2] = t[2], d[3] = t[3];
    } else if (MODE == SCALES_QUAD) {
        typedef int v4i_a4 __attribute__((ext_vector_type(4), aligned(4)));
        v4i_a4 t = *(const v4i_a4 *)p;
        d[0] = t[0], d[1] = t[1], d[2] = t[2], d[3] = t[3];
    } else if (MODE == SCALES_DWORD) {
#pragma unroll
        for (int s = 0; s < 4; s++) d[s] = kb0 + 4 * s < kb_end ? *(const uint32_t *)(p + 4 * s) : 0u;
    } else {
#pragma unroll
        for (int s = 0; s < 4; s++) {
            uint32_t w = 0;
#pragma unroll
            for (int b = 0; b < 4; b++)
                if (kb0 + 4 * s + b < kb_end) w |= (uint32_t)p[4 * s + b] << (8 * b);
            d[s] = w;
        }
    }
}

template <typename S>
__device__ __forceinline__ void park_scales(int srow, uint32_t *ldsSA, uint32_t *ldsSB, int sbuf,
                                            const uint32_t (&d)[4]) {
    uint32_t t[4];
    transpose4x4(d, t);
    if (srow < S::BM) {
        uint32_t *dst = ldsSA + sbuf * 4 * S::PA + srow;
#pragma unroll
        for (int gg = 0; gg < 4; gg++) dst[gg * S::PA] = t[gg];
    } else {
        uint32_t *dst = ldsSB + sbuf * 4 * S::PB + (srow - S::BM);
#pragma unroll
        for (int gg = 0; gg < 4; gg++) dst[gg * S::PB] = t[gg];
    }
}

// SCALES_COPY: the 16 scale bytes from scale column kb0 of this workgroup's BM + BN rows into scale buffer `sbuf`
// (row r of the list at byte 16 r): one copy per wave, waves 0 .. BM / 64 - 1 the A rows.
template <typename S>
__device__ __forceinline__ void issue_scales(const IssueCtx<S> &c, const Lane &L, int kb0, uint8_t *raw) {
    static_assert(S::BM % 64 == 0 && S::BM + S::BN == S::NTHR, "one row of the list per thread, whole waves of A rows");
    const uint8_t *base = uniform_ptr((L.wave < S::BM / 64 ? c.sa_base : c.sb_base) + kb0);
    const uint32_t lds = __builtin_amdgcn_readfirstlane(lds_addr(raw) + L.wave * 1024);
    dma16(base, c.s_voff, lds);
}
// ... and from the staging area into scale buffer `sbuf` of the planes (the thread's own row; the copy has landed).
template <typename S>
__device__ __forceinline__ void park_staged(const Lane &L, const uint8_t *raw, uint32_t *ldsSA, uint32_t *ldsSB, int sbuf) {
    asm volatile("" ::: "memory");  // behind the vector-memory wait that covers the copy
    const v4i t = *(const v4i *)(raw + L.tid * 16);
    const uint32_t d[4] = {(uint32_t)t[0], (uint32_t)t[1], (uint32_t)t[2], (uint32_t)t[3]};
    park_scales<S>(L.tid, ldsSA, ldsSB, sbuf, d);
}

// One K stage of the workgroup tile: this wave's MT x NT accumulators advance by 128 of K,
// and, woven between the MFMAs, the wave issues its share of the direct-to-LDS copies that
// fetch stage `kt_next` (of the tile described by `c`) into LDS buffer `buf_next`.
//
// The copies are spread over the first half of the stage on purpose.  The texture path takes
// 64 bytes per clock, so the 64 KB a stage needs occupy it for ~1000 clocks per CU; issued in
// one burst at the top of the stage they stall every wave (and the MFMA pipe) for that long,
// issued late they would not land before the stage-ending barrier.
//
// AHEAD (the A look-ahead, see persistent_gemm): the stage fetches the B rows of stage `kt_next` into buffer `buf_next`
// in its first steps and, in steps 4 and 5, the A rows of stage `kt_a` of the tile `ca` describes -- the stage after
// `kt_next` in the workgroup's sequence of stages -- into the A half of the buffer it is itself reading, once every wave
// has its A fragments of this stage in registers (`counter` has reached `target`).  MASKED_A: `a_exec` is the execution
// mask of those A copies, zero when the stage two on is not known yet (persistent_gemm, tiles of one stage).
template <typename S, int OPSEL, bool AHEAD = false, bool MASKED_A = false>
__device__ __forceinline__ void compute_stage(const uint8_t *__restrict__ la, const uint8_t *__restrict__ lb, int a_lo,
                                              int a_hi, int b_lo, int b_hi, const int (&sa)[S::MT],
                                              const int (&sb)[S::NT], v4f (&acc)[S::MT][S::NT],
                                              const IssueCtx<S> &c, const Lane &L, int kt_next, uint8_t *ldsA,
                                              uint8_t *ldsB, int buf_next, const IssueCtx<S> &ca, int kt_a,
                                              uint32_t counter, uint32_t target, uint32_t a_exec = ~0u) {
    const uint8_t *ga = uniform_ptr((AHEAD ? ca.a_base + (int64_t)kt_a * ca.a_ks : c.a_base + (int64_t)kt_next * c.a_ks) - COPY_BIAS);
    const uint8_t *gb = uniform_ptr(c.b_base + (int64_t)kt_next * c.b_ks - COPY_BIAS);
    const uint32_t wa =
        __builtin_amdgcn_readfirstlane(lds_addr(ldsA) + (AHEAD ? buf_next ^ 1 : buf_next) * S::DATA_A + L.wave * S::QA * 1024);
    const uint32_t wb = __builtin_amdgcn_readfirstlane(lds_addr(ldsB) + buf_next * S::DATA_B + L.wave * S::QB * 1024);
    typedef CopyRuns<S> Runs;

    // A is held (MT fragments), B streams through two fragment buffers.  Nothing crosses into or
    // out of the stage body, nor from one step of it into the next (sched_barrier).  LDS reads
    // return in order, so the first MFMA's operands (B[0], A[0]) are asked for first.
    constexpr int STEPS = S::NT / 2 > 0 ? S::NT / 2 : 1;  // the copies go out during the first half of the stage
    static_assert(STEPS % Runs::N == 0 || Runs::N % STEPS == 0, "runs spread evenly over the steps");
    __builtin_amdgcn_sched_barrier(0);
    v8i bfr[2];
    {
        v4i lo = *(const v4i *)(lb + b_lo);
        v4i hi = *(const v4i *)(lb + b_hi);
        bfr[0] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
    v8i afr[S::MT];
#pragma unroll
    for (int i = 0; i < S::MT; i++) {
        v4i lo = *(const v4i *)(la + a_lo + i * (16 * 128));
        v4i hi = *(const v4i *)(la + a_hi + i * (16 * 128));
        afr[i] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
    if (AHEAD) lds_count_up(counter);  // this wave's A fragments are in registers
    __builtin_amdgcn_sched_barrier(0);
    constexpr int A_STEP = S::NT / 2;  // AHEAD: the A runs go out in steps A_STEP, A_STEP + 1, ..., the B runs in steps 0, 1, ...
    static_assert(!AHEAD || (Runs::RA <= S::NT - A_STEP && Runs::RB <= A_STEP), "the runs of a stage fit its two halves");
    static_for<S::NT>([&](auto jc) {
        constexpr int j = jc.value;
        if constexpr (AHEAD && j == A_STEP) lds_count_wait(counter, target);
        if (j + 1 < S::NT) {
            v4i lo = *(const v4i *)(lb + b_lo + (j + 1) * (16 * 128));
            v4i hi = *(const v4i *)(lb + b_hi + (j + 1) * (16 * 128));
            bfr[(j + 1) & 1] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
        // run r goes out in step r STEPS / N: evenly over the first half of the stage
        static_for<Runs::N>([&](auto r) {
            if constexpr (AHEAD) {
                constexpr bool isb = r.value >= Runs::RA;
                if constexpr (isb && r.value - Runs::RA == j) Runs::template issue<r.value>(c, L, kt_next, ga, gb, wa, wb);
                if constexpr (!isb && A_STEP + r.value == j) Runs::template issue<r.value, MASKED_A>(ca, L, kt_a, ga, gb, wa, wb, a_exec);
            } else if constexpr (r.value * STEPS / Runs::N == j && j < STEPS) {
                Runs::template issue<r.value>(c, L, kt_next, ga, gb, wa, wb);
            }
        });
#pragma unroll
        for (int i = 0; i < S::MT; i++)
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(afr[i], bfr[j & 1], acc[i][j], 0, 0, OPSEL, sa[i],
                                                                         OPSEL, sb[j]);
        __builtin_amdgcn_sched_barrier(0);
    });
    // The MFMAs have no side effects the compiler can see, so it would sink them past the
    // barrier that ends the stage; an empty volatile asm reading and writing every accumulator
    // pins them here.
#pragma unroll
    for (int i = 0; i < S::MT; i++)
#pragma unroll
        for (int j = 0; j < S::NT; j++) asm volatile("" : "+v"(acc[i][j]));
}

// s_waitcnt with lgkmcnt(0), no expcnt wait, and at most N vector-memory operations left in
// flight.  Vector-memory operations retire in issue order, so this waits for everything except
// the youngest N.
// simm16: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] << 14
template <int N>
__device__ __forceinline__ void wait_vm_allow_c() {
    static_assert(N >= 0 && N <= 63, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt(((N & 15) | (7 << 4) | ((N >> 4) << 14)));
}

// The two halves (A part, B part: DATA_A and DATA_B bytes) of the LDS stage buffer the tile's
// last K stage was read from.  An epilogue may use them as scratch once every wave has left
// the main loop (a workgroup barrier of its own first); the buffer is not written again before
// the barrier that follows the epilogue.
// `c`: the scale planes of the tile's last super-step (4 * PA words), free under the same rule.
struct LdsScratch {
    uint8_t *a, *b, *c;
};

// The persistent tile loop.  `P` (the problem policy) provides
//   bool P::next(Tile &t)                   advance to this workgroup's next tile (false = done);
//                                           tiles with an empty K range are finished inside next()
//   void P::context(const Tile &, const Lane &, IssueCtx<S> &)
//   int  P::epilogue(const Tile &, const Lane &, v4f (&acc)[MT][NT], const LdsScratch &)   returns how many stores each
//                                           lane issued if that number is the same compile-time
//                                           constant P::NST for the whole wave, else -1
//   int  P::kb_end                          scale bytes per row (bound for predicated fetches)
//   bool P::EARLY_WAIT                      wait for the next tile's first stage before the epilogue (see the tile loop)
//
// AHEAD, the A look-ahead.  A stage's copies are all waited for at the end of the stage that issues them, because the
// stage after it reads them; the wait is for the slowest of 64 copies per CU, and a vector-memory wait is for everything
// older, so nothing may be left in flight across the barrier.  The A rows of a stage, however, are dead a few hundred
// clocks into it (every wave reads its A fragments first and holds them), while its B rows are read to the end.  With
// AHEAD the workgroup therefore fetches A TWO stages ahead -- stage g, in its second half, fetches the A rows of stage
// g + 2 into the A half of its own buffer, once an event counter in LDS says that all eight waves have their A fragments
// -- and B one stage ahead as before.  The stage-ending wait then leaves the wave's youngest S::QA copies, those A rows,
// in flight: they have another whole stage to land.  Stages are numbered through the workgroup's whole sequence of
// tiles, so the last two stages of a tile fetch the A rows of the next tile's first two; every tile must therefore have
// at least two stages (the caller's guarantee, or the policy declares SHORT_TILES, below), and the epilogue may not use
// the stage buffer as scratch (no EARLY_WAIT policy does both).  Same products bit for bit: the MFMA sequence does not change.  Measured inside the feed-forward
// step: the batched launch of the three long contractions 457 -> 429 us, the K = 1536 products 1 % faster.
//
// Under AHEAD a tile's context is built twice, for the A rows one stage before it is built for everything else.  A policy
// whose context() reads memory (gathered rows) declares `static constexpr bool REUSE_CONTEXT = true` and the second
// one is a copy of the first.
template <typename P, typename = void>
struct reuse_context_of : std::false_type {};
template <typename P>
struct reuse_context_of<P, std::void_t<decltype(P::REUSE_CONTEXT)>> : std::integral_constant<bool, P::REUSE_CONTEXT> {};

//
// Tiles of a single stage under AHEAD (a policy with `static constexpr bool SHORT_TILES = true`; the others keep the
// two-stage guarantee).  The stage two on then lies in the tile after the next, which is not known yet: the stage
// issues no A copies (masked out) and closes with a full wait, and the stage after it fetches its successor's A rows
// together with the B rows, one stage ahead, before it goes on looking two ahead.
template <typename P, typename = void>
struct short_tiles_of : std::false_type {};
template <typename P>
struct short_tiles_of<P, std::void_t<decltype(P::SHORT_TILES)>> : std::integral_constant<bool, P::SHORT_TILES> {};

template <typename S, int K512, typename P, bool AHEAD = false>  // K512: one of SCALES_*
__device__ __forceinline__ void persistent_gemm(P &prob, uint8_t *smem) {
    constexpr bool SHORT = AHEAD && short_tiles_of<P>::value;
    bool pend = false;  // SHORT: the A rows of the next stage are not in flight yet; this stage fetches them first
    static_assert(!(AHEAD && P::EARLY_WAIT), "an epilogue that borrows the stage buffer cannot share it with the look-ahead");
    uint8_t *const ldsA = smem;                                                  // [2][BM*128]
    uint8_t *const ldsB = smem + 2 * S::DATA_A;                                  // [2][BN*128]
    uint32_t *const ldsSA = (uint32_t *)(smem + 2 * (S::DATA_A + S::DATA_B));    // [2][4][PA]
    uint32_t *const ldsSB = ldsSA + 2 * 4 * S::PA;                               // [2][4][PB]

    constexpr bool COPY = K512 == SCALES_COPY;
    uint8_t *const rawS = smem + S::LDS_BYTES;  // SCALES_COPY: the staging area, [BM + BN rows][16 bytes]

    const Lane L = lane_of<S>();
    const bool has_row0 = L.tid < S::BM + S::BN;
    const int kb_end = prob.kb_end;

    // per-lane LDS read offsets: low half = 16-byte chunk g, high half = chunk g + 4 (= offset ^ 64)
    const int a_row = L.wm * S::WTM + L.r16;
    const int b_row = L.wn * S::WTN + L.r16;
    const int a_rd = a_row * 128 + ((L.g ^ swz_a(a_row)) << 4);
    const int b_rd = b_row * 128 + ((L.g ^ swz_a(b_row)) << 4);

    // AHEAD only: waves whose A fragments are in registers, over all stages
    const uint32_t counter = lds_addr(smem + S::LDS_BYTES + 16 * (S::BM + S::BN));
    typename P::Tile cur, nxt;
    if (!prob.next(cur)) return;
    bool has_next = prob.next(nxt);
    IssueCtx<S> ctx;   // the tile whose B rows and scale bytes are being fetched
    IssueCtx<S> ctxa;  // AHEAD: the tile whose A rows are being fetched (the next tile's, from a tile's second-to-last stage on)
    prob.context(cur, L, ctx);
    if (AHEAD) ctxa = ctx;

    int gstage = 0;  // stages issued so far, over all tiles: LDS data buffer = gstage & 1
    int gsuper = 0;  // super-steps so far: LDS scale buffer = gsuper & 1

    // prologue of the first tile
    {
        uint32_t d0[4], d1[4];
        if constexpr (COPY) {
            issue_scales<S>(ctx, L, ctx.kt0 * 4, rawS);
        } else {
            if (has_row0) load_scales<K512>(ctx.srow0, ctx.kt0 * 4, kb_end, d0);
            if (S::TWO_ROWS) load_scales<K512>(ctx.srow1, ctx.kt0 * 4, kb_end, d1);
        }
        issue_stage<S>(ctx, L, ctx.kt0, ldsA, ldsB, 0);
        if (AHEAD) {
            if (!SHORT || ctx.kt1 - ctx.kt0 >= 2) issue_a<S>(ctx, L, ctx.kt0 + 1, ldsA, 1);
            else pend = true;
            if (L.tid == 0) *(volatile uint32_t *)(smem + S::LDS_BYTES + 16 * (S::BM + S::BN)) = 0;
        }
        if constexpr (!COPY) {
            if (has_row0) park_scales<S>(L.tid, ldsSA, ldsSB, 0, d0);
            if (S::TWO_ROWS) park_scales<S>(L.tid + S::NTHR, ldsSA, ldsSB, 0, d1);
        }
    }
    wait_vm_allow_c<0>();
    if constexpr (COPY) park_staged<S>(L, rawS, ldsSA, ldsSB, 0);
    __syncthreads();

    v4f acc[S::MT][S::NT];
    while (true) {
#pragma unroll
        for (int i = 0; i < S::MT; i++)
#pragma unroll
            for (int j = 0; j < S::NT; j++) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

        const int kt0 = ctx.kt0, KT = ctx.kt1 - ctx.kt0;
        const int nsuper = (KT + 3) >> 2;
        uint32_t d0[4], d1[4];  // scale bytes in flight: next super-step's, or the next tile's first
        for (int ss = 0; ss < nsuper; ss++) {
            const int sbuf = gsuper & 1;
            int sa[S::MT], sb[S::NT];
#pragma unroll
            for (int i = 0; i < S::MT; i++) sa[i] = (int)ldsSA[(sbuf * 4 + L.g) * S::PA + a_row + 16 * i];
#pragma unroll
            for (int j = 0; j < S::NT; j++)
                sb[j] = (int)ldsSB[(sbuf * 4 + L.g) * S::PB + b_row + 16 * j];

            // One K stage.  In every stage but the tile's last, the next stage's operands are
            // put in flight during the stage and waited for at its end.
            // In the last stage nothing of this tile is left to fetch, so the copy context is
            // switched to the next tile and ITS first stage and scales go in flight; the wait
            // and barrier that publish them come after the epilogue.
#define MX_STAGE(SIDX)                                                                                        \
    {                                                                                                         \
        const int k = ss * 4 + SIDX;                                                                          \
        if (k < KT) {                                                                                         \
            const int buf = gstage & 1;                                                                       \
            const bool last = k + 1 == KT;                                                                    \
            int kt_issue = kt0 + k + 1;                                                                       \
            if (!last) {                                                                                      \
                if (SIDX == 3) {                                                                              \
                    if constexpr (COPY) {                                                                     \
                        park_staged<S>(L, rawS, ldsSA, ldsSB, sbuf ^ 1);                                      \
                    } else {                                                                                  \
                        if (has_row0) park_scales<S>(L.tid, ldsSA, ldsSB, sbuf ^ 1, d0);                      \
                        if (S::TWO_ROWS) park_scales<S>(L.tid + S::NTHR, ldsSA, ldsSB, sbuf ^ 1, d1);         \
                    }                                                                                         \
                }                                                                                             \
                if (SIDX == 0 && ss + 1 < nsuper) {                                                           \
                    if constexpr (COPY) {                                                                     \
                        issue_scales<S>(ctx, L, (kt0 + (ss + 1) * 4) * 4, rawS);                              \
                    } else {                                                                                  \
                        if (has_row0) load_scales<K512>(ctx.srow0, (kt0 + (ss + 1) * 4) * 4, kb_end, d0);     \
                        if (S::TWO_ROWS) load_scales<K512>(ctx.srow1, (kt0 + (ss + 1) * 4) * 4, kb_end, d1);  \
                    }                                                                                         \
                }                                                                                             \
            } else if (has_next) {                                                                            \
                if (AHEAD && reuse_context_of<P>::value) ctx = ctxa; /* the next tile's, one stage old */     \
                else prob.context(nxt, L, ctx);                                                               \
                if constexpr (COPY) {                                                                         \
                    issue_scales<S>(ctx, L, ctx.kt0 * 4, rawS);                                               \
                } else {                                                                                      \
                    if (has_row0) load_scales<K512>(ctx.srow0, ctx.kt0 * 4, kb_end, d0);                      \
                    if (S::TWO_ROWS) load_scales<K512>(ctx.srow1, ctx.kt0 * 4, kb_end, d1);                   \
                }                                                                                             \
                kt_issue = ctx.kt0;                                                                           \
            } else {                                                                                          \
                kt_issue = kt0 + k; /* nothing left to fetch: a harmless re-read of this stage */             \
            }                                                                                                 \
            /* AHEAD: the A rows two stages on: this tile's, or the next tile's first two (its context  */    \
            /* from the second-to-last stage on), or, with no tile left, a re-read nobody will look at. */    \
            int kt_a = kt0 + k + 2;                                                                           \
            bool known = true; /* SHORT: whether the stage two on is in this tile or the next */              \
            if (AHEAD && k + 2 >= KT) {                                                                       \
                if (has_next) {                                                                               \
                    if (SHORT ? k == (KT >= 2 ? KT - 2 : 0) : k + 2 == KT) prob.context(nxt, L, ctxa);        \
                    kt_a = ctxa.kt0 + (k + 2 - KT);                                                           \
                    if (SHORT) known = k + 2 - KT < ctxa.kt1 - ctxa.kt0;                                      \
                } else {                                                                                      \
                    kt_a = kt0 + k;                                                                           \
                }                                                                                             \
            }                                                                                                 \
            if constexpr (SHORT) {                                                                            \
                /* the next stage's A rows, which no earlier stage could fetch: with its B rows, up front */  \
                if (pend) issue_a<S>(ctx, L, kt_issue, ldsA, buf ^ 1);                                        \
                pend = !known;                                                                                \
            }                                                                                                 \
            compute_stage<S, SIDX, AHEAD, SHORT>(                                                             \
                ldsA + buf * S::DATA_A, ldsB + buf * S::DATA_B, a_rd, a_rd ^ 64, b_rd, b_rd ^ 64, sa, sb,     \
                acc, ctx, L, kt_issue, ldsA, ldsB, buf ^ 1, ctxa, kt_a, counter,                              \
                (uint32_t)(gstage + 1) * S::NW, __builtin_amdgcn_readfirstlane(known ? ~0u : 0u));            \
            if (!last) {                                                                                      \
                if (SHORT && !known) wait_vm_allow_c<0>();                                                    \
                else wait_vm_allow_c<AHEAD ? S::QA : 0>();                                                    \
                __syncthreads();                                                                              \
            }                                                                                                 \
            gstage++;                                                                                         \
        }                                                                                                     \
    }
            MX_STAGE(0)
            MX_STAGE(1)
            MX_STAGE(2)
            MX_STAGE(3)
#undef MX_STAGE
            gsuper++;
        }
        // The next tile's first stage and scales are already in flight: the epilogue's
        // conversions run under that latency, and when every lane issued the same known number
        // of stores the wait lets exactly those stay in flight,
        // so the stores drain under the next tile's first stage.
        const int lastbuf = (gstage - 1) & 1;
        // P::EARLY_WAIT (epilogues whose lanes issue differing numbers of stores, so that no count of
        // them can be left in flight behind the next tile's copies): the wait for those copies and for
        // the next tile's scale bytes comes BEFORE the epilogue, where only they are outstanding, the
        // scales are parked then (their planes were last read two super-steps ago, with a barrier
        // since), and the barrier behind the epilogue publishes both.  The epilogue's own stores then
        // need no wait at all and drain under the next tile's K loop instead of in front of it.
        static_assert(!(COPY && P::EARLY_WAIT), "the fused epilogues borrow a scale plane and keep the planes");
        if (P::EARLY_WAIT && has_next) {
            wait_vm_allow_c<0>();
            if (has_row0) park_scales<S>(L.tid, ldsSA, ldsSB, gsuper & 1, d0);
            if (S::TWO_ROWS) park_scales<S>(L.tid + S::NTHR, ldsSA, ldsSB, gsuper & 1, d1);
        }
        const int stores = prob.epilogue(cur, L, acc, LdsScratch{ldsA + lastbuf * S::DATA_A, ldsB + lastbuf * S::DATA_B,
                                            (uint8_t *)(ldsSA + ((gsuper - 1) & 1) * 4 * S::PA)});
        if (!P::EARLY_WAIT && has_next && !COPY) {
            if (has_row0) park_scales<S>(L.tid, ldsSA, ldsSB, gsuper & 1, d0);
            if (S::TWO_ROWS) park_scales<S>(L.tid + S::NTHR, ldsSA, ldsSB, gsuper & 1, d1);
        }
        if (!has_next) break;
        if (!P::EARLY_WAIT) {
            if (stores == P::NST) wait_vm_allow_c<P::NST>();
            else wait_vm_allow_c<0>();
        }
        if constexpr (COPY) park_staged<S>(L, rawS, ldsSA, ldsSB, gsuper & 1);  // the next tile's first scale bytes: staged in the last stage
        __syncthreads();
        cur = nxt;
        has_next = prob.next(nxt);
    }
}

// Converts 8 consecutive-N accumulator values of one output row and stores them (one 16-byte
// store for 16-bit outputs when `vec`).
template <int CDT>
__device__ __forceinline__ void store8(void *c, int64_t off, const v4f &lo, const v4f &hi, int nvalid, bool vec) {
    const float v[8] = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    if (CDT == MX_FP32) {
        float *p = (float *)c + off;
        if (vec && nvalid >= 8) {
            ((v4f *)p)[0] = lo;
            ((v4f *)p)[1] = hi;
        } else {
            for (int i = 0; i < 8 && i < nvalid; i++) p[i] = v[i];
        }
    } else {
        uint32_t w[4];
        if (CDT == MX_BF16) {
#pragma unroll
            for (int i = 0; i < 4; i++) w[i] = pack2_bf16(v[2 * i], v[2 * i + 1]);
        } else {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                typedef _Float16 h2 __attribute__((ext_vector_type(2)));
                h2 h = {(_Float16)v[2 * i], (_Float16)v[2 * i + 1]};
                w[i] = __builtin_bit_cast(uint32_t, h);
            }
        }
        uint16_t *p = (uint16_t *)c + off;
        if (vec && nvalid >= 8) {
            *(v4i *)p = v4i{(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
        } else {
            for (int i = 0; i < 8 && i < nvalid; i++) p[i] = (uint16_t)(w[i >> 1] >> ((i & 1) * 16));
        }
    }
}

// The same for a lane that owns NT consecutive N (NT = 8: store8; NT = 4: one 8-byte store of 16-bit values).
template <int CDT, int NT>
__device__ __forceinline__ void store_run(void *c, int64_t off, const float (&v)[NT], int nvalid, bool vec) {
    if (NT == 8) {
        store8<CDT>(c, off, v4f{v[0], v[1], v[2], v[3]}, v4f{v[NT - 4], v[NT - 3], v[NT - 2], v[NT - 1]}, nvalid, vec);
    } else if (CDT == MX_FP32) {
        float *p = (float *)c + off;
        if (vec && nvalid >= 4) *(v4f *)p = v4f{v[0], v[1], v[2], v[3]};
        else for (int i = 0; i < 4 && i < nvalid; i++) p[i] = v[i];
    } else {
        uint32_t w[2];
#pragma unroll
        for (int i = 0; i < 2; i++) {
            if (CDT == MX_BF16) {
                w[i] = pack2_bf16(v[2 * i], v[2 * i + 1]);
            } else {
                typedef _Float16 h2 __attribute__((ext_vector_type(2)));
                h2 h = {(_Float16)v[2 * i], (_Float16)v[2 * i + 1]};
                w[i] = __builtin_bit_cast(uint32_t, h);
            }
        }
        uint16_t *p = (uint16_t *)c + off;
        if (vec && nvalid >= 4) *(v2i *)p = v2i{(int)w[0], (int)w[1]};
        else for (int i = 0; i < 4 && i < nvalid; i++) p[i] = (uint16_t)(w[i >> 1] >> ((i & 1) * 16));
    }
}

// Maps a flat tile id to (tile_m, tile_n) so that (a) ids congruent mod `xcds` -- which run on
// the same XCD: workgroups are dealt to the 8 XCDs round-robin, the persistent stride is a
// multiple of 8, and a problem that owns only some of the XCDs (a batched launch) numbers its
// workgroups XCD-fastest -- are neighbours in tile space and share A/B panels in that XCD's L2, and
// (b) tiles are walked in column groups of GROUP_M row tiles.
__device__ __forceinline__ void tile_of(int id, int tiles_m, int tiles_n, int &tm, int &tn, bool stagger, int xcds) {
    const int total = tiles_m * tiles_n;
    const int per_xcd = total / xcds;
    if (id < per_xcd * xcds) id = xcds == 8 ? (id & 7) * per_xcd + (id >> 3) : (id % xcds) * per_xcd + id / xcds;
    constexpr int GROUP_M = 4;  // measured in the training step: 4 beats 2, 6, 8 and 16 by 1-5 %
    const int width = GROUP_M * tiles_n;
    const int group = id / width;
    const int first = group * GROUP_M;
    const int rows = tiles_m - first < GROUP_M ? tiles_m - first : GROUP_M;
    const int in = id - group * width;
    tm = first + in % rows;
    // (c) `stagger`: column groups that run at the same time on different XCDs start their walk
    // over the columns at different places, one `xcds`-th of the way round per group position.
    // Otherwise all XCDs miss on the same B panel at the same moment and every miss goes to HBM;
    // staggered, the panel one XCD reads now was read by its neighbour a round of tiles ago and
    // comes from the last-level cache -- provided a round is short enough for it to still be
    // there, so callers ask for it only for short K (long K: a round moves several hundred MB and
    // the simultaneous misses, which the memory side merges, are the cheaper pattern).  Measured
    // with operands that are not cache-resident, as inside a training step: 16384 x 8192 x 1536
    // 234 -> 199 us; a batch of three K = 8192 / 16384 products 494 -> 517 us.
    const int groups = (tiles_m + GROUP_M - 1) / GROUP_M;
    tn = in / rows;
    if (stagger) tn = (tn + (group * xcds / groups) * tiles_n / xcds) % tiles_n;
}

// Host-side launch helpers shared by the GEMM translation units (defined in mx_gemm.hip).
int num_cus();                            // CUs of the current device (cached per device ordinal)
bool stream_is_capturing(hipStream_t st);  // true also when the capture status cannot be read
// hipFuncSetAttribute(MaxDynamicSharedMemorySize) once per device; `done` has one bit per device ordinal.
bool allow_dynamic_lds(const void *kernel, int bytes, std::atomic<uint64_t> &done);

// Launch of a kernel that needs more than 64 KiB of dynamic LDS.  The "attribute already set" word is a
// function-local static of this instantiation, i.e. one per kernel: no table shared between kernels, no lock.
template <auto Kern, typename Args>
int launch_with_lds(dim3 grid, dim3 block, int lds_bytes, hipStream_t st, const Args &a) {
    static std::atomic<uint64_t> done{0};
    if (!allow_dynamic_lds((const void *)Kern, lds_bytes, done)) return MX_ELAUNCH;
    Kern<<<grid, block, lds_bytes, st>>>(a);
    return MX_OK;
}

}  // namespace mx
