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

__device__ __forceinline__ uint32_t lds_addr(const void *p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)p;
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
    // LDS row (of the A tile, of the B tile) of this lane's 16-byte chunk of copy q: copy q of wave w moves
    // the 8 rows from (q NW + w) 8
    static __device__ __forceinline__ int a_row(const Lane &L, int q) { return (q * S::NW + L.wave) * 8 + (L.lane >> 3); }
    static __device__ __forceinline__ int b_row(const Lane &L, int q) { return (q * S::NW + L.wave) * 8 + (L.lane >> 3); }
    const uint8_t *a_base, *b_base;
    int64_t a_ks = 128, b_ks = 128;  // bytes from one K stage of an operand to the next (128: row-major)
    uint32_t a_voff[S::QA], b_voff[S::QB];
    const uint8_t *srow0, *srow1;  // scale rows tid and tid + NTHR of the [A rows; B rows] list
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

template <typename S>
__device__ __forceinline__ uint32_t tail_fix(const IssueCtx<S> &c, const Lane &L, int kt, int q) {
    return tail_fix_row(c, L, kt, (q * S::NW + L.wave) * 8 + (L.lane >> 3));
}

// Row r (0..BM-1) of the A tile and row r of the B tile as the DMA engine sees them.
template <typename S>
__device__ __forceinline__ int dma_row(const Lane &L, int q) { return (q * S::NW + L.wave) * 8 + (L.lane >> 3); }

// A copy of the lane descriptor the optimiser cannot see through: address arithmetic done on
// it inside the per-tile setup is recomputed once per tile instead of being hoisted out of
// the tile loop and kept in (spilled) registers across the K loop.
__device__ __forceinline__ Lane opaque(const Lane &L) {
    Lane R = L;
    asm volatile("" : "+v"(R.tid), "+v"(R.lane));
    return R;
}

template <typename S>
__device__ __forceinline__ void issue_stage(const IssueCtx<S> &c, const Lane &L, int kt, uint8_t *ldsA, uint8_t *ldsB,
                                            int buf) {
    // The stage's base address is forced into SGPRs so each load is "scalar base + 32-bit
    // lane offset" and costs no 64-bit vector address arithmetic.
    const uint8_t *ga = uniform_ptr(c.a_base + (int64_t)kt * c.a_ks);
    const uint8_t *gb = uniform_ptr(c.b_base + (int64_t)kt * c.b_ks);
    const uint32_t la = __builtin_amdgcn_readfirstlane(lds_addr(ldsA) + buf * S::DATA_A + L.wave * 1024);
    const uint32_t lb = __builtin_amdgcn_readfirstlane(lds_addr(ldsB) + buf * S::DATA_B + L.wave * 1024);
#pragma unroll
    for (int q = 0; q < S::QA; q++) dma16(ga, c.a_voff[q] - tail_fix<S>(c, L, kt, q), la + q * S::NW * 1024);
#pragma unroll
    for (int q = 0; q < S::QB; q++) dma16(gb, c.b_voff[q] - tail_fix<S>(c, L, kt, q), lb + q * S::NW * 1024);
}

// How a row's scale bytes are fetched: one 16-byte load per 512 of K (K % 512 == 0, 16-byte
// aligned rows), one dword per stage (K % 128 == 0, 4-byte aligned rows), or byte by byte (any
// K % 32 == 0 and any pitch; blocks past the end of K read as scale byte 0).  SCALES_QUAD: one
// 16-byte load per 4 stages from a 4-byte aligned address, for K ranges that start on any stage
// (the token ranges of experts); it reads up to 12 bytes past the last stage's bytes, which the
// caller guarantees to lie inside the row's pitch.  Against SCALES_DWORD it asks the L2 for a
// row's line once per four stages instead of once per stage: 512 rows x 4 bytes a stage is half
// as many lines again as the stage's codes.
enum { SCALES_VEC16 = 0, SCALES_DWORD = 1, SCALES_BYTES = 2, SCALES_QUAD = 3 };

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

// One K stage of the workgroup tile: this wave's MT x NT accumulators advance by 128 of K,
// and, woven between the MFMAs, the wave issues its share of the direct-to-LDS copies that
// fetch stage `kt_next` (of the tile described by `c`) into LDS buffer `buf_next`.
//
// The copies are spread over the first half of the stage on purpose.  The texture path takes
// 64 bytes per clock, so the 64 KB a stage needs occupy it for ~1000 clocks per CU; issued in
// one burst at the top of the stage they stall every wave (and the MFMA pipe) for that long,
// issued late they would not land before the stage-ending barrier.
template <typename S, int OPSEL>
__device__ __forceinline__ void compute_stage(const uint8_t *__restrict__ la, const uint8_t *__restrict__ lb, int a_lo,
                                              int a_hi, int b_lo, int b_hi, const int (&sa)[S::MT],
                                              const int (&sb)[S::NT], v4f (&acc)[S::MT][S::NT],
                                              const IssueCtx<S> &c, const Lane &L, int kt_next, uint8_t *ldsA,
                                              uint8_t *ldsB, int buf_next) {
    const uint8_t *ga = uniform_ptr(c.a_base + (int64_t)kt_next * c.a_ks);
    const uint8_t *gb = uniform_ptr(c.b_base + (int64_t)kt_next * c.b_ks);
    const uint32_t wa = __builtin_amdgcn_readfirstlane(lds_addr(ldsA) + buf_next * S::DATA_A + L.wave * 1024);
    const uint32_t wb = __builtin_amdgcn_readfirstlane(lds_addr(ldsB) + buf_next * S::DATA_B + L.wave * 1024);
    constexpr int NQ = S::QA + S::QB;                      // copies this wave issues per stage
    auto issue = [&](int q) {
        if (q < S::QA) dma16(ga, c.a_voff[q] - tail_fix<S>(c, L, kt_next, q), wa + q * S::NW * 1024);
        else dma16(gb, c.b_voff[q - S::QA] - tail_fix<S>(c, L, kt_next, q - S::QA), wb + (q - S::QA) * S::NW * 1024);
    };

    // A is held (MT fragments), B streams through two fragment buffers.  Nothing crosses into or
    // out of the stage body, nor from one step of it into the next (sched_barrier).  LDS reads
    // return in order, so the first MFMA's operands (B[0], A[0]) are asked for first.
    constexpr int STEPS = S::NT / 2 > 0 ? S::NT / 2 : 1;  // the copies go out during the first half of the stage
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
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < S::NT; j++) {
        if (j + 1 < S::NT) {
            v4i lo = *(const v4i *)(lb + b_lo + (j + 1) * (16 * 128));
            v4i hi = *(const v4i *)(lb + b_hi + (j + 1) * (16 * 128));
            bfr[(j + 1) & 1] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
        if (j < STEPS) {
#pragma unroll
            for (int q = j * NQ / STEPS; q < (j + 1) * NQ / STEPS; q++) issue(q);
        }
#pragma unroll
        for (int i = 0; i < S::MT; i++)
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(afr[i], bfr[j & 1], acc[i][j], 0, 0, OPSEL, sa[i],
                                                                         OPSEL, sb[j]);
        __builtin_amdgcn_sched_barrier(0);
    }
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
template <typename S, int K512, typename P>  // K512: one of SCALES_*
__device__ __forceinline__ void persistent_gemm(P &prob, uint8_t *smem) {
    uint8_t *const ldsA = smem;                                                  // [2][BM*128]
    uint8_t *const ldsB = smem + 2 * S::DATA_A;                                  // [2][BN*128]
    uint32_t *const ldsSA = (uint32_t *)(smem + 2 * (S::DATA_A + S::DATA_B));    // [2][4][PA]
    uint32_t *const ldsSB = ldsSA + 2 * 4 * S::PA;                               // [2][4][PB]

    const Lane L = lane_of<S>();
    const bool has_row0 = L.tid < S::BM + S::BN;
    const int kb_end = prob.kb_end;

    // per-lane LDS read offsets: low half = 16-byte chunk g, high half = chunk g + 4 (= offset ^ 64)
    const int a_row = L.wm * S::WTM + L.r16;
    const int b_row = L.wn * S::WTN + L.r16;
    const int a_rd = a_row * 128 + ((L.g ^ swz_a(a_row)) << 4);
    const int b_rd = b_row * 128 + ((L.g ^ swz_a(b_row)) << 4);

    typename P::Tile cur, nxt;
    if (!prob.next(cur)) return;
    bool has_next = prob.next(nxt);
    IssueCtx<S> ctx;
    prob.context(cur, L, ctx);

    int gstage = 0;  // stages issued so far, over all tiles: LDS data buffer = gstage & 1
    int gsuper = 0;  // super-steps so far: LDS scale buffer = gsuper & 1

    // prologue of the first tile
    {
        uint32_t d0[4], d1[4];
        if (has_row0) load_scales<K512>(ctx.srow0, ctx.kt0 * 4, kb_end, d0);
        if (S::TWO_ROWS) load_scales<K512>(ctx.srow1, ctx.kt0 * 4, kb_end, d1);
        issue_stage<S>(ctx, L, ctx.kt0, ldsA, ldsB, 0);
        if (has_row0) park_scales<S>(L.tid, ldsSA, ldsSB, 0, d0);
        if (S::TWO_ROWS) park_scales<S>(L.tid + S::NTHR, ldsSA, ldsSB, 0, d1);
    }
    wait_vm_allow_c<0>();
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
                    if (has_row0) park_scales<S>(L.tid, ldsSA, ldsSB, sbuf ^ 1, d0);                          \
                    if (S::TWO_ROWS) park_scales<S>(L.tid + S::NTHR, ldsSA, ldsSB, sbuf ^ 1, d1);             \
                }                                                                                             \
                if (SIDX == 0 && ss + 1 < nsuper) {                                                           \
                    if (has_row0) load_scales<K512>(ctx.srow0, (kt0 + (ss + 1) * 4) * 4, kb_end, d0);         \
                    if (S::TWO_ROWS) load_scales<K512>(ctx.srow1, (kt0 + (ss + 1) * 4) * 4, kb_end, d1);      \
                }                                                                                             \
            } else if (has_next) {                                                                            \
                prob.context(nxt, L, ctx);                                                                    \
                if (has_row0) load_scales<K512>(ctx.srow0, ctx.kt0 * 4, kb_end, d0);                          \
                if (S::TWO_ROWS) load_scales<K512>(ctx.srow1, ctx.kt0 * 4, kb_end, d1);                       \
                kt_issue = ctx.kt0;                                                                           \
            } else {                                                                                          \
                kt_issue = kt0 + k; /* nothing left to fetch: a harmless re-read of this stage */             \
            }                                                                                                 \
            compute_stage<S, SIDX>(ldsA + buf * S::DATA_A, ldsB + buf * S::DATA_B, a_rd, a_rd ^ 64, b_rd,     \
                                   b_rd ^ 64, sa, sb, acc, ctx, L, kt_issue, ldsA, ldsB, buf ^ 1);            \
            if (!last) {                                                                                      \
                wait_vm_allow_c<0>();                                                                         \
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
        if (P::EARLY_WAIT && has_next) {
            wait_vm_allow_c<0>();
            if (has_row0) park_scales<S>(L.tid, ldsSA, ldsSB, gsuper & 1, d0);
            if (S::TWO_ROWS) park_scales<S>(L.tid + S::NTHR, ldsSA, ldsSB, gsuper & 1, d1);
        }
        const int stores = prob.epilogue(cur, L, acc, LdsScratch{ldsA + lastbuf * S::DATA_A, ldsB + lastbuf * S::DATA_B,
                                            (uint8_t *)(ldsSA + ((gsuper - 1) & 1) * 4 * S::PA)});
        if (!P::EARLY_WAIT && has_next) {
            if (has_row0) park_scales<S>(L.tid, ldsSA, ldsSB, gsuper & 1, d0);
            if (S::TWO_ROWS) park_scales<S>(L.tid + S::NTHR, ldsSA, ldsSB, gsuper & 1, d1);
        }
        if (!has_next) break;
        if (!P::EARLY_WAIT) {
            if (stores == P::NST) wait_vm_allow_c<P::NST>();
            else wait_vm_allow_c<0>();
        }
        __syncthreads();
        cur = nxt;
        has_next = prob.next(nxt);
    }
}

// ---------------------------------------------------------------------------------------------
// The wide-wave schedule (dense kernels, GemmShape<256, 256, 2, 2>): four waves per workgroup, one per SIMD, each
// owning 128 x 128 of the tile.  A wave then has the whole register file of its SIMD: the 64 accumulator tiles live
// in the 256 accumulation registers and the vector registers hold TWO sets of A fragments, so the first fragments of
// stage k + 1 are read while the last MFMAs of stage k run, and no wave ever stands at a barrier with an empty pipe
// and its operands still in LDS (the lockstep schedule's read burst after the barrier and its one-wave tail).
//
// One barrier per stage, in front of step 6 of 8:
//   * steps 0-3: the wave issues its 16 copies of stage k + 1 into the other buffer (free: every wave passed the
//     barrier of stage k - 1 after its last read of that buffer);
//   * step j reads B fragment j + 1, step 5 reads fragments 6 AND 7: nothing of this stage's buffer is left to read;
//   * in front of step 6: wait for those reads and for the wave's own copies, barrier.  Behind it stage k + 1's data
//     is visible to all and this stage's buffer is dead for all, so the copies of stage k + 2 may overwrite it from
//     the next stage's step 0 on;
//   * steps 6-7 (512 clocks of MFMA) cover the reads of stage k + 1's eight A fragments (into the other set) and its
//     first B fragment.
// The last stage of a tile has no such barrier: the next tile's first stage, already in flight, is published by the
// barrier behind the epilogue as in the lockstep schedule, and the tile reads its first fragments itself.
// B fragments rotate through four buffers (fragment j in buffer j % 4), so buffer 0 is free for the next stage's
// first fragment from step 5 on.
//
// Measured (MX_EPI_WIDE_WAVES; results bit-identical to the lockstep schedule): slower, 2.1 against 2.7 PFLOP/s at
// 8192^3.  A wave alone on its SIMD does not issue this MFMA every 32 clocks in a GEMM's operand pattern (eight A
// fragments against one B fragment, accumulators in the accumulation registers): with the copies and all LDS reads
// taken out of the stage it still needs 51 clocks per MFMA, and every copy it hands to the texture path is time in
// which its SIMD issues nothing.  Two waves per SIMD fill each other's gaps; the lockstep schedule stays the default.
template <typename S, int OPSEL>
__device__ __forceinline__ void wide_stage(const uint8_t *__restrict__ la_n, const uint8_t *__restrict__ lb,
                                           const uint8_t *__restrict__ lb_n, int a_lo, int a_hi, int b_lo, int b_hi,
                                           const int (&sa)[S::MT], const int (&sb)[S::NT], v4f (&acc)[S::MT][S::NT],
                                           const v8i (&afr)[S::MT], v8i (&afr_n)[S::MT], v8i (&bfr)[4], const IssueCtx<S> &c,
                                           const Lane &L, int kt_next, uint8_t *ldsA, uint8_t *ldsB, int buf_next, bool more) {
    static_assert(S::NT == 8, "the step numbers below are those of eight B fragments");
    const uint8_t *ga = uniform_ptr(c.a_base + (int64_t)kt_next * c.a_ks);
    const uint8_t *gb = uniform_ptr(c.b_base + (int64_t)kt_next * c.b_ks);
    const uint32_t wa = __builtin_amdgcn_readfirstlane(lds_addr(ldsA) + buf_next * S::DATA_A + L.wave * 1024);
    const uint32_t wb = __builtin_amdgcn_readfirstlane(lds_addr(ldsB) + buf_next * S::DATA_B + L.wave * 1024);
    constexpr int NQ = S::QA + S::QB, COPY_STEPS = 4;
    auto issue = [&](int q) {
        if (q < S::QA) dma16(ga, c.a_voff[q] - tail_fix<S>(c, L, kt_next, q), wa + q * S::NW * 1024);
        else dma16(gb, c.b_voff[q - S::QA] - tail_fix<S>(c, L, kt_next, q - S::QA), wb + (q - S::QA) * S::NW * 1024);
    };
    auto read_b = [&](const uint8_t *base, int frag, v8i &dst) {
        v4i lo = *(const v4i *)(base + b_lo + frag * (16 * 128));
        v4i hi = *(const v4i *)(base + b_hi + frag * (16 * 128));
        dst = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    };
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < S::NT; j++) {
        if (j < 5) read_b(lb, j + 1, bfr[(j + 1) & 3]);
        if (j == 5) {
            read_b(lb, 6, bfr[2]);
            read_b(lb, 7, bfr[3]);
        }
        if (j < COPY_STEPS) {
#pragma unroll
            for (int q = j * NQ / COPY_STEPS; q < (j + 1) * NQ / COPY_STEPS; q++) issue(q);
        }
        // fragments 6 and 7 are waited for on both paths, so that behind the branch nothing older than the next stage's
        // reads is outstanding and steps 6 and 7 do not wait for those
        if (j == 6) wait_vm_allow_c<63>();
        if (j == 6 && more) {
            wait_vm_allow_c<0>();  // this wave's copies of the next stage have landed
            __syncthreads();
            read_b(lb_n, 0, bfr[0]);
#pragma unroll
            for (int i = 0; i < S::MT; i++) {
                v4i lo = *(const v4i *)(la_n + a_lo + i * (16 * 128));
                v4i hi = *(const v4i *)(la_n + a_hi + i * (16 * 128));
                afr_n[i] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            }
        }
#pragma unroll
        for (int i = 0; i < S::MT; i++)
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(afr[i], bfr[j & 3], acc[i][j], 0, 0, OPSEL, sa[i],
                                                                         OPSEL, sb[j]);
        __builtin_amdgcn_sched_barrier(0);
    }
    // pins the MFMAs in front of whatever follows the stage; "a": the accumulators stay in the accumulation registers
#pragma unroll
    for (int i = 0; i < S::MT; i++)
#pragma unroll
        for (int j = 0; j < S::NT; j++) asm volatile("" : "+a"(acc[i][j]));
}

template <typename S, int K512, typename P>
__device__ __forceinline__ void persistent_gemm_wide(P &prob, uint8_t *smem) {
    static_assert(S::NW == 4 && !P::EARLY_WAIT, "one wave per SIMD; dense epilogues");
    uint8_t *const ldsA = smem;
    uint8_t *const ldsB = smem + 2 * S::DATA_A;
    uint32_t *const ldsSA = (uint32_t *)(smem + 2 * (S::DATA_A + S::DATA_B));
    uint32_t *const ldsSB = ldsSA + 2 * 4 * S::PA;

    const Lane L = lane_of<S>();
    const bool has_row0 = L.tid < S::BM + S::BN;
    const int kb_end = prob.kb_end;
    const int a_row = L.wm * S::WTM + L.r16;
    const int b_row = L.wn * S::WTN + L.r16;
    const int a_rd = a_row * 128 + ((L.g ^ swz_a(a_row)) << 4);
    const int b_rd = b_row * 128 + ((L.g ^ swz_a(b_row)) << 4);

    typename P::Tile cur, nxt;
    if (!prob.next(cur)) return;
    bool has_next = prob.next(nxt);
    IssueCtx<S> ctx;
    prob.context(cur, L, ctx);

    int gstage = 0, gsuper = 0;
    {
        uint32_t d0[4], d1[4];
        if (has_row0) load_scales<K512>(ctx.srow0, ctx.kt0 * 4, kb_end, d0);
        if (S::TWO_ROWS) load_scales<K512>(ctx.srow1, ctx.kt0 * 4, kb_end, d1);
        issue_stage<S>(ctx, L, ctx.kt0, ldsA, ldsB, 0);
        if (has_row0) park_scales<S>(L.tid, ldsSA, ldsSB, 0, d0);
        if (S::TWO_ROWS) park_scales<S>(L.tid + S::NTHR, ldsSA, ldsSB, 0, d1);
    }
    wait_vm_allow_c<0>();
    __syncthreads();

    v4f acc[S::MT][S::NT];
    v8i afr[2][S::MT], bfr[4];
    while (true) {
#pragma unroll
        for (int i = 0; i < S::MT; i++)
#pragma unroll
            for (int j = 0; j < S::NT; j++) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

        // the tile's first fragments (every later stage finds its own already in registers)
        {
            const uint8_t *la = ldsA + (gstage & 1) * S::DATA_A, *lb = ldsB + (gstage & 1) * S::DATA_B;
            v4i lo = *(const v4i *)(lb + b_rd);
            v4i hi = *(const v4i *)(lb + (b_rd ^ 64));
            bfr[0] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
#pragma unroll
            for (int i = 0; i < S::MT; i++) {
                v4i l2 = *(const v4i *)(la + a_rd + i * (16 * 128));
                v4i h2 = *(const v4i *)(la + (a_rd ^ 64) + i * (16 * 128));
                afr[0][i] = __builtin_shufflevector(l2, h2, 0, 1, 2, 3, 4, 5, 6, 7);
            }
        }

        const int kt0 = ctx.kt0, KT = ctx.kt1 - ctx.kt0;
        const int nsuper = (KT + 3) >> 2;
        uint32_t d0[4], d1[4];
        for (int ss = 0; ss < nsuper; ss++) {
            const int sbuf = gsuper & 1;
            int sa[S::MT], sb[S::NT];
#pragma unroll
            for (int i = 0; i < S::MT; i++) sa[i] = (int)ldsSA[(sbuf * 4 + L.g) * S::PA + a_row + 16 * i];
#pragma unroll
            for (int j = 0; j < S::NT; j++) sb[j] = (int)ldsSB[(sbuf * 4 + L.g) * S::PB + b_row + 16 * j];

#define MX_WSTAGE(SIDX)                                                                                       \
    {                                                                                                         \
        const int k = ss * 4 + SIDX;                                                                          \
        if (k < KT) {                                                                                         \
            const int buf = gstage & 1;                                                                       \
            const bool last = k + 1 == KT;                                                                    \
            int kt_issue = kt0 + k + 1;                                                                       \
            if (!last) {                                                                                      \
                if (SIDX == 3) {                                                                              \
                    if (has_row0) park_scales<S>(L.tid, ldsSA, ldsSB, sbuf ^ 1, d0);                          \
                    if (S::TWO_ROWS) park_scales<S>(L.tid + S::NTHR, ldsSA, ldsSB, sbuf ^ 1, d1);             \
                }                                                                                             \
                if (SIDX == 0 && ss + 1 < nsuper) {                                                           \
                    if (has_row0) load_scales<K512>(ctx.srow0, (kt0 + (ss + 1) * 4) * 4, kb_end, d0);         \
                    if (S::TWO_ROWS) load_scales<K512>(ctx.srow1, (kt0 + (ss + 1) * 4) * 4, kb_end, d1);      \
                }                                                                                             \
            } else if (has_next) {                                                                            \
                prob.context(nxt, L, ctx);                                                                    \
                if (has_row0) load_scales<K512>(ctx.srow0, ctx.kt0 * 4, kb_end, d0);                          \
                if (S::TWO_ROWS) load_scales<K512>(ctx.srow1, ctx.kt0 * 4, kb_end, d1);                       \
                kt_issue = ctx.kt0;                                                                           \
            } else {                                                                                          \
                kt_issue = kt0 + k;                                                                           \
            }                                                                                                 \
            wide_stage<S, SIDX>(ldsA + (buf ^ 1) * S::DATA_A, ldsB + buf * S::DATA_B, ldsB + (buf ^ 1) * S::DATA_B, a_rd,      \
                                a_rd ^ 64, b_rd, b_rd ^ 64, sa, sb, acc, afr[SIDX & 1], afr[(SIDX + 1) & 1], bfr, ctx, L,      \
                                kt_issue, ldsA, ldsB, buf ^ 1, !last);                                        \
            gstage++;                                                                                         \
        }                                                                                                     \
    }
            MX_WSTAGE(0)
            MX_WSTAGE(1)
            MX_WSTAGE(2)
            MX_WSTAGE(3)
#undef MX_WSTAGE
            gsuper++;
        }
        const int lastbuf = (gstage - 1) & 1;
        const int stores = prob.epilogue(cur, L, acc, LdsScratch{ldsA + lastbuf * S::DATA_A, ldsB + lastbuf * S::DATA_B,
                                            (uint8_t *)(ldsSA + ((gsuper - 1) & 1) * 4 * S::PA)});
        if (has_next) {
            if (has_row0) park_scales<S>(L.tid, ldsSA, ldsSB, gsuper & 1, d0);
            if (S::TWO_ROWS) park_scales<S>(L.tid + S::NTHR, ldsSA, ldsSB, gsuper & 1, d1);
        }
        if (!has_next) break;
        if (stores == P::NST && P::NST <= 63) wait_vm_allow_c<(P::NST <= 63 ? P::NST : 0)>();
        else wait_vm_allow_c<0>();
        __syncthreads();
        cur = nxt;
        has_next = prob.next(nxt);
    }
}

// ---------------------------------------------------------------------------------------------
// The phased schedule (dense kernels).  Same tile, same LDS layout, same K-stage arithmetic as
// persistent_gemm above, but the eight waves run as two groups of four -- one wave of each group on
// every SIMD -- HALF A STAGE APART: waves 0-3 (group 0, the tile's columns 0-127) begin a stage when
// waves 4-7 (group 1, columns 128-255) are in the middle of theirs.  In the lockstep schedule every
// wave of the workgroup stands at the stage-ending barrier at the same time and then waits for its
// first LDS reads at the same time, so each SIMD's MFMA pipe idles for the barrier, for the read
// latency (230-310 clocks) and for the tail in which only the later of its two waves still has work:
// about a quarter of a stage.  Half a stage apart, one wave of every SIMD is in the middle of its
// MFMAs, operands in registers, whenever the other one waits.
//
// How it stays correct with one hardware barrier.  All eight waves execute the same number of
// s_barrier, two per stage: in the middle of a stage and at its end.  Group 1 executes one extra
// barrier before its first stage (and group 0 one after its last), which is the whole offset: group
// 0's mid-stage barrier is group 1's stage-ending one and vice versa.  Barrier epochs of global stage
// g (tile number tau adds one epoch per tile, see below): group 0 works g in epochs 2g, 2g+1, group
// 1 in 2g+1, 2g+2.
//   * A is read from LDS only at the start of a stage (its fragments stay in registers for the
//     stage); it is shared by both groups, so buffer A[g&1] is read in epochs 2g (group 0) and 2g+1
//     (group 1).  Group 0 copies ALL of A(g+1) (and its own half of B(g+1)) during the first half of
//     stage g, epoch 2g, into A[(g+1)&1], last read in epoch 2g-1; it waits for its copies before the
//     barrier that ends epoch 2g+1, and both groups read A(g+1) no earlier than epoch 2g+2.
//   * The B half of a group is private to it and streamed through the stage: group 1 copies its
//     half of B(g+1) during the first half of ITS stage g (epoch 2g+1) into a buffer it last read in
//     epoch 2g, waits before the barrier ending epoch 2g+2 and reads it from epoch 2g+3.
//   * Scale bytes: every thread loads and parks one row's bytes as in the lockstep schedule; parks
//     always precede a stage-ending barrier of the parking thread's own group that lies before the
//     first read of that plane by either group.
//   * Tile boundary: each group runs its epilogue after its own last stage and then executes one more
//     barrier (epoch + 1 per tile for both groups), so that the pairing mid <-> end is the same in
//     every tile.  The next tile's first stage was copied during the last stage, as above.
// ---------------------------------------------------------------------------------------------
template <typename S>
struct PhasedCtx {
    static constexpr int NA = 2 * S::QA, NB = S::QB;  // group 0: all of A and its half of B; group 1: its half of B
    // Copy q of a wave moves 8 LDS rows; this lane's 16-byte chunk of it belongs to tile row
    //   A: a_row0 + 32 q        (LDS row (4 q + wave % 4) 8 + lane / 8 holds that same row of the tile)
    //   B: b_row0 + 2 q         (LDS row (wave / 4) 128 + (4 q + wave % 4) 8 + lane / 8 holds B row b_row_of_lds of it)
    // clamped to the tile's last valid row; the byte offsets are rebuilt from these at every copy
    // (a multiply-add each) instead of being held in twelve registers across the stage.
    const uint8_t *a_base, *b_base;
    int64_t a_ks = 128, b_ks = 128;
    int a_row0, b_row0, chunk16;  // per lane
    int a_last, b_last;           // last valid row of the tile (uniform)
    int lda, ldb;                 // row pitches in bytes (uniform; 256 rows of either fit 31 bits)
    const uint8_t *srow0, *srow1;
    int kt0, kt1;
    int tail_kt, tail_bytes;
    __device__ __forceinline__ uint32_t a_voff(int q, int kt) const {
        const int row = a_row0 + 32 * q;
        const uint32_t v = (uint32_t)((row < a_last ? row : a_last) * lda) + chunk16;
        return v - (kt == tail_kt && chunk16 >= tail_bytes ? (uint32_t)chunk16 : 0u);
    }
    __device__ __forceinline__ uint32_t b_voff(int q, int kt) const {
        const int row = b_row0 + 2 * q;
        const uint32_t v = (uint32_t)((row < b_last ? row : b_last) * ldb) + chunk16;
        return v - (kt == tail_kt && chunk16 >= tail_bytes ? (uint32_t)chunk16 : 0u);
    }
    // fills the per-lane part; the caller sets bases, pitches, limits, scale rows and the K range
    __device__ __forceinline__ void lanes(const Lane &L) {
        const int in = (L.wave & 3) * 8 + (L.lane >> 3);  // row of copy 0 inside the group's 128-row (A: 256-row) span
        a_row0 = in;
        b_row0 = (L.wave >> 2) * (S::BN / 2) + (in % 16) * S::NT + in / 16;
        chunk16 = ((L.lane & 7) ^ swz_a(in)) << 4;
    }
};

// One half (steps 4 HALF .. 4 HALF + 3 of 8) of a K stage under the phased schedule.  The first half reads
// the A fragments and the first B fragment and weaves the copies of stage `kt_next` between its MFMAs
// (group 0: twelve, three per step; group 1: four, one per step); the fragments live on into the second half.
template <typename S, int OPSEL, int HALF>
__device__ __forceinline__ void phased_half(const uint8_t *__restrict__ la, const uint8_t *__restrict__ lb, int a_lo, int a_hi,
                                            int b_lo, int b_hi, const int (&sa)[S::MT], const int (&sb)[S::NT],
                                            v4f (&acc)[S::MT][S::NT], v8i (&afr)[S::MT], v8i (&bfr)[2], const PhasedCtx<S> &c,
                                            const Lane &L, int grp, int kt_next, uint8_t *ldsA, uint8_t *ldsB, int buf_next) {
    typedef PhasedCtx<S> C;
    const uint8_t *ga = nullptr, *gb = nullptr;
    uint32_t wa = 0, wb = 0;
    if (HALF == 0) {
        ga = uniform_ptr(c.a_base + (int64_t)kt_next * c.a_ks);
        gb = uniform_ptr(c.b_base + (int64_t)kt_next * c.b_ks);
        wa = __builtin_amdgcn_readfirstlane(lds_addr(ldsA) + buf_next * S::DATA_A + (L.wave & 3) * 1024);
        wb = __builtin_amdgcn_readfirstlane(lds_addr(ldsB) + buf_next * S::DATA_B + (L.wave >> 2) * (S::DATA_B / 2) +
                                            (L.wave & 3) * 1024);
    }
    auto copy_a = [&](int q) { dma16(ga, c.a_voff(q, kt_next), wa + q * 4096); };
    auto copy_b = [&](int q) { dma16(gb, c.b_voff(q, kt_next), wb + q * 4096); };
    if (HALF == 0) {
        __builtin_amdgcn_sched_barrier(0);
        {
            v4i lo = *(const v4i *)(lb + b_lo);
            v4i hi = *(const v4i *)(lb + b_hi);
            bfr[0] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
#pragma unroll
        for (int i = 0; i < S::MT; i++) {
            v4i lo = *(const v4i *)(la + a_lo + i * (16 * 128));
            v4i hi = *(const v4i *)(la + a_hi + i * (16 * 128));
            afr[i] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
        __builtin_amdgcn_sched_barrier(0);
    }
    constexpr int STEPS = S::NT / 2;
#pragma unroll
    for (int j = HALF * STEPS; j < (HALF + 1) * STEPS; j++) {
        if (j + 1 < S::NT) {
            v4i lo = *(const v4i *)(lb + b_lo + (j + 1) * (16 * 128));
            v4i hi = *(const v4i *)(lb + b_hi + (j + 1) * (16 * 128));
            bfr[(j + 1) & 1] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
        constexpr int CSTEPS = STEPS;  // the copies go out over the whole first half, as in the lockstep schedule
        if (HALF == 0 && j < CSTEPS) {
            if (grp == 0) {
                constexpr int PER = (C::NA + C::NB) / CSTEPS;
#pragma unroll
                for (int u = 0; u < PER; u++) {
                    const int q = j * PER + u;
                    if (q < C::NA) copy_a(q);
                    else copy_b(q - C::NA);
                }
            } else {
                constexpr int PER = C::NB / CSTEPS;
#pragma unroll
                for (int u = 0; u < PER; u++) copy_b(j * PER + u);
            }
        }
#pragma unroll
        for (int i = 0; i < S::MT; i++)
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(afr[i], bfr[j & 1], acc[i][j], 0, 0, OPSEL, sa[i],
                                                                         OPSEL, sb[j]);
        // The copies sit behind a (wave-uniform) branch on the group, which ends the basic block: a scheduling
        // barrier alone no longer keeps this step's MFMAs in front of the next step's copies (they were all
        // sunk below the last branch of the half, behind one burst of copies).  An empty volatile asm on the
        // step's accumulators does: volatile asm statements keep their order, and the copies are volatile asm.
#pragma unroll
        for (int i = 0; i < S::MT; i++) asm volatile("" : "+v"(acc[i][j]));
        __builtin_amdgcn_sched_barrier(0);
    }
}

// The persistent tile loop under the phased schedule.  `P` as for persistent_gemm, with
// an overload `void context(const Tile &, const Lane &, PhasedCtx<S> &)`; the epilogue must not use LDS
// (the other group is half a stage away from any point of this group's program).
template <typename S, int K512, typename P>
__device__ __forceinline__ void persistent_gemm_phased(P &prob, uint8_t *smem) {
    static_assert(S::NW == 8 && S::WGM == 4 && S::WGN == 2 && !S::TWO_ROWS && S::NT % 2 == 0, "two groups of four waves");
    static_assert((PhasedCtx<S>::NA + PhasedCtx<S>::NB) % (S::NT / 2) == 0 && PhasedCtx<S>::NB % (S::NT / 2) == 0, "copies per step");
    uint8_t *const ldsA = smem;
    uint8_t *const ldsB = smem + 2 * S::DATA_A;
    uint32_t *const ldsSA = (uint32_t *)(smem + 2 * (S::DATA_A + S::DATA_B));
    uint32_t *const ldsSB = ldsSA + 2 * 4 * S::PA;

    Lane L = lane_of<S>();
    L.wm = L.wave & 3;   // group = wave / 4 = the half of N: the four waves of a group sit on the four SIMDs
    L.wn = L.wave >> 2;
    const int grp = L.wn;
    const int kb_end = prob.kb_end;
    const int a_row = L.wm * S::WTM + L.r16;
    const int b_row = L.wn * S::WTN + L.r16;
    const int a_rd = a_row * 128 + ((L.g ^ swz_a(a_row)) << 4);
    const int b_rd = b_row * 128 + ((L.g ^ swz_a(b_row)) << 4);

    typename P::Tile cur, nxt;
    if (!prob.next(cur)) return;
    bool has_next = prob.next(nxt);
    PhasedCtx<S> ctx;
    prob.context(cur, L, ctx);

    int gstage = 0, gsuper = 0;
    {   // first tile: its first stage and scale bytes, published to both groups by one full barrier
        uint32_t d0[4];
        load_scales<K512>(ctx.srow0, ctx.kt0 * 4, kb_end, d0);
        const uint8_t *ga = uniform_ptr(ctx.a_base + (int64_t)ctx.kt0 * ctx.a_ks);
        const uint8_t *gb = uniform_ptr(ctx.b_base + (int64_t)ctx.kt0 * ctx.b_ks);
        const uint32_t wa = __builtin_amdgcn_readfirstlane(lds_addr(ldsA) + (L.wave & 3) * 1024);
        const uint32_t wb = __builtin_amdgcn_readfirstlane(lds_addr(ldsB) + (L.wave >> 2) * (S::DATA_B / 2) + (L.wave & 3) * 1024);
        if (grp == 0) {
#pragma unroll
            for (int q = 0; q < PhasedCtx<S>::NA; q++) dma16(ga, ctx.a_voff(q, ctx.kt0), wa + q * 4096);
        }
#pragma unroll
        for (int q = 0; q < PhasedCtx<S>::NB; q++) dma16(gb, ctx.b_voff(q, ctx.kt0), wb + q * 4096);
        park_scales<S>(L.tid, ldsSA, ldsSB, 0, d0);
    }
    wait_vm_allow_c<0>();
    __syncthreads();
    if (grp == 1) __builtin_amdgcn_s_barrier();  // the offset: from here group 1 is one barrier, half a stage, behind

    v4f acc[S::MT][S::NT];
    while (true) {
#pragma unroll
        for (int i = 0; i < S::MT; i++)
#pragma unroll
            for (int j = 0; j < S::NT; j++) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

        const int kt0 = ctx.kt0, KT = ctx.kt1 - ctx.kt0;
        const int nsuper = (KT + 3) >> 2;
        uint32_t d0[4];
        for (int ss = 0; ss < nsuper; ss++) {
            const int sbuf = gsuper & 1;
            int sa[S::MT], sb[S::NT];
#pragma unroll
            for (int i = 0; i < S::MT; i++) sa[i] = (int)ldsSA[(sbuf * 4 + L.g) * S::PA + a_row + 16 * i];
#pragma unroll
            for (int j = 0; j < S::NT; j++) sb[j] = (int)ldsSB[(sbuf * 4 + L.g) * S::PB + b_row + 16 * j];
            v8i afr[S::MT], bfr[2];
#define MX_PHASED_STAGE(SIDX)                                                                                   \
    {                                                                                                           \
        const int k = ss * 4 + SIDX;                                                                            \
        if (k < KT) {                                                                                           \
            const int buf = gstage & 1;                                                                         \
            const bool last = k + 1 == KT;                                                                      \
            int kt_issue = kt0 + k + 1;                                                                         \
            if (!last) {                                                                                        \
                if (SIDX == 3) park_scales<S>(L.tid, ldsSA, ldsSB, sbuf ^ 1, d0);                               \
                if (SIDX == 0 && ss + 1 < nsuper) load_scales<K512>(ctx.srow0, (kt0 + (ss + 1) * 4) * 4, kb_end, d0); \
            } else if (has_next) {                                                                              \
                prob.context(nxt, L, ctx);                                                                      \
                load_scales<K512>(ctx.srow0, ctx.kt0 * 4, kb_end, d0);                                          \
                kt_issue = ctx.kt0;                                                                             \
            } else {                                                                                            \
                kt_issue = kt0 + k; /* nothing left to fetch: a harmless re-read of this stage */               \
            }                                                                                                   \
            phased_half<S, SIDX, 0>(ldsA + buf * S::DATA_A, ldsB + buf * S::DATA_B, a_rd, a_rd ^ 64, b_rd, b_rd ^ 64, sa, \
                                    sb, acc, afr, bfr, ctx, L, grp, kt_issue, ldsA, ldsB, buf ^ 1);              \
            __builtin_amdgcn_s_barrier(); /* middle of this group's stage, end of the other's */                \
            phased_half<S, SIDX, 1>(ldsA + buf * S::DATA_A, ldsB + buf * S::DATA_B, a_rd, a_rd ^ 64, b_rd, b_rd ^ 64, sa, \
                                    sb, acc, afr, bfr, ctx, L, grp, kt_issue, ldsA, ldsB, buf ^ 1);              \
            /* the next tile's scale bytes go to their plane ahead of this group's stage-ending barrier */       \
            if (last && has_next) park_scales<S>(L.tid, ldsSA, ldsSB, sbuf ^ 1, d0);                            \
            wait_vm_allow_c<0>();                                                                               \
            __builtin_amdgcn_s_barrier();                                                                       \
            gstage++;                                                                                           \
        }                                                                                                       \
    }
            MX_PHASED_STAGE(0)
            MX_PHASED_STAGE(1)
            MX_PHASED_STAGE(2)
            MX_PHASED_STAGE(3)
#undef MX_PHASED_STAGE
            gsuper++;
        }
        prob.epilogue(cur, L, acc, LdsScratch{nullptr, nullptr, nullptr});
        if (!has_next) break;
        __builtin_amdgcn_s_barrier();  // one more per tile and group: keeps the two groups' barriers paired mid <-> end
        cur = nxt;
        has_next = prob.next(nxt);
    }
    if (grp == 0) __builtin_amdgcn_s_barrier();  // closes the offset: pairs with group 1's last stage-ending barrier
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
