// Three alternative kernels for the dense product, kept as measured evidence and built only into the variants
// library (-DMX_BENCH_VARIANTS: libmxfp8_hip_variants.so, which the GEMM benchmark and the bit-equality test load).
// The product library does not contain them and refuses their flags.  All three give the shipped kernel's results bit
// for bit and were measured slower on every benchmark shape:
//   MX_EPI_TILE_128    128 x 128 tiles, two workgroups per CU (the persistent loop of mx_gemm_core.h on another shape)
//   MX_EPI_PHASED      the 256 x 256 tile with its eight waves as two groups of four half a K stage apart
//   MX_EPI_WIDE_WAVES  the 256 x 256 tile on four waves, one per SIMD, 128 x 128 each, accumulators in the
//                      accumulation registers
// At most one of them may be set in `epilogue` of mx_gemm_nt, not together with MX_EPI_ACCUMULATE / MX_EPI_SPLIT_K.
#pragma once

#include "mx_gemm_core.h"

#define MX_EPI_TILE_128 0x10
#define MX_EPI_PHASED 0x20
#define MX_EPI_WIDE_WAVES 0x40

namespace mx {

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
    const uint8_t *ga = uniform_ptr(c.a_base + (int64_t)kt_next * c.a_ks - COPY_BIAS);
    const uint8_t *gb = uniform_ptr(c.b_base + (int64_t)kt_next * c.b_ks - COPY_BIAS);
    const uint32_t wa = __builtin_amdgcn_readfirstlane(lds_addr(ldsA) + buf_next * S::DATA_A + L.wave * S::QA * 1024);
    const uint32_t wb = __builtin_amdgcn_readfirstlane(lds_addr(ldsB) + buf_next * S::DATA_B + L.wave * S::QB * 1024);
    typedef CopyRuns<S> Runs;
    constexpr int COPY_STEPS = 4;
    static_assert(Runs::N % COPY_STEPS == 0, "whole runs per step");
    auto read_b = [&](const uint8_t *base, int frag, v8i &dst) {
        v4i lo = *(const v4i *)(base + b_lo + frag * (16 * 128));
        v4i hi = *(const v4i *)(base + b_hi + frag * (16 * 128));
        dst = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    };
    __builtin_amdgcn_sched_barrier(0);
    static_for<S::NT>([&](auto jc) {
        constexpr int j = jc.value;
        if (j < 5) read_b(lb, j + 1, bfr[(j + 1) & 3]);
        if (j == 5) {
            read_b(lb, 6, bfr[2]);
            read_b(lb, 7, bfr[3]);
        }
        static_for<Runs::N>([&](auto r) {
            if constexpr (r.value * COPY_STEPS / Runs::N == j && j < COPY_STEPS)
                Runs::template issue<r.value>(c, L, kt_next, ga, gb, wa, wb);
        });
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
    });
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

}  // namespace mx
