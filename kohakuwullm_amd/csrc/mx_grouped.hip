// Routed-expert (grouped) MXFP8 GEMMs for gfx950.
//
// Rows are sorted by expert; `offsets (E+1)` int32 on the DEVICE is the exclusive prefix sum
// of the per-expert row counts and is never read on the host: the grid is a bound
// (ceil(M/BM) + E row tiles) and every workgroup resolves its row tile to (expert, start, end)
// itself, as tile_owner does in the reference (src/kohakuwullm/kernels/mxfp8/grouped.py:26-48).
// Empty experts contribute no tiles; row tiles past the last real one are skipped.
//
// One kernel body (mx_gemm_core.h) serves four problems, selected by the policy's MODE:
//   PLAIN      out[m] = xq[index[m] or m] . wq[e(m)]^T                    grouped.py:65-149
//   GEMM1      gather by token, both halves of x . w_in^T, round to the storage dtype, SwiGLU,
//              requantize: hq (M,H), hs (M,H/32), optional pre (M,2H)     experts.py:25-135
//   SCATTER    out[token(m)] += scale(m) * (a[m] . w[e(m)]^T), packed 16-bit atomics;
//              scale = gate[order[m]] (GEMM2, experts.py:138-222) or 1 (GEMM1 dgrad,
//              experts_bwd.py:167-247)
//   DGRAD2     acc = dq[token(m)] . w_out_dgrad[e]^T; dgate[pair] += <acc, h>; dh = acc * gate;
//              SwiGLU' from the stored pre; dpre (M,2H) stored and requantized
//                                                                         experts_bwd.py:29-164
// The row gather costs nothing: every lane of the copy engine supplies its own global address.
#include <type_traits>

#include "mx_gemm_core.h"

namespace mx {


enum { MODE_PLAIN = 0, MODE_GEMM1 = 1, MODE_SCATTER = 2, MODE_DGRAD2 = 3 };

struct GroupedArgs {
    // A operand: rows (R,K) + scales, optionally gathered through index[sorted position]
    const uint8_t *xq, *xs;
    int64_t ldx, ldxs;
    int64_t x_rows;  // R, where the caller states it (mx_grouped_gemm_nt), else 0
    const int32_t *index;
    // B operand: per-expert (E, NB, K) codes + scales
    const uint8_t *wq, *ws;
    int64_t stride_we, ldw, stride_wse, ldws;
    const int32_t *offsets;
    int E, M, N, K;  // M: bound on sorted rows; N: output width (hidden units H for GEMM1/DGRAD2)
    int tiles_n, tbound;
    // outputs / side inputs
    void *out;  // PLAIN: (M,N); SCATTER: (T,N) accumulated
    int64_t ldo;
    int out_vec;
    const int32_t *token_of, *order;
    const void *gate;  // (pairs,) in the 16-bit activation dtype or fp32 (gate_f32)
    int gate_f32;
    uint8_t *hq, *hs;  // GEMM1 out / DGRAD2 in: (M,H), (M,H/32)
    int64_t ldhq, ldhs;
    uint8_t *htq, *hts;  // GEMM1 out (optional): h quantized along the tokens, (H,Mpad), (H,Mpad/32)
    int64_t ldhtq, ldhts;
    int64_t htq_ks;  // 0, or htq stage-major: the 128 positions of panel j of every row together, panel j at j * htq_ks, row r at r * 128
    void *pre;  // GEMM1 out (optional) / DGRAD2 in: (M,2H) 16-bit
    int64_t ldpre;
    void *dpre;  // DGRAD2 out: (M,2H) 16-bit
    uint8_t *dpq, *dps;  // DGRAD2 out: (M,2H), (M,2H/32)
    int64_t lddpq, lddps;
    float *dgate;  // DGRAD2 out: (pairs,) fp32, accumulated
};

template <int CDT>
__device__ __forceinline__ float load_act(const void *p, int64_t i) {
    if (CDT == MX_BF16) return bits2f((uint32_t)((const uint16_t *)p)[i] << 16);
    if (CDT == MX_FP16) return (float)((const _Float16 *)p)[i];
    return ((const float *)p)[i];
}

// Round to the 16-bit storage dtype and come back: what the next consumer will read.
template <int CDT>
__device__ __forceinline__ void round_pair(float &a, float &b, uint32_t &packed) {
    if (CDT == MX_BF16) {
        packed = pack2_bf16(a, b);
        a = bits2f(packed << 16);
        b = bits2f(packed & 0xFFFF0000u);
    } else {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        h2 h = {(_Float16)a, (_Float16)b};
        packed = __builtin_bit_cast(uint32_t, h);
        a = (float)h[0];
        b = (float)h[1];
    }
}

template <int CDT>
__device__ __forceinline__ void unpack8(const v4i &w, float (&v)[8]) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
        if (CDT == MX_BF16) {
            v[2 * i] = bits2f((uint32_t)w[i] << 16);
            v[2 * i + 1] = bits2f((uint32_t)w[i] & 0xFFFF0000u);
        } else {
            typedef _Float16 h2 __attribute__((ext_vector_type(2)));
            h2 h = __builtin_bit_cast(h2, w[i]);
            v[2 * i] = (float)h[0];
            v[2 * i + 1] = (float)h[1];
        }
    }
}

// One 16-bit storage value (in the low half of `bits`) as fp32.
template <int CDT>
__device__ __forceinline__ float unpack1(uint32_t bits) {
    if (CDT == MX_BF16) return bits2f(bits << 16);
    return (float)__builtin_bit_cast(_Float16, (uint16_t)bits);
}

template <int CDT>
__device__ __forceinline__ void atomic_add2(void *base, int64_t off, float a, float b) {
    if (CDT == MX_BF16) {
        typedef float f2 __attribute__((ext_vector_type(2)));
        typedef __bf16 b2 __attribute__((ext_vector_type(2)));
        f2 v = {a, b};
        __builtin_amdgcn_global_atomic_fadd_v2bf16((__attribute__((address_space(1))) b2 *)((uint16_t *)base + off),
                                                   __builtin_convertvector(v, b2));
    } else if (CDT == MX_FP16) {
        typedef _Float16 h2 __attribute__((ext_vector_type(2)));
        h2 v = {(_Float16)a, (_Float16)b};
        __builtin_amdgcn_global_atomic_fadd_v2f16((__attribute__((address_space(1))) h2 *)((_Float16 *)base + off), v);
    } else {
        atomicAdd((float *)base + off, a);
        atomicAdd((float *)base + off + 1, b);
    }
}

__device__ __forceinline__ float sigmoid_f(float x) { return sigmoid_f32(x); }

// Reductions over neighbouring lanes.  A lane owns 8 (GEMM1: 4) consecutive channels of a row
// and its neighbours own the next ones, so a 32-channel MX block is a quad (GEMM1: 8 lanes)
// and a wave's whole row segment is a 16-lane DPP row.
__device__ __forceinline__ float oct_max(float a) {
    a = quad_max(a);
    return fmaxf(a, __shfl_xor(a, 4, 64));
}
__device__ __forceinline__ float row16_sum(float a) {
    a += __shfl_xor(a, 1, 64);
    a += __shfl_xor(a, 2, 64);
    a += __shfl_xor(a, 4, 64);
    return a + __shfl_xor(a, 8, 64);
}

// Per-expert prefix tables in LDS, built once per workgroup by its first wave (coalesced reads
// of `offsets`, wave scans), so that finding the expert of a tile is a binary search or an
// indexed read instead of a walk over `offsets` with one dependent scalar load per expert:
// with 250 empty experts in front of the busy ones that walk cost every workgroup ~100 us per
// launch.  More experts than the tables hold fall back to the walk.
#define MX_TABLE_MAX 1024
template <int MAX>
struct ExpertTableN {
    static constexpr int CAPACITY = MAX;
    int a[MAX + 1];
    int b[MAX + 1];
    int n;
    int longest;  // build_live_table: the K stages of the expert with the most rows
};
typedef ExpertTableN<MX_TABLE_MAX> ExpertTable;
// The expert dW kernel that stages its scale bytes through LDS has 6 KB left for its table (the dynamic part starts
// on a multiple of 1 KB: 6 KB + the stage buffers, scale planes and staging area are 159 of the CU's 160 KB).
#define MX_TABLE_MAX_STAGED 760
typedef ExpertTableN<MX_TABLE_MAX_STAGED> ExpertTableStaged;

// a[e] = row tiles (of `bm` rows) of experts before e, b[e] = 128-row tiles of the padded token
// axis before e, for e in [0, E]; n = E.
__device__ __forceinline__ void build_row_tile_table(int *__restrict__ tab_a, int *__restrict__ tab_b,
                                                     const int32_t *__restrict__ offsets, int E, int bm) {
    if (threadIdx.x < 64) {
        const int lane = threadIdx.x;
        int carry_t = 0, carry_p = 0;
        for (int e0 = 0; e0 < E; e0 += 64) {
            const int e = e0 + lane;
            const int rows = e < E ? offsets[e + 1] - offsets[e] : 0;
            const int tiles = (rows + bm - 1) / bm, pads = (rows + 127) / 128;
            const int it = wave_incl_scan(tiles, lane), ip = wave_incl_scan(pads, lane);
            if (e < E) {
                tab_a[e] = carry_t + it - tiles;
                tab_b[e] = carry_p + ip - pads;
            }
            carry_t += __shfl(it, 63, 64);
            carry_p += __shfl(ip, 63, 64);
        }
        if (lane == 0) {
            tab_a[E] = carry_t;
            tab_b[E] = carry_p;
        }
    }
    __syncthreads();
}

// a[j] = the j-th expert with rows, b[j] = 128-token K stages of the experts before it; n = how many;
// b[n] = K stages of all experts.
template <typename TB>
__device__ __forceinline__ void build_live_table(TB &tb, const int32_t *__restrict__ offsets, int E) {
    if (threadIdx.x < 64) {
        const int lane = threadIdx.x;
        const uint64_t below = lane ? ~0ull >> (64 - lane) : 0ull;
        int carry_l = 0, carry_p = 0, most = 0;
        for (int e0 = 0; e0 < E; e0 += 64) {
            const int e = e0 + lane;
            const int rows = e < E ? offsets[e + 1] - offsets[e] : 0;
            const int pads = (rows + 127) / 128;
            most = pads > most ? pads : most;
            const int ip = wave_incl_scan(pads, lane);
            const uint64_t mask = __ballot(rows > 0);
            if (rows > 0) {
                const int rank = carry_l + __builtin_popcountll(mask & below);
                tb.a[rank] = e;
                tb.b[rank] = carry_p + ip - pads;
            }
            carry_l += __builtin_popcountll(mask);
            carry_p += __shfl(ip, 63, 64);
        }
#pragma unroll
        for (int d = 32; d; d >>= 1) {
            const int other = __shfl_xor(most, d, 64);
            most = other > most ? other : most;
        }
        if (lane == 0) {
            tb.n = carry_l;
            tb.b[carry_l] = carry_p;  // one past the last expert's K stages
            tb.longest = most;
        }
    }
    __syncthreads();
}

template <typename S, int MODE, int CDT>
struct GroupedProblem {
    struct Tile {
        int n0, row0, end, expert, kt0, kt1;
        int ppos;  // position of row0 in the padded token axis (each expert padded to 128-row tiles)
    };
    const GroupedArgs p;  // a copy: fields live in scalar registers
    int next_id;
    int kb_end;
    // incremental tile_owner: experts [0, scan_e) own row tiles [0, scan_tiles) and the first
    // scan_pad 128-row tiles of the padded token axis
    int scan_e, scan_tiles, scan_pad;

    // Accumulator layout: lane (r16, g) holds, for sub-tile (i, j) and
    // register v, row 16 i + 4 g + v of the wave's 64 rows and column 8 r16 + j of its 128.
    // GEMM1 fills each wave's 128-row slice of the B tile with 64 gate rows (sub-tiles 0-3) and
    // the 64 value rows of the same hidden units (sub-tiles 4-7), so a tile spans BN/2 hidden
    // units and a lane owns 4 consecutive ones, gate and value.
    static constexpr int N_PER_TILE = MODE == MODE_GEMM1 ? S::BN / 2 : S::BN;
    static constexpr int NST = S::MT * 4 * (CDT == MX_FP32 ? 2 : 1);
    // the fused epilogues issue a different number of stores per lane (row and column masks): see persistent_gemm
    static constexpr bool EARLY_WAIT = MODE == MODE_GEMM1 || MODE == MODE_DGRAD2;
    static constexpr bool REUSE_CONTEXT = true;  // context() may read the row indices: see persistent_gemm

    const int *tab_a, *tab_b;  // row-tile prefix tables in LDS (build_row_tile_table), or nullptr (more experts than they hold)

    __device__ GroupedProblem(const GroupedArgs &a, const int *table_a, const int *table_b)
        : p(a), next_id(blockIdx.x), kb_end(a.K >> 5), scan_e(0), scan_tiles(0), scan_pad(0), tab_a(table_a), tab_b(table_b) {}

    __device__ __forceinline__ bool next(Tile &t) {
        // With the table the number of real row tiles is known: ids cover exactly those, so the
        // contiguous id ranges of the XCDs hold equal shares of real work.  (Over the host's bound,
        // rows / BM + E row tiles, the ranges of the last XCDs hold only ids past the end: with 64
        // experts at the benchmark's routing one XCD of eight had nothing to do.)
        const int total = p.tiles_n * (tab_a ? tab_a[p.E] : p.tbound);
        const int per_xcd = total >> 3;
        while (next_id < total) {
            int id = next_id;
            next_id += gridDim.x;
            // ids congruent mod 8 run on one XCD: give each XCD a contiguous range so the
            // N tiles of one row tile (same A rows, same expert weights) share an L2
            if (id < (per_xcd << 3)) id = (id & 7) * per_xcd + (id >> 3);
            const int rt = id / p.tiles_n;
            const int tn = id - rt * p.tiles_n;
            if (tab_a) {
                int lo = 0, hi = p.E;  // a[lo] <= rt < a[hi]: the last expert that starts at or before rt owns it
                while (hi - lo > 1) {
                    const int mid = (lo + hi) >> 1;
                    if (tab_a[mid] <= rt) lo = mid;
                    else hi = mid;
                }
                const int first = tab_a[lo];
                t.expert = lo;
                t.row0 = p.offsets[lo] + (rt - first) * S::BM;
                t.end = p.offsets[lo + 1];
                t.ppos = tab_b[lo] * 128 + (rt - first) * S::BM;
                t.n0 = tn * N_PER_TILE;
                t.kt0 = 0;
                t.kt1 = p.K >> 7;
                return true;
            }
            if (rt < scan_tiles) {  // ids are monotonic per workgroup except across the XCD remap edge
                scan_e = 0;
                scan_tiles = 0;
                scan_pad = 0;
            }
            int e = scan_e, before = scan_tiles, pad = scan_pad, start = 0, end = 0;
            bool found = false;
            while (e < p.E) {
                start = p.offsets[e];
                end = p.offsets[e + 1];
                const int tiles = (end - start + S::BM - 1) / S::BM;
                if (rt < before + tiles) {
                    found = true;
                    break;
                }
                before += tiles;
                pad += (end - start + 127) / 128;
                e++;
            }
            scan_e = e;
            scan_tiles = before;
            scan_pad = pad;
            if (!found) continue;  // past the last real row tile
            t.expert = e;
            t.row0 = start + (rt - before) * S::BM;
            t.end = end;
            t.ppos = pad * 128 + (rt - before) * S::BM;
            t.n0 = tn * N_PER_TILE;
            t.kt0 = 0;
            t.kt1 = p.K >> 7;
            return true;
        }
        return false;
    }

    // source row of the A operand for tile row r (rows past the expert's end repeat its last row)
    __device__ __forceinline__ int a_src_row(const Tile &t, int r) const {
        int pos = t.row0 + r;
        pos = pos < t.end ? pos : t.end - 1;
        return p.index ? p.index[pos] : pos;
    }
    // row of the expert's weight matrix kept in LDS row r of the B tile
    __device__ __forceinline__ int b_src_row(const Tile &t, int r) const {
        if (MODE == MODE_GEMM1) {
            const int slice = r / S::WTN, within = r % S::WTN;
            const int j = within >> 4, rr = within & 15;
            int h = t.n0 + slice * (S::WTN / 2) + 4 * rr + (j & 3);
            h = h < p.N ? h : p.N - 1;
            return j < 4 ? h : p.N + h;
        }
        const int n = t.n0 + b_row_of_lds<S>(r);
        return n < p.N ? n : p.N - 1;
    }

    __device__ __forceinline__ void context(const Tile &t, const Lane &L0, IssueCtx<S> &c) const {
        const Lane L = opaque(L0);
        c.a_base = p.xq;
        c.b_base = p.wq + (int64_t)t.expert * p.stride_we;
        c.kt0 = t.kt0;
        c.kt1 = t.kt1;
        c.tail_kt = -1, c.tail_bytes = 0;  // K % 128 == 0 is a precondition of these kernels
#pragma unroll
        for (int q = 0; q < S::QA; q++) {
            const int row = dma_row<S>(L, q);
            c.a_voff[q] = (uint32_t)((int64_t)a_src_row(t, row) * p.ldx) + (((L.lane & 7) ^ swz_a(row)) << 4) + copy_bias(q);
        }
#pragma unroll
        for (int q = 0; q < S::QB; q++) {
            const int row = dma_row<S>(L, q);
            c.b_voff[q] = (uint32_t)((int64_t)b_src_row(t, row) * p.ldw) + (((L.lane & 7) ^ swz_a(row)) << 4) + copy_bias(q);
        }
        auto srow = [&](int r) -> const uint8_t * {
            if (r < S::BM) return p.xs + (int64_t)a_src_row(t, r) * p.ldxs;
            return p.ws + (int64_t)t.expert * p.stride_wse + (int64_t)b_src_row(t, r - S::BM) * p.ldws;
        };
        c.srow0 = srow(L.tid < S::BM + S::BN ? L.tid : 0);
        c.srow1 = S::TWO_ROWS ? srow(L.tid + S::NTHR < S::BM + S::BN ? L.tid + S::NTHR : 0) : nullptr;
        // SCALES_COPY: the same row through the copy engine, as a 32-bit offset from its matrix
        c.sa_base = p.xs, c.sb_base = p.ws;
        c.s_voff = (uint32_t)(c.srow0 - (L.tid < S::BM ? p.xs : p.ws));
    }

    __device__ __forceinline__ int epilogue(const Tile &t, const Lane &L, v4f (&acc)[S::MT][S::NT],
                                            const LdsScratch &lds) const {
        if constexpr (MODE == MODE_PLAIN) return epilogue_plain(t, L, acc);
        else if constexpr (MODE == MODE_GEMM1) return epilogue_gemm1(t, L, acc, lds);
        else if constexpr (MODE == MODE_SCATTER) return epilogue_scatter(t, L, acc);
        else return epilogue_dgrad2(t, L, acc, lds);
    }

    // sorted row of (i, v) for this lane
    __device__ __forceinline__ int row_of(const Tile &t, const Lane &L, int i, int v) const {
        return t.row0 + L.wm * S::WTM + 16 * i + 4 * L.g + v;
    }

    // ---- PLAIN: rows of the expert's range are written, nothing else is touched
    __device__ __forceinline__ int epilogue_plain(const Tile &t, const Lane &L, v4f (&acc)[S::MT][S::NT]) const {
        const bool interior = t.row0 + S::BM <= t.end && t.n0 + S::BN <= p.N && p.out_vec;
        const int n = t.n0 + L.wn * S::WTN + 8 * L.r16;
#pragma unroll
        for (int i = 0; i < S::MT; i++) {
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int m = row_of(t, L, i, v);
                const int64_t off = (int64_t)m * p.ldo + n;
                const v4f lo = {acc[i][0][v], acc[i][1][v], acc[i][2][v], acc[i][3][v]};
                const v4f hi = {acc[i][4][v], acc[i][5][v], acc[i][6][v], acc[i][7][v]};
                if (interior) store8<CDT>(p.out, off, lo, hi, 8, true);
                else if (m < t.end && n < p.N) store8<CDT>(p.out, off, lo, hi, p.N - n < 8 ? p.N - n : 8, p.out_vec != 0);
            }
        }
        return interior ? NST : -1;
    }

    // Byte offset in the token-axis code matrix of 16-byte chunk `ch` of a tile's positions (the tile starts at padded
    // position `pbase`, a multiple of 128) in row `row`: row-major, or stage-major panels of 128 positions.
    __device__ __forceinline__ int64_t token_axis_offset(int row, int64_t pbase, int ch) const {
        return p.htq_ks ? ((pbase >> 7) + (ch >> 3)) * p.htq_ks + (int64_t)row * 128 + (ch & 7) * 16
                        : (int64_t)row * p.ldhtq + pbase + ch * 16;
    }

    // ---- GEMM1: sub-tiles 0-3 are gate, 4-7 value of the lane's 4 hidden units
    // Outputs: pre (rounded accumulators), h quantized along the hidden axis (hq, hs) for GEMM2,
    // and, when htq is given, h quantized along the tokens for GEMM2's WGRAD.  The token-axis
    // blocks are the 32-row groups (i, i+1) x g x v of a wave; their codes are transposed through
    // the LDS stage buffer the main loop has just left, so they reach memory as 256-byte runs.
    // (The epilogue is bound by its vector ALU work -- rounding, sigmoid, two quantizers per
    // value -- not by its stores: staging the row-direction outputs through LDS for wider
    // stores was measured and did not pay.)
    __device__ __forceinline__ int epilogue_gemm1(const Tile &t, const Lane &L0, v4f (&acc)[S::MT][S::NT],
                                                  const LdsScratch &lds) const {
        const Lane L = rebuilt<S>(L0);  // no per-lane column or row number of the epilogue lives across the K loop
        static_assert(S::MT % 2 == 0 && N_PER_TILE * S::BM <= S::DATA_A, "token-axis staging: one A half holds the tile");
        static_assert(S::NT == 8 && S::BM % 128 == 0, "four gate and four value sub-tiles per lane; whole 128-token tiles");
        constexpr int CH = S::BM / 16;  // 16-byte chunks of a staged column (its BM tokens)
        const int hblock = t.n0 + L.wn * (S::WTN / 2) + 32 * (L.r16 >> 3);  // the 32 hidden units of 8 lanes
        const int h = t.n0 + L.wn * (S::WTN / 2) + 4 * L.r16;
        const bool tok = p.htq != nullptr;
        if (tok) __syncthreads();  // every wave is out of the main loop: the stage buffer is free
#pragma unroll
        for (int blk = 0; blk < S::MT / 2; blk++) {
            float a[2][4][4];  // [i in block][v][hidden unit]
#pragma unroll
            for (int ii = 0; ii < 2; ii++) {
                const int i = 2 * blk + ii;
#pragma unroll
                for (int v = 0; v < 4; v++) {
                    const int m = row_of(t, L, i, v);
                    const bool row_ok = m < t.end;
                    const bool ok = row_ok && hblock < p.N;  // H % 32 == 0: a block is in or out
                    float gv[4], vv[4];
                    uint32_t gp[2], vp[2];
#pragma unroll
                    for (int e = 0; e < 4; e++) gv[e] = acc[i][e][v], vv[e] = acc[i][4 + e][v];
                    // h is rounded to the storage dtype before the activation, so the backward
                    // differentiates the function the forward evaluated (experts.py:116-119)
#pragma unroll
                    for (int e = 0; e < 2; e++) {
                        round_pair<CDT>(gv[2 * e], gv[2 * e + 1], gp[e]);
                        round_pair<CDT>(vv[2 * e], vv[2 * e + 1], vp[e]);
                    }
                    if (ok && p.pre) {
                        uint16_t *pp = (uint16_t *)p.pre + (int64_t)m * p.ldpre + h;
                        *(v2i *)pp = v2i{(int)gp[0], (int)gp[1]};
                        *(v2i *)(pp + p.N) = v2i{(int)vp[0], (int)vp[1]};
                    }
                    float r[4];
#pragma unroll
                    for (int e = 0; e < 4; e++) r[e] = gv[e] * sigmoid_f(gv[e]) * vv[e];
                    const float amax = oct_max(fmaxf(fmaxf(fabsf(r[0]), fabsf(r[1])), fmaxf(fabsf(r[2]), fabsf(r[3]))));
                    const uint32_t byte = scale_byte(amax);
                    const float inv = inv_scale(byte);
                    if (ok) {
                        *(uint32_t *)(p.hq + (int64_t)m * p.ldhq + h) = pack4_e4m3(r[0] * inv, r[1] * inv, r[2] * inv, r[3] * inv);
                        if ((L.r16 & 7) == 0) p.hs[(int64_t)m * p.ldhs + (hblock >> 5)] = (uint8_t)byte;
                    }
#pragma unroll
                    for (int e = 0; e < 4; e++) a[ii][v][e] = row_ok ? r[e] : 0.0f;  // rows past the expert are padding
                }
            }
            if (!tok) continue;
            // token axis: the block's 32 rows are this lane's 8 values and the lanes 16, 32, 48 away
#pragma unroll
            for (int e = 0; e < 4; e++) {
                float cm = 0.0f;
#pragma unroll
                for (int ii = 0; ii < 2; ii++)
#pragma unroll
                    for (int v = 0; v < 4; v++) cm = fmaxf(cm, fabsf(a[ii][v][e]));
                cm = fmaxf(cm, __shfl_xor(cm, 16, 64));
                cm = fmaxf(cm, __shfl_xor(cm, 32, 64));
                const uint32_t byte = scale_byte(cm);
                const float inv = inv_scale(byte);
                const int col = L.wn * (S::WTN / 2) + 4 * L.r16 + e;  // hidden unit inside the tile
#pragma unroll
                for (int ii = 0; ii < 2; ii++) {
                    const int row = L.wm * S::WTM + 16 * (2 * blk + ii) + 4 * L.g;  // 4 consecutive rows: one dword
                    const uint32_t w = pack4_e4m3(a[ii][0][e] * inv, a[ii][1][e] * inv, a[ii][2][e] * inv, a[ii][3][e] * inv);
                    // column-major, BM bytes per hidden unit, 16-byte chunks XOR-swizzled by the lane's r16
                    *(uint32_t *)(lds.a + col * S::BM + ((((row >> 4) ^ (col >> 2)) & (CH - 1)) << 4) + (row & 15)) = w;
                }
                if (L.g == 0) lds.b[col * (S::BM / 32) + L.wm * (S::WTM / 32) + blk] = (uint8_t)byte;
            }
        }
        if (!tok) return -1;
        __syncthreads();
        // CH consecutive lanes write the BM bytes of one hidden unit's BM tokens; a 128-row part
        // that starts past the expert's rows belongs to the next expert's padding and is skipped
        // wave-uniform and lane-dependent parts of the addresses below are rebuilt here (scalar register,
        // opaque lane id): as invariants of the tile loop they were spilled and reloaded behind full waits
        const int64_t pbase = __builtin_amdgcn_readfirstlane(t.ppos);
        const int o_tid = opaque(L).tid;
        static_assert((N_PER_TILE * S::BM / 16) % S::NTHR == 0, "whole rounds of 16-byte chunks");
#pragma unroll
        for (int k = 0; k < N_PER_TILE * S::BM / 16 / S::NTHR; k++) {
            const int q = o_tid + k * S::NTHR;
            const int col = q / CH, ch = q % CH;
            const bool part_ok = t.row0 + (ch >> 3) * 128 < t.end;
            if (t.n0 + col < p.N && part_ok) {
                const v4i w = *(const v4i *)(lds.a + col * S::BM + (((ch ^ (col >> 2)) & (CH - 1)) << 4));
                *(v4i *)(p.htq + token_axis_offset(t.n0 + col, pbase, ch)) = w;
            }
        }
        if (o_tid < N_PER_TILE && t.n0 + o_tid < p.N) {
            const uint32_t *src = (const uint32_t *)(lds.b + o_tid * (S::BM / 32));
            uint8_t *dst = p.hts + (int64_t)(t.n0 + o_tid) * p.ldhts + (pbase >> 5);
#pragma unroll
            for (int part = 0; part < S::BM / 128; part++)  // a dword of scale bytes per 128 tokens
                if (t.row0 + part * 128 < t.end) *(uint32_t *)(dst + 4 * part) = src[part];
        }
        return -1;
    }

    // ---- SCATTER: out[token(m)] += scale(m) * acc, packed 16-bit (or fp32) atomics
    __device__ __forceinline__ int epilogue_scatter(const Tile &t, const Lane &L, v4f (&acc)[S::MT][S::NT]) const {
        const int n = t.n0 + L.wn * S::WTN + 8 * L.r16;
#pragma unroll
        for (int i = 0; i < S::MT; i++) {
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int m = row_of(t, L, i, v);
                if (m >= t.end) continue;
                const int target = p.token_of[m];
                float scale = 1.0f;
                if (p.gate) scale = p.gate_f32 ? ((const float *)p.gate)[p.order[m]] : load_act<CDT>(p.gate, p.order[m]);
                const int64_t off = (int64_t)target * p.ldo + n;
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const float a = acc[i][2 * e][v] * scale, b = acc[i][2 * e + 1][v] * scale;
                    if (n + 2 * e + 1 < p.N) atomic_add2<CDT>(p.out, off + 2 * e, a, b);  // N is even
                }
            }
        }
        return -1;
    }

    // ---- DGRAD2: the accumulator dout[t] . W_out is consumed three ways in registers
    // Everything a 16-row slab (one i: the lane's 4 rows) reads from memory -- pair index, gate,
    // the fp8 copy of h, the stored pre -- is requested before any of it is used: issued row by
    // row, each dependent chain (order -> gate) and each row's loads would expose a full memory
    // latency 16 times per tile, which made this epilogue several times longer than the K loop.
    //
    // Token axis (p.htq given): dpre is also wanted quantized along the tokens, for dW_in.  The
    // lane keeps its 16 rows x 16 columns of dpre as packed 16-bit values -- the stored, rounded
    // ones, which is what a column quantizer reading dpre back would see -- in place of the
    // accumulators they were computed from, and a second phase quantizes them in 32-row blocks and
    // transposes them through the free stage buffer, 128 columns of dpre at a time.
    __device__ __forceinline__ int epilogue_dgrad2(const Tile &t, const Lane &L, v4f (&acc)[S::MT][S::NT],
                                                   const LdsScratch &lds) const {
        static_assert(S::MT % 2 == 0 && (S::BN / 2) * S::BM <= S::DATA_A && (S::BN / 2) * S::BM <= S::DATA_B &&
                          2 * (S::BN / 2) * (S::BM / 32) <= 4 * S::PA * 4,
                      "token-axis staging: half the tile's columns per pass, two passes in flight");
        static_assert(S::NT == 8 && S::BM % 128 == 0, "eight consecutive columns per lane; whole 128-token tiles");
        constexpr int CH = S::BM / 16;  // 16-byte chunks of a staged column (its BM tokens)
        const bool tok = p.htq != nullptr;
        uint32_t keep[2][S::MT][4][4];  // [gate | value][slab][row][pair of columns]
        const int H = p.N;
        // Lane-dependent offsets are derived from an opaque copy of the lane id.  From the plain one they are
        // invariants of the tile loop: the compiler computes them once (sixteen row numbers alone), cannot keep them
        // in registers across the main loop, and reloads each from scratch memory right before its use behind a full
        // vector-memory wait -- which also waits for every load and store in flight.
        const Lane Lo = opaque(L);
        const int o_tid = Lo.tid, o_r16 = Lo.lane & 15, o_g = Lo.lane >> 4;
        const int hblock = t.n0 + L.wn * S::WTN + 32 * (o_r16 >> 2);  // the 32 hidden units of a quad
        const int h = t.n0 + L.wn * S::WTN + 8 * o_r16;
        const bool col_ok = hblock < H;
        auto row_at = [&](int i, int v) { return t.row0 + L.wm * S::WTM + 16 * i + 4 * o_g + v; };
        // Row metadata once per tile: lane l of a wave fetches the pair index and the gate factor of the wave's row l
        // (two dependent loads per tile); a step takes its rows' values from those lanes.  Fetched per slab of rows by
        // the lanes that use them, the chain order -> gate cost two memory round trips per slab.
        const int meta_m = t.row0 + L.wm * S::WTM + (Lo.lane < S::WTM ? Lo.lane : S::WTM - 1);
        const int pair_l = p.order[meta_m < t.end ? meta_m : t.end - 1];
        asm volatile("" ::: "memory");  // the first step's requests go out behind this load, not behind the chain's second
        // The rows of a lane are taken RS at a time, and what a step reads from memory -- the fp8 copy of h, its scale
        // byte, the stored pre -- is requested one step ahead, in front of the previous step's arithmetic and stores.
        // Vector memory operations retire in order: loads issued behind a step's stores would wait for those stores
        // to reach the L2, and all eight waves of the workgroup would then sit through a memory round trip per step
        // with nothing to issue.  The compiler barriers keep the order written here.
        constexpr int RS = 1, STEPS = S::MT * 4 / RS;  // more rows per step, or requests further ahead, spill and are slower
        struct StepLoads {
            v2i hc[RS];
            uint32_t hsb[RS];
            v4i pg[RS], pv[RS];
        };
        const int hh = col_ok ? h : 0, hb = col_ok ? hblock : 0;  // clamped: loaded, never used
        auto request = [&](int s, StepLoads &d) {
#pragma unroll
            for (int vv = 0; vv < RS; vv++) {
                const int m = row_at(s * RS / 4, s * RS % 4 + vv);
                const int mm = m < t.end ? m : t.end - 1;
                d.hc[vv] = *(const v2i *)(p.hq + (int64_t)mm * p.ldhq + hh);
                d.hsb[vv] = p.hs[(int64_t)mm * p.ldhs + (hb >> 5)];
                const uint16_t *pp = (const uint16_t *)p.pre + (int64_t)mm * p.ldpre + hh;
                d.pg[vv] = *(const v4i *)pp;
                d.pv[vv] = *(const v4i *)(pp + H);
            }
        };
        constexpr int AHEAD = 1;
        StepLoads buf[AHEAD + 1];
#pragma unroll
        for (int s = 0; s < AHEAD; s++) request(s, buf[s]);
        asm volatile("" ::: "memory");
        float gate_l;
        if (p.gate_f32) {
            gate_l = ((const float *)p.gate)[pair_l];
        } else {
            const uint16_t raw = ((const uint16_t *)p.gate)[pair_l];
            gate_l = CDT == MX_BF16 ? bits2f((uint32_t)raw << 16) : (float)__builtin_bit_cast(_Float16, raw);
        }
#pragma unroll
        for (int s = 0; s < STEPS; s++) {
            if (s + AHEAD < STEPS) request(s + AHEAD, buf[(s + AHEAD) % (AHEAD + 1)]);
            asm volatile("" ::: "memory");
            const StepLoads &d = buf[s % (AHEAD + 1)];
#pragma unroll
            for (int vv = 0; vv < RS; vv++) {
                const int i = s * RS / 4, v = s * RS % 4 + vv;
                const int m = row_at(i, v);
                const bool row_ok = m < t.end;
                const bool ok = row_ok && col_ok;
                const int src = 16 * i + 4 * o_g + v;  // the lane of this wave that holds row (i, g, v)'s metadata
                const int pair = __shfl(pair_l, src, 64);
                const float gate = __shfl(gate_l, src, 64);
                float a[8];
#pragma unroll
                for (int e = 0; e < 8; e++) a[e] = acc[i][e][v];
                float dg[8], dv[8], dot = 0.0f;
                if (ok) {
                    // h read back from its fp8 copy: the forward multiplied those values
                    const float hscale = bits2f(d.hsb[vv] << 23);
                    float gq[8], vq[8];
                    unpack8<CDT>(d.pg[vv], gq);
                    unpack8<CDT>(d.pv[vv], vq);
#pragma unroll
                    for (int e = 0; e < 8; e++) {
                        typedef float v2f __attribute__((ext_vector_type(2)));
                        const int word = d.hc[vv][e >> 2];
                        const v2f pairv = (e & 2) ? __builtin_amdgcn_cvt_pk_f32_fp8(word, true)
                                                  : __builtin_amdgcn_cvt_pk_f32_fp8(word, false);
                        dot += a[e] * pairv[e & 1];  // times the block's power-of-two scale once, below (exact)
                        const float sg = sigmoid_f(gq[e]);
                        const float dhs = a[e] * gate * sg;
                        dg[e] = dhs * vq[e] * (1.0f + gq[e] * (1.0f - sg));
                        dv[e] = dhs * gq[e];
                    }
                    dot *= hscale;
                } else {
#pragma unroll
                    for (int e = 0; e < 8; e++) dg[e] = dv[e] = 0.0f;
                }
                // both halves: store dpre in the storage dtype, quantize from the fp32 values
                const float amax_g = quad_max(amax8(dg));
                const float amax_v = quad_max(amax8(dv));
                const uint32_t bg = scale_byte(amax_g), bv = scale_byte(amax_v);
                const float ig = inv_scale(bg), iv = inv_scale(bv);
                if (ok) {
                    uint32_t w[4], x[4];
                    float tg[8], tv[8];
#pragma unroll
                    for (int e = 0; e < 8; e++) tg[e] = dg[e], tv[e] = dv[e];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        round_pair<CDT>(tg[2 * e], tg[2 * e + 1], w[e]);
                        round_pair<CDT>(tv[2 * e], tv[2 * e + 1], x[e]);
                    }
                    if (p.dpre) {
                        uint16_t *dp = (uint16_t *)p.dpre + (int64_t)m * p.ldpre + h;
                        *(v4i *)dp = v4i{(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
                        *(v4i *)(dp + H) = v4i{(int)x[0], (int)x[1], (int)x[2], (int)x[3]};
                    }
#pragma unroll
                    for (int e = 0; e < 4; e++) keep[0][i][v][e] = w[e], keep[1][i][v][e] = x[e];
                    v2i cg, cv;
                    cg[0] = (int)pack4_e4m3(dg[0] * ig, dg[1] * ig, dg[2] * ig, dg[3] * ig);
                    cg[1] = (int)pack4_e4m3(dg[4] * ig, dg[5] * ig, dg[6] * ig, dg[7] * ig);
                    cv[0] = (int)pack4_e4m3(dv[0] * iv, dv[1] * iv, dv[2] * iv, dv[3] * iv);
                    cv[1] = (int)pack4_e4m3(dv[4] * iv, dv[5] * iv, dv[6] * iv, dv[7] * iv);
                    uint8_t *qp = p.dpq + (int64_t)m * p.lddpq + h;
                    *(v2i *)qp = cg;
                    *(v2i *)(qp + H) = cv;
                    if ((o_r16 & 3) == 0) {
                        uint8_t *sp = p.dps + (int64_t)m * p.lddps + (hblock >> 5);
                        sp[0] = (uint8_t)bg;
                        sp[H >> 5] = (uint8_t)bv;
                    }
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++) keep[0][i][v][e] = keep[1][i][v][e] = 0u;  // padding rows and columns
                }
                // the dot product over the expert width is split across lanes, waves and N tiles
                dot = row16_sum(dot);
                if (row_ok && o_r16 == 0) atomicAdd(p.dgate + pair, dot);
            }
            asm volatile("" ::: "memory");
        }
        if (!tok) return -1;

        __syncthreads();  // every wave is out of the main loop: the stage buffer is free
        const int64_t pbase = __builtin_amdgcn_readfirstlane(t.ppos);
        // Lane-dependent offsets of the passes below are derived from an opaque copy of the lane id.
        // From the plain one they are invariants of the tile loop: the compiler computed them once,
        // could not keep them in registers across the main loop, and reloaded each from scratch
        // memory right before its use behind a full vector-memory wait, which also waited for the
        // pass's previous global store: the stores of a pass went out one round trip at a time
        // (127 reloads per tile; C4: 235 -> 224 us).
#pragma unroll
        for (int pass = 0; pass < 4; pass++) {
            // pass = (gate | value, low | high four of the lane's eight columns); staged column
            // c = 64 wn + 4 r16 + e holds tile column 8 (c / 4) + 4 sub + c % 4
            // The passes alternate between the two halves of the stage buffer (and of the scale
            // area), so one barrier per pass is enough: a half is rewritten two passes later, with
            // the next pass's barrier in between, and a pass's global stores drain under the
            // arithmetic of the next.
            const int half = pass >> 1, sub = pass & 1;
            uint8_t *const codes = (pass & 1) ? lds.b : lds.a;
            uint8_t *const bytes = lds.c + (pass & 1) * ((S::BN / 2) * (S::BM / 32));
#pragma unroll
            for (int blk = 0; blk < S::MT / 2; blk++) {
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    float val[2][4];
                    float cm = 0.0f;
#pragma unroll
                    for (int ii = 0; ii < 2; ii++)
#pragma unroll
                        for (int v = 0; v < 4; v++) {
                            const uint32_t word = keep[half][2 * blk + ii][v][2 * sub + (e >> 1)];
                            val[ii][v] = unpack1<CDT>((e & 1) ? word >> 16 : word & 0xFFFFu);
                            cm = fmaxf(cm, fabsf(val[ii][v]));
                        }
                    // the block's 32 rows are this lane's 8 values and the lanes 16, 32, 48 away
                    cm = fmaxf(cm, __shfl_xor(cm, 16, 64));
                    cm = fmaxf(cm, __shfl_xor(cm, 32, 64));
                    const uint32_t byte = scale_byte(cm);
                    const float inv = inv_scale(byte);
                    const int col = L.wn * (S::WTN / 2) + 4 * o_r16 + e;
#pragma unroll
                    for (int ii = 0; ii < 2; ii++) {
                        const int row = L.wm * S::WTM + 16 * (2 * blk + ii) + 4 * o_g;  // 4 consecutive rows: one dword
                        const uint32_t w = pack4_e4m3(val[ii][0] * inv, val[ii][1] * inv, val[ii][2] * inv, val[ii][3] * inv);
                        // column-major, BM bytes per column, 16-byte chunks XOR-swizzled by the lane's r16
                        *(uint32_t *)(codes + col * S::BM + ((((row >> 4) ^ (col >> 2)) & (CH - 1)) << 4) + (row & 15)) = w;
                    }
                    if (o_g == 0) bytes[col * (S::BM / 32) + L.wm * (S::WTM / 32) + blk] = (uint8_t)byte;
                }
            }
            __syncthreads();
            // CH consecutive lanes write the BM bytes of one column's BM tokens; a 128-row part
            // that starts past the expert's rows belongs to the next expert's padding and is skipped
            static_assert(((S::BN / 2) * S::BM / 16) % S::NTHR == 0, "whole rounds of 16-byte chunks");
#pragma unroll
            for (int k = 0; k < (S::BN / 2) * S::BM / 16 / S::NTHR; k++) {
                const int q = o_tid + k * S::NTHR;
                const int col = q / CH, ch = q % CH;
                const int hcol = t.n0 + 8 * (col >> 2) + 4 * sub + (col & 3);
                const bool part_ok = t.row0 + (ch >> 3) * 128 < t.end;
                if (hcol < H && part_ok) {
                    const v4i w = *(const v4i *)(codes + col * S::BM + (((ch ^ (col >> 2)) & (CH - 1)) << 4));
                    *(v4i *)(p.htq + token_axis_offset(half * H + hcol, pbase, ch)) = w;
                }
            }
            if (o_tid < S::BN / 2) {
                const int hcol = t.n0 + 8 * (o_tid >> 2) + 4 * sub + (o_tid & 3);
                if (hcol < H) {
                    const uint32_t *src = (const uint32_t *)(bytes + o_tid * (S::BM / 32));
                    uint8_t *dst = p.hts + (int64_t)(half * H + hcol) * p.ldhts + (pbase >> 5);
#pragma unroll
                    for (int part = 0; part < S::BM / 128; part++)  // a dword of scale bytes per 128 tokens
                        if (t.row0 + part * 128 < t.end) *(uint32_t *)(dst + 4 * part) = src[part];
                }
            }
        }
        return -1;
    }
};

// ---- combine: out[t] = sum_k scale(t,k) * y[pos(t,k)] ---------------------------------------------
// The scatter-add of the routed rows back to their tokens, as a gather: pair p = t * top_k + k
// sits at sorted position inv[p] (or nowhere: -1, a dropped pair).  One writer per output
// element, fp32 sum in slot order, one rounding: deterministic, and an order of magnitude
// faster than 16-bit atomics for top_k rows per token.
__global__ __launch_bounds__(256) void fill_i32_kernel(int32_t *dst, int64_t n, int32_t value) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = value;
}

__global__ __launch_bounds__(256) void invert_order_kernel(const int32_t *__restrict__ order,
                                                            const int32_t *__restrict__ offsets, int E, int64_t M,
                                                            int64_t pairs, int32_t *__restrict__ inv) {
    const int64_t m = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (m >= M || m >= offsets[E]) return;  // rows past the last expert belong to nobody
    const int64_t p = order[m];
    if (p >= 0 && p < pairs) inv[p] = (int32_t)m;
}

template <int CDT>
__global__ __launch_bounds__(256) void combine_kernel(const uint16_t *__restrict__ y, int64_t ldy,
                                                       const int32_t *__restrict__ inv, const void *__restrict__ gate,
                                                       int gate_f32, int top_k, uint16_t *__restrict__ out, int64_t ldo,
                                                       int64_t T, int N8) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t t = idx / N8;
    const int c = (int)(idx - t * N8) * 8;
    if (t >= T) return;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; e++) acc[e] = 0.0f;
    // Eight slots at a time: their positions and gate factors first, then all their rows, then the sums in slot order.
    // One slot after the other, every slot waited for its position and then for its row: two memory round trips
    // per slot in a kernel that does nothing else (61 -> 47 us for six slots per token at the benchmark's routing).
    for (int k0 = 0; k0 < top_k; k0 += 8) {
        int pos[8];
        float scale[8];
        v4i row[8];
#pragma unroll
        for (int k = 0; k < 8; k++) {
            const int64_t pair = t * top_k + k0 + k;
            pos[k] = k0 + k < top_k ? inv[pair] : -1;
            scale[k] = 1.0f;
            if (gate && k0 + k < top_k) scale[k] = gate_f32 ? ((const float *)gate)[pair] : load_act<CDT>(gate, pair);
        }
#pragma unroll
        for (int k = 0; k < 8; k++)
            if (pos[k] >= 0) row[k] = *(const v4i *)(y + (int64_t)pos[k] * ldy + c);
#pragma unroll
        for (int k = 0; k < 8; k++) {
            if (pos[k] < 0) continue;
            float v[8];
            unpack8<CDT>(row[k], v);
#pragma unroll
            for (int e = 0; e < 8; e++) acc[e] += scale[k] * v[e];
        }
    }
    uint32_t w[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
        float a = acc[2 * e], b = acc[2 * e + 1];
        round_pair<CDT>(a, b, w[e]);
    }
    *(v4i *)(out + t * ldo + c) = v4i{(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
}

// Experts the row-tile tables of a workgroup hold.  Two workgroups share a CU's 160 KB under the 128 x 128 shape: their
// stage buffers take 2 x 73 KB, which leaves room for 512 experts each.
// With the look-ahead the staging area of the scale bytes takes 8 KB more: 760 experts (the host selects it for no more).
template <typename S, bool AHEAD>
constexpr int row_table_max() { return AHEAD ? MX_TABLE_MAX_STAGED : S::BM + S::BN > 256 ? MX_TABLE_MAX : 512; }

template <typename S, int MODE, int CDT, int K512, bool AHEAD = false>
__device__ __forceinline__ void grouped_body(const GroupedArgs &args, uint8_t *smem) {
    constexpr int TMAX = row_table_max<S, AHEAD>();
    __shared__ int table_a[TMAX + 1], table_b[TMAX + 1];
    const bool tabled = args.E <= TMAX;
    if (tabled) build_row_tile_table(table_a, table_b, args.offsets, args.E, S::BM);
    GroupedProblem<S, MODE, CDT> prob(args, tabled ? table_a : nullptr, tabled ? table_b : nullptr);
    persistent_gemm<S, K512, GroupedProblem<S, MODE, CDT>, AHEAD>(prob, smem);
}

template <typename S, int MODE, int CDT, int K512, bool AHEAD = false>
__global__ __launch_bounds__(S::NTHR) void grouped_kernel(GroupedArgs args) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    grouped_body<S, MODE, CDT, K512, AHEAD>(args, smem);
}

#ifdef MX_BENCH_VARIANTS
// The same body on the 128 x 128 tile of four waves (one per SIMD), two workgroups resident per CU, so that one
// workgroup's epilogue can run while the other one's MFMAs do.  The register budget is the one of two waves per SIMD.
template <typename S, int MODE, int CDT, int K512>
__global__ __launch_bounds__(S::NTHR) __attribute__((amdgpu_waves_per_eu(2, 2))) void grouped_pair_kernel(GroupedArgs args) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    grouped_body<S, MODE, CDT, K512>(args, smem);
}
#endif

// Slow path for shapes the tiled kernel does not take (PLAIN only): one thread per output element.
template <int CDT>
__global__ __launch_bounds__(256) void grouped_generic_kernel(GroupedArgs p) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int last = p.offsets[p.E];
    const int64_t m = idx / p.N, n = idx - m * p.N;
    if (m >= last || m >= p.M) return;
    int e = 0;
    while (e + 1 < p.E && p.offsets[e + 1] <= m) e++;
    const int64_t src = p.index ? p.index[m] : m;
    const uint8_t *pa = p.xq + src * p.ldx, *pb = p.wq + e * p.stride_we + n * p.ldw;
    const uint8_t *sa = p.xs + src * p.ldxs, *sb = p.ws + e * p.stride_wse + n * p.ldws;
    float acc = 0.0f;
    for (int kb = 0; kb < p.K / MX_BLOCK; kb++) {
        float part = 0.0f;
        for (int i = 0; i < MX_BLOCK; i += 2) {
            typedef float v2f __attribute__((ext_vector_type(2)));
            uint32_t wa = pa[kb * MX_BLOCK + i] | ((uint32_t)pa[kb * MX_BLOCK + i + 1] << 8);
            uint32_t wb = pb[kb * MX_BLOCK + i] | ((uint32_t)pb[kb * MX_BLOCK + i + 1] << 8);
            v2f fa = __builtin_amdgcn_cvt_pk_f32_fp8((int)wa, false);
            v2f fb = __builtin_amdgcn_cvt_pk_f32_fp8((int)wb, false);
            part += fa[0] * fb[0] + fa[1] * fb[1];
        }
        acc += ldexpf(part, (int)sa[kb] + (int)sb[kb] - 254);
    }
    if (CDT == MX_FP32) ((float *)p.out)[m * p.ldo + n] = acc;
    else if (CDT == MX_BF16) ((uint16_t *)p.out)[m * p.ldo + n] = (uint16_t)f2bf16(acc);
    else ((_Float16 *)p.out)[m * p.ldo + n] = (_Float16)acc;
}

// ---- grouped WGRAD: dW[e] (N,Kout) = AT[:, seg(e)] . BT[:, seg(e)]^T ------------------------------
// AT (N, Mpad) and BT (Kout, Mpad) are the token-axis quantizations written by
// mx_quantize_cols_grouped: expert e owns the padded positions of its 128-row tiles, i.e. K
// stages [tiles_before(e), tiles_before(e) + tiles(e)).  One writer per element; an expert
// with no rows gets zeros (grouped.py:152-247 of the reference has the same contract).
struct WgradArgs {
    const uint8_t *aq, *as, *bq, *bs;
    int64_t lda, ldas, ldb, ldbs;
    // Stage-major code matrices (0: row-major): the 128 positions of K stage kt of every row lie together, stage kt at
    // kt * a_ks, row r of it at r * 128 (lda is 128 then), so a tile's stage is one contiguous run; b_ks likewise.
    int64_t a_ks, b_ks;
    void *dw;
    int64_t stride_dwe, lddw;
    const int32_t *offsets;
    int E, N, Kout, KB;  // KB: scale bytes per row of the padded space
    int tiles_m, tiles_n, c_vec;
    // K split for few, long tiles (a handful of busy experts): `slots` fp32 tile slots; every
    // workgroup derives the same number of K slices per tile from the offsets (wgrad_slices),
    // slice s of the j-th tile of a non-empty expert leaves its partial sum in slot j * slices + s,
    // and wgrad_reduce_kernel adds the slices in order.  slots == 0: whole tiles only.
    float *ws;
    int slots;
};

// Even K split (needs the LDS table of the experts with rows).  The K stages of those experts,
// laid end to end, are cut into G / tiles_per_expert equal ranges of `q` stages; a group of
// tiles_per_expert workgroups, one per output tile, takes each range.  A range that covers an
// expert's stages only in part leaves fp32 partial sums: at most two per workgroup (the end of
// an expert an earlier group began, the beginning of one a later group ends), in slots 2 u and
// 2 u + 1 of workgroup-unit u, and wgrad_reduce_kernel adds an expert's pieces in group order.
// Every workgroup works one range of equal length, where whole K slices left a ragged second
// round and one fp32 partial tile per slice (measured at six busy experts of 16384 rows:
// 480 partial tiles and two rounds against 336 and one).
struct WgradEven {
    int per_e, groups, q, total;
};

template <typename TB>
__device__ __forceinline__ WgradEven wgrad_even_plan(const WgradArgs &p, int workgroups, const TB &tb) {
    WgradEven v;
    v.per_e = p.tiles_m * p.tiles_n;
    v.groups = workgroups / v.per_e;  // > 0: the split is only chosen when the tiles leave workgroups idle
    v.total = tb.b[tb.n];
    v.q = (v.total + v.groups - 1) / v.groups;
    return v;
}

// The workgroups of one XCD (b % 8) take consecutive unit numbers, so that the tiles of one
// (expert, K range), which read the same operand panels, share that XCD's L2.
__device__ __forceinline__ int wgrad_unit_of(int b, int g) { return (g & 7) == 0 ? (b & 7) * (g >> 3) + (b >> 3) : b; }

// Number of K slices per tile: as many as fill the GPU about twice over, at most 8, and 1 when
// the tiles of the non-empty experts already fill three quarters of it.  Also counts the
// non-empty experts.  (With the table, any result above 1 selects the even split.)
template <typename TB>
__device__ __forceinline__ int wgrad_slices(const WgradArgs &p, int workgroups, int &live, const TB *tb) {
    if (tb) {
        live = tb->n;
    } else {
        live = 0;
        for (int e = 0; e < p.E; e++) live += p.offsets[e + 1] > p.offsets[e] ? 1 : 0;
    }
    const int per_e = p.tiles_m * p.tiles_n;
    const int tiles = live * per_e;
    if (!p.slots || tiles == 0) return 1;
    if (tiles * 4 >= workgroups * 3) {
        // Plenty of tiles: dealt whole and round-robin they balance, unless a few experts hold most of the
        // rows -- then one workgroup's tile is as long as `longest` K stages while the average workgroup has
        // total * per_e / workgroups to do, and the launch lasts as long as that one tile.  Routed loads
        // follow a power law, so this is the usual case: split evenly when the longest tile is more than
        // twice the average load (the split costs each workgroup up to two fp32 partial tiles).
        if (!tb || workgroups < per_e) return 1;
        return (int64_t)tb->longest * workgroups > 2 * (int64_t)tb->b[tb->n] * per_e ? 2 : 1;
    }
    int s = 2 * workgroups / tiles;
    s = s < p.slots / tiles ? s : p.slots / tiles;
    return s < 1 ? 1 : (s > 8 ? 8 : s);
}

template <typename S, int CDT, typename TB = ExpertTable>
struct WgradProblem {
    struct Tile {
        int m0, n0, kt0, kt1, expert;
        int slot;  // fp32 scratch slot of this K slice, or -1 for a whole tile
    };
    const WgradArgs p;
    // Units are dealt round-robin over the workgroups: the (tile, K slice) units of the non-empty
    // experts, compactly numbered so they spread evenly wherever those experts sit among the E.
    // (The dW of an expert without rows is zero-filled by wgrad_zero_kernel, launched first.)
    int next_unit, kb_end;
    int live, slices;
    // incremental scan: expert scan_e is the scan_live-th non-empty one and its first K stage
    // is scan_tiles
    int scan_e, scan_tiles, scan_live;
    // even K split: this workgroup's unit number, its remaining range of K stages, the split's plan
    bool even;
    int unit, pos, end;
    WgradEven ev;
    static constexpr int NST = S::MT * 4 * (CDT == MX_FP32 ? 2 : 1);
    static constexpr bool EARLY_WAIT = false;
    // an expert of up to 128 rows is one K stage, and so is the end of a range of the even split: see persistent_gemm
    static constexpr bool SHORT_TILES = true;

    // Workgroups are dealt to the 8 XCDs round-robin, so workgroup b starts at unit
    // (b % 8) * (G / 8) + b / 8: the workgroups of one XCD take consecutive units, i.e. the tiles
    // of one (expert, K slice), which read the same operand panels, share that XCD's L2 (measured:
    // the kernel's fabric reads equal the operand bytes).
    const TB *tb;  // the experts with rows, in LDS, or nullptr (more experts than it holds)

    __device__ WgradProblem(const WgradArgs &a, const TB *table)
        : p(a), kb_end(a.KB), scan_e(0), scan_tiles(0), scan_live(0), tb(table) {
        const int g = (int)gridDim.x, b = (int)blockIdx.x;
        next_unit = wgrad_unit_of(b, g);
        slices = wgrad_slices(p, g, live, tb);
        even = tb && slices > 1;
        if (even) {
            ev = wgrad_even_plan(p, g, *tb);
            unit = next_unit;
            const int grp = unit / ev.per_e;
            pos = grp < ev.groups ? grp * ev.q : ev.total;
            pos = pos < ev.total ? pos : ev.total;
            end = pos + ev.q < ev.total ? pos + ev.q : ev.total;
        }
    }

    __device__ __forceinline__ void zero_slot(int slot) const {
        v4f *dst = (v4f *)p.ws + (int64_t)slot * (S::BM * S::BN / 4);
        for (int idx = threadIdx.x; idx < S::BM * S::BN / 4; idx += S::NTHR) dst[idx] = v4f{0.f, 0.f, 0.f, 0.f};
    }

    __device__ __forceinline__ bool next(Tile &t) {
        const int per_e = p.tiles_m * p.tiles_n;
        if (even) {
            if (pos >= end) return false;
            // the expert whose K stages hold `pos`: the last j with b[j] <= pos
            int lo = 0, hi = tb->n - 1;
            while (lo < hi) {
                const int mid = (lo + hi + 1) >> 1;
                if (tb->b[mid] <= pos) lo = mid;
                else hi = mid - 1;
            }
            const int first = tb->b[lo], past = tb->b[lo + 1];
            const int rem = unit % per_e;
            t.expert = tb->a[lo];
            t.m0 = (rem / p.tiles_n) * S::BM;
            t.n0 = (rem % p.tiles_n) * S::BN;
            t.kt0 = pos;
            t.kt1 = end < past ? end : past;
            t.slot = (t.kt0 == first && t.kt1 == past) ? -1 : 2 * unit + (t.kt0 > first ? 0 : 1);
            pos = t.kt1;
            return true;
        }
        const int per_live = per_e * slices;
        while (next_unit < live * per_live) {
            const int unit = next_unit;
            next_unit += gridDim.x;
            const int j = unit / per_live, r = unit - j * per_live;
            const int slice = r / per_e, rem = r - slice * per_e;  // slice-major: neighbours share operand panels
            // advance to the j-th non-empty expert (units, hence j, only grow for one workgroup)
            if (tb) {
                scan_e = tb->a[j];
                scan_tiles = tb->b[j];
            } else while (true) {
                const int rows = p.offsets[scan_e + 1] - p.offsets[scan_e];
                if (rows > 0 && scan_live == j) break;
                scan_tiles += (rows + 127) / 128;
                scan_live += rows > 0 ? 1 : 0;
                scan_e++;
            }
            t.expert = scan_e;
            t.m0 = (rem / p.tiles_n) * S::BM;
            t.n0 = (rem % p.tiles_n) * S::BN;
            const int len = (p.offsets[scan_e + 1] - p.offsets[scan_e] + 127) / 128;
            const int per = (len + slices - 1) / slices;
            const int lo = slice * per < len ? slice * per : len;
            const int hi = lo + per < len ? lo + per : len;
            t.kt0 = scan_tiles + lo;
            t.kt1 = scan_tiles + hi;
            t.slot = slices > 1 ? (j * per_e + rem) * slices + slice : -1;
            if (lo == hi) {
                zero_slot(t.slot);  // only a slice can be empty: a whole tile of a non-empty expert has K stages
                continue;
            }
            return true;
        }
        return false;
    }

    __device__ __forceinline__ void context(const Tile &t, const Lane &L0, IssueCtx<S> &c) const {
        const Lane L = opaque(L0);
        c.a_base = p.aq + (int64_t)t.m0 * p.lda;
        c.b_base = p.bq + (int64_t)t.n0 * p.ldb;
        c.kt0 = t.kt0;
        c.kt1 = t.kt1;
        c.tail_kt = -1, c.tail_bytes = 0;  // K % 128 == 0 is a precondition of these kernels
        c.a_ks = p.a_ks ? p.a_ks : 128;
        c.b_ks = p.b_ks ? p.b_ks : 128;
        const int mrem = p.N - t.m0, nrem = p.Kout - t.n0;
#pragma unroll
        for (int q = 0; q < S::QA; q++) {
            const int row = dma_row<S>(L, q);
            c.a_voff[q] = (uint32_t)((int64_t)(row < mrem ? row : mrem - 1) * p.lda) + (((L.lane & 7) ^ swz_a(row)) << 4) + copy_bias(q);
        }
#pragma unroll
        for (int q = 0; q < S::QB; q++) {
            const int row = dma_row<S>(L, q);
            const int brow = b_row_of_lds<S>(row);
            c.b_voff[q] = (uint32_t)((int64_t)(brow < nrem ? brow : nrem - 1) * p.ldb) + (((L.lane & 7) ^ swz_a(row)) << 4) + copy_bias(q);
        }
        auto srow = [&](int r) -> const uint8_t * {
            if (r < S::BM) return p.as + (int64_t)(t.m0 + (r < mrem ? r : mrem - 1)) * p.ldas;
            r = b_row_of_lds<S>(r - S::BM);
            return p.bs + (int64_t)(t.n0 + (r < nrem ? r : nrem - 1)) * p.ldbs;
        };
        c.srow0 = srow(L.tid < S::BM + S::BN ? L.tid : 0);
        c.srow1 = S::TWO_ROWS ? srow(L.tid + S::NTHR < S::BM + S::BN ? L.tid + S::NTHR : 0) : nullptr;
        // SCALES_COPY: the same row through the copy engine, as a 32-bit offset from its matrix
        c.sa_base = p.as, c.sb_base = p.bs;
        c.s_voff = (uint32_t)(c.srow0 - (L.tid < S::BM ? p.as : p.bs));
    }

    __device__ __forceinline__ int epilogue(const Tile &t, const Lane &L0, v4f (&acc)[S::MT][S::NT], const LdsScratch &) const {
        const Lane L = rebuilt<S>(L0);  // no per-lane address of the epilogue lives across the K loop
        if (t.slot >= 0) {  // one K slice: fp32 partial, laid out [sub-tile][thread]
            v4f *dst = (v4f *)p.ws + (int64_t)t.slot * (S::BM * S::BN / 4);
#pragma unroll
            for (int i = 0; i < S::MT; i++)
#pragma unroll
                for (int j = 0; j < S::NT; j++) dst[(i * S::NT + j) * S::NTHR + L.tid] = acc[i][j];
            return -1;
        }
        const bool interior = t.m0 + S::BM <= p.N && t.n0 + S::BN <= p.Kout && p.c_vec;
        const int64_t base = (int64_t)t.expert * p.stride_dwe;
        const int n = t.n0 + L.wn * S::WTN + 8 * L.r16;
#pragma unroll
        for (int i = 0; i < S::MT; i++) {
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int m = t.m0 + L.wm * S::WTM + 16 * i + 4 * L.g + v;
                const int64_t off = base + (int64_t)m * p.lddw + n;
                const v4f lo = {acc[i][0][v], acc[i][1][v], acc[i][2][v], acc[i][3][v]};
                const v4f hi = {acc[i][4][v], acc[i][5][v], acc[i][6][v], acc[i][7][v]};
                if (interior) store8<CDT>(p.dw, off, lo, hi, 8, true);
                else if (m < p.N && n < p.Kout) store8<CDT>(p.dw, off, lo, hi, p.Kout - n < 8 ? p.Kout - n : 8, p.c_vec != 0);
            }
        }
        return interior ? NST : -1;
    }
};

// dW of the experts without rows: zeros.  A plain streaming fill, launched ahead of the GEMM.  (As
// part of it, in one burst, the fills of 58 empty experts cost three times what they cost here: vector
// memory operations retire in order, so the first stage's wait for its copies waits for every store
// issued before them.  Spread over the K stages, a few stores per thread in front of each stage's
// copies, they cost the GEMM exactly the 14 us the separate launch takes.)  One block per (expert, 64 rows).
template <int CDT>
__global__ __launch_bounds__(256) void wgrad_zero_kernel(WgradArgs p, int chunks) {
    const int e = blockIdx.x / chunks, m0 = (blockIdx.x % chunks) * 64;
    if (p.offsets[e + 1] > p.offsets[e]) return;
    const int esz = CDT == MX_FP32 ? 4 : 2;
    char *base = (char *)p.dw + ((int64_t)e * p.stride_dwe + (int64_t)m0 * p.lddw) * esz;
    const int rows = p.N - m0 < 64 ? p.N - m0 : 64;
    if (p.c_vec && (p.Kout * esz) % 16 == 0) {
        const int per_row = p.Kout * esz / 16;
        for (int idx = threadIdx.x; idx < rows * per_row; idx += 256) {
            const int m = idx / per_row, c = idx - m * per_row;
            *(v4i *)(base + (int64_t)m * p.lddw * esz + c * 16) = v4i{0, 0, 0, 0};
        }
        return;
    }
    for (int idx = threadIdx.x; idx < rows * p.Kout; idx += 256) {
        const int m = idx / p.Kout, n = idx - m * p.Kout;
        char *dst = base + ((int64_t)m * p.lddw + n) * esz;
        if (esz == 4) *(float *)dst = 0.0f;
        else *(uint16_t *)dst = 0;
    }
}

template <typename S, int CDT, int SCALES>
__global__ __launch_bounds__(S::NTHR) void grouped_wgrad_kernel(WgradArgs args) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    // SCALES_COPY (the host selects it only for E <= MX_TABLE_MAX_STAGED): the smaller table beside the staging area
    typedef typename std::conditional<SCALES == SCALES_COPY, ExpertTableStaged, ExpertTable>::type TB;
    __shared__ TB table;
    const bool tabled = args.E <= TB::CAPACITY;
    if (tabled) build_live_table(table, args.offsets, args.E);
    WgradProblem<S, CDT, TB> prob(args, tabled ? &table : nullptr);
    // with the staged scale bytes goes the A look-ahead of the dense kernels (its K loop then holds no vector load)
    persistent_gemm<S, SCALES, WgradProblem<S, CDT, TB>, SCALES == SCALES_COPY>(prob, smem);
}

// Adds the K slices of every tile of every non-empty expert, in slice order, and stores dW.
// One unit per (tile of a non-empty expert, i), numbered compactly as in the GEMM; the host does
// not know how many experts have rows, so a fixed number of workgroups stride over the units
// (none when the GEMM kept its tiles whole).
template <typename S, int CDT>
__global__ __launch_bounds__(S::NTHR) void wgrad_reduce_kernel(WgradArgs p, int workgroups) {
    __shared__ ExpertTable table;
    const bool tabled = p.E <= MX_TABLE_MAX;
    if (tabled) build_live_table(table, p.offsets, p.E);
    int live;
    const int slices = wgrad_slices(p, workgroups, live, tabled ? &table : nullptr);
    if (slices == 1) return;
    const int per_e = p.tiles_m * p.tiles_n;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int wm = wave / S::WGN, wn = wave % S::WGN;
    for (int unit = blockIdx.x; unit < live * per_e * S::MT; unit += gridDim.x) {
        const int id = unit / S::MT, i = unit % S::MT;
        const int j = id / per_e, rem = id - j * per_e;
        int e = 0;
        if (tabled) {
            e = table.a[j];
        } else {
            for (int seen = 0;; e++) {
                if (p.offsets[e + 1] > p.offsets[e]) {
                    if (seen == j) break;
                    seen++;
                }
            }
        }
        v4f sum[S::NT];
#pragma unroll
        for (int jj = 0; jj < S::NT; jj++) sum[jj] = v4f{0.f, 0.f, 0.f, 0.f};
        if (tabled) {  // even K split: the pieces of the groups whose ranges meet this expert's stages
            const WgradEven ev = wgrad_even_plan(p, workgroups, table);
            const int g_lo = table.b[j] / ev.q, g_hi = (table.b[j + 1] - 1) / ev.q;
            if (g_lo == g_hi) continue;  // one group had all of it and stored the tile itself
            for (int g = g_lo; g <= g_hi; g++) {
                const int slot = 2 * (g * per_e + rem) + (g == g_lo ? 1 : 0);
                const v4f *src = (const v4f *)p.ws + (int64_t)slot * (S::BM * S::BN / 4);
#pragma unroll
                for (int jj = 0; jj < S::NT; jj++) sum[jj] += src[(i * S::NT + jj) * S::NTHR + tid];
            }
        } else {
            for (int sl = 0; sl < slices; sl++) {
                const v4f *src = (const v4f *)p.ws + (int64_t)((j * per_e + rem) * slices + sl) * (S::BM * S::BN / 4);
#pragma unroll
                for (int jj = 0; jj < S::NT; jj++) sum[jj] += src[(i * S::NT + jj) * S::NTHR + tid];
            }
        }
        const int n = (rem % p.tiles_n) * S::BN + wn * S::WTN + 8 * (lane & 15);
#pragma unroll
        for (int v = 0; v < 4; v++) {
            const int m = (rem / p.tiles_n) * S::BM + wm * S::WTM + 16 * i + 4 * (lane >> 4) + v;
            if (m < p.N && n < p.Kout) {
                const v4f lo = {sum[0][v], sum[1][v], sum[2][v], sum[3][v]};
                const v4f hi = {sum[4][v], sum[5][v], sum[6][v], sum[7][v]};
                store8<CDT>(p.dw, (int64_t)e * p.stride_dwe + (int64_t)m * p.lddw + n, lo, hi, p.Kout - n < 8 ? p.Kout - n : 8,
                            p.c_vec != 0);
            }
        }
    }
}

}  // namespace mx

using namespace mx;

static inline bool aligned(const void *p, uintptr_t a) { return ((uintptr_t)p & (a - 1)) == 0; }

// 256 x 256 x 128 tile, 8 waves as 4 (M) x 2 (N): a wave owns 64 x 128, a lane 8 consecutive N.
typedef GemmShape<256, 256, 4, 2> Big;

static bool tiled_ok(const GroupedArgs &a, int64_t a_rows) {
    return a.K % 128 == 0 && aligned(a.xq, 16) && aligned(a.wq, 16) && a.ldx % 16 == 0 && a.ldw % 16 == 0 &&
           a.stride_we % 16 == 0 && aligned(a.xs, 4) && aligned(a.ws, 4) && a.ldxs % 4 == 0 && a.ldws % 4 == 0 &&
           a.stride_wse % 4 == 0 && a_rows * a.ldx < ((int64_t)1 << 32) && (int64_t)a.N * 2 * a.ldw < ((int64_t)1 << 32);
}

// 128 x 128 x 128 tile, 4 waves as 4 (M) x 1 (N), one per SIMD: a wave owns 32 x 128 -- the same eight consecutive N per
// lane as under Big, so the fused epilogues' column logic is shared -- and two workgroups fit a CU (2 x 73 KB of LDS,
// 256 registers per lane each).  Twice the operand bytes per flop of Big: for the fused expert epilogues only, whose
// vector ALU work dwarfs their short K loops.
typedef GemmShape<128, 128, 4, 1> Slim;

// Built into the variants library only (-DMX_BENCH_VARIANTS), where it replaces Big for the two fused expert kernels:
// bit-identical outputs, measured slower at the benchmark's routing (GEMM1 148 -> 185 us, GEMM2-dgrad 192 -> 209 us).
// The eight waves of a CU issue the same vector ALU work either way, and the K loops of a 128 x 128 tile, whose copies
// must land within a stage of 512 MFMA clocks, cost more than their overlap with the other workgroup's epilogue returns.
#ifdef MX_BENCH_VARIANTS
#define MX_EXPERT_SLIM 1
#else
#define MX_EXPERT_SLIM 0
#endif

template <typename S, int MODE, int CDT>
static int launch_grouped_shape(GroupedArgs a, hipStream_t st) {
    constexpr int npt = MODE == MODE_GEMM1 ? S::BN / 2 : S::BN;
    constexpr bool pair = S::NW == 4;  // two workgroups per CU
    a.tiles_n = (a.N + npt - 1) / npt;
    a.tbound = (a.M + S::BM - 1) / S::BM + a.E;
    const int64_t work = (int64_t)a.tiles_n * a.tbound;
    if (work >= 0x7FFFFFFF) return MX_EUNSUPPORTED;
    const bool k512 = a.K % 512 == 0 && aligned(a.xs, 16) && aligned(a.ws, 16) && a.ldxs % 16 == 0 &&
                      a.ldws % 16 == 0 && a.stride_wse % 16 == 0;
    const int wgs = num_cus() * (pair ? 2 : 1);
    dim3 grid((unsigned)(work < wgs ? work : wgs)), block(S::NTHR);
    int rc;
#ifdef MX_BENCH_VARIANTS
    if constexpr (pair)
        rc = k512 ? launch_with_lds<grouped_pair_kernel<S, MODE, CDT, SCALES_VEC16>>(grid, block, S::LDS_BYTES, st, a)
                  : launch_with_lds<grouped_pair_kernel<S, MODE, CDT, SCALES_DWORD>>(grid, block, S::LDS_BYTES, st, a);
    else
#endif
    {
        // The plain product on whole 512s of K (every tile then has four stages or more): the A operand two stages ahead
        // and scale bytes through the copy engine (32-bit lane offsets: both scale matrices under 4 GB), as the dense
        // kernels; 90 -> 81 us and 132 -> 120 us on 98304 routed rows at K = 512 and 1024.
        bool ahead = false;
        if constexpr (MODE == MODE_PLAIN && !pair)
            ahead = k512 && a.E <= MX_TABLE_MAX_STAGED && a.x_rows > 0 && a.x_rows * a.ldxs < ((int64_t)1 << 32) &&
                    ((int64_t)a.E - 1) * a.stride_wse + (int64_t)a.N * a.ldws < ((int64_t)1 << 32);
        if constexpr (MODE == MODE_PLAIN && !pair) {
            if (ahead) rc = launch_with_lds<grouped_kernel<S, MODE, CDT, SCALES_COPY, true>>(grid, block, S::LDS_BYTES_AHEAD, st, a);
        }
        if (!ahead)
            rc = k512 ? launch_with_lds<grouped_kernel<S, MODE, CDT, SCALES_VEC16>>(grid, block, S::LDS_BYTES, st, a)
                      : launch_with_lds<grouped_kernel<S, MODE, CDT, SCALES_DWORD>>(grid, block, S::LDS_BYTES, st, a);
    }
    if (rc != MX_OK) return rc;
    return hipGetLastError() == hipSuccess ? MX_OK : MX_ELAUNCH;
}

template <int MODE, int CDT>
static int launch_grouped(const GroupedArgs &a, hipStream_t st) {
    if constexpr (MX_EXPERT_SLIM && (MODE == MODE_GEMM1 || MODE == MODE_DGRAD2)) return launch_grouped_shape<Slim, MODE, CDT>(a, st);
    else return launch_grouped_shape<Big, MODE, CDT>(a, st);
}

template <int MODE>
static int launch_grouped_dt(int dt, const GroupedArgs &a, hipStream_t st) {
    switch (dt) {
    case MX_BF16: return launch_grouped<MODE, MX_BF16>(a, st);
    case MX_FP16: return launch_grouped<MODE, MX_FP16>(a, st);
    default: return MX_EINVAL;
    }
}

static GroupedArgs base_args(const uint8_t *xq, const uint8_t *xs, int64_t ldx, int64_t ldxs, const int32_t *index,
                             const uint8_t *wq, const uint8_t *ws, int64_t stride_we, int64_t ldw, int64_t stride_wse,
                             int64_t ldws, const int32_t *offsets, int64_t E, int64_t M, int64_t N, int64_t K) {
    GroupedArgs a = {};
    a.xq = xq, a.xs = xs, a.ldx = ldx, a.ldxs = ldxs, a.index = index;
    a.wq = wq, a.ws = ws, a.stride_we = stride_we, a.ldw = ldw, a.stride_wse = stride_wse, a.ldws = ldws;
    a.offsets = offsets, a.E = (int)E, a.M = (int)M, a.N = (int)N, a.K = (int)K;
    return a;
}

static bool sizes_ok(int64_t E, int64_t M, int64_t N, int64_t K) {
    return E > 0 && E < (1 << 20) && M >= 0 && M < 0x7FFFFFFF && N >= 0 && N < 0x7FFFFFFF && K >= 0 && K < 0x7FFFFFFF &&
           K % MX_BLOCK == 0;
}

extern "C" int mx_grouped_gemm_nt(const uint8_t *xq, const uint8_t *xs, int64_t a_rows, int64_t ldx, int64_t ldxs,
                                  const int32_t *index, const uint8_t *wq, const uint8_t *ws, int64_t stride_we,
                                  int64_t ldw, int64_t stride_wse, int64_t ldws, const int32_t *offsets, int64_t E,
                                  void *out, int out_dtype, int64_t ldo, int64_t M, int64_t N, int64_t K, void *stream) {
    if (!sizes_ok(E, M, N, K) || ldx < K || ldw < K || ldo < N) return MX_EINVAL;
    if (M == 0 || N == 0) return MX_OK;
    hipStream_t st = (hipStream_t)stream;
    if (mx::stream_is_capturing(st)) return MX_ECAPTURE;
    GroupedArgs a = base_args(xq, xs, ldx, ldxs, index, wq, ws, stride_we, ldw, stride_wse, ldws, offsets, E, M, N, K);
    a.out = out, a.ldo = ldo, a.x_rows = a_rows;
    const int esz = out_dtype == MX_FP32 ? 4 : 2;
    a.out_vec = aligned(out, 16) && (ldo * esz) % 16 == 0;
    if (K == 0 || !tiled_ok(a, a_rows)) {
        if (K == 0) return MX_EUNSUPPORTED;
        int64_t blocks = (M * N + 255) / 256;
        if (blocks > 0x7FFFFFFF) return MX_EUNSUPPORTED;
        switch (out_dtype) {
        case MX_BF16: grouped_generic_kernel<MX_BF16><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(a); break;
        case MX_FP16: grouped_generic_kernel<MX_FP16><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(a); break;
        case MX_FP32: grouped_generic_kernel<MX_FP32><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(a); break;
        default: return MX_EINVAL;
        }
        return hipGetLastError() == hipSuccess ? MX_OK : MX_ELAUNCH;
    }
    switch (out_dtype) {
    case MX_BF16: return launch_grouped<MODE_PLAIN, MX_BF16>(a, st);
    case MX_FP16: return launch_grouped<MODE_PLAIN, MX_FP16>(a, st);
    case MX_FP32: return launch_grouped<MODE_PLAIN, MX_FP32>(a, st);
    default: return MX_EINVAL;
    }
}

extern "C" int mx_experts_gemm1(const uint8_t *xq, const uint8_t *xs, int64_t T, int64_t ldx, int64_t ldxs,
                                const int32_t *token_of, const uint8_t *wq, const uint8_t *ws, int64_t stride_we,
                                int64_t ldw, int64_t stride_wse, int64_t ldws, const int32_t *offsets, int64_t E,
                                uint8_t *hq, int64_t ldhq, uint8_t *hs, int64_t ldhs, void *pre, int64_t ldpre,
                                uint8_t *htq, int64_t ldhtq, uint8_t *hts, int64_t ldhts, int act_dtype, int64_t M,
                                int64_t H, int64_t K, void *stream) {
    if (!sizes_ok(E, M, H, K) || H % MX_BLOCK || ldx < K || ldw < K || ldhq < H || ldhs < H / MX_BLOCK ||
        (pre && ldpre < 2 * H) || (htq != nullptr) != (hts != nullptr))
        return MX_EINVAL;
    const int64_t mpad = ((M + 127) / 128 + E) * 128;
    // a leading dimension of exactly 128 on a wider padded axis: htq stage-major, (Mpad/128, H, 128)
    const bool t_panels = htq && ldhtq == 128 && mpad > 128;
    if (htq && ((ldhtq < mpad - 128 * E && !t_panels) || ldhts < (mpad - 128 * E) / MX_BLOCK)) return MX_EINVAL;
    if (M == 0 || H == 0) return MX_OK;
    GroupedArgs a = base_args(xq, xs, ldx, ldxs, token_of, wq, ws, stride_we, ldw, stride_wse, ldws, offsets, E, M, H, K);
    a.hq = hq, a.ldhq = ldhq, a.hs = hs, a.ldhs = ldhs, a.pre = pre, a.ldpre = ldpre;
    a.htq = htq, a.ldhtq = ldhtq, a.hts = hts, a.ldhts = ldhts, a.htq_ks = t_panels ? H * 128 : 0;
    if (K == 0 || !tiled_ok(a, T) || !aligned(hq, 8) || ldhq % 8 || (pre && (!aligned(pre, 8) || ldpre % 4)) ||
        (htq && (!aligned(htq, 16) || ldhtq % 16 || !aligned(hts, 4) || ldhts % 4)))
        return MX_EUNSUPPORTED;
    if (mx::stream_is_capturing((hipStream_t)stream)) return MX_ECAPTURE;
    return launch_grouped_dt<MODE_GEMM1>(act_dtype, a, (hipStream_t)stream);
}

extern "C" int mx_experts_scatter_gemm(const uint8_t *aq, const uint8_t *as, int64_t a_rows, int64_t lda, int64_t ldas,
                                       const int32_t *index, const uint8_t *wq, const uint8_t *ws, int64_t stride_we,
                                       int64_t ldw, int64_t stride_wse, int64_t ldws, const int32_t *offsets,
                                       int64_t E, const int32_t *token_of, const int32_t *order, const void *gate,
                                       int gate_dtype, void *out, int out_dtype, int64_t ldo, int64_t M, int64_t N,
                                       int64_t K, void *stream) {
    if (!sizes_ok(E, M, N, K) || N % 2 || lda < K || ldw < K || ldo < N || !token_of || (gate && !order)) return MX_EINVAL;
    if (gate && gate_dtype != MX_FP32 && gate_dtype != out_dtype) return MX_EINVAL;
    if (M == 0 || N == 0) return MX_OK;
    GroupedArgs a = base_args(aq, as, lda, ldas, index, wq, ws, stride_we, ldw, stride_wse, ldws, offsets, E, M, N, K);
    a.token_of = token_of, a.order = order, a.gate = gate, a.gate_f32 = gate_dtype == MX_FP32;
    a.out = out, a.ldo = ldo;
    if (K == 0 || !tiled_ok(a, a_rows) || !aligned(out, 4) || ldo % 2) return MX_EUNSUPPORTED;
    if (mx::stream_is_capturing((hipStream_t)stream)) return MX_ECAPTURE;
    return launch_grouped_dt<MODE_SCATTER>(out_dtype, a, (hipStream_t)stream);
}

extern "C" int mx_experts_gemm2_dgrad(const uint8_t *dq, const uint8_t *ds, int64_t T, int64_t lddq, int64_t ldds,
                                      const int32_t *token_of, const int32_t *order, const void *gate, int gate_dtype,
                                      const uint8_t *wq, const uint8_t *ws, int64_t stride_we, int64_t ldw,
                                      int64_t stride_wse, int64_t ldws, const int32_t *offsets, int64_t E,
                                      const uint8_t *hq, int64_t ldhq, const uint8_t *hs, int64_t ldhs, const void *pre,
                                      void *dpre, int64_t ldpre, uint8_t *dpq, int64_t lddpq, uint8_t *dps,
                                      int64_t lddps, uint8_t *ptq, int64_t ldptq, uint8_t *pts, int64_t ldpts,
                                      float *dgate, int act_dtype, int64_t M, int64_t H, int64_t K, void *stream) {
    if (!sizes_ok(E, M, H, K) || H % MX_BLOCK || lddq < K || ldw < K || ldhq < H || ldpre < 2 * H || lddpq < 2 * H ||
        lddps < 2 * H / MX_BLOCK || !token_of || !order || !gate || !pre || !dgate || (!dpre && !ptq) ||
        (ptq != nullptr) != (pts != nullptr))
        return MX_EINVAL;
    if (gate_dtype != MX_FP32 && gate_dtype != act_dtype) return MX_EINVAL;
    const int64_t mpad = ((M + 127) / 128 + E) * 128;
    // a leading dimension of exactly 128 on a wider padded axis: ptq stage-major, (Mpad/128, 2H, 128)
    const bool t_panels = ptq && ldptq == 128 && mpad > 128;
    if (ptq && ((ldptq < mpad - 128 * E && !t_panels) || ldpts < (mpad - 128 * E) / MX_BLOCK)) return MX_EINVAL;
    if (M == 0 || H == 0) return MX_OK;
    GroupedArgs a = base_args(dq, ds, lddq, ldds, token_of, wq, ws, stride_we, ldw, stride_wse, ldws, offsets, E, M, H, K);
    a.token_of = token_of, a.order = order, a.gate = gate, a.gate_f32 = gate_dtype == MX_FP32;
    a.hq = (uint8_t *)hq, a.ldhq = ldhq, a.hs = (uint8_t *)hs, a.ldhs = ldhs;
    a.pre = (void *)pre, a.dpre = dpre, a.ldpre = ldpre, a.dpq = dpq, a.lddpq = lddpq, a.dps = dps, a.lddps = lddps;
    a.dgate = dgate;
    a.htq = ptq, a.ldhtq = ldptq, a.hts = pts, a.ldhts = ldpts, a.htq_ks = t_panels ? 2 * H * 128 : 0;
    if (K == 0 || !tiled_ok(a, T) || !aligned(hq, 8) || ldhq % 8 || !aligned(pre, 16) || (dpre && !aligned(dpre, 16)) ||
        ldpre % 8 || H % 8 || !aligned(dpq, 8) || lddpq % 8 ||
        (ptq && (!aligned(ptq, 16) || ldptq % 16 || !aligned(pts, 4) || ldpts % 4)))
        return MX_EUNSUPPORTED;
    if (mx::stream_is_capturing((hipStream_t)stream)) return MX_ECAPTURE;
    return launch_grouped_dt<MODE_DGRAD2>(act_dtype, a, (hipStream_t)stream);
}

extern "C" int mx_experts_combine(const void *y, int64_t ldy, const int32_t *order, const int32_t *offsets, int64_t E,
                                  const void *gate, int gate_dtype, int32_t *inv, int64_t T, int64_t top_k, void *out,
                                  int dtype, int64_t ldo, int64_t M, int64_t N, void *stream) {
    if (E <= 0 || E >= (1 << 20) || T < 0 || top_k <= 0 || top_k > 0x7FFF || M < 0 || N < 0 || M >= 0x7FFFFFFF ||
        T * top_k >= 0x7FFFFFFF || ldy < N || ldo < N || (order && !offsets) || !inv)
        return MX_EINVAL;
    if (dtype != MX_BF16 && dtype != MX_FP16) return MX_EINVAL;
    if (gate && gate_dtype != MX_FP32 && gate_dtype != dtype) return MX_EINVAL;
    if (T == 0 || N == 0) return MX_OK;
    if (N % 8 || !aligned(y, 16) || !aligned(out, 16) || ldy % 8 || ldo % 8) return MX_EUNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    if (mx::stream_is_capturing(st)) return MX_ECAPTURE;
    const int64_t pairs = T * top_k;
    if (order) {  // order == NULL: inv already holds the positions of this routing (an earlier call filled it)
        fill_i32_kernel<<<dim3((unsigned)((pairs + 255) / 256)), dim3(256), 0, st>>>(inv, pairs, -1);
        if (M) invert_order_kernel<<<dim3((unsigned)((M + 255) / 256)), dim3(256), 0, st>>>(order, offsets, (int)E, M, pairs, inv);
    }
    const int n8 = (int)(N / 8);
    const int64_t blocks = (T * n8 + 255) / 256;
    if (blocks > 0x7FFFFFFF) return MX_EUNSUPPORTED;
    if (dtype == MX_BF16)
        combine_kernel<MX_BF16><<<dim3((unsigned)blocks), dim3(256), 0, st>>>((const uint16_t *)y, ldy, inv, gate,
                                                                             gate_dtype == MX_FP32, (int)top_k,
                                                                             (uint16_t *)out, ldo, T, n8);
    else
        combine_kernel<MX_FP16><<<dim3((unsigned)blocks), dim3(256), 0, st>>>((const uint16_t *)y, ldy, inv, gate,
                                                                             gate_dtype == MX_FP32, (int)top_k,
                                                                             (uint16_t *)out, ldo, T, n8);
    return hipGetLastError() == hipSuccess ? MX_OK : MX_ELAUNCH;
}

template <int CDT>
static int launch_wgrad(WgradArgs a, float *ws, int64_t ws_bytes, hipStream_t st) {
    typedef Big S;
    a.tiles_m = (a.N + S::BM - 1) / S::BM;
    a.tiles_n = (a.Kout + S::BN - 1) / S::BN;
    const int esz = CDT == MX_FP32 ? 4 : 2;
    a.c_vec = aligned(a.dw, 16) && (a.lddw * esz) % 16 == 0 && (a.stride_dwe * esz) % 16 == 0;
    const int64_t work = (int64_t)a.tiles_m * a.tiles_n * a.E;
    if (work >= 0x7FFFFFFF) return MX_EUNSUPPORTED;
    const int cus = num_cus();
    // With more tile ids than workgroups the K split can still pay: the ids of experts without
    // rows are empty, and how many those are is only known on the device.
    const bool fits = ws && !((uintptr_t)ws & 15) && ws_bytes >= 2 * (int64_t)cus * S::BM * S::BN * (int64_t)sizeof(float);
    a.ws = work < (1 << 27) && fits ? ws : nullptr;  // two fp32 tile slots per workgroup, or whole tiles only
    a.slots = a.ws ? 2 * cus : 0;
    dim3 grid((unsigned)(work * (a.slots ? 8 : 1) < cus ? work * (a.slots ? 8 : 1) : cus)), block(S::NTHR);
    // scale rows with 12 readable bytes behind their last stage take one 16-byte fetch per four stages ...
    const bool quad = a.ldas >= a.KB + 12 && a.ldbs >= a.KB + 12;
    // ... and that fetch goes through the copy engine into an LDS staging area (no vector load in the K loop for
    // the compiler to put a full wait in front of: 10 us of 155 on six experts of 16384 rows) when the lane
    // offsets fit 32 bits and the experts fit the smaller table that leaves room for the staging area
    const bool staged = quad && a.E <= MX_TABLE_MAX_STAGED && (int64_t)a.N * a.ldas < ((int64_t)1 << 32) &&
                        (int64_t)a.Kout * a.ldbs < ((int64_t)1 << 32);
    const int chunks = (a.N + 63) / 64;
    if ((int64_t)a.E * chunks >= 0x7FFFFFFF) return MX_EUNSUPPORTED;
    wgrad_zero_kernel<CDT><<<dim3((unsigned)(a.E * chunks)), dim3(256), 0, st>>>(a, chunks);
    const int rc = staged ? launch_with_lds<grouped_wgrad_kernel<S, CDT, SCALES_COPY>>(grid, block, S::LDS_BYTES_AHEAD, st, a)
                   : quad ? launch_with_lds<grouped_wgrad_kernel<S, CDT, SCALES_QUAD>>(grid, block, S::LDS_BYTES, st, a)
                          : launch_with_lds<grouped_wgrad_kernel<S, CDT, SCALES_DWORD>>(grid, block, S::LDS_BYTES, st, a);
    if (rc != MX_OK) return rc;
    // tiles are only split while (tiles x slices) fit the 2 * cus slots, so 4 * cus workgroups cover every unit at once
    const int64_t units = work * S::MT < 4 * (int64_t)cus ? work * S::MT : 4 * (int64_t)cus;
    if (a.slots) wgrad_reduce_kernel<S, CDT><<<dim3((unsigned)units), block, 0, st>>>(a, (int)grid.x);
    return hipGetLastError() == hipSuccess ? MX_OK : MX_ELAUNCH;
}

extern "C" int mx_grouped_wgrad_nt(const uint8_t *aq, const uint8_t *as, int64_t lda, int64_t ldas, const uint8_t *bq,
                                   const uint8_t *bs, int64_t ldb, int64_t ldbs, const int32_t *offsets, int64_t E,
                                   int64_t M, void *dw, int dw_dtype, int64_t stride_dwe, int64_t lddw, int64_t N,
                                   int64_t Kout, void *workspace, int64_t workspace_bytes, void *stream) {
    if (E <= 0 || E >= (1 << 20) || M < 0 || M >= 0x7FFFFFFF || N < 0 || Kout < 0 || N >= 0x7FFFFFFF ||
        Kout >= 0x7FFFFFFF || lddw < Kout || workspace_bytes < 0)
        return MX_EINVAL;
    const int64_t mpad = ((M + 127) / 128 + E) * 128;
    // a leading dimension of exactly 128 on the wider padded axis is the stage-major layout (see the header)
    const bool a_panels = lda == 128 && mpad > 128, b_panels = ldb == 128 && mpad > 128;
    if ((lda < mpad && !a_panels) || (ldb < mpad && !b_panels) || ldas < mpad / MX_BLOCK || ldbs < mpad / MX_BLOCK)
        return MX_EINVAL;
    if (N == 0 || Kout == 0) return MX_OK;
    if (!aligned(aq, 16) || !aligned(bq, 16) || lda % 16 || ldb % 16 || !aligned(as, 4) || !aligned(bs, 4) || ldas % 4 ||
        ldbs % 4 || 256 * lda >= ((int64_t)1 << 32) || 256 * ldb >= ((int64_t)1 << 32))
        return MX_EUNSUPPORTED;
    WgradArgs a = {};
    a.aq = aq, a.as = as, a.bq = bq, a.bs = bs, a.lda = lda, a.ldas = ldas, a.ldb = ldb, a.ldbs = ldbs;
    a.dw = dw, a.stride_dwe = stride_dwe, a.lddw = lddw, a.offsets = offsets, a.E = (int)E, a.N = (int)N,
    a.Kout = (int)Kout, a.KB = (int)(mpad / MX_BLOCK);
    a.a_ks = a_panels ? N * 128 : 0, a.b_ks = b_panels ? Kout * 128 : 0;
    hipStream_t st = (hipStream_t)stream;
    if (mx::stream_is_capturing(st)) return MX_ECAPTURE;
    switch (dw_dtype) {
    case MX_BF16: return launch_wgrad<MX_BF16>(a, (float *)workspace, workspace_bytes, st);
    case MX_FP16: return launch_wgrad<MX_FP16>(a, (float *)workspace, workspace_bytes, st);
    case MX_FP32: return launch_wgrad<MX_FP32>(a, (float *)workspace, workspace_bytes, st);
    default: return MX_EINVAL;
    }
}
