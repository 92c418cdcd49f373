// Dense MXFP8 NT GEMM for gfx950: C (M,N) = deq(A) deq(B)^T, A (M,K) and B (N,K) e4m3,
// K-minor, one UE8M0 byte per 32 K elements, fp32 accumulation, bf16/fp16/fp32 output.
// Semantics: mxfp8_matmul_pq of the reference (src/kohakuwullm/kernels/mxfp8/quantize.py:242-371).
// The kernel body lives in mx_gemm_core.h; this file supplies the dense problem policy,
// the slow generic kernel for shapes the tiled kernel does not take, and the C entry point.
#include <atomic>

#include "mx_gemm_core.h"
#ifdef MX_BENCH_VARIANTS
#include "mx_gemm_variants.h"
#endif

namespace mx {

struct DenseArgs {
    const uint8_t *aq, *as, *bq, *bs;
    void *c;
    int M, N, K;
    int64_t lda, ldas, ldb, ldbs, ldc;
    int tiles_m, tiles_n;
    int c_vec;
    int accumulate;  // fp32 atomic add into C (split-K)
    int split_k;     // number of K slices; tile ids run over tiles_m * tiles_n * split_k
    float *slice_ws;  // with split_k > 1 and no accumulate: slice s of tile i leaves its fp32 partial in slot
                      // i * split_k + s of this buffer and slice_reduce_kernel adds the slices
    // Even K split of the last, partial round of tiles.  Tile ids [0, dp_tiles) are whole tiles
    // dealt round-robin; the K stages of the remaining sk_tiles tiles are laid end to end (each
    // tile padded to KT4 stages) and cut into gridDim.x equal ranges of sk_q stages, one per
    // workgroup.  A workgroup whose range covers only part of a tile leaves its fp32 partial
    // in sk_ws; split_reduce_kernel, launched behind the GEMM, adds the pieces and stores C.
    // (Letting the last workgroup to arrive at a tile add the pieces inside the GEMM was
    // measured slower: one CU pulls the other pieces at ~40 GB/s, a kernel of its own at TB/s.)
    int dp_tiles, sk_tiles, sk_q;
    float *sk_ws;
    int xcds;  // XCDs this problem's workgroups are spread over (8; fewer inside a batched launch)
    // Stage-major operands (0: row-major).  a_ks: A is stored as K/128 panels of 128 bytes of every
    // row, panel kt at kt * a_ks, row m of it at m * 128 (lda is 128 then); b_ks likewise.  A K stage
    // of a tile is then one contiguous run instead of 256 rows a pitch apart.
    int64_t a_ks, b_ks;
    int phased;  // which schedule wrote the fp32 partial tiles: it decides which part of a tile a wave owns
};

// Whether tile_of staggers the column walk (see there): up to 64 K stages per tile.
__host__ __device__ inline bool stagger_columns(int64_t K) { return K <= 64 * 128; }

template <typename S, int CDT>
struct DenseProblem {
    struct Tile {
        int m0, n0, kt0, kt1;
        int sk;    // index among the K-split tiles when this unit is one piece of several, else -1
        int slot;  // slot of slice_ws this K slice is written to, else -1
    };
    const DenseArgs p;  // a copy: its fields live in scalar registers, never re-read through a pointer
    int next_id;
    int kb_end;
    int sk_pos, sk_end;  // this workgroup's remaining range in the K-split stage space
    const int first, stride;  // this workgroup is number `first` of the `stride` working on the problem

    __device__ DenseProblem(const DenseArgs &args, int first_, int stride_)
        : p(args), next_id(first_), kb_end(args.K >> 5), first(first_), stride(stride_) {
        const int KT4 = ((((p.K + 127) >> 7)) + 3) & ~3;
        const int total = p.sk_tiles * KT4;
        sk_pos = first * p.sk_q;
        sk_end = sk_pos + p.sk_q < total ? sk_pos + p.sk_q : total;
    }

    __device__ __forceinline__ bool next(Tile &t) {
        const int per_slice = p.tiles_m * p.tiles_n;
        if (sk_pos < sk_end) {
            const int KT = ((p.K + 127) >> 7), KT4 = (KT + 3) & ~3;
            const int local = sk_pos / KT4;
            const int k0 = sk_pos - local * KT4;
            const int stop = k0 + (sk_end - sk_pos);
            int tm, tn;
            tile_of(p.dp_tiles + local, p.tiles_m, p.tiles_n, tm, tn, stagger_columns(p.K), p.xcds);
            t.m0 = tm * S::BM;
            t.n0 = tn * S::BN;
            t.kt0 = k0;
            t.kt1 = stop < KT ? stop : KT;
            t.sk = (k0 == 0 && stop >= KT) ? -1 : local;
            t.slot = -1;
            sk_pos += (stop < KT4 ? stop : KT4) - k0;
            return true;
        }
        t.sk = -1;
        if (p.sk_tiles && next_id >= p.dp_tiles) return false;
        if (next_id >= per_slice * p.split_k) return false;
        const int slice = next_id / per_slice;
        const int index = next_id - slice * per_slice;
        int tm, tn;
        tile_of(index, p.tiles_m, p.tiles_n, tm, tn, stagger_columns(p.K), p.xcds);
        t.slot = p.slice_ws ? index * p.split_k + slice : -1;
        t.m0 = tm * S::BM;
        t.n0 = tn * S::BN;
        const int KT = ((p.K + 127) >> 7);
        // K slices are multiples of 4 stages so every slice starts on a 16-byte scale boundary
        const int per = (((KT + p.split_k - 1) / p.split_k) + 3) & ~3;
        t.kt0 = slice * per < KT ? slice * per : KT;
        t.kt1 = t.kt0 + per < KT ? t.kt0 + per : KT;
        next_id += stride;
        if (t.kt0 == t.kt1) return next(t);  // an empty trailing slice adds nothing
        return true;
    }

    __device__ __forceinline__ const uint8_t *scale_row(const Tile &t, int r) const {
        const int mrem = p.M - t.m0, nrem = p.N - t.n0;
        if (r < S::BM) return p.as + (int64_t)(t.m0 + (r < mrem ? r : mrem - 1)) * p.ldas;
        r = b_row_of_lds<S>(r - S::BM);
        return p.bs + (int64_t)(t.n0 + (r < nrem ? r : nrem - 1)) * p.ldbs;
    }

    __device__ __forceinline__ void context(const Tile &t, const Lane &L0, IssueCtx<S> &c) const {
        const Lane L = opaque(L0);
        c.a_base = p.aq + (int64_t)t.m0 * p.lda;
        c.b_base = p.bq + (int64_t)t.n0 * p.ldb;
        c.a_ks = p.a_ks ? p.a_ks : 128;
        c.b_ks = p.b_ks ? p.b_ks : 128;
        c.kt0 = t.kt0;
        c.kt1 = t.kt1;
        c.tail_bytes = p.K & 127;
        c.tail_kt = c.tail_bytes ? p.K >> 7 : -1;
        const int mrem = p.M - t.m0, nrem = p.N - t.n0;
#pragma unroll
        for (int q = 0; q < S::QA; q++) {
            int row = dma_row<S>(L, q);
            int chunk = (L.lane & 7) ^ swz_a(row);
            int grow = row < mrem ? row : mrem - 1;  // rows past M re-read the last row; never stored
            c.a_voff[q] = (uint32_t)(grow * p.lda) + chunk * 16 + copy_bias(q);
        }
#pragma unroll
        for (int q = 0; q < S::QB; q++) {
            int row = dma_row<S>(L, q);  // LDS row; it holds B row b_row_of_lds(row) of the tile
            int chunk = (L.lane & 7) ^ swz_a(row);
            int brow = b_row_of_lds<S>(row);
            int grow = brow < nrem ? brow : nrem - 1;
            c.b_voff[q] = (uint32_t)(grow * p.ldb) + chunk * 16 + copy_bias(q);
        }
        c.srow0 = scale_row(t, L.tid < S::BM + S::BN ? L.tid : 0);
        c.srow1 = S::TWO_ROWS ? scale_row(t, L.tid + S::NTHR < S::BM + S::BN ? L.tid + S::NTHR : 0) : nullptr;
        // SCALES_COPY: the same row as srow0, as an offset into its scale matrix (the launcher checked that it fits)
        c.sa_base = p.as;
        c.sb_base = p.bs;
        c.s_voff = (uint32_t)(c.srow0 - (L.tid < S::BM ? p.as : p.bs));
    }

#ifdef MX_BENCH_VARIANTS
    // the phased schedule's description of a tile: bases, pitches and limits; the lanes rebuild their offsets from them
    __device__ __forceinline__ void context(const Tile &t, const Lane &L0, PhasedCtx<S> &c) const {
        const Lane L = opaque(L0);
        c.a_base = p.aq + (int64_t)t.m0 * p.lda;
        c.b_base = p.bq + (int64_t)t.n0 * p.ldb;
        c.a_ks = p.a_ks ? p.a_ks : 128;
        c.b_ks = p.b_ks ? p.b_ks : 128;
        c.kt0 = t.kt0;
        c.kt1 = t.kt1;
        c.tail_bytes = p.K & 127;
        c.tail_kt = c.tail_bytes ? p.K >> 7 : -1;
        c.a_last = (p.M - t.m0 < S::BM ? p.M - t.m0 : S::BM) - 1;
        c.b_last = (p.N - t.n0 < S::BN ? p.N - t.n0 : S::BN) - 1;
        c.lda = (int)p.lda;
        c.ldb = (int)p.ldb;
        c.lanes(L);
        c.srow0 = scale_row(t, L.tid);
        c.srow1 = nullptr;
    }
#endif

    // stores an interior tile issues per lane: one per (i, v), two when a lane's run is 8 fp32 values (32 bytes)
    static constexpr int NST = S::MT * 4 * (CDT == MX_FP32 && S::NT == 8 ? 2 : 1);
    static constexpr bool EARLY_WAIT = false;  // interior tiles leave exactly NST stores in flight instead

    // Slot of workgroup `wg`'s piece of the split tile whose stages start at `begin` in the
    // split stage space: a workgroup has at most two partial units, the first one continuing
    // a tile that an earlier workgroup started.
    __device__ __forceinline__ static v4f *piece_slot(const DenseArgs &p, int wg, int begin) {
        const int second = begin > wg * p.sk_q ? 1 : 0;
        return (v4f *)p.sk_ws + (int64_t)(2 * wg + second) * (S::BM * S::BN / 4);
    }

    // One piece of a K-split tile: the fp32 accumulators go to the workgroup's slot, laid out
    // [sub-tile][thread] so the stores and the reduction kernel's loads are contiguous.
    __device__ __forceinline__ void write_piece(const Tile &t, const Lane &L, v4f (&acc)[S::MT][S::NT]) const {
        const int KT4 = ((((p.K + 127) >> 7)) + 3) & ~3;
        v4f *mine = piece_slot(p, first, t.sk * KT4);
#pragma unroll
        for (int i = 0; i < S::MT; i++)
#pragma unroll
            for (int j = 0; j < S::NT; j++) mine[(i * S::NT + j) * S::NTHR + L.tid] = acc[i][j];
    }

    __device__ __forceinline__ int epilogue(const Tile &t, const Lane &L, v4f (&acc)[S::MT][S::NT], const LdsScratch &) const {
        if (t.sk >= 0) {
            write_piece(t, L, acc);
            return -1;
        }
        if (t.slot >= 0) {
            v4f *dst = (v4f *)p.slice_ws + (int64_t)t.slot * (S::BM * S::BN / 4);
#pragma unroll
            for (int i = 0; i < S::MT; i++)
#pragma unroll
                for (int j = 0; j < S::NT; j++) dst[(i * S::NT + j) * S::NTHR + L.tid] = acc[i][j];
            return -1;
        }
        // Interior tiles of a vector-aligned C store unconditionally: every lane issues NST stores.
        const bool interior = t.m0 + S::BM <= p.M && t.n0 + S::BN <= p.N && p.c_vec && !p.accumulate;
        // component v of a lane's NT sub-tiles (i, 0..NT-1): row 16 i + 4 g + v, NT consecutive N from NT r16
        const int n = t.n0 + L.wn * S::WTN + S::NT * L.r16;
#pragma unroll
        for (int i = 0; i < S::MT; i++) {
#pragma unroll
            for (int v = 0; v < 4; v++) {
                const int m = t.m0 + L.wm * S::WTM + 16 * i + 4 * L.g + v;
                const int64_t off = (int64_t)m * p.ldc + n;
                float run[S::NT];
#pragma unroll
                for (int j = 0; j < S::NT; j++) run[j] = acc[i][j][v];
                if (interior) {
                    store_run<CDT, S::NT>(p.c, off, run, S::NT, true);
                } else if (m < p.M && n < p.N) {
                    const int nvalid = p.N - n < S::NT ? p.N - n : S::NT;
                    if (CDT == MX_FP32 && p.accumulate) {
                        float *dst = (float *)p.c + off;
                        for (int e = 0; e < S::NT && e < nvalid; e++) atomicAdd(dst + e, run[e]);
                    } else {
                        store_run<CDT, S::NT>(p.c, off, run, nvalid, p.c_vec != 0);
                    }
                }
            }
        }
        return interior ? NST : -1;
    }
};

// AHEAD: the A operand is fetched two K stages ahead (persistent_gemm); every tile, K-split piece and K slice of the
// launch must then have at least two stages.  Instantiated for SCALES_VEC16 only, whose K % 512 == 0 makes every
// one of them a multiple of four stages.
template <typename S, int CDT, int K512, bool AHEAD = false>
__global__ __launch_bounds__(S::NTHR) void gemm_nt_kernel(DenseArgs args) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    DenseProblem<S, CDT> prob(args, (int)blockIdx.x, (int)gridDim.x);
    persistent_gemm<S, K512, DenseProblem<S, CDT>, AHEAD>(prob, smem);
}

#ifdef MX_BENCH_VARIANTS
// The same tiles under the phased schedule (two groups of four waves half a K stage apart): MX_EPI_PHASED.
template <typename S, int CDT, int K512>
__global__ __launch_bounds__(S::NTHR) void gemm_nt_phased_kernel(DenseArgs args) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    DenseProblem<S, CDT> prob(args, (int)blockIdx.x, (int)gridDim.x);
    persistent_gemm_phased<S, K512>(prob, smem);
}

// The same tiles under the wide-wave schedule (four waves, one per SIMD, 128 x 128 each, accumulators in the
// accumulation registers, the next stage's first fragments read under the last MFMAs of the current one).
template <typename S, int CDT, int K512>
__global__ __launch_bounds__(S::NTHR) void gemm_nt_wide_kernel(DenseArgs args) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    DenseProblem<S, CDT> prob(args, (int)blockIdx.x, (int)gridDim.x);
    persistent_gemm_wide<S, K512>(prob, smem);
}

// The same kernel body on a 128 x 128 tile with two workgroups resident per CU (4 waves each, one per SIMD and
// workgroup): the second workgroup's K loop runs under the first one's epilogue, barrier waits and start-up.
template <typename S, int CDT, int K512>
__global__ __launch_bounds__(S::NTHR) __attribute__((amdgpu_waves_per_eu(2, 2))) void gemm_nt_pair_kernel(DenseArgs args) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    DenseProblem<S, CDT> prob(args, (int)blockIdx.x, (int)gridDim.x);
    persistent_gemm<S, K512>(prob, smem);
}
#endif

// Several independent products in one launch.  The XCDs are partitioned among the problems
// (x_lo[j] .. x_lo[j+1]) in proportion to their work, so a product with too few
// tiles to fill the GPU runs beside the others instead of leaving most of it idle.
#define MX_BATCH_MAX 4
// Problem j owns XCDs [x_lo[j], x_lo[j + 1]) whole: all 32 CUs of an XCD then work on one product
// and share its panels in that XCD's L2.  (Dealing every problem a few CUs of every XCD instead
// was measured: the three backward products of the feed-forward block pulled 1957 MiB through
// the fabric in 490 us, which is the part's bandwidth.)
struct DenseBatchArgs {
    DenseArgs prob[MX_BATCH_MAX];
    int x_lo[MX_BATCH_MAX + 1];
    int count;
};

template <typename S, int CDT, int K512, bool AHEAD = false>
__global__ __launch_bounds__(S::NTHR) void gemm_nt_batch_kernel(DenseBatchArgs b) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    // workgroups go to the XCDs round-robin: this one runs on XCD blockIdx.x % 8
    const int x = (int)blockIdx.x & 7, slot = (int)blockIdx.x >> 3;
    int j = 0;
    while (j + 1 < b.count && x >= b.x_lo[j + 1]) j++;
    const int nx = b.x_lo[j + 1] - b.x_lo[j];
    DenseProblem<S, CDT> prob(b.prob[j], (x - b.x_lo[j]) + nx * slot, nx * ((int)gridDim.x >> 3));
    persistent_gemm<S, K512, DenseProblem<S, CDT>, AHEAD>(prob, smem);
}

// Second half of the even K split: each thread owns what one lane of the GEMM epilogue owns
// for one i (4 rows x 8 consecutive N of one split tile), adds that piece of every workgroup
// that worked on the tile, in workgroup order, and stores it.  Tiles a single workgroup
// covered whole were stored by the GEMM itself.
template <typename S, int CDT>
__global__ __launch_bounds__(S::NTHR) void split_reduce_kernel(DenseArgs p) {
    const int KT = ((p.K + 127) >> 7), KT4 = (KT + 3) & ~3;
    const int local = blockIdx.x / S::MT;
    const int i = blockIdx.x % S::MT;
    const int begin = local * KT4;
    const int c_lo = begin / p.sk_q, c_hi = (begin + KT - 1) / p.sk_q;
    if (c_lo == c_hi) return;
    const int tid = threadIdx.x;
    v4f sum[S::NT];
#pragma unroll
    for (int j = 0; j < S::NT; j++) sum[j] = v4f{0.f, 0.f, 0.f, 0.f};
    for (int c = c_lo; c <= c_hi; c++) {
        const v4f *src = DenseProblem<S, CDT>::piece_slot(p, c, begin);
#pragma unroll
        for (int j = 0; j < S::NT; j++) sum[j] += src[(i * S::NT + j) * S::NTHR + tid];
    }
    int tm, tn;
    tile_of(p.dp_tiles + local, p.tiles_m, p.tiles_n, tm, tn, stagger_columns(p.K), p.xcds);
    const int wave = tid >> 6, lane = tid & 63;
    const int wm = p.phased ? wave & 3 : wave / S::WGN, wn = p.phased ? wave >> 2 : wave % S::WGN;
    const int n = tn * S::BN + wn * S::WTN + 8 * (lane & 15);
#pragma unroll
    for (int v = 0; v < 4; v++) {
        const int m = tm * S::BM + wm * S::WTM + 16 * i + 4 * (lane >> 4) + v;
        if (m < p.M && n < p.N) {
            const int nvalid = p.N - n < 8 ? p.N - n : 8;
            const v4f lo = {sum[0][v], sum[1][v], sum[2][v], sum[3][v]};
            const v4f hi = {sum[4][v], sum[5][v], sum[6][v], sum[7][v]};
            store8<CDT>(p.c, (int64_t)m * p.ldc + n, lo, hi, nvalid, p.c_vec != 0);
        }
    }
}

// Adds the split_k fp32 slices of every tile, in slice order, and stores C.  One block per (tile, i).
template <typename S, int CDT>
__global__ __launch_bounds__(S::NTHR) void slice_reduce_kernel(DenseArgs p) {
    const int index = blockIdx.x / S::MT, i = blockIdx.x % S::MT;
    const int tid = threadIdx.x;
    v4f sum[S::NT];
#pragma unroll
    for (int j = 0; j < S::NT; j++) sum[j] = v4f{0.f, 0.f, 0.f, 0.f};
    for (int sl = 0; sl < p.split_k; sl++) {
        const v4f *src = (const v4f *)p.slice_ws + (int64_t)(index * p.split_k + sl) * (S::BM * S::BN / 4);
#pragma unroll
        for (int j = 0; j < S::NT; j++) sum[j] += src[(i * S::NT + j) * S::NTHR + tid];
    }
    int tm, tn;
    tile_of(index, p.tiles_m, p.tiles_n, tm, tn, stagger_columns(p.K), p.xcds);
    const int wave = tid >> 6, lane = tid & 63;
    const int wm = p.phased ? wave & 3 : wave / S::WGN, wn = p.phased ? wave >> 2 : wave % S::WGN;
    const int n = tn * S::BN + wn * S::WTN + 8 * (lane & 15);
#pragma unroll
    for (int v = 0; v < 4; v++) {
        const int m = tm * S::BM + wm * S::WTM + 16 * i + 4 * (lane >> 4) + v;
        if (m < p.M && n < p.N) {
            const v4f lo = {sum[0][v], sum[1][v], sum[2][v], sum[3][v]};
            const v4f hi = {sum[4][v], sum[5][v], sum[6][v], sum[7][v]};
            store8<CDT>(p.c, (int64_t)m * p.ldc + n, lo, hi, p.N - n < 8 ? p.N - n : 8, p.c_vec != 0);
        }
    }
}

// Any K % 32 == 0, any alignment: one thread per output element.  The slow path.
template <int CDT>
__global__ __launch_bounds__(256) void gemm_nt_generic_kernel(const uint8_t *__restrict__ aq,
                                                               const uint8_t *__restrict__ as,
                                                               const uint8_t *__restrict__ bq,
                                                               const uint8_t *__restrict__ bs, void *__restrict__ c,
                                                               int64_t M, int64_t N, int64_t K, int64_t lda,
                                                               int64_t ldas, int64_t ldb, int64_t ldbs, int64_t ldc) {
    int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= M * N) return;
    int64_t m = idx / N, n = idx - m * N;
    const uint8_t *pa = aq + m * lda, *pb = bq + n * ldb;
    float acc = 0.0f;
    for (int64_t kb = 0; kb < K / MX_BLOCK; kb++) {
        float part = 0.0f;
        for (int i = 0; i < MX_BLOCK; i += 2) {
            typedef float v2f __attribute__((ext_vector_type(2)));
            uint32_t wa = pa[kb * MX_BLOCK + i] | ((uint32_t)pa[kb * MX_BLOCK + i + 1] << 8);
            uint32_t wb = pb[kb * MX_BLOCK + i] | ((uint32_t)pb[kb * MX_BLOCK + i + 1] << 8);
            v2f fa = __builtin_amdgcn_cvt_pk_f32_fp8((int)wa, false);
            v2f fb = __builtin_amdgcn_cvt_pk_f32_fp8((int)wb, false);
            part += fa[0] * fb[0] + fa[1] * fb[1];
        }
        int e = (int)as[m * ldas + kb] + (int)bs[n * ldbs + kb] - 254;
        acc += ldexpf(part, e);
    }
    if (CDT == MX_FP32) ((float *)c)[m * ldc + n] = acc;
    else if (CDT == MX_BF16) ((uint16_t *)c)[m * ldc + n] = (uint16_t)f2bf16(acc);
    else ((_Float16 *)c)[m * ldc + n] = (_Float16)acc;
}

}  // namespace mx

using namespace mx;

static inline bool aligned(const void *p, uintptr_t a) { return ((uintptr_t)p & (a - 1)) == 0; }

namespace mx {
// CUs of the current device, asked of the runtime once per device ordinal.  The cache is a word per
// ordinal written with the one value it can ever hold: no lock, no table that grows.
int num_cus() {
    static std::atomic<int> cached[64];
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    int n = cached[dev].load(std::memory_order_relaxed);
    if (n) return n;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev].store(n, std::memory_order_relaxed);
    return n;
}

bool allow_dynamic_lds(const void *kernel, int bytes, std::atomic<uint64_t> &done) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return false;
    const uint64_t bit = 1ull << dev;
    if (done.load(std::memory_order_acquire) & bit) return true;
    if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) {
        (void)hipGetLastError();
        return false;
    }
    done.fetch_or(bit, std::memory_order_release);
    return true;
}

bool stream_is_capturing(hipStream_t st) {
    hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
    const hipError_t e = hipStreamIsCapturing(st, &cap);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        // the capture family of errors (e.g. the legacy stream while another stream captures in global
        // mode) counts as capturing; anything else (no device) is left for the launch itself to report
        return e >= hipErrorStreamCaptureUnsupported && e <= hipErrorStreamCaptureWrongThread;
    }
    return cap != hipStreamCaptureStatusNone;
}
}  // namespace mx

// fp32 tile slots a caller's workspace holds for the K splits (dense and expert WGRAD): the kernels use at
// most two per workgroup, so 2 x CUs slots of one 256 x 256 tile are all they can ever take.
static inline int64_t slot_bytes() { return (int64_t)256 * 256 * sizeof(float); }
static inline int workspace_slots(const void *ws, int64_t bytes) {
    if (!ws || bytes <= 0 || ((uintptr_t)ws & 15)) return 0;
    const int64_t n = bytes / slot_bytes();
    return n > 0x7FFFFFFF ? 0x7FFFFFFF : (int)n;
}

// Which scale fetch (SCALES_*) a problem's K and scale pointers allow.
// Whether the A look-ahead (persistent_gemm) is used: whenever the scale bytes can go through the copy engine
// (SCALES_COPY) and K spans at least two groups of four stages.  It wins on long contractions (the three of the
// feed-forward backward, K = 8192 and 16384, in one launch: 442 -> 416 us) and is level on short ones (K = 1536:
// 183 -> 183 us; K = 4096 with its K-split pieces of 16 stages: 105 -> 107 us).  (With the scale bytes loaded through
// registers it lost 3 % on the short ones: the compiler, which cannot see the copies, put a full vector-memory wait in
// front of every use of those loads, once per four stages and once per tile, and the A rows meant to stay in flight
// were waited for half a stage after their issue.)
#ifndef MX_AHEAD_MIN_K
#define MX_AHEAD_MIN_K 1024
#endif
static bool ahead_pays(const DenseArgs &a) {
    // its scale bytes go through the copy engine, whose lane offsets are 32 bits
    return a.K >= MX_AHEAD_MIN_K && (int64_t)a.M * a.ldas < ((int64_t)1 << 32) && (int64_t)a.N * a.ldbs < ((int64_t)1 << 32);
}

static int scale_mode(const DenseArgs &a) {
    if (a.K % 512 == 0 && aligned(a.as, 16) && aligned(a.bs, 16) && a.ldas % 16 == 0 && a.ldbs % 16 == 0) return SCALES_VEC16;
    if (a.K % 128 == 0 && aligned(a.as, 4) && aligned(a.bs, 4) && a.ldas % 4 == 0 && a.ldbs % 4 == 0) return SCALES_DWORD;
    return SCALES_BYTES;
}

template <typename S, int CDT>
static int launch_tiled(DenseArgs a, float *ws, int ws_slots, hipStream_t st, bool phased = false) {
    a.tiles_m = (a.M + S::BM - 1) / S::BM;
    a.tiles_n = (a.N + S::BN - 1) / S::BN;
    const int esz = CDT == MX_FP32 ? 4 : 2;
    a.c_vec = aligned(a.c, 16) && (a.ldc * esz) % 16 == 0;
    const int mode = scale_mode(a);
    const int64_t work = (int64_t)a.tiles_m * a.tiles_n * a.split_k;
    const int cus = num_cus();
    a.dp_tiles = (int)work, a.sk_tiles = 0, a.sk_q = 0, a.sk_ws = nullptr;
    // The last round of tiles occupies `rest` of the `cus` workgroups for a whole tile time.
    // Dealing the K stages of those tiles evenly over all workgroups instead saves
    // (cus - rest) / cus of a tile time and costs an fp32 round trip of every piece plus a
    // second launch; in units of one K stage, measured: 4 + 0.15 per piece.  Ranges are sk_q
    // stages, a multiple of 4 (scale fetches are 16-byte aligned) and at least an eighth of a
    // tile, so no tile is cut into more than 9 pieces.
    const int rest = (int)(work % cus);
    const int KT = ((a.K + 127) >> 7), KT4 = (KT + 3) & ~3;
    if (a.split_k == 1 && !a.accumulate && rest > 0 && KT4 >= 8) {
        int64_t q = ((int64_t)rest * KT4 + cus - 1) / cus;
        if (q < KT4 / 8) q = KT4 / 8;
        q = (q + 3) & ~(int64_t)3;
        const double pieces = (double)rest * KT4 / q + rest;
        const double gain = (double)(KT4 - q), cost = 4.0 + 0.15 * pieces;
        float *slots = gain > 1.25 * cost && ws_slots >= 2 * cus ? ws : nullptr;  // two slots per workgroup
        if (slots) {
            a.sk_tiles = rest;
            a.dp_tiles = (int)work - rest;
            a.sk_q = (int)q;
            a.sk_ws = slots;
        }
    }
    dim3 grid((unsigned)(work < cus && !a.sk_tiles ? work : cus)), block(S::NTHR);
    int rc;
    a.phased = phased ? 1 : 0;
#ifdef MX_BENCH_VARIANTS
    if constexpr (S::NW == 4)
        rc = mode == SCALES_VEC16   ? launch_with_lds<gemm_nt_wide_kernel<S, CDT, SCALES_VEC16>>(grid, block, S::LDS_BYTES, st, a)
             : mode == SCALES_DWORD ? launch_with_lds<gemm_nt_wide_kernel<S, CDT, SCALES_DWORD>>(grid, block, S::LDS_BYTES, st, a)
                                    : launch_with_lds<gemm_nt_wide_kernel<S, CDT, SCALES_BYTES>>(grid, block, S::LDS_BYTES, st, a);
    else if (phased)
        rc = mode == SCALES_VEC16   ? launch_with_lds<gemm_nt_phased_kernel<S, CDT, SCALES_VEC16>>(grid, block, S::LDS_BYTES, st, a)
             : mode == SCALES_DWORD ? launch_with_lds<gemm_nt_phased_kernel<S, CDT, SCALES_DWORD>>(grid, block, S::LDS_BYTES, st, a)
                                    : launch_with_lds<gemm_nt_phased_kernel<S, CDT, SCALES_BYTES>>(grid, block, S::LDS_BYTES, st, a);
    else
#endif
        rc = mode == SCALES_VEC16 && ahead_pays(a)
                 ? launch_with_lds<gemm_nt_kernel<S, CDT, SCALES_COPY, true>>(grid, block, S::LDS_BYTES_AHEAD, st, a)
             : mode == SCALES_VEC16 ? launch_with_lds<gemm_nt_kernel<S, CDT, SCALES_VEC16>>(grid, block, S::LDS_BYTES, st, a)
             : mode == SCALES_DWORD ? launch_with_lds<gemm_nt_kernel<S, CDT, SCALES_DWORD>>(grid, block, S::LDS_BYTES, st, a)
                                    : launch_with_lds<gemm_nt_kernel<S, CDT, SCALES_BYTES>>(grid, block, S::LDS_BYTES, st, a);
    if (rc != MX_OK) return rc;
    if (a.sk_tiles)
        split_reduce_kernel<S, CDT><<<dim3((unsigned)(a.sk_tiles * S::MT)), dim3(S::NTHR), 0, st>>>(a);
    return hipGetLastError() == hipSuccess ? MX_OK : MX_ELAUNCH;
}

// 256 x 256 x 128 tile, 8 waves as 4 (M) x 2 (N): a wave owns 64 x 128, a lane 8 consecutive N.
typedef GemmShape<256, 256, 4, 2> DenseShape;
#ifdef MX_BENCH_VARIANTS
// 128 x 128 x 128 tile, 4 waves as 2 x 2: a wave owns 64 x 64, a lane 4 consecutive N; 73 KiB of LDS, two per CU.
typedef GemmShape<128, 128, 2, 2> PairShape;
// 256 x 256 x 128 tile, 4 waves as 2 x 2, one per SIMD: a wave owns 128 x 128 (the wide-wave schedule).
typedef GemmShape<256, 256, 2, 2> WideShape;

template <int CDT>
static int launch_pair(DenseArgs a, hipStream_t st) {
    typedef PairShape S;
    a.tiles_m = (a.M + S::BM - 1) / S::BM;
    a.tiles_n = (a.N + S::BN - 1) / S::BN;
    a.c_vec = aligned(a.c, 16) && (a.ldc * (CDT == MX_FP32 ? 4 : 2)) % 16 == 0;
    const int mode = scale_mode(a);
    const int64_t work = (int64_t)a.tiles_m * a.tiles_n * a.split_k;
    a.dp_tiles = (int)work, a.sk_tiles = 0, a.sk_q = 0, a.sk_ws = nullptr;
    const int wgs = 2 * num_cus();
    dim3 grid((unsigned)(work < wgs ? work : wgs)), block(S::NTHR);
    const int rc = mode == SCALES_VEC16   ? launch_with_lds<gemm_nt_pair_kernel<S, CDT, SCALES_VEC16>>(grid, block, S::LDS_BYTES, st, a)
                   : mode == SCALES_DWORD ? launch_with_lds<gemm_nt_pair_kernel<S, CDT, SCALES_DWORD>>(grid, block, S::LDS_BYTES, st, a)
                                          : launch_with_lds<gemm_nt_pair_kernel<S, CDT, SCALES_BYTES>>(grid, block, S::LDS_BYTES, st, a);
    if (rc != MX_OK) return rc;
    return hipGetLastError() == hipSuccess ? MX_OK : MX_ELAUNCH;
}
#endif

static bool tiled_ok(const DenseArgs &a) {
    const int64_t M = a.M, N = a.N;
    return a.K % MX_BLOCK == 0 && aligned(a.aq, 16) && aligned(a.bq, 16) && a.lda % 16 == 0 && a.ldb % 16 == 0 &&
           256 * a.lda < (int64_t)0x7FFFFFFF && 256 * a.ldb < (int64_t)0x7FFFFFFF &&
           ((M + 255) / 256) * ((N + 255) / 256) * a.split_k < 0x7FFFFFFF;
}

template <int CDT>
static int gemm_dispatch(DenseArgs a, float *ws, int ws_slots, hipStream_t st, bool pair = false, bool phased = false,
                         bool wide = false) {
    const int64_t M = a.M, N = a.N;
#ifdef MX_BENCH_VARIANTS
    if (pair && tiled_ok(a) && a.split_k == 1 && !a.slice_ws) return launch_pair<CDT>(a, st);
    if (wide && tiled_ok(a)) return launch_tiled<WideShape, CDT>(a, ws, ws_slots, st, false);
#else
    if (pair || phased || wide) return MX_EUNSUPPORTED;
#endif
    if (!tiled_ok(a)) {
        if (a.accumulate || a.a_ks || a.b_ks) return MX_EUNSUPPORTED;  // the element-wise kernel reads row-major only
        int64_t blocks = (M * N + 255) / 256;
        if (blocks > 0x7FFFFFFF) return MX_EUNSUPPORTED;
        gemm_nt_generic_kernel<CDT><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(a.aq, a.as, a.bq, a.bs, a.c, M, N, a.K,
                                                                                  a.lda, a.ldas, a.ldb, a.ldbs, a.ldc);
        return hipGetLastError() == hipSuccess ? MX_OK : MX_ELAUNCH;
    }
    return launch_tiled<DenseShape, CDT>(a, ws, ws_slots, st, phased);
}

// Several products behind one launch, the eight XCDs shared out among them whole.  Every problem
// gets one XCD, the rest go, one at a time, to the problem that would otherwise finish last; cost
// of a problem on n workgroups = rounds of tiles x (K stages + 4 for the tile's prologue and
// epilogue).  A problem with few, long tiles (a weight gradient) may in addition be cut into 2 or
// 4 K slices that run as independent tiles and leave fp32 partial sums for slice_reduce_kernel;
// every combination of slice counts is priced (a partial tile costs about 0.1 stage of
// everyone's time) and the cheapest plan wins, against running the products one after the other
// as well.
template <int CDT>
static int batch_dispatch(DenseArgs *probs, int count, float *ws, int ws_slots, hipStream_t st) {
    typedef DenseShape S;
    const int cus = num_cus();
    bool fuse = count > 1 && count <= MX_BATCH_MAX;
    DenseBatchArgs b;
    int64_t tiles[MX_BATCH_MAX], alone = 0;
    int KT[MX_BATCH_MAX];
    int mode = SCALES_VEC16;  // the least capable fetch any problem needs serves them all
    for (int j = 0; j < count && fuse; j++) {
        DenseArgs &a = probs[j];
        if (!tiled_ok(a)) {
            fuse = false;
            break;
        }
        a.tiles_m = (a.M + S::BM - 1) / S::BM;
        a.tiles_n = (a.N + S::BN - 1) / S::BN;
        a.c_vec = aligned(a.c, 16) && (a.ldc * (CDT == MX_FP32 ? 4 : 2)) % 16 == 0;
        a.dp_tiles = a.tiles_m * a.tiles_n, a.sk_tiles = 0, a.sk_q = 0, a.sk_ws = nullptr;
        mode = scale_mode(a) > mode ? scale_mode(a) : mode;
        tiles[j] = a.dp_tiles;
        KT[j] = ((a.K + 127) >> 7);
        // a launch of its own: whole rounds of tiles, then the last round with the same even K
        // split launch_tiled would choose
        const int64_t rest = tiles[j] % cus, KT4 = (KT[j] + 3) & ~3;
        alone += tiles[j] / cus * (KT[j] + 4);
        if (rest) {
            int64_t q = (rest * KT4 + cus - 1) / cus;
            q = ((q < KT4 / 8 ? KT4 / 8 : q) + 3) & ~(int64_t)3;
            const double pieces = (double)rest * KT4 / q + rest, cost = 4.0 + 0.15 * pieces;
            alone += KT4 >= 8 && ws_slots >= 2 * cus && (double)(KT4 - q) > 1.25 * cost ? q + (int64_t)cost : KT[j] + 4;
        }
        // A product with several full rounds of tiles runs well on its own (each XCD's 32 CUs
        // share A/B panels in L2, the ragged last round is K-split); confined to a part of the
        // GPU beside another product it shares less and both become bound by HBM.  Measured
        // with operands that are not cache-resident: 32768 x 2048 x 3072 beside its weight
        // gradient 479 us in one launch, 404 us one after the other; the three backward
        // products of the feed-forward block (1.5, 0.75 and 0.4 rounds) 482 against 536.
        if (tiles[j] >= 2 * (int64_t)cus) fuse = false;
    }
    // Plan: a number of whole XCDs for every problem (they add up to 8) and a number of K slices,
    // chosen together by pricing every combination.
    int share[MX_BATCH_MAX], slices[MX_BATCH_MAX], best_share[MX_BATCH_MAX], best_slices[MX_BATCH_MAX];
    int64_t best = -1;
    fuse = fuse && cus % 8 == 0 && count <= 8;
    if (fuse) {
        const int per_xcd = cus / 8;
        const int slots = ws_slots < 2 * cus ? ws_slots : 2 * cus;  // fp32 tile slots the caller's workspace offers
        auto per_slice = [&](int j) { return (((KT[j] + slices[j] - 1) / slices[j]) + 3) & ~3; };
        auto units = [&](int j) { return tiles[j] * slices[j]; };
        auto finish = [&](int j) {
            return (units(j) + per_xcd * share[j] - 1) / (per_xcd * share[j]) * (per_slice(j) + 4);
        };
        int combos = 1;
        for (int j = 0; j < count; j++) combos *= 3;
        for (int code = 0; code < combos; code++) {
            int64_t partial = 0;
            bool ok = true;
            for (int j = 0, c = code; j < count; j++, c /= 3) {
                slices[j] = 1 << (c % 3);
                // every slice must own K stages, and at least 16 of them to be worth a partial tile
                if (slices[j] > 1 && (KT[j] < 16 * slices[j] || (slices[j] - 1) * per_slice(j) >= KT[j])) ok = false;
                if (slices[j] > 1) partial += units(j);
                share[j] = 1;
            }
            if (!ok || partial > slots) continue;
            // the XCDs beyond one each go, one at a time, to the problem that would finish last
            for (int left = 8 - count; left > 0; left--) {
                int worst = 0;
                for (int j = 1; j < count; j++)
                    if (finish(j) > finish(worst)) worst = j;
                share[worst]++;
            }
            int64_t together = partial ? 4 + partial / 10 : 0;
            int64_t longest = 0;
            for (int j = 0; j < count; j++) longest = finish(j) > longest ? finish(j) : longest;
            together += longest;
            if (best < 0 || together < best) {
                best = together;
                for (int j = 0; j < count; j++) best_share[j] = share[j], best_slices[j] = slices[j];
            }
        }
        fuse = best >= 0 && best < alone;
    }
    float *scratch = nullptr;
    if (fuse) {
        bool any = false;
        for (int j = 0; j < count; j++) any = any || best_slices[j] > 1;
        if (any) scratch = ws;  // the plan fitted its partial tiles into the workspace's slots
    }
    if (!fuse) {
        for (int j = 0; j < count; j++) {
            int rc = gemm_dispatch<CDT>(probs[j], ws, ws_slots, st);
            if (rc != MX_OK) return rc;
        }
        return MX_OK;
    }
    b.x_lo[0] = 0;
    int64_t slot_base = 0;
    for (int j = 0; j < count; j++) {
        DenseArgs &a = probs[j];
        a.split_k = best_slices[j];
        a.xcds = best_share[j];
        if (a.split_k > 1) {
            a.slice_ws = scratch + slot_base * (S::BM * S::BN);
            slot_base += tiles[j] * a.split_k;
        }
        b.x_lo[j + 1] = b.x_lo[j] + best_share[j];
        b.prob[j] = a;
    }
    b.count = count;
    const dim3 grid((unsigned)cus), block(S::NTHR);
    bool ahead = mode == SCALES_VEC16;
    for (int j = 0; j < count; j++) ahead = ahead && ahead_pays(probs[j]);
    const int rc = ahead ? launch_with_lds<gemm_nt_batch_kernel<S, CDT, SCALES_COPY, true>>(grid, block, S::LDS_BYTES_AHEAD, st, b)
                   : mode == SCALES_VEC16 ? launch_with_lds<gemm_nt_batch_kernel<S, CDT, SCALES_VEC16>>(grid, block, S::LDS_BYTES, st, b)
                   : mode == SCALES_DWORD
                       ? launch_with_lds<gemm_nt_batch_kernel<S, CDT, SCALES_DWORD>>(grid, block, S::LDS_BYTES, st, b)
                       : launch_with_lds<gemm_nt_batch_kernel<S, CDT, SCALES_BYTES>>(grid, block, S::LDS_BYTES, st, b);
    if (rc != MX_OK) return rc;
    for (int j = 0; j < count; j++)
        if (probs[j].split_k > 1)
            slice_reduce_kernel<S, CDT><<<dim3((unsigned)(tiles[j] * S::MT)), dim3(S::NTHR), 0, st>>>(probs[j]);
    return hipGetLastError() == hipSuccess ? MX_OK : MX_ELAUNCH;
}

static int fill_args(DenseArgs &a, const uint8_t *aq, const uint8_t *as, const uint8_t *bq, const uint8_t *bs, void *c,
                     int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldas, int64_t ldb, int64_t ldbs, int64_t ldc) {
    // a leading dimension of exactly 128 with K > 128 is the stage-major layout (see the header)
    const bool a_panels = lda == 128 && K > 128, b_panels = ldb == 128 && K > 128;
    if (M < 0 || N < 0 || K < 0 || K % MX_BLOCK || (lda < K && !a_panels) || (ldb < K && !b_panels) ||
        ((a_panels || b_panels) && K % 128) || ldas < K / MX_BLOCK || ldbs < K / MX_BLOCK || ldc < N ||
        M > 0x7FFFFFFF || N > 0x7FFFFFFF || K > 0x7FFFFFFF)
        return MX_EINVAL;
    a.aq = aq, a.as = as, a.bq = bq, a.bs = bs, a.c = c;
    a.M = (int)M, a.N = (int)N, a.K = (int)K;
    a.lda = lda, a.ldas = ldas, a.ldb = ldb, a.ldbs = ldbs, a.ldc = ldc;
    a.accumulate = 0, a.split_k = 1;
    a.slice_ws = nullptr;
    a.tiles_m = a.tiles_n = a.c_vec = 0;
    a.dp_tiles = a.sk_tiles = a.sk_q = 0;
    a.sk_ws = nullptr;
    a.xcds = 8;
    a.a_ks = a_panels ? M * 128 : 0;
    a.b_ks = b_panels ? N * 128 : 0;
    a.phased = 0;
    return MX_OK;
}

// An empty contraction: C = 0.  A fill kernel, not a memset, so the call can sit in a captured graph.
__global__ __launch_bounds__(256) static void zero_matrix_kernel(uint8_t *c, int64_t row_bytes, int64_t pitch_bytes,
                                                                  int64_t total) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < total) c[(i / row_bytes) * pitch_bytes + i % row_bytes] = 0;
}

static int zero_matrix(void *c, int c_dtype, int64_t M, int64_t N, int64_t ldc, hipStream_t st) {
    const int esz = c_dtype == MX_FP32 ? 4 : 2;
    const int64_t total = M * N * esz, blocks = (total + 255) / 256;
    if (blocks > 0x7FFFFFFF) return MX_EUNSUPPORTED;
    zero_matrix_kernel<<<dim3((unsigned)blocks), dim3(256), 0, st>>>((uint8_t *)c, N * esz, ldc * esz, total);
    return hipGetLastError() == hipSuccess ? MX_OK : MX_ELAUNCH;
}

extern "C" int64_t mx_gemm_workspace_bytes(void) { return 2 * (int64_t)num_cus() * slot_bytes(); }

extern "C" int mx_gemm_nt_batch(const mx_gemm_problem *problems, int count, int c_dtype, void *workspace,
                                int64_t workspace_bytes, void *stream) {
    if (count < 0 || (count > 0 && !problems) || workspace_bytes < 0) return MX_EINVAL;
    if (c_dtype != MX_BF16 && c_dtype != MX_FP16 && c_dtype != MX_FP32) return MX_EINVAL;
    hipStream_t st = (hipStream_t)stream;
    float *const ws = (float *)workspace;
    const int ws_slots = workspace_slots(workspace, workspace_bytes);
    DenseArgs live[MX_BATCH_MAX];
    int n = 0;
    auto flush = [&]() -> int {
        int rc = MX_OK;
        if (n) {
            switch (c_dtype) {
            case MX_BF16: rc = batch_dispatch<MX_BF16>(live, n, ws, ws_slots, st); break;
            case MX_FP16: rc = batch_dispatch<MX_FP16>(live, n, ws, ws_slots, st); break;
            default: rc = batch_dispatch<MX_FP32>(live, n, ws, ws_slots, st); break;
            }
        }
        n = 0;
        return rc;
    };
    for (int j = 0; j < count; j++) {  // validate everything before launching anything
        const mx_gemm_problem &q = problems[j];
        DenseArgs probe;
        int rc = fill_args(probe, q.aq, q.a_scale, q.bq, q.b_scale, q.c, q.M, q.N, q.K, q.lda, q.ldas, q.ldb, q.ldbs, q.ldc);
        if (rc != MX_OK) return rc;
    }
    if (count && stream_is_capturing(st)) return MX_ECAPTURE;
    for (int j = 0; j < count; j++) {
        const mx_gemm_problem &q = problems[j];
        if (q.M == 0 || q.N == 0) continue;
        if (q.K == 0) {
            int rc = zero_matrix(q.c, c_dtype, q.M, q.N, q.ldc, st);
            if (rc != MX_OK) return rc;
            continue;
        }
        fill_args(live[n++], q.aq, q.a_scale, q.bq, q.b_scale, q.c, q.M, q.N, q.K, q.lda, q.ldas, q.ldb, q.ldbs, q.ldc);
        if (n == MX_BATCH_MAX) {
            int rc = flush();
            if (rc != MX_OK) return rc;
        }
    }
    return flush();
}

extern "C" int mx_gemm_nt(const uint8_t *aq, const uint8_t *as, const uint8_t *bq, const uint8_t *bs, void *c,
                          int c_dtype, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldas, int64_t ldb,
                          int64_t ldbs, int64_t ldc, int epilogue, void *workspace, int64_t workspace_bytes,
                          void *stream) {
    if (workspace_bytes < 0) return MX_EINVAL;
    DenseArgs a;
    int rc = fill_args(a, aq, as, bq, bs, c, M, N, K, lda, ldas, ldb, ldbs, ldc);
    if (rc != MX_OK) return rc;
    if (epilogue < 0) return MX_EINVAL;
    const int split_k = epilogue >> 8;  // MX_EPI_SPLIT_K(n)
    const int epi = epilogue & 0x0F;
    if (epi != MX_EPI_NONE && epi != MX_EPI_ACCUMULATE) return MX_EUNSUPPORTED;
#ifdef MX_BENCH_VARIANTS
    const bool pair = (epilogue & MX_EPI_TILE_128) != 0, phased = (epilogue & MX_EPI_PHASED) != 0;
    const bool wide = (epilogue & MX_EPI_WIDE_WAVES) != 0;
    // one alternative kernel at a time, on a plain product: no unknown bit, no accumulation, no caller-driven K slices
    if ((epilogue & 0x80) || (int)pair + (int)phased + (int)wide > 1) return MX_EUNSUPPORTED;
    if ((pair || phased || wide) && (epi != MX_EPI_NONE || split_k > 1)) return MX_EUNSUPPORTED;
#else
    const bool pair = false, phased = false, wide = false;
    if (epilogue & 0xF0) return MX_EUNSUPPORTED;  // bits 4-7 select nothing in this library
#endif
    if (epi == MX_EPI_ACCUMULATE && c_dtype != MX_FP32) return MX_EINVAL;
    if (split_k > 1 && epi != MX_EPI_ACCUMULATE) return MX_EINVAL;
    if (c_dtype != MX_BF16 && c_dtype != MX_FP16 && c_dtype != MX_FP32) return MX_EINVAL;
    if (M == 0 || N == 0) return MX_OK;
    hipStream_t st = (hipStream_t)stream;
    if (stream_is_capturing(st)) return MX_ECAPTURE;
    float *const ws = (float *)workspace;
    const int ws_slots = workspace_slots(workspace, workspace_bytes);
    if (K == 0)  // an empty contraction is a zero matrix
        return epi == MX_EPI_ACCUMULATE ? MX_OK : zero_matrix(c, c_dtype, M, N, ldc, st);
    a.accumulate = epi == MX_EPI_ACCUMULATE;
    a.split_k = split_k > 1 ? split_k : 1;
    switch (c_dtype) {
    case MX_BF16: return gemm_dispatch<MX_BF16>(a, ws, ws_slots, st, pair, phased, wide);
    case MX_FP16: return gemm_dispatch<MX_FP16>(a, ws, ws_slots, st, pair, phased, wide);
    default: return gemm_dispatch<MX_FP32>(a, ws, ws_slots, st, pair, phased, wide);
    }
}
