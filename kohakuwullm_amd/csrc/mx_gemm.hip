// Dense MXFP8 NT GEMM for gfx950: C (M,N) = deq(A) deq(B)^T, A (M,K) and B (N,K) e4m3,
// K-minor, one UE8M0 byte per 32 K elements, fp32 accumulation, bf16/fp16/fp32 output.
// Semantics: mxfp8_matmul_pq of the reference (src/kohakuwullm/kernels/mxfp8/quantize.py:242-371).
// The kernel body lives in mx_gemm_core.h; this file supplies the dense problem policy,
// the slow generic kernel for shapes the tiled kernel does not take, and the C entry point.
#include "mx_gemm_core.h"

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
};

template <typename S, int CDT>
struct DenseProblem {
    struct Tile {
        int m0, n0, kt0, kt1;
    };
    const DenseArgs p;  // a copy: its fields live in scalar registers, never re-read through a pointer
    int next_id;
    int kb_end;

    __device__ DenseProblem(const DenseArgs &args) : p(args), next_id(blockIdx.x), kb_end(args.K >> 5) {}

    __device__ __forceinline__ bool next(Tile &t) {
        const int per_slice = p.tiles_m * p.tiles_n;
        if (next_id >= per_slice * p.split_k) return false;
        const int slice = next_id / per_slice;
        int tm, tn;
        tile_of(next_id - slice * per_slice, p.tiles_m, p.tiles_n, tm, tn);
        t.m0 = tm * S::BM;
        t.n0 = tn * S::BN;
        const int KT = p.K >> 7;
        // K slices are multiples of 4 stages so every slice starts on a 16-byte scale boundary
        const int per = (((KT + p.split_k - 1) / p.split_k) + 3) & ~3;
        t.kt0 = slice * per < KT ? slice * per : KT;
        t.kt1 = t.kt0 + per < KT ? t.kt0 + per : KT;
        next_id += gridDim.x;
        if (t.kt0 == t.kt1) return next(t);  // an empty trailing slice adds nothing
        return true;
    }

    __device__ __forceinline__ void context(const Tile &t, const Lane &L0, IssueCtx<S> &c) const {
        const Lane L = opaque(L0);
        c.a_base = p.aq + (int64_t)t.m0 * p.lda;
        c.b_base = p.bq + (int64_t)t.n0 * p.ldb;
        c.kt0 = t.kt0;
        c.kt1 = t.kt1;
        const int mrem = p.M - t.m0, nrem = p.N - t.n0;
#pragma unroll
        for (int q = 0; q < S::QA; q++) {
            int row = dma_row<S>(L, q);
            int chunk = (L.lane & 7) ^ swz_a(row);
            int grow = row < mrem ? row : mrem - 1;  // rows past M re-read the last row; never stored
            c.a_voff[q] = (uint32_t)(grow * p.lda) + chunk * 16;
        }
#pragma unroll
        for (int q = 0; q < S::QB; q++) {
            int row = dma_row<S>(L, q);
            int chunk = (L.lane & 7) ^ swz_b(row);
            int grow = row < nrem ? row : nrem - 1;
            c.b_voff[q] = (uint32_t)(grow * p.ldb) + chunk * 16;
        }
        auto srow = [&](int r) -> const uint8_t * {
            if (r < S::BM) return p.as + (int64_t)(t.m0 + (r < mrem ? r : mrem - 1)) * p.ldas;
            r -= S::BM;
            return p.bs + (int64_t)(t.n0 + (r < nrem ? r : nrem - 1)) * p.ldbs;
        };
        c.srow0 = srow(L.tid < S::BM + S::BN ? L.tid : 0);
        c.srow1 = S::TWO_ROWS ? srow(L.tid + S::NTHR < S::BM + S::BN ? L.tid + S::NTHR : 0) : nullptr;
    }

    // Address of K byte 0 of row r of the tile's [A rows; B rows] list.
    __device__ __forceinline__ const uint8_t *line(const Tile &t, int r) const {
        if (r < S::BM) {
            const int mrem = p.M - t.m0;
            return p.aq + (int64_t)(t.m0 + (r < mrem ? r : mrem - 1)) * p.lda;
        }
        r -= S::BM;
        const int nrem = p.N - t.n0;
        return p.bq + (int64_t)(t.n0 + (r < nrem ? r : nrem - 1)) * p.ldb;
    }

    static constexpr int NST = S::MT * (S::NT / 2) * (CDT == MX_FP32 ? 2 : 1);

    __device__ __forceinline__ int epilogue(const Tile &t, const Lane &L, v4f (&acc)[S::MT][S::NT]) const {
        // Interior tiles of a vector-aligned C store unconditionally: every lane issues NST stores.
        const bool interior = t.m0 + S::BM <= p.M && t.n0 + S::BN <= p.N && p.c_vec && !p.accumulate;
        // sub-tiles (2h, 2h+1) of a lane hold 8 consecutive N starting at b_sub_off(2h) + 8 g
#pragma unroll
        for (int i = 0; i < S::MT; i++) {
            const int m = t.m0 + L.wm * S::WTM + 16 * i + L.r16;
#pragma unroll
            for (int h = 0; h < S::NT / 2; h++) {
                const int n = t.n0 + L.wn * S::WTN + b_sub_off(2 * h) + 8 * L.g;
                const int64_t off = (int64_t)m * p.ldc + n;
                if (interior) {
                    store8<CDT>(p.c, off, acc[i][2 * h], acc[i][2 * h + 1], 8, true);
                } else if (m < p.M && n < p.N) {
                    const int nvalid = p.N - n < 8 ? p.N - n : 8;
                    if (CDT == MX_FP32 && p.accumulate) {
                        float *dst = (float *)p.c + off;
                        for (int e = 0; e < 8 && e < nvalid; e++) atomicAdd(dst + e, e < 4 ? acc[i][2 * h][e] : acc[i][2 * h + 1][e - 4]);
                    } else {
                        store8<CDT>(p.c, off, acc[i][2 * h], acc[i][2 * h + 1], nvalid, p.c_vec != 0);
                    }
                }
            }
        }
        return interior ? NST : -1;
    }
};

template <typename S, int CDT, bool K512>
__global__ __launch_bounds__(S::NTHR) void gemm_nt_kernel(DenseArgs args) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    DenseProblem<S, CDT> prob(args);
    persistent_gemm<S, K512>(prob, smem);
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

static int num_cus() {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess) return 256;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return 256;
    return n;
}

template <typename S, int CDT>
static int launch_tiled(DenseArgs a, hipStream_t st) {
    a.tiles_m = (a.M + S::BM - 1) / S::BM;
    a.tiles_n = (a.N + S::BN - 1) / S::BN;
    const int esz = CDT == MX_FP32 ? 4 : 2;
    a.c_vec = aligned(a.c, 16) && (a.ldc * esz) % 16 == 0;
    const bool k512 = a.K % 512 == 0 && aligned(a.as, 16) && aligned(a.bs, 16) && a.ldas % 16 == 0 && a.ldbs % 16 == 0;
    const int64_t work = (int64_t)a.tiles_m * a.tiles_n * a.split_k;
    const int cus = num_cus();
    dim3 grid((unsigned)(work < cus ? work : cus)), block(S::NTHR);
    auto kern = k512 ? gemm_nt_kernel<S, CDT, true> : gemm_nt_kernel<S, CDT, false>;
    if (hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, S::LDS_BYTES) != hipSuccess)
        return MX_ELAUNCH;
    kern<<<grid, block, S::LDS_BYTES, st>>>(a);
    return hipGetLastError() == hipSuccess ? MX_OK : MX_ELAUNCH;
}

template <int CDT>
static int gemm_dispatch(DenseArgs a, hipStream_t st) {
    const int64_t M = a.M, N = a.N;
    const bool tiled_ok = a.K % 128 == 0 && aligned(a.aq, 16) && aligned(a.bq, 16) && a.lda % 16 == 0 &&
                          a.ldb % 16 == 0 && aligned(a.as, 4) && aligned(a.bs, 4) && a.ldas % 4 == 0 &&
                          a.ldbs % 4 == 0 && 256 * a.lda < (int64_t)0x7FFFFFFF && 256 * a.ldb < (int64_t)0x7FFFFFFF &&
                          ((M + 255) / 256) * ((N + 255) / 256) * a.split_k < 0x7FFFFFFF;
    if (!tiled_ok) {
        if (a.accumulate) return MX_EUNSUPPORTED;
        int64_t blocks = (M * N + 255) / 256;
        if (blocks > 0x7FFFFFFF) return MX_EUNSUPPORTED;
        gemm_nt_generic_kernel<CDT><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(a.aq, a.as, a.bq, a.bs, a.c, M, N, a.K,
                                                                                  a.lda, a.ldas, a.ldb, a.ldbs, a.ldc);
        return hipGetLastError() == hipSuccess ? MX_OK : MX_ELAUNCH;
    }
    typedef GemmShape<256, 256, 2, 4> Big;
    return launch_tiled<Big, CDT>(a, st);
}

extern "C" int mx_gemm_nt(const uint8_t *aq, const uint8_t *as, const uint8_t *bq, const uint8_t *bs, void *c,
                          int c_dtype, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldas, int64_t ldb,
                          int64_t ldbs, int64_t ldc, int epilogue, void *stream) {
    if (M < 0 || N < 0 || K < 0 || K % MX_BLOCK || lda < K || ldb < K || ldas < K / MX_BLOCK || ldbs < K / MX_BLOCK ||
        ldc < N || M > 0x7FFFFFFF || N > 0x7FFFFFFF || K > 0x7FFFFFFF)
        return MX_EINVAL;
    const int split_k = epilogue >> 8;  // MX_EPI_SPLIT_K(n)
    const int epi = epilogue & 0xFF;
    if (epi != MX_EPI_NONE && epi != MX_EPI_ACCUMULATE) return MX_EUNSUPPORTED;
    if (epi == MX_EPI_ACCUMULATE && c_dtype != MX_FP32) return MX_EINVAL;
    if (split_k > 1 && epi != MX_EPI_ACCUMULATE) return MX_EINVAL;
    if (M == 0 || N == 0) return MX_OK;
    hipStream_t st = (hipStream_t)stream;
    if (K == 0) {
        if (epi == MX_EPI_ACCUMULATE) return MX_OK;
        // An empty contraction is a zero matrix.
        int esz = c_dtype == MX_FP32 ? 4 : 2;
        hipError_t e = hipMemset2DAsync(c, (size_t)ldc * esz, 0, (size_t)N * esz, (size_t)M, st);
        return e == hipSuccess ? MX_OK : MX_ELAUNCH;
    }
    DenseArgs a;
    a.aq = aq, a.as = as, a.bq = bq, a.bs = bs, a.c = c;
    a.M = (int)M, a.N = (int)N, a.K = (int)K;
    a.lda = lda, a.ldas = ldas, a.ldb = ldb, a.ldbs = ldbs, a.ldc = ldc;
    a.accumulate = epi == MX_EPI_ACCUMULATE;
    a.split_k = split_k > 1 ? split_k : 1;
    a.tiles_m = a.tiles_n = a.c_vec = 0;
    switch (c_dtype) {
    case MX_BF16: return gemm_dispatch<MX_BF16>(a, st);
    case MX_FP16: return gemm_dispatch<MX_FP16>(a, st);
    case MX_FP32: return gemm_dispatch<MX_FP32>(a, st);
    default: return MX_EINVAL;
    }
}
