// Dense MXFP8 NT GEMM for gfx950: C (M,N) = deq(A) deq(B)^T, A (M,K) and B (N,K) e4m3,
// K-minor, with one UE8M0 byte per 32 K elements, fp32 accumulation on
// v_mfma_scale_f32_16x16x128_f8f6f4, bf16/fp16/fp32 output.
//
// Semantics: mxfp8_matmul_pq of the reference (src/kohakuwullm/kernels/mxfp8/quantize.py:242-371).
//
// Shape of the kernel
//   * workgroup tile BM x BN x 128, 64-lane waves arranged WGM x WGN, each wave owning a
//     (BM/WGM) x (BN/WGN) sub-tile as 16x16 MFMA accumulators;
//   * operand tiles travel HBM -> LDS with the direct global-to-LDS load (16 bytes per
//     lane), double buffered, one workgroup barrier per 128-wide K stage;
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
//   * the MFMA is issued "B rows x A rows", so a lane's 4 accumulator registers are 4
//     consecutive N of one output row; the B rows feeding sub-tiles 4j..4j+3 are permuted
//     so a lane ends up with 16 consecutive N and stores two 16-byte vectors.
#include "mx_common.h"

namespace mx {

typedef __attribute__((address_space(1))) const void gptr_t;
typedef __attribute__((address_space(3))) void lptr_t;

__device__ __forceinline__ void dma16(const uint8_t *g, uint8_t *l) {
    // Each lane supplies its own global address; the wave's 64 x 16 bytes land contiguously
    // in LDS starting at `l` (wave-uniform).
    __builtin_amdgcn_global_load_lds((gptr_t *)g, (lptr_t *)l, 16, 0, 0);
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
    static constexpr int SC_A = 4 * BM * 4, SC_B = 4 * BN * 4;  // bytes per super-step
    static constexpr int LDS_BYTES = 2 * (DATA_A + DATA_B + SC_A + SC_B);
    static_assert(WTN % 64 == 0, "a wave's N extent must be a multiple of 64");
    static_assert(WTM % 16 == 0, "a wave's M extent must be a multiple of 16");
    static_assert((BM / 8) % NW == 0 && (BN / 8) % NW == 0, "DMA rows must divide over the waves");
    static_assert(BM + BN <= 2 * NTHR, "scale loader assumes at most two rows per thread");
};

// chunk swizzles: position of logical 16-byte chunk c of LDS row r is c ^ swz(r)
__device__ __forceinline__ int swz_a(int r) { return (r >> 1) & 7; }
__device__ __forceinline__ int swz_b(int r) { return (((r >> 4) & 3) << 1) | ((r >> 1) & 1); }

// 4x4 byte transpose: in d[s] = bytes {4s+0..4s+3}; out t[g] = bytes {g, 4+g, 8+g, 12+g}.
__device__ __forceinline__ void transpose4x4(const uint32_t d[4], uint32_t t[4]) {
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

template <typename S, int OPSEL>
__device__ __forceinline__ void compute_stage(const uint8_t *__restrict__ la, const uint8_t *__restrict__ lb, int a_lo,
                                              int a_hi, int b_lo, int b_hi, const int (&sa)[S::MT],
                                              const int (&sb)[S::NT], v4f (&acc)[S::MT][S::NT]) {
    v8i bf[S::NT];
#pragma unroll
    for (int j = 0; j < S::NT; j++) {
        const int o = (j >> 2) * (64 * 128) + (j & 3) * (4 * 128);
        v4i lo = *(const v4i *)(lb + b_lo + o);
        v4i hi = *(const v4i *)(lb + b_hi + o);
        bf[j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
    // A fragments are double buffered in registers: the reads for sub-tile i+1 are in
    // flight while the MFMAs of sub-tile i issue.
    v8i af[2];
    {
        v4i lo = *(const v4i *)(la + a_lo);
        v4i hi = *(const v4i *)(la + a_hi);
        af[0] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
#pragma unroll
    for (int i = 0; i < S::MT; i++) {
        if (i + 1 < S::MT) {
            v4i lo = *(const v4i *)(la + a_lo + (i + 1) * (16 * 128));
            v4i hi = *(const v4i *)(la + a_hi + (i + 1) * (16 * 128));
            af[(i + 1) & 1] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
#pragma unroll
        for (int j = 0; j < S::NT; j++)
            acc[i][j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(bf[j], af[i & 1], acc[i][j], 0, 0, OPSEL,
                                                                         sb[j], OPSEL, sa[i]);
    }
}

template <int CDT>
__device__ __forceinline__ void store16(void *c, int64_t off, const float (&v)[16], int nvalid, bool vec) {
    if (CDT == MX_FP32) {
        float *p = (float *)c + off;
        if (vec && nvalid == 16) {
#pragma unroll
            for (int i = 0; i < 4; i++) ((v4f *)p)[i] = v4f{v[4 * i], v[4 * i + 1], v[4 * i + 2], v[4 * i + 3]};
        } else {
            for (int i = 0; i < 16 && i < nvalid; i++) p[i] = v[i];
        }
    } else {
        uint32_t w[8];
        if (CDT == MX_BF16) {
#pragma unroll
            for (int i = 0; i < 8; i++) w[i] = pack2_bf16(v[2 * i], v[2 * i + 1]);
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) {
                typedef _Float16 h2 __attribute__((ext_vector_type(2)));
                h2 h = {(_Float16)v[2 * i], (_Float16)v[2 * i + 1]};
                w[i] = __builtin_bit_cast(uint32_t, h);
            }
        }
        uint16_t *p = (uint16_t *)c + off;
        if (vec && nvalid == 16) {
            ((v4i *)p)[0] = v4i{(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
            ((v4i *)p)[1] = v4i{(int)w[4], (int)w[5], (int)w[6], (int)w[7]};
        } else {
            for (int i = 0; i < 16 && i < nvalid; i++) p[i] = (uint16_t)(w[i >> 1] >> ((i & 1) * 16));
        }
    }
}

// Maps the flat workgroup id to a tile so that (a) ids that land on the same XCD (id % 8)
// are neighbours in tile space and share A/B panels in that XCD's L2, and (b) tiles are
// walked in column groups of GROUP_M row tiles.
__device__ __forceinline__ void tile_of(int pid, int tiles_m, int tiles_n, int &tm, int &tn) {
    const int total = tiles_m * tiles_n;
    const int per_xcd = total >> 3;
    int id = pid;
    if (pid < (per_xcd << 3)) id = (pid & 7) * per_xcd + (pid >> 3);
    constexpr int GROUP_M = 8;
    const int width = GROUP_M * tiles_n;
    const int group = id / width;
    const int first = group * GROUP_M;
    const int rows = tiles_m - first < GROUP_M ? tiles_m - first : GROUP_M;
    const int in = id - group * width;
    tm = first + in % rows;
    tn = in / rows;
}

template <typename S, int CDT, bool K512>
__global__ __launch_bounds__(S::NTHR) void gemm_nt_kernel(const uint8_t *__restrict__ aq, const uint8_t *__restrict__ as,
                                                           const uint8_t *__restrict__ bq, const uint8_t *__restrict__ bs,
                                                           void *__restrict__ c, int M, int N, int K, int64_t lda,
                                                           int64_t ldas, int64_t ldb, int64_t ldbs, int64_t ldc,
                                                           int tiles_m, int tiles_n, int c_vec) {
    extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
    uint8_t *const ldsA = smem;                                   // [2][BM*128]
    uint8_t *const ldsB = smem + 2 * S::DATA_A;                   // [2][BN*128]
    uint32_t *const ldsSA = (uint32_t *)(smem + 2 * (S::DATA_A + S::DATA_B));  // [2][4][BM]
    uint32_t *const ldsSB = ldsSA + 2 * 4 * S::BM;                // [2][4][BN]

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / S::WGN, wn = wave % S::WGN;
    const int r16 = lane & 15, g = lane >> 4;

    int tm, tn;
    tile_of(blockIdx.x, tiles_m, tiles_n, tm, tn);
    const int m0 = tm * S::BM, n0 = tn * S::BN;

    // ---- global -> LDS copy plan (per lane byte offsets relative to the tile's first row)
    const uint8_t *const a_tile = aq + (int64_t)m0 * lda;
    const uint8_t *const b_tile = bq + (int64_t)n0 * ldb;
    uint32_t a_voff[S::QA], b_voff[S::QB];
#pragma unroll
    for (int q = 0; q < S::QA; q++) {
        int row = (q * S::NW + wave) * 8 + (lane >> 3);
        int chunk = (lane & 7) ^ swz_a(row);
        int grow = row < M - m0 ? row : M - m0 - 1;
        a_voff[q] = (uint32_t)(grow * lda) + chunk * 16;
    }
#pragma unroll
    for (int q = 0; q < S::QB; q++) {
        int row = (q * S::NW + wave) * 8 + (lane >> 3);
        int chunk = (lane & 7) ^ swz_b(row);
        int grow = row < N - n0 ? row : N - n0 - 1;
        b_voff[q] = (uint32_t)(grow * ldb) + chunk * 16;
    }

    // ---- scale loader: thread t owns A row t (t < BM) and/or B row t - BM.
    // rows 0..BM-1 -> A, BM..BM+BN-1 -> B; a thread handles row tid and row tid + NTHR.
    const int KB = K >> 5;  // scale bytes per row
    auto load_scales = [&](int srow, int kb0, uint32_t (&d)[4]) {
        const uint8_t *p;
        if (srow < S::BM) {
            int r = srow < M - m0 ? srow : M - m0 - 1;
            p = as + (int64_t)(m0 + r) * ldas + kb0;
        } else {
            int r = srow - S::BM;
            r = r < N - n0 ? r : N - n0 - 1;
            p = bs + (int64_t)(n0 + r) * ldbs + kb0;
        }
        if (K512) {
            v4i t = *(const v4i *)p;
            d[0] = t[0], d[1] = t[1], d[2] = t[2], d[3] = t[3];
        } else {
#pragma unroll
            for (int s = 0; s < 4; s++) d[s] = kb0 + 4 * s < KB ? *(const uint32_t *)(p + 4 * s) : 0u;
        }
    };
    auto park_scales = [&](int srow, int buf, const uint32_t (&d)[4]) {
        uint32_t t[4];
        transpose4x4(d, t);
        uint32_t *dst = srow < S::BM ? ldsSA + buf * 4 * S::BM + srow : ldsSB + buf * 4 * S::BN + (srow - S::BM);
        const int stride = srow < S::BM ? S::BM : S::BN;
#pragma unroll
        for (int gg = 0; gg < 4; gg++) dst[gg * stride] = t[gg];
    };
    constexpr int SROWS = S::BM + S::BN;
    constexpr bool TWO_ROWS = SROWS > S::NTHR;
    const bool has_row0 = tid < SROWS;

    auto issue_stage = [&](int kt, int buf) {
        // The stage's base address is forced into SGPRs so each load is "scalar base + 32-bit
        // lane offset" and costs no 64-bit vector address arithmetic.
        const uint8_t *ga = uniform_ptr(a_tile + (int64_t)kt * 128);
        const uint8_t *gb = uniform_ptr(b_tile + (int64_t)kt * 128);
        uint8_t *la = ldsA + buf * S::DATA_A + wave * 1024;
        uint8_t *lb = ldsB + buf * S::DATA_B + wave * 1024;
#pragma unroll
        for (int q = 0; q < S::QA; q++) dma16(ga + a_voff[q], la + q * S::NW * 1024);
#pragma unroll
        for (int q = 0; q < S::QB; q++) dma16(gb + b_voff[q], lb + q * S::NW * 1024);
    };

    // ---- per-lane LDS read bases
    const int a_row = wm * S::WTM + r16;
    const int b_row = wn * S::WTN + 16 * (r16 >> 2) + (r16 & 3);
    // low half = 16-byte chunk g, high half = chunk g + 4 (= address ^ 64)
    const int a_rd = a_row * 128 + ((g ^ swz_a(a_row)) << 4);
    const int b_rd = b_row * 128 + ((g ^ swz_b(b_row)) << 4);

    v4f acc[S::MT][S::NT];
#pragma unroll
    for (int i = 0; i < S::MT; i++)
#pragma unroll
        for (int j = 0; j < S::NT; j++) acc[i][j] = v4f{0.f, 0.f, 0.f, 0.f};

    const int KT = K >> 7;  // K % 128 == 0 (host checked)

    // ---- prologue: scales of super-step 0 and data of stage 0
    {
        uint32_t d0[4], d1[4];
        if (has_row0) load_scales(tid, 0, d0);
        if (TWO_ROWS) load_scales(tid + S::NTHR, 0, d1);
        issue_stage(0, 0);
        if (has_row0) park_scales(tid, 0, d0);
        if (TWO_ROWS) park_scales(tid + S::NTHR, 0, d1);
    }
    __builtin_amdgcn_s_waitcnt(0);  // vmcnt(0) expcnt(0) lgkmcnt(0)
    __syncthreads();

    const int nsuper = (KT + 3) >> 2;
    for (int ss = 0; ss < nsuper; ss++) {
        const int sbuf = ss & 1;
        // scales of this super-step: one dword per sub-tile, byte s = stage s
        int sa[S::MT], sb[S::NT];
#pragma unroll
        for (int i = 0; i < S::MT; i++) sa[i] = (int)ldsSA[(sbuf * 4 + g) * S::BM + a_row + 16 * i];
#pragma unroll
        for (int j = 0; j < S::NT; j++)
            sb[j] = (int)ldsSB[(sbuf * 4 + g) * S::BN + b_row + (j >> 2) * 64 + (j & 3) * 4];

        // prefetch the next super-step's scales into registers
        uint32_t d0[4], d1[4];
        const bool more = ss + 1 < nsuper;
        if (more) {
            if (has_row0) load_scales(tid, (ss + 1) * 16, d0);
            if (TWO_ROWS) load_scales(tid + S::NTHR, (ss + 1) * 16, d1);
        }

#define MX_STAGE(SIDX)                                                                              \
    {                                                                                               \
        const int kt = ss * 4 + SIDX;                                                               \
        if (kt < KT) {                                                                              \
            const int buf = kt & 1;                                                                 \
            if (kt + 1 < KT) issue_stage(kt + 1, buf ^ 1);                                          \
            if (SIDX == 3 && more) {                                                                \
                if (has_row0) park_scales(tid, sbuf ^ 1, d0);                                       \
                if (TWO_ROWS) park_scales(tid + S::NTHR, sbuf ^ 1, d1);                             \
            }                                                                                       \
            compute_stage<S, SIDX>(ldsA + buf * S::DATA_A, ldsB + buf * S::DATA_B, a_rd, a_rd ^ 64, b_rd, b_rd ^ 64, sa, sb, acc); \
            __builtin_amdgcn_s_waitcnt(0);                                                          \
            __syncthreads();                                                                        \
        }                                                                                           \
    }
        MX_STAGE(0)
        MX_STAGE(1)
        MX_STAGE(2)
        MX_STAGE(3)
#undef MX_STAGE
    }

    // ---- epilogue: lane holds, per (i, group of 4 j), 16 consecutive N of row a_row + 16 i
#pragma unroll
    for (int i = 0; i < S::MT; i++) {
        const int m = m0 + wm * S::WTM + 16 * i + r16;
#pragma unroll
        for (int jq = 0; jq < S::NT / 4; jq++) {
            const int n = n0 + wn * S::WTN + jq * 64 + 16 * g;
            float v[16];
#pragma unroll
            for (int jj = 0; jj < 4; jj++)
#pragma unroll
                for (int e = 0; e < 4; e++) v[4 * jj + e] = acc[i][jq * 4 + jj][e];
            if (m < M && n < N) store16<CDT>(c, (int64_t)m * ldc + n, v, N - n < 16 ? N - n : 16, c_vec != 0);
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

template <typename S, int CDT>
static int launch_tiled(const uint8_t *aq, const uint8_t *as, const uint8_t *bq, const uint8_t *bs, void *c, int64_t M,
                        int64_t N, int64_t K, int64_t lda, int64_t ldas, int64_t ldb, int64_t ldbs, int64_t ldc,
                        hipStream_t st) {
    const int tiles_m = (int)((M + S::BM - 1) / S::BM), tiles_n = (int)((N + S::BN - 1) / S::BN);
    const int esz = CDT == MX_FP32 ? 4 : 2;
    const int c_vec = aligned(c, 16) && (ldc * esz) % 16 == 0;
    const bool k512 = K % 512 == 0 && aligned(as, 16) && aligned(bs, 16) && ldas % 16 == 0 && ldbs % 16 == 0;
    dim3 grid((unsigned)(tiles_m * tiles_n)), block(S::NTHR);
    hipError_t e;
    if (k512) {
        auto kern = gemm_nt_kernel<S, CDT, true>;
        e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, S::LDS_BYTES);
        if (e != hipSuccess) return MX_ELAUNCH;
        kern<<<grid, block, S::LDS_BYTES, st>>>(aq, as, bq, bs, c, (int)M, (int)N, (int)K, lda, ldas, ldb, ldbs, ldc,
                                                tiles_m, tiles_n, c_vec);
    } else {
        auto kern = gemm_nt_kernel<S, CDT, false>;
        e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, S::LDS_BYTES);
        if (e != hipSuccess) return MX_ELAUNCH;
        kern<<<grid, block, S::LDS_BYTES, st>>>(aq, as, bq, bs, c, (int)M, (int)N, (int)K, lda, ldas, ldb, ldbs, ldc,
                                                tiles_m, tiles_n, c_vec);
    }
    return hipGetLastError() == hipSuccess ? MX_OK : MX_ELAUNCH;
}

template <int CDT>
static int gemm_dispatch(const uint8_t *aq, const uint8_t *as, const uint8_t *bq, const uint8_t *bs, void *c, int64_t M,
                         int64_t N, int64_t K, int64_t lda, int64_t ldas, int64_t ldb, int64_t ldbs, int64_t ldc,
                         hipStream_t st) {
    const bool tiled_ok = K % 128 == 0 && aligned(aq, 16) && aligned(bq, 16) && lda % 16 == 0 && ldb % 16 == 0 &&
                          aligned(as, 4) && aligned(bs, 4) && ldas % 4 == 0 && ldbs % 4 == 0 &&
                          M * lda < (int64_t)1 << 40 && 256 * lda < (int64_t)0x7FFFFFFF && 256 * ldb < (int64_t)0x7FFFFFFF &&
                          M < 0x7FFFFFFF && N < 0x7FFFFFFF && K < 0x7FFFFFFF &&
                          ((M + 255) / 256) * ((N + 255) / 256) < 0x7FFFFFFF;
    if (!tiled_ok) {
        int64_t blocks = (M * N + 255) / 256;
        if (blocks > 0x7FFFFFFF) return MX_EUNSUPPORTED;
        gemm_nt_generic_kernel<CDT><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(aq, as, bq, bs, c, M, N, K, lda, ldas,
                                                                                  ldb, ldbs, ldc);
        return hipGetLastError() == hipSuccess ? MX_OK : MX_ELAUNCH;
    }
    typedef GemmShape<256, 256, 2, 4> Big;
    return launch_tiled<Big, CDT>(aq, as, bq, bs, c, M, N, K, lda, ldas, ldb, ldbs, ldc, st);
}

extern "C" int mx_gemm_nt(const uint8_t *aq, const uint8_t *as, const uint8_t *bq, const uint8_t *bs, void *c,
                          int c_dtype, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldas, int64_t ldb,
                          int64_t ldbs, int64_t ldc, int epilogue, void *stream) {
    if (M < 0 || N < 0 || K < 0 || K % MX_BLOCK || lda < K || ldb < K || ldas < K / MX_BLOCK || ldbs < K / MX_BLOCK ||
        ldc < N)
        return MX_EINVAL;
    if (epilogue != MX_EPI_NONE) return MX_EUNSUPPORTED;
    if (M == 0 || N == 0) return MX_OK;
    hipStream_t st = (hipStream_t)stream;
    if (K == 0) {
        // An empty contraction is a zero matrix.
        int esz = c_dtype == MX_FP32 ? 4 : 2;
        hipError_t e = hipMemset2DAsync(c, (size_t)ldc * esz, 0, (size_t)N * esz, (size_t)M, st);
        return e == hipSuccess ? MX_OK : MX_ELAUNCH;
    }
    switch (c_dtype) {
    case MX_BF16: return gemm_dispatch<MX_BF16>(aq, as, bq, bs, c, M, N, K, lda, ldas, ldb, ldbs, ldc, st);
    case MX_FP16: return gemm_dispatch<MX_FP16>(aq, as, bq, bs, c, M, N, K, lda, ldas, ldb, ldbs, ldc, st);
    case MX_FP32: return gemm_dispatch<MX_FP32>(aq, as, bq, bs, c, M, N, K, lda, ldas, ldb, ldbs, ldc, st);
    default: return MX_EINVAL;
    }
}
