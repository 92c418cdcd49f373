// MXFP8 quantizers for gfx950: row axis, column axis, both at once, and SwiGLU -> MXFP8.
//
// All of them are HBM-streaming kernels: 16-byte coalesced loads, per-32 amax by a
// DPP quad reduction (row axis) or an in-register + cross-lane reduction (column
// axis), the UE8M0 byte from the fp32 exponent/mantissa bits, an exact multiply by
// 2^-e, and the hardware RTNE e4m3 conversion.  Semantics follow _quantize_block of
// the reference (src/kohakuwullm/kernels/mxfp8/quantize.py:39-56).
#include "mx_common.h"

namespace mx {
int num_cus();  // CUs of the current device (mx_gemm.hip)
}

namespace mx {

// ------------------------------------------------------------------------------------
// Row axis.  One lane owns 8 consecutive elements; the 4 lanes of a quad own one block.
// ------------------------------------------------------------------------------------

// OR the quad's byte into a dword holding the 4 bytes of a 16-lane row, in block order.
__device__ __forceinline__ uint32_t gather_row_scales(uint32_t byte, int lane) {
    uint32_t v = byte << ((lane & 12) << 1);
    v |= (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x124, 0xF, 0xF, true);  // row_ror:4
    v |= (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x128, 0xF, 0xF, true);  // row_ror:8
    return v;
}

template <int DT, int U, bool FLAT>
__global__ __launch_bounds__(256) void quant_rows_kernel(const void *__restrict__ x, uint32_t chunks_per_row,
                                                          int64_t sx_row, uint8_t *__restrict__ q, int64_t ldq,
                                                          uint8_t *__restrict__ s, int64_t lds, uint32_t total_chunks,
                                                          int pack_scales) {
    typedef typename Elem<DT>::type T;
    const int lane = threadIdx.x & 63;
    const uint32_t base = blockIdx.x * (uint32_t)(U * 256) + threadIdx.x;
    float v[U][8];
    int64_t qoff[U], soff[U];
    bool ok[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        uint32_t chunk = base + u * 256;
        ok[u] = chunk < total_chunks;
        int64_t xoff;
        if (FLAT) {
            xoff = (int64_t)chunk * 8;
            qoff[u] = (int64_t)chunk * 8;
            soff[u] = chunk >> 2;
        } else {
            uint32_t row = chunk / chunks_per_row;
            uint32_t col = chunk - row * chunks_per_row;
            xoff = (int64_t)row * sx_row + (int64_t)col * 8;
            qoff[u] = (int64_t)row * ldq + (int64_t)col * 8;
            soff[u] = (int64_t)row * lds + (col >> 2);
        }
        if (ok[u]) {
            Elem<DT>::load8((const T *)x + xoff, v[u]);
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) v[u][i] = 0.0f;
        }
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
        float amax = quad_max(amax8(v[u]));
        uint32_t byte = scale_byte(amax);
        float inv = inv_scale(byte);
        uint32_t packed = gather_row_scales(byte, lane);
        if (ok[u]) {
            v2i codes;
            codes[0] = (int)pack4_e4m3(v[u][0] * inv, v[u][1] * inv, v[u][2] * inv, v[u][3] * inv);
            codes[1] = (int)pack4_e4m3(v[u][4] * inv, v[u][5] * inv, v[u][6] * inv, v[u][7] * inv);
            *(v2i *)(q + qoff[u]) = codes;
            // The 16 lanes of a DPP row hold 4 consecutive blocks.  They are all valid or
            // the tail of the tensor cuts the group, in which case bytes are stored singly.
            bool group_full = ((base + u * 256) | 15u) < total_chunks;
            if (pack_scales && group_full) {
                if ((lane & 15) == 0) *(uint32_t *)(s + soff[u]) = packed;
            } else if ((lane & 3) == 0) {
                s[soff[u]] = (uint8_t)byte;
            }
        }
    }
}

// (T, H, D) attention operand, blocks along D: the row quantizer with a head stride and an
// optional per-(head, channel) fp32 mean subtracted in registers (the smoothing of the MXFP8
// QK^T operands: no shifted copy of the operand reaches memory).  Outputs are contiguous
// (T, H*D) codes and (T, H*D/32) scale bytes.  D % 32 == 0, so a chunk of 8 stays inside a head.
template <int DT, bool SMOOTH>
__global__ __launch_bounds__(256) void quant_heads_kernel(const void *__restrict__ x, uint32_t chunks_per_row,
                                                           uint32_t chunks_per_head, int64_t stride_t, int64_t stride_h,
                                                           const float *__restrict__ mu, uint8_t *__restrict__ q,
                                                           uint8_t *__restrict__ s, uint32_t total_chunks,
                                                           int pack_scales) {
    typedef typename Elem<DT>::type T;
    constexpr int U = 4;
    const int lane = threadIdx.x & 63;
    const uint32_t base = blockIdx.x * (uint32_t)(U * 256) + threadIdx.x;
    float v[U][8];
    bool ok[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        const uint32_t chunk = base + u * 256;
        ok[u] = chunk < total_chunks;
        const uint32_t row = chunk / chunks_per_row, col = chunk - row * chunks_per_row;
        const uint32_t head = col / chunks_per_head, d = col - head * chunks_per_head;
        if (ok[u]) {
            Elem<DT>::load8((const T *)x + (int64_t)row * stride_t + (int64_t)head * stride_h + (int64_t)d * 8, v[u]);
            if (SMOOTH) {
                const v4f a = ((const v4f *)(mu + (int64_t)col * 8))[0], b = ((const v4f *)(mu + (int64_t)col * 8))[1];
#pragma unroll
                for (int i = 0; i < 4; i++) v[u][i] -= a[i], v[u][4 + i] -= b[i];
            }
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) v[u][i] = 0.0f;
        }
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
        const uint32_t chunk = base + u * 256;
        float amax = quad_max(amax8(v[u]));
        uint32_t byte = scale_byte(amax);
        float inv = inv_scale(byte);
        uint32_t packed = gather_row_scales(byte, lane);
        if (ok[u]) {
            v2i codes;
            codes[0] = (int)pack4_e4m3(v[u][0] * inv, v[u][1] * inv, v[u][2] * inv, v[u][3] * inv);
            codes[1] = (int)pack4_e4m3(v[u][4] * inv, v[u][5] * inv, v[u][6] * inv, v[u][7] * inv);
            *(v2i *)(q + (int64_t)chunk * 8) = codes;
            bool group_full = (chunk | 15u) < total_chunks;
            if (pack_scales && group_full) {
                if ((lane & 15) == 0) *(uint32_t *)(s + (chunk >> 2)) = packed;
            } else if ((lane & 3) == 0) {
                s[chunk >> 2] = (uint8_t)byte;
            }
        }
    }
}

// Any strides: one thread per block.  The slow path for doubly-strided views.
template <int DT>
__global__ __launch_bounds__(256) void quant_rows_generic_kernel(const void *__restrict__ x, int64_t M, int64_t KB,
                                                                  int64_t sx_row, int64_t sx_col,
                                                                  uint8_t *__restrict__ q, int64_t ldq,
                                                                  uint8_t *__restrict__ s, int64_t lds) {
    typedef typename Elem<DT>::type T;
    int64_t blk = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (blk >= M * KB) return;
    int64_t row = blk / KB, kb = blk - row * KB;
    const T *p = (const T *)x + row * sx_row + kb * MX_BLOCK * sx_col;
    float v[MX_BLOCK];
    float amax = 0.0f;
#pragma unroll
    for (int i = 0; i < MX_BLOCK; i++) {
        v[i] = Elem<DT>::load1(p + i * sx_col);
        amax = fmaxf(amax, fabsf(v[i]));
    }
    uint32_t byte = scale_byte(amax);
    float inv = inv_scale(byte);
    uint8_t *qo = q + row * ldq + kb * MX_BLOCK;
#pragma unroll
    for (int i = 0; i < MX_BLOCK; i += 4) {
        uint32_t c = pack4_e4m3(v[i] * inv, v[i + 1] * inv, v[i + 2] * inv, v[i + 3] * inv);
        qo[i] = (uint8_t)c;
        qo[i + 1] = (uint8_t)(c >> 8);
        qo[i + 2] = (uint8_t)(c >> 16);
        qo[i + 3] = (uint8_t)(c >> 24);
    }
    s[row * lds + kb] = (uint8_t)byte;
}

// ------------------------------------------------------------------------------------
// Column axis (and dual).  A 256-thread workgroup owns a 128 (M) x 128 (K) tile.  Thread
// (cg = t%16, rg = t/16) holds rows rg*8..+7 x columns cg*8..+7, so wave w holds exactly
// the w-th 32-row block of the tile: the column amax is an in-register max over 8 rows
// and a max across the wave's 4 row groups (lanes l, l^16, l^32, l^48).  Codes are
// transposed through LDS so the (K,M) output is written in full 128-byte rows.
//
// The same with R = 4 rows per thread: a 128 (M) x 64 (K) tile, thread (cg = t%8, rg = t/8)
// holds rows rg*4..+3 x columns cg*8..+7, wave w again the w-th 32-row block (8 row groups:
// lanes l^8, l^16, l^32).  Half the values per thread, half the registers (63 against 90 for
// both axes, 98 against 162 for SwiGLU'), twice the resident waves -- and slower: inside a
// feed-forward step on 16384 x 1536 / 16384 x 4096 bf16, both axes 28.5 against 26.8 us, SwiGLU
// 91.8 against 80.8, SwiGLU' 172.9 against 149.3.  A tile row of 64 columns is a 128-byte run
// where R = 8 reads and writes 256-byte ones, and every scale row is cut into twice as many
// pieces.  Bit-identical results; R = 8 is what the launchers below instantiate.
// ------------------------------------------------------------------------------------

#define QC_TILE 128
#define QC_PITCH 136  // bytes per transposed LDS row (8-byte aligned, staggers banks)

struct QuantTileOut {
    uint8_t *qT;  // (K,M) codes, blocks along M
    int64_t ldqT;
    uint8_t *sT;  // (K,M/32)
    int64_t ldsT;
    uint8_t *q;  // (M,K) codes, blocks along K (only when ROWS)
    int64_t ldq;
    uint8_t *s;  // (M,K/32)
    int64_t lds;
    int pack_row_scales, pack_col_scales;
    // Stage-major code layouts (0: row-major with the pitches above).  q_ks: 128-column panels
    // of q, panel p at p * q_ks, row m of it at m * 128.  qT_ks: the same for qT (panels of 128
    // of its M columns).  A GEMM then finds a K stage of a tile in one contiguous run.
    int64_t q_ks, qT_ks;
};

// Quantizes the 128 x TK tile (TK = 16 R columns) held as v[R][8] per thread (rows m0 + rg*R + i,
// columns kc0 + cg*8 + c of the OUTPUT matrix, which has K columns and M rows) along the column
// axis, and along the row axis too when ROWS.  `tile`/`tscale` are the workgroup's LDS
// staging buffers; the caller must not touch them until the function's trailing barrier.
template <int R>
struct TileGeom {
    static_assert(R == 8 || R == 4, "8 rows x 8 columns or 4 rows x 8 columns per thread");
    static constexpr int CGS = 2 * R;        // column groups (of 8) across the tile: lanes of one tile row
    static constexpr int TK = 8 * CGS;       // tile columns
    static constexpr int RGS = 256 / CGS;    // row groups (of R rows): 128 rows
    static __device__ __forceinline__ int cg(int t) { return t % CGS; }
    static __device__ __forceinline__ int rg(int t) { return t / CGS; }
};

template <bool ROWS, int R = 8, bool NTS = false>  // NTS: the code stores carry the non-temporal hint
__device__ __forceinline__ void quant_tile(float (&v)[R][8], const QuantTileOut &o, int64_t M, int64_t K, int64_t m0,
                                           int64_t kc0, uint8_t *tile, uint8_t *tscale) {
    typedef TileGeom<R> G;
    const int t = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;
    const int cg = G::cg(t), rg = G::rg(t);
    const int64_t col = kc0 + cg * 8;
    const int64_t row0 = m0 + rg * R;
    const bool col_ok = col < K;
    const bool blk_ok = m0 + wave * 32 < M;

    if (ROWS) {
        // Row-axis outputs: the 4 lanes of a quad hold 32 consecutive columns of a row.
#pragma unroll
        for (int i = 0; i < R; i++) {
            float amax = quad_max(amax8(v[i]));
            uint32_t byte = scale_byte(amax);
            float inv = inv_scale(byte);
            // the scale bytes of a tile row in one word: four (R = 8, 16 lanes) or two (R = 4, 8 lanes)
            uint32_t packed;
            if (R == 8) {
                packed = gather_row_scales(byte, lane);
            } else {
                packed = byte << ((lane & 4) << 1);
                // row_ror:12 = every lane takes the word of the lane 4 above it in its 16-lane row: lane 0 (8) of a tile
                // row gets block 1's byte from lane 4 (12)
                packed |= (uint32_t)__builtin_amdgcn_mov_dpp((int)packed, 0x12C, 0xF, 0xF, true);
            }
            if (col_ok && blk_ok) {
                v2i codes;
                codes[0] = (int)pack4_e4m3(v[i][0] * inv, v[i][1] * inv, v[i][2] * inv, v[i][3] * inv);
                codes[1] = (int)pack4_e4m3(v[i][4] * inv, v[i][5] * inv, v[i][6] * inv, v[i][7] * inv);
                stream_store<NTS>((v2i *)(o.q + (o.q_ks ? (col >> 7) * o.q_ks + (row0 + i) * 128 + (col & 127) : (row0 + i) * o.ldq + col)), codes);
                uint8_t *sp = o.s + (row0 + i) * o.lds + (col >> 5);
                bool full = kc0 + G::TK <= K;
                if (o.pack_row_scales && full) {
                    if (cg == 0) {
                        if (R == 8) *(uint32_t *)sp = packed;
                        else *(uint16_t *)sp = (uint16_t)packed;
                    }
                } else if ((cg & 3) == 0) {
                    *sp = (uint8_t)byte;
                }
            }
        }
    }

    // Column amax over this wave's 32 rows.
    float cm[8];
#pragma unroll
    for (int c = 0; c < 8; c++) {
        float a = fmaxf(fabsf(v[0][c]), fabsf(v[1][c]));
#pragma unroll
        for (int i = 2; i < R; i++) a = fmaxf(a, fabsf(v[i][c]));
        cm[c] = a;
    }
#pragma unroll
    for (int c = 0; c < 8; c++) {
        if (R == 4) {  // lane ^ 8: the other half of the 16-lane row
            const int x = __builtin_amdgcn_mov_dpp((int)f2bits(cm[c]), 0x128, 0xF, 0xF, true);  // row_ror:8
            cm[c] = fmaxf(cm[c], bits2f((uint32_t)x));
        }
        cm[c] = fmaxf(cm[c], __shfl_xor(cm[c], 16, 64));
        cm[c] = fmaxf(cm[c], __shfl_xor(cm[c], 32, 64));
    }
#pragma unroll
    for (int c = 0; c < 8; c++) {
        uint32_t byte = scale_byte(cm[c]);
        float inv = inv_scale(byte);
        uint8_t *dst = tile + (cg * 8 + c) * QC_PITCH + rg * R;
        if (R == 8) {
            v2i codes;
            codes[0] = (int)pack4_e4m3(v[0][c] * inv, v[1][c] * inv, v[2][c] * inv, v[3][c] * inv);
            codes[1] = (int)pack4_e4m3(v[R - 4][c] * inv, v[R - 3][c] * inv, v[R - 2][c] * inv, v[R - 1][c] * inv);
            *(v2i *)dst = codes;
        } else {
            *(uint32_t *)dst = pack4_e4m3(v[0][c] * inv, v[1][c] * inv, v[2][c] * inv, v[3][c] * inv);
        }
        if (rg % (32 / R) == 0) tscale[(cg * 8 + c) * 4 + wave] = (uint8_t)byte;
    }
    __syncthreads();

    // Transposed codes: TK rows of 128 bytes, 16 bytes per thread per pass.
#pragma unroll
    for (int j = 0; j < G::TK / 32; j++) {
        int kr = j * 32 + (t >> 3), ch = t & 7;
        if (kc0 + kr < K && m0 + ch * 16 < M) {
            const v2i *src = (const v2i *)(tile + kr * QC_PITCH + ch * 16);
            v4i w;
            v2i a = src[0], b = src[1];
            w[0] = a[0];
            w[1] = a[1];
            w[2] = b[0];
            w[3] = b[1];
            stream_store<NTS>((v4i *)(o.qT + (o.qT_ks ? (m0 >> 7) * o.qT_ks + (kc0 + kr) * 128 : (kc0 + kr) * o.ldqT + m0) + ch * 16), w);
        }
    }
    if (t < G::TK && kc0 + t < K) {
        uint8_t *sp = o.sT + (kc0 + t) * o.ldsT + (m0 >> 5);
        int64_t nb = (M - m0) >> 5;
        if (o.pack_col_scales && nb >= 4) {
            *(uint32_t *)sp = *(const uint32_t *)(tscale + t * 4);
        } else {
            for (int b = 0; b < 4 && b < nb; b++) sp[b] = tscale[t * 4 + b];
        }
    }
    __syncthreads();
}

// quant_tile<ROWS, 8, NTS> for a tile of 16-bit values kept as loaded (r[i]: row i's eight values, packed): every value
// is converted where it is used, three times instead of once, and the thread holds 32 registers of tile instead of 64.
// The plain row + token axis quantizer then fits 64 registers and eight waves per SIMD (90 registers and five with the
// tile in fp32), so that the 1536 tiles of a 16384 x 1536 activation are resident at once instead of in 1.2 rounds.
// Same arithmetic on the same values: bit-identical outputs.
template <int DT, bool ROWS, bool NTS>
__device__ __forceinline__ void quant_tile_raw(typename Elem<DT>::raw (&r)[8], bool ok, const QuantTileOut &o, int64_t M,
                                               int64_t K, int64_t m0, int64_t kc0, uint8_t *tile, uint8_t *tscale) {
    typedef TileGeom<8> G;
    typedef Elem<DT> E;
    const int t = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;
    const int cg = G::cg(t), rg = G::rg(t);
    const int64_t col = kc0 + cg * 8;
    const int64_t row0 = m0 + rg * 8;
    auto val = [&](int i, int c) { return ok ? E::elem(r[i], c) : 0.0f; };

    if (ROWS) {
#pragma unroll
        for (int i = 0; i < 8; i++) {
            float v[8];
#pragma unroll
            for (int c = 0; c < 8; c++) v[c] = val(i, c);
            const float amax = quad_max(amax8(v));
            const uint32_t byte = scale_byte(amax);
            const float inv = inv_scale(byte);
            const uint32_t packed = gather_row_scales(byte, lane);
            if (ok) {
                v2i codes;
                codes[0] = (int)pack4_e4m3(v[0] * inv, v[1] * inv, v[2] * inv, v[3] * inv);
                codes[1] = (int)pack4_e4m3(v[4] * inv, v[5] * inv, v[6] * inv, v[7] * inv);
                stream_store<NTS>((v2i *)(o.q + (o.q_ks ? (col >> 7) * o.q_ks + (row0 + i) * 128 + (col & 127) : (row0 + i) * o.ldq + col)), codes);
                uint8_t *sp = o.s + (row0 + i) * o.lds + (col >> 5);
                const bool full = kc0 + G::TK <= K;
                if (o.pack_row_scales && full) {
                    if (cg == 0) *(uint32_t *)sp = packed;
                } else if ((cg & 3) == 0) {
                    *sp = (uint8_t)byte;
                }
            }
        }
    }
    // The column pass converts the raw values again.  Without this the compiler keeps the 64 conversions of the row
    // pass alive for it, which is the register cost this function exists to avoid.
#pragma unroll
    for (int i = 0; i < 8; i++) asm volatile("" : "+v"(r[i]));
#pragma unroll
    for (int c = 0; c < 8; c++) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = val(i, c);
        float cm = amax8(v);
        cm = fmaxf(cm, __shfl_xor(cm, 16, 64));
        cm = fmaxf(cm, __shfl_xor(cm, 32, 64));
        const uint32_t byte = scale_byte(cm);
        const float inv = inv_scale(byte);
        v2i codes;
        codes[0] = (int)pack4_e4m3(v[0] * inv, v[1] * inv, v[2] * inv, v[3] * inv);
        codes[1] = (int)pack4_e4m3(v[4] * inv, v[5] * inv, v[6] * inv, v[7] * inv);
        *(v2i *)(tile + (cg * 8 + c) * QC_PITCH + rg * 8) = codes;
        if ((rg & 3) == 0) tscale[(cg * 8 + c) * 4 + wave] = (uint8_t)byte;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < G::TK / 32; j++) {
        const int kr = j * 32 + (t >> 3), ch = t & 7;
        if (kc0 + kr < K && m0 + ch * 16 < M) {
            const v2i *src = (const v2i *)(tile + kr * QC_PITCH + ch * 16);
            const v2i a = src[0], b = src[1];
            stream_store<NTS>((v4i *)(o.qT + (o.qT_ks ? (m0 >> 7) * o.qT_ks + (kc0 + kr) * 128 : (kc0 + kr) * o.ldqT + m0) + ch * 16),
                              v4i{a[0], a[1], b[0], b[1]});
        }
    }
    if (t < G::TK && kc0 + t < K) {
        uint8_t *sp = o.sT + (kc0 + t) * o.ldsT + (m0 >> 5);
        const int64_t nb = (M - m0) >> 5;
        if (o.pack_col_scales && nb >= 4) {
            *(uint32_t *)sp = *(const uint32_t *)(tscale + t * 4);
        } else {
            for (int b = 0; b < 4 && b < nb; b++) sp[b] = tscale[t * 4 + b];
        }
    }
    __syncthreads();
}

// Loads the thread's R rows of 8 values of one operand raw (all loads in flight before any conversion).
template <int DT, int R, bool NT>
__device__ __forceinline__ void load_rows(const void *x, int64_t first, int64_t ld, typename Elem<DT>::raw (&r)[R]) {
    typedef typename Elem<DT>::type T;
#pragma unroll
    for (int i = 0; i < R; i++) r[i] = Elem<DT>::template load_raw<NT>((const T *)x + first + i * ld);
}

// RAW (16-bit inputs, R = 8): the tile stays packed as loaded (quant_tile_raw): 64 registers, eight waves per SIMD.
template <int DT, bool DUAL, int R, bool RAW = false>
__global__ __launch_bounds__(256) void quant_cols_kernel(const void *__restrict__ x, int64_t M, int64_t K, int64_t ldx,
                                                          QuantTileOut o) {
    typedef TileGeom<R> G;
    __shared__ __attribute__((aligned(16))) uint8_t tile[G::TK * QC_PITCH];
    __shared__ __attribute__((aligned(4))) uint8_t tscale[G::TK * 4];
    const int t = threadIdx.x;
    const int64_t m0 = (int64_t)blockIdx.y * QC_TILE, k0 = (int64_t)blockIdx.x * G::TK;
    const int64_t col = k0 + G::cg(t) * 8;
    const int64_t row0 = m0 + G::rg(t) * R;
    const bool ok = col < K && m0 + (t >> 6) * 32 < M;  // K % 8 == 0 and M % 32 == 0
    // the thread's loads go out together (row by row, each waited for the one before it)
    typename Elem<DT>::raw r[R];
    // both axes at once is the activation path of a training step, where the 16-bit input is not read again soon: its
    // loads carry the non-temporal hint; the codes are read by the next GEMM and are stored plainly
    if (ok) load_rows<DT, R, DUAL>(x, row0 * ldx + col, ldx, r);
    if constexpr (RAW) {
        static_assert(DT != MX_FP32 && R == 8, "a packed tile of 16-bit values");
        quant_tile_raw<DT, DUAL, false>(r, ok, o, M, K, m0, k0, tile, tscale);
        return;
    }
    float v[R][8];
#pragma unroll
    for (int i = 0; i < R; i++) {
        if (ok) {
            Elem<DT>::unpack(r[i], v[i]);
        } else {
#pragma unroll
            for (int c = 0; c < 8; c++) v[i][c] = 0.0f;
        }
    }
    quant_tile<DUAL, R>(v, o, M, K, m0, k0, tile, tscale);
}

// RMSNorm in front of both quantizers: y = (x * rstd[row]) * w[col] in fp32 -- the two products in the order
// rmsnorm_quant_kernel forms them, so the row-axis pair equals that kernel's bit for bit -- then the tile quantizer.
// rstd comes from a first pass over x (mx_rmsnorm_quantize asked for nothing else); the second read of an activation
// that fits the last-level cache is served from there.  Neither the 16-bit normalized activation nor a transposed copy
// of it reaches memory.
template <int DT, int WDT>
__global__ __launch_bounds__(256) void rmsnorm_quant_dual_kernel(const void *__restrict__ x, int64_t M, int64_t K, int64_t ldx,
                                                                  const void *__restrict__ w, const float *__restrict__ rstd,
                                                                  QuantTileOut o) {
    typedef TileGeom<8> G;
    typedef typename Elem<WDT>::type TW;
    __shared__ __attribute__((aligned(16))) uint8_t tile[G::TK * QC_PITCH];
    __shared__ __attribute__((aligned(4))) uint8_t tscale[G::TK * 4];
    const int t = threadIdx.x;
    const int64_t m0 = (int64_t)blockIdx.y * QC_TILE, k0 = (int64_t)blockIdx.x * G::TK;
    const int64_t col = k0 + G::cg(t) * 8;
    const int64_t row0 = m0 + G::rg(t) * 8;
    const bool ok = col < K && m0 + (t >> 6) * 32 < M;  // K % 8 == 0 and M % 32 == 0
    float v[8][8];
    typename Elem<DT>::raw r[8];
    float wv[8], rs[8];
    if (ok) {
        load_rows<DT, 8, false>(x, row0 * ldx + col, ldx, r);
        const v4f r0 = *(const v4f *)(rstd + row0), r1 = *(const v4f *)(rstd + row0 + 4);
#pragma unroll
        for (int i = 0; i < 4; i++) rs[i] = r0[i], rs[4 + i] = r1[i];
        if (w) {
            Elem<WDT>::load8((const TW *)w + col, wv);
        } else {
#pragma unroll
            for (int c = 0; c < 8; c++) wv[c] = 1.0f;
        }
    }
#pragma unroll
    for (int i = 0; i < 8; i++) {
        if (ok) {
            Elem<DT>::unpack(r[i], v[i]);
#pragma unroll
            for (int c = 0; c < 8; c++) v[i][c] = w ? v[i][c] * rs[i] * wv[c] : v[i][c] * rs[i];
        } else {
#pragma unroll
            for (int c = 0; c < 8; c++) v[i][c] = 0.0f;
        }
    }
    quant_tile<true, 8>(v, o, M, K, m0, k0, tile, tscale);
}

// Several matrices behind one launch: workgroup `id` finds its matrix in the running tile
// totals and quantizes one 128 x 128 tile of it along both axes.  For the once-per-step
// requantization of all weight matrices of a model, where a launch per matrix (and per axis)
// costs more than the bytes it moves.
#define MX_QUANT_BATCH_MAX 24
struct QuantBatchArgs {
    const void *x[MX_QUANT_BATCH_MAX];
    int64_t M[MX_QUANT_BATCH_MAX], K[MX_QUANT_BATCH_MAX], ldx[MX_QUANT_BATCH_MAX];
    QuantTileOut o[MX_QUANT_BATCH_MAX];
    int tile_end[MX_QUANT_BATCH_MAX];  // tiles of problems 0..j
    int tiles_k[MX_QUANT_BATCH_MAX];
    int count;
};

template <int DT>
__global__ __launch_bounds__(256) void quant_dual_batch_kernel(QuantBatchArgs b) {
    typedef typename Elem<DT>::type T;
    __shared__ __attribute__((aligned(16))) uint8_t tile[QC_TILE * QC_PITCH];
    __shared__ __attribute__((aligned(4))) uint8_t tscale[QC_TILE * 4];
    const int t = threadIdx.x;
    int j = 0;
    while (j + 1 < b.count && (int)blockIdx.x >= b.tile_end[j]) j++;
    const int local = (int)blockIdx.x - (j ? b.tile_end[j - 1] : 0);
    const int64_t M = b.M[j], K = b.K[j], ldx = b.ldx[j];
    const void *x = b.x[j];
    const int64_t m0 = (int64_t)(local / b.tiles_k[j]) * QC_TILE, k0 = (int64_t)(local % b.tiles_k[j]) * QC_TILE;
    const int64_t col = k0 + (t & 15) * 8;
    const int64_t row0 = m0 + (t >> 4) * 8;
    const bool ok = col < K && m0 + (t >> 6) * 32 < M;
    float v[8][8];
    typename Elem<DT>::raw r[8];  // eight loads in flight, then the conversions
    if (ok) {
#pragma unroll
        for (int i = 0; i < 8; i++) r[i] = Elem<DT>::load_raw((const T *)x + (row0 + i) * ldx + col);
    }
#pragma unroll
    for (int i = 0; i < 8; i++) {
        if (ok) {
            Elem<DT>::unpack(r[i], v[i]);
        } else {
#pragma unroll
            for (int c = 0; c < 8; c++) v[i][c] = 0.0f;
        }
    }
    quant_tile<true>(v, b.o[j], M, K, m0, k0, tile, tscale);
}

__device__ __forceinline__ float sigmoid_fast(float x) { return sigmoid_f32(x); }

// h = silu(g) * u from the fused projection output gu (M, 2H) (gate half first), quantized
// along both axes: (q,s) (M,H) for the down projection's forward, (qT,sT) (H,M) for its wgrad.
template <int DT, int R>
__global__ __launch_bounds__(256) void swiglu_quant_dual_kernel(const void *__restrict__ gu, int64_t M, int64_t H,
                                                                 int64_t ldgu, QuantTileOut o) {
    typedef TileGeom<R> G;
    __shared__ __attribute__((aligned(16))) uint8_t tile[G::TK * QC_PITCH];
    __shared__ __attribute__((aligned(4))) uint8_t tscale[G::TK * 4];
    const int t = threadIdx.x;
    const int64_t m0 = (int64_t)blockIdx.y * QC_TILE, k0 = (int64_t)blockIdx.x * G::TK;
    const int64_t col = k0 + G::cg(t) * 8;
    const int64_t row0 = m0 + G::rg(t) * R;
    const bool ok = col < H && m0 + (t >> 6) * 32 < M;
    float v[R][8];
    typename Elem<DT>::raw rg[R], ru[R];  // all loads in flight before the first conversion
    if (ok) {
        load_rows<DT, R, true>(gu, row0 * ldgu + col, ldgu, rg);
        load_rows<DT, R, true>(gu, row0 * ldgu + H + col, ldgu, ru);
    }
#pragma unroll
    for (int i = 0; i < R; i++) {
        if (ok) {
            float g[8], u[8];
            Elem<DT>::unpack(rg[i], g);
            Elem<DT>::unpack(ru[i], u);
#pragma unroll
            for (int c = 0; c < 8; c++) v[i][c] = g[c] * sigmoid_fast(g[c]) * u[c];
        } else {
#pragma unroll
            for (int c = 0; c < 8; c++) v[i][c] = 0.0f;
        }
    }
    // hundreds of MB in, hundreds out, nothing of it small enough to be found in a cache by its consumer: all hinted
    quant_tile<true, R, true>(v, o, M, H, m0, k0, tile, tscale);
}

// SwiGLU backward fused with both quantizers.  Reads dh (M,H) and the saved projection
// output gu (M,2H); forms dgate = dh * u * s * (1 + g (1 - s)) and dup = dh * g * s with
// s = sigmoid(g) in fp32 (elementwise/swiglu.py:108-119, experts_bwd.py:145-148 of the
// reference); writes dpre = [dgate | dup] quantized along 2H ((q,s): (M,2H)) for the input
// projection's dgrad and along M ((qT,sT): (2H,M)) for its wgrad.  o.q/o.qT address the
// full (M,2H) / (2H,M) outputs.
template <int DT, int R>
__global__ __launch_bounds__(256) void swiglu_bwd_quant_dual_kernel(const void *__restrict__ dh, int64_t lddh,
                                                                     const void *__restrict__ gu, int64_t ldgu,
                                                                     int64_t M, int64_t H, QuantTileOut o) {
    typedef TileGeom<R> G;
    __shared__ __attribute__((aligned(16))) uint8_t tile[G::TK * QC_PITCH];
    __shared__ __attribute__((aligned(4))) uint8_t tscale[G::TK * 4];
    const int t = threadIdx.x;
    const int64_t m0 = (int64_t)blockIdx.y * QC_TILE, k0 = (int64_t)blockIdx.x * G::TK;
    const int64_t col = k0 + G::cg(t) * 8;
    const int64_t row0 = m0 + G::rg(t) * R;
    const bool ok = col < H && m0 + (t >> 6) * 32 < M;
    float v[R][8], w[R][8];
    // All loads of the thread go out before the first conversion.  Written row by row (load three,
    // convert, next row) the compiler kept that order and every thread had 48 bytes in flight at a time,
    // with a memory latency in front of each of its rows.
    typename Elem<DT>::raw rg[R], ru[R], rd[R];
    if (ok) {
        load_rows<DT, R, true>(gu, row0 * ldgu + col, ldgu, rg);
        load_rows<DT, R, true>(gu, row0 * ldgu + H + col, ldgu, ru);
        load_rows<DT, R, true>(dh, row0 * lddh + col, lddh, rd);
    }
#pragma unroll
    for (int i = 0; i < R; i++) {
        if (ok) {
            float g[8], u[8], d[8];
            Elem<DT>::unpack(rg[i], g);
            Elem<DT>::unpack(ru[i], u);
            Elem<DT>::unpack(rd[i], d);
#pragma unroll
            for (int c = 0; c < 8; c++) {
                float sg = sigmoid_fast(g[c]);
                v[i][c] = d[c] * u[c] * sg * (1.0f + g[c] * (1.0f - sg));
                w[i][c] = d[c] * g[c] * sg;
            }
        } else {
#pragma unroll
            for (int c = 0; c < 8; c++) v[i][c] = w[i][c] = 0.0f;
        }
    }
    // The gate half occupies output columns [0,H), the up half [H,2H): same tile, shifted.
    // Columns at or beyond H inside the gate-half tile are masked by passing K = H.
    quant_tile<true, R, true>(v, o, M, H, m0, k0, tile, tscale);
    QuantTileOut o2 = o;
    o2.q += o.q_ks ? (H >> 7) * o.q_ks : H;
    o2.s += H / MX_BLOCK;
    o2.qT += o.qT_ks ? H * 128 : H * o.ldqT;
    o2.sT += H * o.ldsT;
    quant_tile<true, R, true>(w, o2, M, H, m0, k0, tile, tscale);
}

// ------------------------------------------------------------------------------------
// silu(gate) * up in fp32 -> row-axis MXFP8 (fused_act.py:37-66 of the reference).
// ------------------------------------------------------------------------------------

template <int DT, int U>
__global__ __launch_bounds__(256) void swiglu_quant_rows_kernel(const void *__restrict__ g, const void *__restrict__ up,
                                                                 uint32_t chunks_per_row, int64_t ldg, int64_t ldu,
                                                                 uint8_t *__restrict__ q, int64_t ldq,
                                                                 uint8_t *__restrict__ s, int64_t lds,
                                                                 uint32_t total_chunks, int pack_scales) {
    typedef typename Elem<DT>::type T;
    const int lane = threadIdx.x & 63;
    const uint32_t base = blockIdx.x * (uint32_t)(U * 256) + threadIdx.x;
    float a[U][8], b[U][8];
    int64_t qoff[U], soff[U];
    bool ok[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
        uint32_t chunk = base + u * 256;
        ok[u] = chunk < total_chunks;
        uint32_t row = chunk / chunks_per_row;
        uint32_t col = chunk - row * chunks_per_row;
        qoff[u] = (int64_t)row * ldq + (int64_t)col * 8;
        soff[u] = (int64_t)row * lds + (col >> 2);
        if (ok[u]) {
            Elem<DT>::load8((const T *)g + (int64_t)row * ldg + (int64_t)col * 8, a[u]);
            Elem<DT>::load8((const T *)up + (int64_t)row * ldu + (int64_t)col * 8, b[u]);
        } else {
#pragma unroll
            for (int i = 0; i < 8; i++) a[u][i] = b[u][i] = 0.0f;
        }
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; i++) {
            float gv = a[u][i];
            v[i] = gv * sigmoid_f32(gv) * b[u][i];
        }
        float amax = quad_max(amax8(v));
        uint32_t byte = scale_byte(amax);
        float inv = inv_scale(byte);
        uint32_t packed = gather_row_scales(byte, lane);
        if (ok[u]) {
            v2i codes;
            codes[0] = (int)pack4_e4m3(v[0] * inv, v[1] * inv, v[2] * inv, v[3] * inv);
            codes[1] = (int)pack4_e4m3(v[4] * inv, v[5] * inv, v[6] * inv, v[7] * inv);
            *(v2i *)(q + qoff[u]) = codes;
            bool group_full = ((base + u * 256) | 15u) < total_chunks;
            if (pack_scales && group_full) {
                if ((lane & 15) == 0) *(uint32_t *)(s + soff[u]) = packed;
            } else if ((lane & 3) == 0) {
                s[soff[u]] = (uint8_t)byte;
            }
        }
    }
}

// ------------------------------------------------------------------------------------
// Column-axis quantizer over expert-sorted rows, for the routed experts' MXFP8 WGRAD.
// WGRAD contracts the rows an expert owns, so the 32-row blocks must not straddle two experts:
// every expert's segment is laid out from a fresh multiple of 128 in a padded position space
// (tile t of 128 rows = positions [128 t, 128 t + 128)), rows past the segment's end are zero.
// Row tile -> (expert, first row) is resolved on the device from `offsets`, like the GEMMs.
// Sources: SRC_PLAIN  x[index[m] or m] (optionally times row_scale[scale_index[m]] in fp32,
//                     the gate applied to dout rows: grouped.py:218-221 of the reference)
//          SRC_SWIGLU silu(pre[m][c]) * pre[m][H + c] in fp32 (moe.py:288-290 rebuilds h from pre)
// ------------------------------------------------------------------------------------

enum { SRC_PLAIN = 0, SRC_SWIGLU = 1 };

struct GroupedQuantArgs {
    const void *x;
    int64_t ldx;
    int C;  // output columns of x to quantize (H for SRC_SWIGLU, whose x has 2H columns)
    const int32_t *index;
    const void *row_scale;
    const int32_t *scale_index;
    int scale_f32;
    const int32_t *offsets;
    int E;
    int span;  // column tiles per workgroup
};

template <int DT, int SRC>
__global__ __launch_bounds__(256) void quant_cols_grouped_kernel(GroupedQuantArgs a, QuantTileOut o, int64_t mpad) {
    typedef typename Elem<DT>::type T;
    __shared__ __attribute__((aligned(16))) uint8_t tile[QC_TILE * QC_PITCH];
    __shared__ __attribute__((aligned(4))) uint8_t tscale[QC_TILE * 4];
    const int t = threadIdx.x;
    const int rt = blockIdx.y;
    // tile_owner: the expert whose tiles contain rt.  The first wave looks at 64 experts at a time
    // (one coalesced read of `offsets`, a wave scan of their tile counts) instead of walking the
    // experts with a dependent scalar load each: with hundreds of experts, most of them empty,
    // that walk took longer than the tile itself.
    __shared__ int owner[4];
    if (t < 64) {
        int carry = 0;
        bool done = false;
        for (int e0 = 0; e0 < a.E && !done; e0 += 64) {
            const int e = e0 + t;
            const int lo = e < a.E ? a.offsets[e] : 0, hi = e < a.E ? a.offsets[e + 1] : 0;
            const int tiles = (hi - lo + QC_TILE - 1) / QC_TILE;
            const int incl = wave_incl_scan(tiles, t);
            const int first = carry + incl - tiles;
            const bool mine = e < a.E && rt >= first && rt < first + tiles;
            if (__ballot(mine)) {
                if (mine) owner[0] = e, owner[1] = first, owner[2] = lo, owner[3] = hi;
                done = true;
            }
            carry += __shfl(incl, 63, 64);
        }
        if (!done && t == 0) owner[0] = -1;
    }
    __syncthreads();
    if (owner[0] < 0) return;  // beyond the last real tile: that part of the padded space is never read
    const int before = owner[1], start = owner[2], end = owner[3];
    const int row_base = start + (rt - before) * QC_TILE;
    const int64_t k0 = (int64_t)blockIdx.x * QC_TILE;
    const int64_t col = k0 + (t & 15) * 8;
    const bool col_ok = col < a.C;
    float v[8][8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int pos = row_base + (t >> 4) * 8 + i;
        if (col_ok && pos < end) {
            const int64_t src = a.index ? a.index[pos] : pos;
            if (SRC == SRC_PLAIN) {
                Elem<DT>::load8((const T *)a.x + src * a.ldx + col, v[i]);
                if (a.row_scale) {
                    const int si = a.scale_index ? a.scale_index[pos] : pos;
                    const float sc = a.scale_f32 ? ((const float *)a.row_scale)[si] : Elem<DT>::load1((const T *)a.row_scale + si);
#pragma unroll
                    for (int c = 0; c < 8; c++) v[i][c] *= sc;
                }
            } else {
                float g[8], u[8];
                Elem<DT>::load8((const T *)a.x + src * a.ldx + col, g);
                Elem<DT>::load8((const T *)a.x + src * a.ldx + a.C + col, u);
#pragma unroll
                for (int c = 0; c < 8; c++) v[i][c] = g[c] * sigmoid_fast(g[c]) * u[c];
            }
        } else {
#pragma unroll
            for (int c = 0; c < 8; c++) v[i][c] = 0.0f;
        }
    }
    quant_tile<false>(v, o, mpad, a.C, (int64_t)rt * QC_TILE, k0, tile, tscale);
}

// The same quantizer for wide inputs: a workgroup keeps its 128 rows and walks `span` column tiles.
// Measured at 98304 routed rows x 1024 columns with a row scale: 72 us one tile per workgroup,
// 60 us four tiles (one expert search, one read of the row indices and scales, 1 KB runs of every
// source row); without the row scale 56 and 57 us.  One tile per workgroup stays with the kernel
// above, which is the faster of the two then.
template <int DT, int SRC>
__global__ __launch_bounds__(256) void quant_cols_grouped_walk_kernel(GroupedQuantArgs a, QuantTileOut o, int64_t mpad) {
    typedef typename Elem<DT>::type T;
    __shared__ __attribute__((aligned(16))) uint8_t tile[QC_TILE * QC_PITCH];
    __shared__ __attribute__((aligned(4))) uint8_t tscale[QC_TILE * 4];
    const int t = threadIdx.x;
    const int rt = blockIdx.y;
    // tile_owner: the expert whose tiles contain rt.  The first wave looks at 64 experts at a time
    // (one coalesced read of `offsets`, a wave scan of their tile counts) instead of walking the
    // experts with a dependent scalar load each: with hundreds of experts, most of them empty,
    // that walk took longer than the tile itself.
    __shared__ int owner[4];
    if (t < 64) {
        int carry = 0;
        bool done = false;
        for (int e0 = 0; e0 < a.E && !done; e0 += 64) {
            const int e = e0 + t;
            const int lo = e < a.E ? a.offsets[e] : 0, hi = e < a.E ? a.offsets[e + 1] : 0;
            const int tiles = (hi - lo + QC_TILE - 1) / QC_TILE;
            const int incl = wave_incl_scan(tiles, t);
            const int first = carry + incl - tiles;
            const bool mine = e < a.E && rt >= first && rt < first + tiles;
            if (__ballot(mine)) {
                if (mine) owner[0] = e, owner[1] = first, owner[2] = lo, owner[3] = hi;
                done = true;
            }
            carry += __shfl(incl, 63, 64);
        }
        if (!done && t == 0) owner[0] = -1;
    }
    __syncthreads();
    if (owner[0] < 0) return;  // beyond the last real tile: that part of the padded space is never read
    const int before = owner[1], start = owner[2], end = owner[3];
    const int row_base = start + (rt - before) * QC_TILE;
    // this thread's 8 source rows (and their scale factors) serve every column tile of the workgroup
    int64_t src[8];
    float sc[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const int pos = row_base + (t >> 4) * 8 + i;
        src[i] = -1;
        sc[i] = 1.0f;
        if (pos < end) {
            src[i] = a.index ? a.index[pos] : pos;
            if (SRC == SRC_PLAIN && a.row_scale) {
                const int si = a.scale_index ? a.scale_index[pos] : pos;
                sc[i] = a.scale_f32 ? ((const float *)a.row_scale)[si] : Elem<DT>::load1((const T *)a.row_scale + si);
            }
        }
    }
    // A workgroup walks `span` neighbouring column tiles of its 128 rows: it reads span x 256
    // contiguous bytes of every source row instead of 256, and finds its expert once.
    const int ctiles = (a.C + QC_TILE - 1) / QC_TILE;
    const int kt_end = (int)(blockIdx.x + 1) * a.span < ctiles ? (int)(blockIdx.x + 1) * a.span : ctiles;
    for (int kt = (int)blockIdx.x * a.span; kt < kt_end; kt++) {
        const int64_t k0 = (int64_t)kt * QC_TILE;
        const int64_t col = k0 + (t & 15) * 8;
        const bool col_ok = col < a.C;
        float v[8][8];
        typename Elem<DT>::raw r[8];  // the eight row loads of this column tile go out together
        if (SRC == SRC_PLAIN) {
#pragma unroll
            for (int i = 0; i < 8; i++)
                if (col_ok && src[i] >= 0) r[i] = Elem<DT>::load_raw((const T *)a.x + src[i] * a.ldx + col);
        }
#pragma unroll
        for (int i = 0; i < 8; i++) {
            if (col_ok && src[i] >= 0) {
                if (SRC == SRC_PLAIN) {
                    Elem<DT>::unpack(r[i], v[i]);
                    if (a.row_scale) {
#pragma unroll
                        for (int c = 0; c < 8; c++) v[i][c] *= sc[i];
                    }
                } else {
                    float g[8], u[8];
                    Elem<DT>::load8((const T *)a.x + src[i] * a.ldx + col, g);
                    Elem<DT>::load8((const T *)a.x + src[i] * a.ldx + a.C + col, u);
#pragma unroll
                    for (int c = 0; c < 8; c++) v[i][c] = g[c] * sigmoid_fast(g[c]) * u[c];
                }
            } else {
#pragma unroll
                for (int c = 0; c < 8; c++) v[i][c] = 0.0f;
            }
        }
        quant_tile<false>(v, o, mpad, a.C, (int64_t)rt * QC_TILE, k0, tile, tscale);
    }
}

}  // namespace mx

// ------------------------------------------------------------------------------------
// C ABI
// ------------------------------------------------------------------------------------

using namespace mx;

static inline bool aligned(const void *p, uintptr_t a) { return ((uintptr_t)p & (a - 1)) == 0; }
static inline int esize(int dt) { return dt == MX_FP32 ? 4 : 2; }

#define MX_LAUNCH_CHECK()                                   \
    do {                                                    \
        if (hipGetLastError() != hipSuccess) return MX_ELAUNCH; \
    } while (0)

template <int DT>
static int launch_rows(const void *x, int64_t M, int64_t K, int64_t sx_row, int64_t sx_col, uint8_t *q, int64_t ldq,
                       uint8_t *s, int64_t lds, hipStream_t st) {
    const int64_t KB = K / MX_BLOCK;
    const bool vec_ok = sx_col == 1 && aligned(x, 16) && (sx_row * esize(DT)) % 16 == 0 && aligned(q, 8) &&
                        ldq % 8 == 0 && M * (K / 8) < (int64_t)0x7FFFFF00;
    if (!vec_ok) {
        int64_t blocks = M * KB;
        if ((blocks + 255) / 256 > 0x7FFFFFFF) return MX_EUNSUPPORTED;
        quant_rows_generic_kernel<DT><<<dim3((unsigned)((blocks + 255) / 256)), dim3(256), 0, st>>>(
            x, M, KB, sx_row, sx_col, q, ldq, s, lds);
        MX_LAUNCH_CHECK();
        return MX_OK;
    }
    // 16-byte chunks per thread.  Measured on 128 MB and more of bf16: 4 chunks 5.6 TB/s, 2 chunks 6.0, 1 chunk 5.75
    constexpr int U = 2;
    const uint32_t cpr = (uint32_t)(K / 8);
    const uint32_t total = (uint32_t)(M * (K / 8));
    const unsigned grid = (total + U * 256 - 1) / (U * 256);
    const bool flat = sx_row == K && ldq == K && lds == KB;
    if (flat) {
        int pack = aligned(s, 4);
        quant_rows_kernel<DT, U, true><<<dim3(grid), dim3(256), 0, st>>>(x, cpr, sx_row, q, ldq, s, lds, total, pack);
    } else {
        int pack = aligned(s, 4) && lds % 4 == 0 && KB % 4 == 0;
        quant_rows_kernel<DT, U, false><<<dim3(grid), dim3(256), 0, st>>>(x, cpr, sx_row, q, ldq, s, lds, total, pack);
    }
    MX_LAUNCH_CHECK();
    return MX_OK;
}

// A leading dimension of exactly 128 for a matrix wider than 128 columns asks for the stage-major
// layout: 128-column panels, each holding every row (pitch 128), panel p at p * rows * 128.
static bool stage_major(int64_t ld, int64_t cols) { return ld == 128 && cols > 128; }

static QuantTileOut tile_out(uint8_t *qT, int64_t ldqT, uint8_t *sT, int64_t ldsT, uint8_t *q, int64_t ldq, uint8_t *s,
                             int64_t lds, int64_t q_ks = 0, int64_t qT_ks = 0) {
    QuantTileOut o;
    o.qT = qT, o.ldqT = ldqT, o.sT = sT, o.ldsT = ldsT, o.q = q, o.ldq = ldq, o.s = s, o.lds = lds;
    o.q_ks = q_ks, o.qT_ks = qT_ks;
    o.pack_row_scales = s != nullptr && aligned(s, 4) && lds % 4 == 0;
    o.pack_col_scales = aligned(sT, 4) && ldsT % 4 == 0;
    return o;
}

// Rows per thread of the dense tile quantizers (see TileGeom): 8 = 128 x 128 tiles.
constexpr int MX_QR_COLS = 8, MX_QR_SWIGLU = 8, MX_QR_SWIGLU_BWD = 8;

template <int R>
static bool tile_grid(int64_t M, int64_t K, dim3 &grid) {
    grid = dim3((unsigned)((K + TileGeom<R>::TK - 1) / TileGeom<R>::TK), (unsigned)((M + QC_TILE - 1) / QC_TILE));
    return grid.y <= 65535u;
}

template <int DT, bool DUAL>
static int launch_cols(const void *x, int64_t M, int64_t K, int64_t ldx, uint8_t *qT, int64_t ldqT, uint8_t *sT,
                       int64_t ldsT, uint8_t *q, int64_t ldq, uint8_t *s, int64_t lds, hipStream_t st, int64_t qT_ks = 0) {
    dim3 grid;
    if (!tile_grid<MX_QR_COLS>(M, K, grid)) return MX_EUNSUPPORTED;
    const QuantTileOut o = tile_out(qT, ldqT, sT, ldsT, q, ldq, s, lds, 0, qT_ks);
    // Both axes of a 16-bit matrix whose tiles are all resident at once with eight waves per SIMD, but not with the five
    // the fp32 tile allows, go to the packed-tile kernel: 16384 x 1536 (1536 tiles on 256 CUs) 27.0 -> 24.9 us.  Larger
    // matrices run several rounds either way and are faster with fewer, fatter waves (16384 x 4096: 54.4 against 58.9 us).
    bool raw = false;
    if constexpr (DT != MX_FP32 && DUAL) raw = (int64_t)grid.x * grid.y <= 8 * (int64_t)num_cus();
    if constexpr (DT != MX_FP32 && DUAL) {
        if (raw) quant_cols_kernel<DT, DUAL, MX_QR_COLS, true><<<grid, dim3(256), 0, st>>>(x, M, K, ldx, o);
    }
    if (!raw) quant_cols_kernel<DT, DUAL, MX_QR_COLS><<<grid, dim3(256), 0, st>>>(x, M, K, ldx, o);
    MX_LAUNCH_CHECK();
    return MX_OK;
}

static bool cols_vec_ok(const void *x, int dt, int64_t K, int64_t ldx, const uint8_t *qT, int64_t ldqT) {
    return K % 8 == 0 && aligned(x, 16) && (ldx * esize(dt)) % 16 == 0 && aligned(qT, 16) && ldqT % 16 == 0;
}

template <int DT>
static int launch_norm_dual(const void *x, int64_t M, int64_t K, int64_t ldx, const void *w, int w_dtype, const float *rstd,
                            const QuantTileOut &o, hipStream_t st) {
    dim3 grid;
    if (!tile_grid<8>(M, K, grid)) return MX_EUNSUPPORTED;
    switch (w ? w_dtype : (int)MX_FP32) {
    case MX_BF16: rmsnorm_quant_dual_kernel<DT, MX_BF16><<<grid, dim3(256), 0, st>>>(x, M, K, ldx, w, rstd, o); break;
    case MX_FP16: rmsnorm_quant_dual_kernel<DT, MX_FP16><<<grid, dim3(256), 0, st>>>(x, M, K, ldx, w, rstd, o); break;
    default: rmsnorm_quant_dual_kernel<DT, MX_FP32><<<grid, dim3(256), 0, st>>>(x, M, K, ldx, w, rstd, o); break;
    }
    MX_LAUNCH_CHECK();
    return MX_OK;
}

extern "C" int mx_rmsnorm_quantize_dual(const void *x, int x_dtype, int64_t M, int64_t K, int64_t ldx, const void *weight,
                                        int w_dtype, float eps, float *rstd, uint8_t *q, int64_t ldq, uint8_t *s,
                                        int64_t lds, uint8_t *qT, int64_t ldqT, uint8_t *sT, int64_t ldsT, void *stream) {
    const bool panels = stage_major(ldqT, M);
    if (M < 0 || K <= 0 || M % MX_BLOCK || K % MX_BLOCK || !x || !rstd || !q || !s || !qT || !sT || ldx < K || ldq < K ||
        lds < K / MX_BLOCK || (ldqT < M && !panels) || (panels && M % 128) || ldsT < M / MX_BLOCK)
        return MX_EINVAL;
    if (x_dtype != MX_BF16 && x_dtype != MX_FP16 && x_dtype != MX_FP32) return MX_EINVAL;
    if (weight && w_dtype != MX_BF16 && w_dtype != MX_FP16 && w_dtype != MX_FP32) return MX_EINVAL;
    if (M == 0) return MX_OK;
    if (!cols_vec_ok(x, x_dtype, K, ldx, qT, ldqT) || !aligned(q, 8) || ldq % 8 || !aligned(rstd, 16) ||
        (weight && !aligned(weight, 16)))
        return MX_EUNSUPPORTED;
    // first pass: the rows' reciprocal root mean squares (the row kernel, asked for nothing but rstd)
    int rc = mx_rmsnorm_quantize(x, x_dtype, M, K, ldx, nullptr, 0, eps, nullptr, 0, rstd, nullptr, 0, nullptr, 0, stream);
    if (rc != MX_OK) return rc;
    hipStream_t st = (hipStream_t)stream;
    const QuantTileOut o = tile_out(qT, ldqT, sT, ldsT, q, ldq, s, lds, 0, panels ? K * 128 : 0);
    switch (x_dtype) {
    case MX_BF16: return launch_norm_dual<MX_BF16>(x, M, K, ldx, weight, w_dtype, rstd, o, st);
    case MX_FP16: return launch_norm_dual<MX_FP16>(x, M, K, ldx, weight, w_dtype, rstd, o, st);
    default: return launch_norm_dual<MX_FP32>(x, M, K, ldx, weight, w_dtype, rstd, o, st);
    }
}

extern "C" int mx_quantize_cols(const void *x, int x_dtype, int64_t M, int64_t K, int64_t ldx, uint8_t *qT,
                                int64_t ldqT, uint8_t *sT, int64_t ldsT, void *stream) {
    if (M < 0 || K < 0 || M % MX_BLOCK || ldx < K || ldqT < M || ldsT < M / MX_BLOCK) return MX_EINVAL;
    if (M == 0 || K == 0) return MX_OK;
    hipStream_t st = (hipStream_t)stream;
    if (mx::stream_is_capturing(st)) return MX_ECAPTURE;
    if (!cols_vec_ok(x, x_dtype, K, ldx, qT, ldqT)) {
        // Rows of the transposed view, one thread per block.
        switch (x_dtype) {
        case MX_BF16: return launch_rows<MX_BF16>(x, K, M, 1, ldx, qT, ldqT, sT, ldsT, st);
        case MX_FP16: return launch_rows<MX_FP16>(x, K, M, 1, ldx, qT, ldqT, sT, ldsT, st);
        case MX_FP32: return launch_rows<MX_FP32>(x, K, M, 1, ldx, qT, ldqT, sT, ldsT, st);
        default: return MX_EINVAL;
        }
    }
    switch (x_dtype) {
    case MX_BF16: return launch_cols<MX_BF16, false>(x, M, K, ldx, qT, ldqT, sT, ldsT, nullptr, 0, nullptr, 0, st);
    case MX_FP16: return launch_cols<MX_FP16, false>(x, M, K, ldx, qT, ldqT, sT, ldsT, nullptr, 0, nullptr, 0, st);
    case MX_FP32: return launch_cols<MX_FP32, false>(x, M, K, ldx, qT, ldqT, sT, ldsT, nullptr, 0, nullptr, 0, st);
    default: return MX_EINVAL;
    }
}

extern "C" int mx_quantize_rows(const void *x, int x_dtype, int64_t M, int64_t K, int64_t sx_row, int64_t sx_col,
                                uint8_t *q, int64_t ldq, uint8_t *s, int64_t lds, void *stream) {
    if (M < 0 || K < 0 || K % MX_BLOCK || ldq < K || lds < K / MX_BLOCK) return MX_EINVAL;
    if (M == 0 || K == 0) return MX_OK;
    hipStream_t st = (hipStream_t)stream;
    if (mx::stream_is_capturing(st)) return MX_ECAPTURE;
    // A transposed view (unit stride down the rows) is the column quantizer of the
    // matrix underneath it: no copy is made.
    if (sx_col != 1 && sx_row == 1 && M > 1 && cols_vec_ok(x, x_dtype, M, sx_col, q, ldq))
        return mx_quantize_cols(x, x_dtype, K, M, sx_col, q, ldq, s, lds, stream);
    switch (x_dtype) {
    case MX_BF16: return launch_rows<MX_BF16>(x, M, K, sx_row, sx_col, q, ldq, s, lds, st);
    case MX_FP16: return launch_rows<MX_FP16>(x, M, K, sx_row, sx_col, q, ldq, s, lds, st);
    case MX_FP32: return launch_rows<MX_FP32>(x, M, K, sx_row, sx_col, q, ldq, s, lds, st);
    default: return MX_EINVAL;
    }
}

template <int DT>
static int launch_heads(const void *x, int64_t T, int64_t H, int64_t D, int64_t stride_t, int64_t stride_h,
                        const float *mu, uint8_t *q, uint8_t *s, hipStream_t st) {
    const uint32_t cpr = (uint32_t)(H * D / 8), cph = (uint32_t)(D / 8), total = (uint32_t)(T * (H * D / 8));
    const unsigned grid = (total + 4 * 256 - 1) / (4 * 256);
    // the outputs are contiguous, so a 16-lane group's 4 scale bytes are one aligned dword whatever the row length
    const int pack = aligned(s, 4);
    if (mu)
        quant_heads_kernel<DT, true><<<dim3(grid), dim3(256), 0, st>>>(x, cpr, cph, stride_t, stride_h, mu, q, s, total, pack);
    else
        quant_heads_kernel<DT, false><<<dim3(grid), dim3(256), 0, st>>>(x, cpr, cph, stride_t, stride_h, mu, q, s, total, pack);
    MX_LAUNCH_CHECK();
    return MX_OK;
}

extern "C" int mx_quantize_heads(const void *x, int x_dtype, int64_t T, int64_t H, int64_t D, int64_t stride_t,
                                 int64_t stride_h, const float *mu, uint8_t *q, uint8_t *s, void *stream) {
    if (T < 0 || H < 0 || D < 0 || D % MX_BLOCK || (H > 1 && stride_h < D) || stride_t < 0) return MX_EINVAL;
    if (x_dtype != MX_BF16 && x_dtype != MX_FP16 && x_dtype != MX_FP32) return MX_EINVAL;
    if (T == 0 || H == 0 || D == 0) return MX_OK;
    if (!x || !q || !s) return MX_EINVAL;
    if (!aligned(x, 16) || (stride_t * esize(x_dtype)) % 16 || (stride_h * esize(x_dtype)) % 16 || !aligned(q, 8) ||
        (mu && !aligned(mu, 16)) || T * (H * D / 8) >= (int64_t)0x7FFFFF00)
        return MX_EUNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    if (mx::stream_is_capturing(st)) return MX_ECAPTURE;
    switch (x_dtype) {
    case MX_BF16: return launch_heads<MX_BF16>(x, T, H, D, stride_t, stride_h, mu, q, s, st);
    case MX_FP16: return launch_heads<MX_FP16>(x, T, H, D, stride_t, stride_h, mu, q, s, st);
    default: return launch_heads<MX_FP32>(x, T, H, D, stride_t, stride_h, mu, q, s, st);
    }
}

extern "C" int mx_quantize_dual(const void *x, int x_dtype, int64_t M, int64_t K, int64_t ldx, uint8_t *q, int64_t ldq,
                                uint8_t *s, int64_t lds, uint8_t *qT, int64_t ldqT, uint8_t *sT, int64_t ldsT,
                                void *stream) {
    const bool panels = stage_major(ldqT, M);  // qT as 128-token panels
    if (M < 0 || K < 0 || M % MX_BLOCK || K % MX_BLOCK || ldx < K || ldq < K || lds < K / MX_BLOCK ||
        (ldqT < M && !panels) || (panels && M % 128) || ldsT < M / MX_BLOCK)
        return MX_EINVAL;
    if (M == 0 || K == 0) return MX_OK;
    hipStream_t st = (hipStream_t)stream;
    if (mx::stream_is_capturing(st)) return MX_ECAPTURE;
    if (!cols_vec_ok(x, x_dtype, K, ldx, qT, ldqT) || !aligned(q, 8) || ldq % 8) {
        if (panels) return MX_EUNSUPPORTED;
        int rc = mx_quantize_rows(x, x_dtype, M, K, ldx, 1, q, ldq, s, lds, stream);
        if (rc != MX_OK) return rc;
        return mx_quantize_cols(x, x_dtype, M, K, ldx, qT, ldqT, sT, ldsT, stream);
    }
    const int64_t ks = panels ? K * 128 : 0;
    switch (x_dtype) {
    case MX_BF16: return launch_cols<MX_BF16, true>(x, M, K, ldx, qT, ldqT, sT, ldsT, q, ldq, s, lds, st, ks);
    case MX_FP16: return launch_cols<MX_FP16, true>(x, M, K, ldx, qT, ldqT, sT, ldsT, q, ldq, s, lds, st, ks);
    case MX_FP32: return launch_cols<MX_FP32, true>(x, M, K, ldx, qT, ldqT, sT, ldsT, q, ldq, s, lds, st, ks);
    default: return MX_EINVAL;
    }
}

extern "C" int mx_quantize_dual_batch(const mx_quant_problem *problems, int count, int x_dtype, void *stream) {
    if (count < 0 || (count > 0 && !problems)) return MX_EINVAL;
    if (x_dtype != MX_BF16 && x_dtype != MX_FP16 && x_dtype != MX_FP32) return MX_EINVAL;
    for (int j = 0; j < count; j++) {  // validate everything before launching anything
        const mx_quant_problem &p = problems[j];
        if (p.M < 0 || p.K < 0 || p.M % MX_BLOCK || p.K % MX_BLOCK || p.ldx < p.K || p.ldq < p.K ||
            p.lds < p.K / MX_BLOCK || p.ldqT < p.M || p.ldsT < p.M / MX_BLOCK)
            return MX_EINVAL;
        if (p.M && p.K && (!p.x || !p.q || !p.s || !p.qT || !p.sT)) return MX_EINVAL;
    }
    hipStream_t st = (hipStream_t)stream;
    if (mx::stream_is_capturing(st)) return MX_ECAPTURE;
    QuantBatchArgs b;
    b.count = 0;
    int64_t total = 0;
    auto flush = [&]() -> int {
        if (b.count) {
            const dim3 grid((unsigned)total), block(256);
            switch (x_dtype) {
            case MX_BF16: quant_dual_batch_kernel<MX_BF16><<<grid, block, 0, st>>>(b); break;
            case MX_FP16: quant_dual_batch_kernel<MX_FP16><<<grid, block, 0, st>>>(b); break;
            default: quant_dual_batch_kernel<MX_FP32><<<grid, block, 0, st>>>(b); break;
            }
            MX_LAUNCH_CHECK();
        }
        b.count = 0, total = 0;
        return MX_OK;
    };
    for (int j = 0; j < count; j++) {
        const mx_quant_problem &p = problems[j];
        if (p.M == 0 || p.K == 0) continue;
        const int64_t tiles_k = (p.K + QC_TILE - 1) / QC_TILE, tiles = tiles_k * ((p.M + QC_TILE - 1) / QC_TILE);
        if (!cols_vec_ok(p.x, x_dtype, p.K, p.ldx, p.qT, p.ldqT) || !aligned(p.q, 8) || p.ldq % 8 ||
            tiles > 0x3FFFFFFF) {
            // an operand the tiled kernel does not take goes through the single-matrix entry point
            int rc = mx_quantize_dual(p.x, x_dtype, p.M, p.K, p.ldx, p.q, p.ldq, p.s, p.lds, p.qT, p.ldqT, p.sT, p.ldsT,
                                      stream);
            if (rc != MX_OK) return rc;
            continue;
        }
        if (b.count == MX_QUANT_BATCH_MAX || total + tiles > 0x3FFFFFFF) {
            int rc = flush();
            if (rc != MX_OK) return rc;
        }
        const int k = b.count++;
        b.x[k] = p.x, b.M[k] = p.M, b.K[k] = p.K, b.ldx[k] = p.ldx;
        b.o[k] = tile_out(p.qT, p.ldqT, p.sT, p.ldsT, p.q, p.ldq, p.s, p.lds);
        total += tiles;
        b.tile_end[k] = (int)total, b.tiles_k[k] = (int)tiles_k;
    }
    return flush();
}

template <int DT>
static int launch_swiglu(const void *g, const void *u, int64_t M, int64_t K, int64_t ldg, int64_t ldu, uint8_t *q,
                         int64_t ldq, uint8_t *s, int64_t lds, hipStream_t st) {
    constexpr int U = 2;
    const uint32_t total = (uint32_t)(M * (K / 8));
    const unsigned grid = (total + U * 256 - 1) / (U * 256);
    int pack = aligned(s, 4) && lds % 4 == 0 && (K / MX_BLOCK) % 4 == 0;
    swiglu_quant_rows_kernel<DT, U><<<dim3(grid), dim3(256), 0, st>>>(g, u, (uint32_t)(K / 8), ldg, ldu, q, ldq, s, lds,
                                                                      total, pack);
    MX_LAUNCH_CHECK();
    return MX_OK;
}

extern "C" int mx_swiglu_quantize_rows(const void *gate, const void *up, int dtype, int64_t M, int64_t K, int64_t ldg,
                                       int64_t ldu, uint8_t *q, int64_t ldq, uint8_t *s, int64_t lds, void *stream) {
    if (M < 0 || K < 0 || K % MX_BLOCK || ldg < K || ldu < K || ldq < K || lds < K / MX_BLOCK) return MX_EINVAL;
    if (M == 0 || K == 0) return MX_OK;
    if (dtype != MX_BF16 && dtype != MX_FP16) return MX_EUNSUPPORTED;
    if (!aligned(gate, 16) || !aligned(up, 16) || (ldg * 2) % 16 || (ldu * 2) % 16 || !aligned(q, 8) || ldq % 8 ||
        M * (K / 8) >= (int64_t)0x7FFFFF00)
        return MX_EUNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    if (mx::stream_is_capturing(st)) return MX_ECAPTURE;
    return dtype == MX_BF16 ? launch_swiglu<MX_BF16>(gate, up, M, K, ldg, ldu, q, ldq, s, lds, st)
                            : launch_swiglu<MX_FP16>(gate, up, M, K, ldg, ldu, q, ldq, s, lds, st);
}

extern "C" int mx_swiglu_quantize_dual(const void *gu, int dtype, int64_t M, int64_t H, int64_t ldgu, uint8_t *q,
                                       int64_t ldq, uint8_t *s, int64_t lds, uint8_t *qT, int64_t ldqT, uint8_t *sT,
                                       int64_t ldsT, void *stream) {
    const bool panels = stage_major(ldqT, M);  // qT as 128-token panels
    if (M < 0 || H < 0 || M % MX_BLOCK || H % MX_BLOCK || ldgu < 2 * H || ldq < H || lds < H / MX_BLOCK ||
        (ldqT < M && !panels) || (panels && M % 128) || ldsT < M / MX_BLOCK)
        return MX_EINVAL;
    if (M == 0 || H == 0) return MX_OK;
    if (dtype != MX_BF16 && dtype != MX_FP16) return MX_EUNSUPPORTED;
    if (!aligned(gu, 16) || (ldgu * 2) % 16 || !aligned(q, 8) || ldq % 8 || !aligned(qT, 16) || ldqT % 16)
        return MX_EUNSUPPORTED;
    dim3 grid;
    if (!tile_grid<MX_QR_SWIGLU>(M, H, grid)) return MX_EUNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    if (mx::stream_is_capturing(st)) return MX_ECAPTURE;
    QuantTileOut o = tile_out(qT, ldqT, sT, ldsT, q, ldq, s, lds, 0, panels ? H * 128 : 0);
    if (dtype == MX_BF16) swiglu_quant_dual_kernel<MX_BF16, MX_QR_SWIGLU><<<grid, dim3(256), 0, st>>>(gu, M, H, ldgu, o);
    else swiglu_quant_dual_kernel<MX_FP16, MX_QR_SWIGLU><<<grid, dim3(256), 0, st>>>(gu, M, H, ldgu, o);
    MX_LAUNCH_CHECK();
    return MX_OK;
}

extern "C" int mx_swiglu_bwd_quantize_dual(const void *dh, int64_t lddh, const void *gu, int64_t ldgu, int dtype,
                                           int64_t M, int64_t H, uint8_t *q, int64_t ldq, uint8_t *s, int64_t lds,
                                           uint8_t *qT, int64_t ldqT, uint8_t *sT, int64_t ldsT, void *stream) {
    const bool q_panels = stage_major(ldq, 2 * H), qt_panels = stage_major(ldqT, M);
    if (M < 0 || H < 0 || M % MX_BLOCK || H % MX_BLOCK || lddh < H || ldgu < 2 * H || (ldq < 2 * H && !q_panels) ||
        (q_panels && H % 128) || lds < 2 * H / MX_BLOCK || (ldqT < M && !qt_panels) || (qt_panels && M % 128) ||
        ldsT < M / MX_BLOCK)
        return MX_EINVAL;
    if (M == 0 || H == 0) return MX_OK;
    if (dtype != MX_BF16 && dtype != MX_FP16) return MX_EUNSUPPORTED;
    if (!aligned(gu, 16) || (ldgu * 2) % 16 || !aligned(dh, 16) || (lddh * 2) % 16 || !aligned(q, 8) || ldq % 8 ||
        !aligned(qT, 16) || ldqT % 16)
        return MX_EUNSUPPORTED;
    dim3 grid;
    if (!tile_grid<MX_QR_SWIGLU_BWD>(M, H, grid)) return MX_EUNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    if (mx::stream_is_capturing(st)) return MX_ECAPTURE;
    QuantTileOut o = tile_out(qT, ldqT, sT, ldsT, q, ldq, s, lds, q_panels ? M * 128 : 0, qt_panels ? 2 * H * 128 : 0);
    if (H % 128) o.pack_row_scales = 0;  // the up half's scale columns start at H/32: keep the packed stores aligned
    if (dtype == MX_BF16)
        swiglu_bwd_quant_dual_kernel<MX_BF16, MX_QR_SWIGLU_BWD><<<grid, dim3(256), 0, st>>>(dh, lddh, gu, ldgu, M, H, o);
    else swiglu_bwd_quant_dual_kernel<MX_FP16, MX_QR_SWIGLU_BWD><<<grid, dim3(256), 0, st>>>(dh, lddh, gu, ldgu, M, H, o);
    MX_LAUNCH_CHECK();
    return MX_OK;
}

extern "C" int mx_quantize_cols_grouped(const void *x, int dtype, int64_t ldx, int64_t C, int source,
                                        const int32_t *index, const void *row_scale, int row_scale_dtype,
                                        const int32_t *scale_index, const int32_t *offsets, int64_t E, int64_t M,
                                        uint8_t *qT, int64_t ldqT, uint8_t *sT, int64_t ldsT, void *stream) {
    if (M < 0 || C < 0 || E <= 0 || E >= (1 << 20) || M >= 0x7FFFFFFF || C >= 0x7FFFFFFF) return MX_EINVAL;
    if (source != SRC_PLAIN && source != SRC_SWIGLU) return MX_EINVAL;
    const int64_t tiles = (M + QC_TILE - 1) / QC_TILE + E;
    const int64_t mpad = tiles * QC_TILE;
    // a leading dimension of exactly 128 on the wider padded axis: qT stage-major, (Mpad/128, C, 128)
    const bool qt_panels = ldqT == 128 && mpad > 128;
    if ((ldqT < mpad && !qt_panels) || ldsT < mpad / MX_BLOCK || ldx < (source == SRC_SWIGLU ? 2 * C : C)) return MX_EINVAL;
    if (row_scale && row_scale_dtype != MX_FP32 && row_scale_dtype != dtype) return MX_EINVAL;
    if (dtype != MX_BF16 && dtype != MX_FP16) return MX_EUNSUPPORTED;
    if (C % 8 || !aligned(x, 16) || (ldx * 2) % 16 || !aligned(qT, 16) || ldqT % 16 || tiles > 65535) return MX_EUNSUPPORTED;
    if (C == 0) return MX_OK;
    GroupedQuantArgs a;
    a.x = x, a.ldx = ldx, a.C = (int)C, a.index = index, a.row_scale = row_scale, a.scale_index = scale_index;
    a.scale_f32 = row_scale_dtype == MX_FP32, a.offsets = offsets, a.E = (int)E;
    QuantTileOut o = tile_out(qT, ldqT, sT, ldsT, nullptr, 0, nullptr, 0, 0, qt_panels ? C * 128 : 0);
    const int ctiles = (int)((C + QC_TILE - 1) / QC_TILE);
    // four column tiles per workgroup while that still leaves every CU several workgroups
    a.span = ctiles >= 4 && (int64_t)tiles * (ctiles / 4) >= 2 * (int64_t)mx::num_cus() ? 4 : 1;
    dim3 grid((unsigned)((ctiles + a.span - 1) / a.span), (unsigned)tiles);
    hipStream_t st = (hipStream_t)stream;
    if (mx::stream_is_capturing(st)) return MX_ECAPTURE;
#define MX_QCG_LAUNCH(DT, SRC)                                                                     \
    do {                                                                                           \
        if (a.span > 1) quant_cols_grouped_walk_kernel<DT, SRC><<<grid, dim3(256), 0, st>>>(a, o, mpad); \
        else quant_cols_grouped_kernel<DT, SRC><<<grid, dim3(256), 0, st>>>(a, o, mpad);           \
    } while (0)
    if (dtype == MX_BF16) {
        if (source == SRC_PLAIN) MX_QCG_LAUNCH(MX_BF16, SRC_PLAIN);
        else MX_QCG_LAUNCH(MX_BF16, SRC_SWIGLU);
    } else {
        if (source == SRC_PLAIN) MX_QCG_LAUNCH(MX_FP16, SRC_PLAIN);
        else MX_QCG_LAUNCH(MX_FP16, SRC_SWIGLU);
    }
#undef MX_QCG_LAUNCH
    MX_LAUNCH_CHECK();
    return MX_OK;
}

// ---- cuBLAS SWIZZLE_32_4_4 scale layout (interop) -------------------------------------------------
// 128-row x 4-column tiles of 512 bytes, row-tile major; inside a tile scale (r, c) sits at
// (r % 32) * 16 + (r / 32) * 4 + c; zero padded to whole tiles.  One thread moves the 4 bytes
// of one row of one tile.  (src/kohakuwullm/kernels/mxfp8/interop.py:24-41, quantize.py:175-180.)
namespace mx {
template <bool TO_SWIZZLED>
__global__ __launch_bounds__(256) void swizzle_scales_kernel(uint8_t *__restrict__ natural, int64_t lds,
                                                             uint8_t *__restrict__ swizzled, int64_t rows, int64_t cols,
                                                             int64_t col_tiles, int64_t total) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;  // one dword of the swizzled buffer
    if (idx >= total) return;
    const int64_t tile = idx >> 7;
    const int in = (int)(idx & 127);        // (r % 32) * 4 + r / 32
    const int rr = (in >> 2) + 32 * (in & 3);
    const int64_t r = (tile / col_tiles) * 128 + rr;
    const int64_t c0 = (tile % col_tiles) * 4;
    if (TO_SWIZZLED) {
        uint32_t w = 0;
        if (r < rows)
            for (int c = 0; c < 4; c++)
                if (c0 + c < cols) w |= (uint32_t)natural[r * lds + c0 + c] << (8 * c);
        ((uint32_t *)swizzled)[idx] = w;
    } else if (r < rows) {
        const uint32_t w = ((const uint32_t *)swizzled)[idx];
        for (int c = 0; c < 4; c++)
            if (c0 + c < cols) natural[r * lds + c0 + c] = (uint8_t)(w >> (8 * c));
    }
}
}  // namespace mx

static int swizzle_launch(bool to_swizzled, uint8_t *natural, int64_t lds, uint8_t *swizzled, int64_t rows, int64_t cols,
                          void *stream) {
    if (rows < 0 || cols < 0 || lds < cols) return MX_EINVAL;
    if (((uintptr_t)swizzled & 3) != 0) return MX_EINVAL;
    const int64_t row_tiles = (rows + 127) / 128, col_tiles = (cols + 3) / 4;
    const int64_t total = row_tiles * col_tiles * 128;
    if (total == 0) return MX_OK;
    const int64_t blocks = (total + 255) / 256;
    if (blocks > 0x7FFFFFFF) return MX_EUNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    if (mx::stream_is_capturing(st)) return MX_ECAPTURE;
    if (to_swizzled)
        mx::swizzle_scales_kernel<true><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(natural, lds, swizzled, rows, cols,
                                                                                    col_tiles, total);
    else
        mx::swizzle_scales_kernel<false><<<dim3((unsigned)blocks), dim3(256), 0, st>>>(natural, lds, swizzled, rows, cols,
                                                                                     col_tiles, total);
    return hipGetLastError() == hipSuccess ? MX_OK : MX_ELAUNCH;
}

extern "C" int mx_swizzle_scales(const uint8_t *s, int64_t rows, int64_t cols, int64_t lds, uint8_t *swizzled,
                                 void *stream) {
    return swizzle_launch(true, (uint8_t *)s, lds, swizzled, rows, cols, stream);
}

extern "C" int mx_unswizzle_scales(const uint8_t *swizzled, int64_t rows, int64_t cols, uint8_t *s, int64_t lds,
                                   void *stream) {
    return swizzle_launch(false, s, lds, (uint8_t *)swizzled, rows, cols, stream);
}
