// RMSNorm as a producer of MXFP8 operands for gfx950: y = x * rstd * w in fp32, written as the
// 16-bit activation and/or as e4m3 codes + UE8M0 bytes per 32 of K, in one pass over x.
// Semantics follow _rmsnorm_fwd / _rmsnorm_bwd of the reference
// (src/kohakuwullm/kernels/elementwise/rmsnorm.py:20-128) and _rmsnorm_mx_kernel
// (src/kohakuwullm/kernels/mxfp8/fused_act.py:104-143): rstd = 1 / sqrt(mean(x^2) + eps), the
// codes are quantized from the fp32 y, not from the rounded 16-bit output.
//
// HBM-streaming kernels, one wave per row: a lane owns 8 consecutive elements of every 512
// (16-byte loads, 1 KB per wave instruction), so the four lanes of a quad own one MX block and
// the block maximum is a DPP quad reduction.  The sum of squares is accumulated in fp64: the
// squares of 16-bit inputs are exact, so the sum does not depend on the order of the additions
// beyond the last bits of an fp64, and rstd comes out the same fp32 number whatever the
// reduction tree.
#include "mx_common.h"

namespace mx {

__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// OR the quad's byte into a dword holding the 4 bytes of a 16-lane row, in block order.
__device__ __forceinline__ uint32_t gather16(uint32_t byte, int lane) {
    uint32_t v = byte << ((lane & 12) << 1);
    v |= (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x124, 0xF, 0xF, true);  // row_ror:4
    v |= (uint32_t)__builtin_amdgcn_mov_dpp((int)v, 0x128, 0xF, 0xF, true);  // row_ror:8
    return v;
}

template <int DT>
__device__ __forceinline__ void store8(void *p, const float (&y)[8]) {
    if (DT == MX_FP32) {
        ((v4f *)p)[0] = v4f{y[0], y[1], y[2], y[3]};
        ((v4f *)p)[1] = v4f{y[4], y[5], y[6], y[7]};
    } else if (DT == MX_BF16) {
        *(v4i *)p = v4i{(int)pack2_bf16(y[0], y[1]), (int)pack2_bf16(y[2], y[3]), (int)pack2_bf16(y[4], y[5]),
                        (int)pack2_bf16(y[6], y[7])};
    } else {
        typedef _Float16 h8 __attribute__((ext_vector_type(8)));
        h8 h;
#pragma unroll
        for (int i = 0; i < 8; i++) h[i] = (_Float16)y[i];
        *(h8 *)p = h;
    }
}

struct NormArgs {
    const void *x, *w;
    void *out;
    float *rstd;
    uint8_t *q, *s;
    int64_t M, ldx, ldo, ldq, lds;
    int K;
    float eps;
};

// One 8-element chunk of the second phase: scale, store the activation, quantize.
template <int DT, int WDT>
__device__ __forceinline__ void norm_chunk(const NormArgs &a, int64_t row, int c, int chunks, int lane, float rstd,
                                           float (&y)[8]) {
    typedef typename Elem<DT>::type T;
    typedef typename Elem<WDT>::type TW;
    const bool ok = c < chunks;
    if (a.w && ok) {
        float w[8];
        Elem<WDT>::load8((const TW *)a.w + c * 8, w);
#pragma unroll
        for (int i = 0; i < 8; i++) y[i] = y[i] * rstd * w[i];
    } else {
#pragma unroll
        for (int i = 0; i < 8; i++) y[i] = y[i] * rstd;
    }
    if (a.out && ok) store8<DT>((T *)a.out + row * a.ldo + c * 8, y);
    if (!a.q) return;
    const float amax = quad_max(amax8(y));
    const uint32_t byte = scale_byte(amax);
    const float inv = inv_scale(byte);
    const uint32_t packed = gather16(byte, lane);
    if (!ok) return;
    v2i codes;
    codes[0] = (int)pack4_e4m3(y[0] * inv, y[1] * inv, y[2] * inv, y[3] * inv);
    codes[1] = (int)pack4_e4m3(y[4] * inv, y[5] * inv, y[6] * inv, y[7] * inv);
    *(v2i *)(a.q + row * a.ldq + c * 8) = codes;
    // 16 lanes hold 4 consecutive blocks: one dword when all four exist and the scale row is
    // dword-aligned there, single bytes otherwise
    uint8_t *sp = a.s + row * a.lds + (c >> 2);
    const bool group_full = (c | 15) < chunks && (a.lds & 3) == 0 && ((uintptr_t)a.s & 3) == 0;
    if (group_full) {
        if ((lane & 15) == 0) *(uint32_t *)sp = packed;
    } else if ((lane & 3) == 0) {
        *sp = (uint8_t)byte;
    }
}

template <int DT>
__device__ __forceinline__ double load_squares(const void *p, bool ok, float (&t)[8]) {
    typedef typename Elem<DT>::type T;
    if (ok) {
        Elem<DT>::load8((const T *)p, t);
    } else {
#pragma unroll
        for (int i = 0; i < 8; i++) t[i] = 0.0f;
    }
    double ss = 0.0;
#pragma unroll
    for (int i = 0; i < 8; i++) {
        const double d = (double)t[i];
        ss = __builtin_fma(d, d, ss);
    }
    return ss;
}

// The reference's fp32 arithmetic on the (exact) sum: mean + eps, square root, reciprocal, each
// correctly rounded.  The divide and the square root go through fp64 and are rounded once more
// to fp32, which is the correctly rounded fp32 result for fp32 operands (53 >= 2 * 24 + 2 bits)
// and does not depend on how the compiler is told to expand the fp32 forms.
__device__ __forceinline__ float rstd_of(double ss, int K, float eps) {
    const float mean = (float)((double)(float)ss / (double)(float)K) + eps;
    const float root = (float)__builtin_sqrt((double)mean);
    return (float)(1.0 / (double)root);
}

// CH > 0: the row (K <= 512 CH) stays in registers between the two phases.  CH == 0: any K,
// the row is read a second time (from L2: the same wave has just streamed it).
template <int DT, int WDT, int CH>
__global__ __launch_bounds__(256) void rmsnorm_quant_kernel(NormArgs a) {
    typedef typename Elem<DT>::type T;
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (row >= a.M) return;
    const int chunks = a.K >> 3;
    const T *xr = (const T *)a.x + row * a.ldx;
    if constexpr (CH > 0) {
        float v[CH][8];
        double ss = 0.0;
#pragma unroll
        for (int u = 0; u < CH; u++) {
            const int c = u * 64 + lane;
            ss += load_squares<DT>(xr + c * 8, c < chunks, v[u]);
        }
        const float rstd = rstd_of(wave_sum(ss), a.K, a.eps);
        if (a.rstd && lane == 0) a.rstd[row] = rstd;
#pragma unroll
        for (int u = 0; u < CH; u++) norm_chunk<DT, WDT>(a, row, u * 64 + lane, chunks, lane, rstd, v[u]);
    } else {
        const int passes = (chunks + 63) >> 6;
        double ss = 0.0;
        for (int u = 0; u < passes; u++) {
            const int c = u * 64 + lane;
            float t[8];
            ss += load_squares<DT>(xr + c * 8, c < chunks, t);
        }
        const float rstd = rstd_of(wave_sum(ss), a.K, a.eps);
        if (a.rstd && lane == 0) a.rstd[row] = rstd;
        for (int u = 0; u < passes; u++) {
            const int c = u * 64 + lane;
            float t[8];
            load_squares<DT>(xr + c * 8, c < chunks, t);
            norm_chunk<DT, WDT>(a, row, c, chunks, lane, rstd, t);
        }
    }
}

struct NormBwdArgs {
    const void *x, *w, *dout;
    const float *rstd;
    void *dx;
    float *dw_part;  // (gridDim.x, K) fp32, or NULL
    int64_t M, ldx, lddo, lddx;
    int K;
};

// dx = (dy - xhat * mean(dy * xhat)) * rstd with dy = dout * w, xhat = x * rstd; the weight
// gradient sum_rows(dout * xhat) is kept per lane for the lane's own columns across all rows of
// the wave, added over the workgroup's four waves through LDS and written as one partial row
// per workgroup (the caller sums the partial rows; a workgroup without rows writes zeros).
// K <= 512 CH.  (A variant that kept the row packed and fetched the next row ahead was measured
// 1.5x slower: the conditional prefetch makes the compiler wait for all loads at once, and the
// extra registers halve the waves per SIMD.)
template <int DT, int WDT, int CH>
__global__ __launch_bounds__(256) void rmsnorm_bwd_kernel(NormBwdArgs a) {
    typedef typename Elem<DT>::type T;
    typedef typename Elem<WDT>::type TW;
    __shared__ float red[3][64 * 8];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int chunks = a.K >> 3;
    float dw[CH][8];
#pragma unroll
    for (int u = 0; u < CH; u++)
#pragma unroll
        for (int i = 0; i < 8; i++) dw[u][i] = 0.0f;
    for (int64_t row = (int64_t)blockIdx.x * 4 + wave; row < a.M; row += (int64_t)gridDim.x * 4) {
        const T *xr = (const T *)a.x + row * a.ldx;
        const T *gr = (const T *)a.dout + row * a.lddo;
        const float rstd = a.rstd[row];
        float xh[CH][8], dy[CH][8];
        float dot = 0.0f;
#pragma unroll
        for (int u = 0; u < CH; u++) {
            const int c = u * 64 + lane;
            if (c < chunks) {
                float g[8], w[8];
                Elem<DT>::load8(xr + c * 8, xh[u]);
                Elem<DT>::load8(gr + c * 8, g);
                if (a.w) {  // from L1/L2 after the first row: held in registers it would cost 8 CH of them
                    Elem<WDT>::load8((const TW *)a.w + c * 8, w);
                } else {
#pragma unroll
                    for (int i = 0; i < 8; i++) w[i] = 1.0f;
                }
#pragma unroll
                for (int i = 0; i < 8; i++) {
                    xh[u][i] *= rstd;
                    dw[u][i] += g[i] * xh[u][i];
                    dy[u][i] = g[i] * w[i];
                    dot += dy[u][i] * xh[u][i];
                }
            } else {
#pragma unroll
                for (int i = 0; i < 8; i++) xh[u][i] = dy[u][i] = 0.0f;
            }
        }
        const float m = wave_sum(dot) / (float)a.K;
#pragma unroll
        for (int u = 0; u < CH; u++) {
            const int c = u * 64 + lane;
            if (c < chunks) {
                float r[8];
#pragma unroll
                for (int i = 0; i < 8; i++) r[i] = (dy[u][i] - xh[u][i] * m) * rstd;
                store8<DT>((T *)a.dx + row * a.lddx + c * 8, r);
            }
        }
    }
    if (!a.dw_part) return;
    // waves 1..3 hand their sums to wave 0, one 512-column slice at a time
#pragma unroll
    for (int u = 0; u < CH; u++) {
        __syncthreads();
        if (wave > 0) {
#pragma unroll
            for (int i = 0; i < 8; i++) red[wave - 1][i * 64 + lane] = dw[u][i];
        }
        __syncthreads();
        const int c = u * 64 + lane;
        if (wave == 0 && c < chunks) {
            float r[8];
#pragma unroll
            for (int i = 0; i < 8; i++) r[i] = dw[u][i] + red[0][i * 64 + lane] + red[1][i * 64 + lane] + red[2][i * 64 + lane];
            store8<MX_FP32>(a.dw_part + (int64_t)blockIdx.x * a.K + c * 8, r);
        }
    }
}

}  // namespace mx

using namespace mx;

static inline bool aligned(const void *p, uintptr_t n) { return ((uintptr_t)p & (n - 1)) == 0; }
static inline int esize(int dt) { return dt == MX_FP32 ? 4 : 2; }
static inline bool dtype_ok(int dt) { return dt == MX_BF16 || dt == MX_FP16 || dt == MX_FP32; }

template <int DT, int WDT>
static int launch_norm(const NormArgs &a, hipStream_t st) {
    const dim3 grid((unsigned)((a.M + 3) / 4)), block(256);
    const int ch = (a.K + 511) / 512;
    if (ch <= 1) rmsnorm_quant_kernel<DT, WDT, 1><<<grid, block, 0, st>>>(a);
    else if (ch <= 2) rmsnorm_quant_kernel<DT, WDT, 2><<<grid, block, 0, st>>>(a);
    else if (ch <= 3) rmsnorm_quant_kernel<DT, WDT, 3><<<grid, block, 0, st>>>(a);
    else if (ch <= 4) rmsnorm_quant_kernel<DT, WDT, 4><<<grid, block, 0, st>>>(a);
    else if (ch <= 6) rmsnorm_quant_kernel<DT, WDT, 6><<<grid, block, 0, st>>>(a);
    else if (ch <= 8) rmsnorm_quant_kernel<DT, WDT, 8><<<grid, block, 0, st>>>(a);
    else rmsnorm_quant_kernel<DT, WDT, 0><<<grid, block, 0, st>>>(a);
    return hipGetLastError() == hipSuccess ? MX_OK : MX_ELAUNCH;
}

template <int DT>
static int launch_norm_w(const NormArgs &a, int w_dtype, hipStream_t st) {
    if (!a.w || w_dtype == DT) return launch_norm<DT, DT>(a, st);
    if (w_dtype == MX_FP32) return launch_norm<DT, MX_FP32>(a, st);
    return MX_EUNSUPPORTED;  // a 16-bit weight of the other 16-bit type
}

extern "C" int mx_rmsnorm_quantize(const void *x, int x_dtype, int64_t M, int64_t K, int64_t ldx, const void *weight,
                                   int w_dtype, float eps, void *out, int64_t ldo, float *rstd, uint8_t *q,
                                   int64_t ldq, uint8_t *s, int64_t lds, void *stream) {
    if (M < 0 || K <= 0 || K >= (1 << 28) || !x || !dtype_ok(x_dtype) || (weight && !dtype_ok(w_dtype)) || ldx < K ||
        (out && ldo < K) || (q != nullptr) != (s != nullptr) || (q && (K % MX_BLOCK || ldq < K || lds < K / MX_BLOCK)) ||
        (!out && !q && !rstd))
        return MX_EINVAL;
    if (M == 0) return MX_OK;
    const int ex = esize(x_dtype);
    if (K % 8 || !aligned(x, 16) || (ldx * ex) % 16 || (out && (!aligned(out, 16) || (ldo * ex) % 16)) ||
        (weight && !aligned(weight, 16)) || (q && (!aligned(q, 8) || ldq % 8)) || (M + 3) / 4 > 0x7FFFFFFF)
        return MX_EUNSUPPORTED;
    NormArgs a = {x, weight, out, rstd, q, s, M, ldx, ldo, ldq, lds, (int)K, eps};
    hipStream_t st = (hipStream_t)stream;
    if (mx::stream_is_capturing(st)) return MX_ECAPTURE;
    switch (x_dtype) {
    case MX_BF16: return launch_norm_w<MX_BF16>(a, w_dtype, st);
    case MX_FP16: return launch_norm_w<MX_FP16>(a, w_dtype, st);
    default: return launch_norm_w<MX_FP32>(a, w_dtype, st);
    }
}

template <int DT, int WDT>
static int launch_norm_bwd(const NormBwdArgs &a, int64_t parts, hipStream_t st) {
    const dim3 grid((unsigned)parts), block(256);
    const int ch = (a.K + 511) / 512;
    if (ch <= 1) rmsnorm_bwd_kernel<DT, WDT, 1><<<grid, block, 0, st>>>(a);
    else if (ch <= 2) rmsnorm_bwd_kernel<DT, WDT, 2><<<grid, block, 0, st>>>(a);
    else if (ch <= 3) rmsnorm_bwd_kernel<DT, WDT, 3><<<grid, block, 0, st>>>(a);
    else if (ch <= 4) rmsnorm_bwd_kernel<DT, WDT, 4><<<grid, block, 0, st>>>(a);
    else if (ch <= 6) rmsnorm_bwd_kernel<DT, WDT, 6><<<grid, block, 0, st>>>(a);
    else if (ch <= 8) rmsnorm_bwd_kernel<DT, WDT, 8><<<grid, block, 0, st>>>(a);
    else return MX_EUNSUPPORTED;
    return hipGetLastError() == hipSuccess ? MX_OK : MX_ELAUNCH;
}

extern "C" int mx_rmsnorm_backward(const void *x, int dtype, int64_t M, int64_t K, int64_t ldx, const void *weight,
                                   int w_dtype, const void *dout, int64_t lddo, const float *rstd, void *dx,
                                   int64_t lddx, float *dw_part, int64_t parts, void *stream) {
    if (M < 0 || K <= 0 || !x || !dout || !rstd || !dx || (dtype != MX_BF16 && dtype != MX_FP16) ||
        (weight && !dtype_ok(w_dtype)) || ldx < K || lddo < K || lddx < K || parts <= 0 || parts > 65535)
        return MX_EINVAL;
    if (M == 0 && !dw_part) return MX_OK;
    if (K % 8 || K > 4096 || !aligned(x, 16) || !aligned(dout, 16) || !aligned(dx, 16) || ldx % 8 || lddo % 8 || lddx % 8 ||
        (weight && !aligned(weight, 16)) || (dw_part && !aligned(dw_part, 16)))
        return MX_EUNSUPPORTED;
    NormBwdArgs a = {x, weight, dout, rstd, dx, dw_part, M, ldx, lddo, lddx, (int)K};
    hipStream_t st = (hipStream_t)stream;
    if (mx::stream_is_capturing(st)) return MX_ECAPTURE;
    const bool w32 = weight && w_dtype == MX_FP32;
    if (weight && !w32 && w_dtype != dtype) return MX_EUNSUPPORTED;
    if (dtype == MX_BF16) return w32 ? launch_norm_bwd<MX_BF16, MX_FP32>(a, parts, st) : launch_norm_bwd<MX_BF16, MX_BF16>(a, parts, st);
    return w32 ? launch_norm_bwd<MX_FP16, MX_FP32>(a, parts, st) : launch_norm_bwd<MX_FP16, MX_FP16>(a, parts, st);
}
