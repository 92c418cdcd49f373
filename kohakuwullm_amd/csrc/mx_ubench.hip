// The denominators the kernels of this library are priced against, measured on the device itself:
// streaming bandwidth (read, copy, triad, and the quantizer's own 2-bytes-in 1-byte-out mix) and the
// issue rate of the block-scaled fp8 MFMA from registers.  The reference measures its roofline
// denominators the same way instead of quoting a data sheet (copy / read / triad:
// src/kohakuwullm/bench/core/timing.py:231-268; a register-resident MMA loop with independent
// accumulators: docs/internals/kernel-convention.md:14-33).
#include "mx_common.h"

namespace mx {

int num_cus();  // mx_gemm.hip

// 16 bytes per lane per access, UNROLL accesses of every stream in flight per lane, grid-stride over whole chunks.
// What is swept (mx_ubench_stream_cfg): threads per workgroup, UNROLL, workgroups per CU (0: one chunk per workgroup,
// no loop) and whether loads / stores carry the non-temporal hint.  The default entry point runs one fixed point.
constexpr int STREAM_THREADS = 256;
constexpr int STREAM_UNROLL = 4;
constexpr int STREAM_MAX_THREADS = 1024;

template <bool NT>
__device__ __forceinline__ v4i ld16(const v4i *p) { return NT ? __builtin_nontemporal_load(p) : *p; }
template <bool NT>
__device__ __forceinline__ void st16(v4i *p, v4i v) {
    if (NT) __builtin_nontemporal_store(v, p);
    else *p = v;
}

// kind 0: read only (a); every thread folds what it read into one dword of `c` (one per thread)
// kind 1: copy c = a                                                            (1 : 1)
// kind 2: triad c = a + 2 b on fp32                                             (2 : 1, with arithmetic)
// kind 3: 2 : 1 mix -- reads two 16-byte vectors (a[2i], a[2i+1]) and writes one (their byte-wise fold) to c[i]:
//         the traffic of a 16-bit -> 8-bit cast without its arithmetic, one input stream
// kind 4: 2 : 1 mix from two input streams -- c[i] = fold(a[i], a[n + i]) (a holds 2 n vectors)
// kind 5: 3 : 2 mix -- reads a[i], a[n + i], a[2 n + i], writes c[i] and c[n + i] (a holds 3 n vectors, c 2 n):
//         the traffic of the SwiGLU' quantizer (three 16-bit inputs, four 8-bit outputs)
template <int KIND, int UNROLL, bool NTL, bool NTS>
__global__ __launch_bounds__(STREAM_MAX_THREADS) void stream_kernel(const v4i *__restrict__ a, const v4i *__restrict__ b,
                                                                    v4i *__restrict__ c, int64_t n_out) {
    const int64_t stride = (int64_t)gridDim.x * blockDim.x;
    int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    v4i fold = {0, 0, 0, 0};
    for (; i + (UNROLL - 1) * stride < n_out; i += UNROLL * stride) {
        v4i x[UNROLL], y[UNROLL], z[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            const int64_t at = i + u * stride;
            if (KIND == 3) {
                x[u] = ld16<NTL>(a + 2 * at);
                y[u] = ld16<NTL>(a + 2 * at + 1);
            } else {
                x[u] = ld16<NTL>(a + at);
                if (KIND == 2) y[u] = ld16<NTL>(b + at);
                if (KIND >= 4) y[u] = ld16<NTL>(a + n_out + at);
                if (KIND == 5) z[u] = ld16<NTL>(a + 2 * n_out + at);
            }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; u++) {
            const int64_t at = i + u * stride;
            if (KIND == 0) {
                fold ^= x[u];
            } else if (KIND == 1) {
                st16<NTS>(c + at, x[u]);
            } else if (KIND == 2) {
                v4f fa = __builtin_bit_cast(v4f, x[u]), fb = __builtin_bit_cast(v4f, y[u]);
                st16<NTS>(c + at, __builtin_bit_cast(v4i, fa + 2.0f * fb));
            } else if (KIND == 5) {
                st16<NTS>(c + at, (x[u] & 0x00FF00FF) | ((y[u] & 0x00FF00FF) << 8));
                st16<NTS>(c + n_out + at, (z[u] & 0x00FF00FF) | ((y[u] & 0xFF00FF00)));
            } else {
                st16<NTS>(c + at, (x[u] & 0x00FF00FF) | ((y[u] & 0x00FF00FF) << 8));
            }
        }
    }
    for (; i < n_out; i += stride) {  // the ragged end, one vector at a time
        if (KIND == 0) fold ^= a[i];
        else if (KIND == 1) c[i] = a[i];
        else if (KIND == 2) c[i] = __builtin_bit_cast(v4i, __builtin_bit_cast(v4f, a[i]) + 2.0f * __builtin_bit_cast(v4f, b[i]));
        else if (KIND == 3) c[i] = (a[2 * i] & 0x00FF00FF) | ((a[2 * i + 1] & 0x00FF00FF) << 8);
        else if (KIND == 4) c[i] = (a[i] & 0x00FF00FF) | ((a[n_out + i] & 0x00FF00FF) << 8);
        else {
            c[i] = (a[i] & 0x00FF00FF) | ((a[n_out + i] & 0x00FF00FF) << 8);
            c[n_out + i] = (a[2 * n_out + i] & 0x00FF00FF) | (a[n_out + i] & 0xFF00FF00);
        }
    }
    if (KIND == 0) ((int *)c)[(int64_t)blockIdx.x * blockDim.x + threadIdx.x] = fold[0] ^ fold[1] ^ fold[2] ^ fold[3];
}

template <int KIND, int UNROLL>
static void launch_stream(bool ntl, bool nts, dim3 grid, dim3 block, hipStream_t st, const v4i *a, const v4i *b, v4i *c,
                          int64_t n) {
    if (ntl && nts) stream_kernel<KIND, UNROLL, true, true><<<grid, block, 0, st>>>(a, b, c, n);
    else if (ntl) stream_kernel<KIND, UNROLL, true, false><<<grid, block, 0, st>>>(a, b, c, n);
    else if (nts) stream_kernel<KIND, UNROLL, false, true><<<grid, block, 0, st>>>(a, b, c, n);
    else stream_kernel<KIND, UNROLL, false, false><<<grid, block, 0, st>>>(a, b, c, n);
}

template <int KIND>
static int launch_stream_unroll(int unroll, bool ntl, bool nts, dim3 grid, dim3 block, hipStream_t st, const v4i *a,
                                const v4i *b, v4i *c, int64_t n) {
    switch (unroll) {
    case 1: launch_stream<KIND, 1>(ntl, nts, grid, block, st, a, b, c, n); break;
    case 2: launch_stream<KIND, 2>(ntl, nts, grid, block, st, a, b, c, n); break;
    case 4: launch_stream<KIND, 4>(ntl, nts, grid, block, st, a, b, c, n); break;
    case 8: launch_stream<KIND, 8>(ntl, nts, grid, block, st, a, b, c, n); break;
    default: return MX_EINVAL;
    }
    return MX_OK;
}

// The memory access pattern of the 128 x 128 tile quantizers without their arithmetic: 256 threads, thread (t % 16,
// t / 16) reads 16 bytes of each of 8 rows (a row pitch apart) from every input, writes 8 bytes per row into a (M, K)
// byte matrix (the row-axis codes' place) and, through LDS, the transposed byte tile into a (K, M) byte matrix in
// 16-byte pieces (row-major, or 128-token panels: the stage-major layout).  INPUTS 1: one 16-bit matrix (the plain
// quantizers), 2: the two halves of a (M, 2K) matrix (SwiGLU), 3: those and a (M, K) matrix, two sets of outputs
// (SwiGLU').  What this reaches bounds what those kernels can: the same bytes in the same places, no arithmetic.
template <int INPUTS, bool TRANSPOSED, bool NTL, bool NTS>
__global__ __launch_bounds__(256) void tile_pattern_kernel(const uint16_t *__restrict__ x, const uint16_t *__restrict__ y,
                                                            int64_t M, int64_t K, int64_t ldx, uint8_t *__restrict__ q,
                                                            uint8_t *__restrict__ qT, uint8_t *__restrict__ q2,
                                                            uint8_t *__restrict__ qT2, int panels) {
    __shared__ __attribute__((aligned(16))) uint8_t tile[128 * 136];
    const int t = threadIdx.x, cg = t & 15, rg = t >> 4;
    const int64_t m0 = (int64_t)blockIdx.y * 128, k0 = (int64_t)blockIdx.x * 128;
    const int64_t col = k0 + cg * 8, row0 = m0 + rg * 8;
    v4i a[8], b[8], c[8];
#pragma unroll
    for (int i = 0; i < 8; i++) {
        a[i] = ld16<NTL>((const v4i *)(x + (row0 + i) * ldx + col));
        if (INPUTS >= 2) b[i] = ld16<NTL>((const v4i *)(x + (row0 + i) * ldx + K + col));
        if (INPUTS == 3) c[i] = ld16<NTL>((const v4i *)(y + (row0 + i) * K + col));
    }
#pragma unroll
    for (int pass = 0; pass < (INPUTS == 3 ? 2 : 1); pass++) {
        uint8_t *qq = pass ? q2 : q, *qqT = pass ? qT2 : qT;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            v4i v = a[i];
            if (INPUTS >= 2) v ^= pass ? c[i] : b[i];
            if (INPUTS == 3 && !pass) v ^= c[i];
            typedef int v2i_t __attribute__((ext_vector_type(2)));
            const v2i_t codes = {v[0] ^ v[1], v[2] ^ v[3]};
            v2i_t *dst = (v2i_t *)(qq + (panels ? (col >> 7) * (M * 128) + (row0 + i) * 128 + (col & 127) : (row0 + i) * K + col));
            if (NTS) __builtin_nontemporal_store(codes, dst);
            else *dst = codes;
            if (TRANSPOSED) {
#pragma unroll
                for (int e = 0; e < 8; e++) tile[(cg * 8 + e) * 136 + rg * 8 + i] = (uint8_t)(v[e >> 1] >> ((e & 1) * 16));
            }
        }
        if (TRANSPOSED) {
            __syncthreads();
#pragma unroll
            for (int j = 0; j < 4; j++) {
                const int kr = j * 32 + (t >> 3), ch = t & 7;
                const int *src = (const int *)(tile + kr * 136 + ch * 16);
                st16<NTS>((v4i *)(qqT + (panels ? (m0 >> 7) * (K * 128) + (k0 + kr) * 128 : (k0 + kr) * M + m0) + ch * 16),
                          v4i{src[0], src[1], src[2], src[3]});
            }
            __syncthreads();
        }
    }
}

// Register-resident block-scaled fp8 MFMA loop: ACCS independent accumulator tiles per wave, operands that never
// change, no memory traffic.  `random` fills the operand registers with a per-lane hash (switching activity of
// real data) instead of zeros: the part's clock, and with it this peak, depends on what the multipliers see.
template <bool WIDE, bool VSCALE = false>  // WIDE false: 16x16x128 (4 accumulator registers), true: 32x32x64 (16)
__global__ __launch_bounds__(512) void mfma_peak_kernel(int iters, int random, float *out) {
    typedef float v16f __attribute__((ext_vector_type(16)));
    constexpr int ACCS = WIDE ? 4 : 8;
    const uint32_t lane = threadIdx.x;
    v8i a[2], b[2];
#pragma unroll
    for (int k = 0; k < 2; k++)
#pragma unroll
        for (int i = 0; i < 8; i++) {
            uint32_t h = (lane * 2654435761u) ^ ((uint32_t)(i + 8 * k) * 0x9E3779B9u) ^ (blockIdx.x * 0x85EBCA6Bu);
            h ^= h >> 15, h *= 0x2C1B3C6Du, h ^= h >> 12;
            h &= 0xF7F7F7F7u;  // every byte a finite e4m3 code (exponent field never all ones), both signs
            a[k][i] = random ? (int)h : 0;
            b[k][i] = random ? (int)((h * 0x27D4EB2Fu) & 0xF7F7F7F7u) : 0;
        }
    // VSCALE: the scale bytes come from vector registers the compiler cannot see through (as in a GEMM, where they
    // are data), one register per accumulator tile, instead of an inline constant
    int sc[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        sc[j] = 0x7F7F7F7F;
        if (VSCALE) asm volatile("" : "+v"(sc[j]));
    }
    float sum = 0.f;
    if (!WIDE) {
        v4f acc[ACCS];
#pragma unroll
        for (int j = 0; j < ACCS; j++) acc[j] = v4f{0.f, 0.f, 0.f, 0.f};
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int j = 0; j < ACCS; j++)
                acc[j] = VSCALE ? __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[j & 1], b[(j >> 1) & 1], acc[j], 0, 0, 0, sc[j], 0,
                                                                                   sc[(j + 3) & 7])
                                : __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[j & 1], b[(j >> 1) & 1], acc[j], 0, 0, 0,
                                                                                   0x7F7F7F7F, 0, 0x7F7F7F7F);
        }
#pragma unroll
        for (int j = 0; j < ACCS; j++) sum += acc[j][0] + acc[j][3];
    } else {
        v16f acc[ACCS];
#pragma unroll
        for (int j = 0; j < ACCS; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[j][e] = 0.f;
        for (int it = 0; it < iters; it++) {
#pragma unroll
            for (int j = 0; j < ACCS; j++)
                acc[j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[j & 1], b[(j >> 1) & 1], acc[j], 0, 0, 0, 0x7F7F7F7F, 0,
                                                                         0x7F7F7F7F);
        }
#pragma unroll
        for (int j = 0; j < ACCS; j++) sum += acc[j][0] + acc[j][15];
    }
    out[(int64_t)blockIdx.x * 512 + threadIdx.x] = sum;
}

}  // namespace mx

using namespace mx;

extern "C" int mx_ubench_stream_cfg(int kind, int threads, int unroll, int wgs_per_cu, int nontemporal, const void *a,
                                    const void *b, void *c, int64_t out_bytes, void *stream) {
    if (kind < 0 || kind > 5 || out_bytes < 0 || out_bytes % 16) return MX_EINVAL;
    if (threads < 64 || threads > STREAM_MAX_THREADS || threads % 64 || wgs_per_cu < 0 || nontemporal < 0 || nontemporal > 3)
        return MX_EINVAL;
    if (!a || !c || (kind == 2 && !b) || ((uintptr_t)a & 15) || ((uintptr_t)b & 15) || ((uintptr_t)c & 15)) return MX_EINVAL;
    hipStream_t st = (hipStream_t)stream;
    if (mx::stream_is_capturing(st)) return MX_ECAPTURE;
    const int64_t n = out_bytes / 16;
    // enough resident waves to cover HBM latency on every CU, few enough that the grid-stride loop does the work
    const int64_t want = (n + (int64_t)threads * unroll - 1) / ((int64_t)threads * unroll);
    const int64_t cap = wgs_per_cu ? (int64_t)num_cus() * wgs_per_cu : want;
    if ((want < cap ? want : cap) > 0x7FFFFFFF) return MX_EUNSUPPORTED;
    const dim3 grid((unsigned)(want < 1 ? 1 : want < cap ? want : cap)), block((unsigned)threads);
    const bool ntl = nontemporal & 1, nts = nontemporal & 2;
    const v4i *pa = (const v4i *)a, *pb = (const v4i *)b;
    v4i *pc = (v4i *)c;
    int rc;
    switch (kind) {
    case 0: rc = launch_stream_unroll<0>(unroll, ntl, nts, grid, block, st, pa, pb, pc, n); break;
    case 1: rc = launch_stream_unroll<1>(unroll, ntl, nts, grid, block, st, pa, pb, pc, n); break;
    case 2: rc = launch_stream_unroll<2>(unroll, ntl, nts, grid, block, st, pa, pb, pc, n); break;
    case 3: rc = launch_stream_unroll<3>(unroll, ntl, nts, grid, block, st, pa, pb, pc, n); break;
    case 4: rc = launch_stream_unroll<4>(unroll, ntl, nts, grid, block, st, pa, pb, pc, n); break;
    default: rc = launch_stream_unroll<5>(unroll, ntl, nts, grid, block, st, pa, pb, pc, n); break;
    }
    if (rc != MX_OK) return rc;
    return hipGetLastError() == hipSuccess ? MX_OK : MX_ELAUNCH;
}

template <int INPUTS, bool TRANSPOSED>
static void launch_tile_pattern(int nt, dim3 grid, hipStream_t st, const uint16_t *x, const uint16_t *y, int64_t M, int64_t K,
                                int64_t ldx, uint8_t *q, uint8_t *qT, uint8_t *q2, uint8_t *qT2, int panels) {
    const dim3 block(256);
    switch (nt) {
    case 0: tile_pattern_kernel<INPUTS, TRANSPOSED, false, false><<<grid, block, 0, st>>>(x, y, M, K, ldx, q, qT, q2, qT2, panels); break;
    case 1: tile_pattern_kernel<INPUTS, TRANSPOSED, true, false><<<grid, block, 0, st>>>(x, y, M, K, ldx, q, qT, q2, qT2, panels); break;
    case 2: tile_pattern_kernel<INPUTS, TRANSPOSED, false, true><<<grid, block, 0, st>>>(x, y, M, K, ldx, q, qT, q2, qT2, panels); break;
    default: tile_pattern_kernel<INPUTS, TRANSPOSED, true, true><<<grid, block, 0, st>>>(x, y, M, K, ldx, q, qT, q2, qT2, panels); break;
    }
}

extern "C" int mx_ubench_tile_pattern(int inputs, int transposed, int nontemporal, int panels, const void *x, int64_t ldx,
                                      const void *y, int64_t M, int64_t K, uint8_t *q, uint8_t *qT, uint8_t *q2, uint8_t *qT2,
                                      void *stream) {
    if (inputs < 1 || inputs > 3 || nontemporal < 0 || nontemporal > 3 || M <= 0 || K <= 0 || M % 128 || K % 128) return MX_EINVAL;
    if (!x || !q || (transposed && !qT) || (inputs == 3 && (!y || !q2 || (transposed && !qT2)))) return MX_EINVAL;
    if (ldx < (inputs >= 2 ? 2 * K : K) || ldx % 8 || ((uintptr_t)x & 15) || ((uintptr_t)y & 15) || ((uintptr_t)q & 15) ||
        ((uintptr_t)qT & 15) || ((uintptr_t)q2 & 15) || ((uintptr_t)qT2 & 15) || M / 128 > 65535)
        return MX_EINVAL;
    hipStream_t st = (hipStream_t)stream;
    if (mx::stream_is_capturing(st)) return MX_ECAPTURE;
    const dim3 grid((unsigned)(K / 128), (unsigned)(M / 128));
    const uint16_t *px = (const uint16_t *)x, *py = (const uint16_t *)y;
    const int p = panels ? 1 : 0;
    if (inputs == 1 && transposed) launch_tile_pattern<1, true>(nontemporal, grid, st, px, py, M, K, ldx, q, qT, q2, qT2, p);
    else if (inputs == 1) launch_tile_pattern<1, false>(nontemporal, grid, st, px, py, M, K, ldx, q, qT, q2, qT2, p);
    else if (inputs == 2 && transposed) launch_tile_pattern<2, true>(nontemporal, grid, st, px, py, M, K, ldx, q, qT, q2, qT2, p);
    else if (inputs == 2) launch_tile_pattern<2, false>(nontemporal, grid, st, px, py, M, K, ldx, q, qT, q2, qT2, p);
    else if (transposed) launch_tile_pattern<3, true>(nontemporal, grid, st, px, py, M, K, ldx, q, qT, q2, qT2, p);
    else launch_tile_pattern<3, false>(nontemporal, grid, st, px, py, M, K, ldx, q, qT, q2, qT2, p);
    return hipGetLastError() == hipSuccess ? MX_OK : MX_ELAUNCH;
}

extern "C" int mx_ubench_stream(int kind, const void *a, const void *b, void *c, int64_t out_bytes, void *stream) {
    if (kind > 3) return MX_EINVAL;
    return mx_ubench_stream_cfg(kind, STREAM_THREADS, STREAM_UNROLL, 16, 3, a, b, c, out_bytes, stream);
}

extern "C" int64_t mx_ubench_mfma(int wide, int iters, int random, float *out, int64_t out_floats, void *stream) {
    if (iters <= 0 || !out) return MX_EINVAL;
    hipStream_t st = (hipStream_t)stream;
    if (mx::stream_is_capturing(st)) return MX_ECAPTURE;
    const int cus = num_cus();
    if (out_floats < (int64_t)cus * 512) return MX_EINVAL;
    // bit 0 of `wide`: the 32x32x64 form; bit 1: four waves per CU (one per SIMD) instead of eight; bit 2 (16x16x128
    // only): scale bytes from vector registers instead of an inline constant
    const int waves = (wide & 2) ? 4 : 8;
    if (wide & 1) mfma_peak_kernel<true><<<dim3((unsigned)cus), dim3(waves * 64), 0, st>>>(iters, random, out);
    else if (wide & 4) mfma_peak_kernel<false, true><<<dim3((unsigned)cus), dim3(waves * 64), 0, st>>>(iters, random, out);
    else mfma_peak_kernel<false><<<dim3((unsigned)cus), dim3(waves * 64), 0, st>>>(iters, random, out);
    if (hipGetLastError() != hipSuccess) return MX_ELAUNCH;
    // MFMA instructions issued by the launch: workgroups x waves x iterations x accumulators per wave
    return (int64_t)cus * waves * iters * ((wide & 1) ? 4 : 8);
}
