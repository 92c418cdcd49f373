// The denominators the kernels of this library are priced against, measured on the device itself:
// streaming bandwidth (read, copy, triad, and the quantizer's own 2-bytes-in 1-byte-out mix) and the
// issue rate of the block-scaled fp8 MFMA from registers.  The reference measures its roofline
// denominators the same way instead of quoting a data sheet (copy / read / triad:
// src/kohakuwullm/bench/core/timing.py:231-268; a register-resident MMA loop with independent
// accumulators: docs/internals/kernel-convention.md:14-33).
#include "mx_common.h"

namespace mx {

int num_cus();  // mx_gemm.hip

// 16 bytes per lane per load, UNROLL loads in flight per lane, grid-stride over whole chunks.
constexpr int STREAM_THREADS = 256;
constexpr int STREAM_UNROLL = 4;

__device__ __forceinline__ v4i nt_load(const v4i *p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void nt_store(v4i *p, v4i v) { __builtin_nontemporal_store(v, p); }

// kind 0: read only (a); every thread folds what it read into one dword of `c` (one per thread)
// kind 1: copy c = a
// kind 2: triad c = a + 2 b on fp32
// kind 3: 2 : 1 mix -- reads two 16-byte vectors (a[2i], a[2i+1]) and writes one (their byte-wise fold) to c[i]:
//         the traffic of a 16-bit -> 8-bit cast without its arithmetic
template <int KIND>
__global__ __launch_bounds__(STREAM_THREADS) void stream_kernel(const v4i *__restrict__ a, const v4i *__restrict__ b,
                                                                v4i *__restrict__ c, int64_t n_out) {
    const int64_t stride = (int64_t)gridDim.x * STREAM_THREADS;
    int64_t i = (int64_t)blockIdx.x * STREAM_THREADS + threadIdx.x;
    v4i fold = {0, 0, 0, 0};
    for (; i + (STREAM_UNROLL - 1) * stride < n_out; i += STREAM_UNROLL * stride) {
        v4i x[STREAM_UNROLL], y[STREAM_UNROLL];
#pragma unroll
        for (int u = 0; u < STREAM_UNROLL; u++) {
            if (KIND == 3) {
                x[u] = nt_load(a + 2 * (i + u * stride));
                y[u] = nt_load(a + 2 * (i + u * stride) + 1);
            } else {
                x[u] = nt_load(a + i + u * stride);
                if (KIND == 2) y[u] = nt_load(b + i + u * stride);
            }
        }
#pragma unroll
        for (int u = 0; u < STREAM_UNROLL; u++) {
            if (KIND == 0) {
                fold ^= x[u];
            } else if (KIND == 1) {
                nt_store(c + i + u * stride, x[u]);
            } else if (KIND == 2) {
                v4f fa = __builtin_bit_cast(v4f, x[u]), fb = __builtin_bit_cast(v4f, y[u]);
                nt_store(c + i + u * stride, __builtin_bit_cast(v4i, fa + 2.0f * fb));
            } else {
                nt_store(c + i + u * stride, (x[u] & 0x00FF00FF) | ((y[u] & 0x00FF00FF) << 8));
            }
        }
    }
    for (; i < n_out; i += stride) {  // the ragged end, one vector at a time
        if (KIND == 0) fold ^= a[i];
        else if (KIND == 1) c[i] = a[i];
        else if (KIND == 2) c[i] = __builtin_bit_cast(v4i, __builtin_bit_cast(v4f, a[i]) + 2.0f * __builtin_bit_cast(v4f, b[i]));
        else c[i] = (a[2 * i] & 0x00FF00FF) | ((a[2 * i + 1] & 0x00FF00FF) << 8);
    }
    if (KIND == 0) ((int *)c)[(int64_t)blockIdx.x * STREAM_THREADS + threadIdx.x] = fold[0] ^ fold[1] ^ fold[2] ^ fold[3];
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

extern "C" int mx_ubench_stream(int kind, const void *a, const void *b, void *c, int64_t out_bytes, void *stream) {
    if (kind < 0 || kind > 3 || out_bytes < 0 || out_bytes % 16) return MX_EINVAL;
    if (!a || !c || (kind == 2 && !b) || ((uintptr_t)a & 15) || ((uintptr_t)b & 15) || ((uintptr_t)c & 15)) return MX_EINVAL;
    hipStream_t st = (hipStream_t)stream;
    if (mx::stream_is_capturing(st)) return MX_ECAPTURE;
    const int64_t n = out_bytes / 16;
    // enough resident waves to cover HBM latency on every CU, few enough that the grid-stride loop does the work
    const int64_t want = (n + STREAM_THREADS * STREAM_UNROLL - 1) / (STREAM_THREADS * STREAM_UNROLL);
    const int64_t cap = (int64_t)num_cus() * 16;
    const dim3 grid((unsigned)(want < 1 ? 1 : want < cap ? want : cap)), block(STREAM_THREADS);
    switch (kind) {
    case 0: stream_kernel<0><<<grid, block, 0, st>>>((const v4i *)a, nullptr, (v4i *)c, n); break;
    case 1: stream_kernel<1><<<grid, block, 0, st>>>((const v4i *)a, nullptr, (v4i *)c, n); break;
    case 2: stream_kernel<2><<<grid, block, 0, st>>>((const v4i *)a, (const v4i *)b, (v4i *)c, n); break;
    default: stream_kernel<3><<<grid, block, 0, st>>>((const v4i *)a, nullptr, (v4i *)c, n); break;
    }
    return hipGetLastError() == hipSuccess ? MX_OK : MX_ELAUNCH;
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
