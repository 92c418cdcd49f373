// Shared device helpers for the MXFP8 kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "mxfp8_hip.h"

#define MX_BLOCK 32

namespace mx {

// Whether work on `st` is being recorded into a graph (mx_gemm.hip).  Every entry point asks before it
// launches and returns MX_ECAPTURE: recording this library's launches is switched off.
bool stream_is_capturing(hipStream_t st);

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef unsigned short v8us __attribute__((ext_vector_type(8)));

__device__ __forceinline__ float bits2f(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f2bits(float f) { return __builtin_bit_cast(uint32_t, f); }

// UE8M0 byte of a block from its fp32 amax (>= 0):
// ceil(log2(max(amax,1e-30)/448)) + 127 == E - 8 + (M > 0x600000) because 448 = 1.75 * 2^8.
// quantize.py:53-56 of the reference.
__device__ __forceinline__ uint32_t scale_byte(float amax) {
    uint32_t u = f2bits(amax);
    u = u > 0x0DA24260u ? u : 0x0DA24260u;  // max(amax, 1e-30f) on the bit pattern (amax >= 0)
    uint32_t e = u >> 23;
    uint32_t m = u & 0x7FFFFFu;
    return e - 8u + (m > 0x600000u ? 1u : 0u);
}

// 2^(127 - byte): multiplying by it divides by the block scale exactly.
__device__ __forceinline__ float inv_scale(uint32_t byte) { return bits2f((254u - byte) << 23); }

// Two fp32 -> two e4m3 bytes (RTNE) into the low or high half of `old`.
template <bool HI>
__device__ __forceinline__ int cvt_pk_e4m3(float a, float b, int old) {
    return __builtin_amdgcn_cvt_pk_fp8_f32(a, b, old, HI);
}

__device__ __forceinline__ uint32_t pack4_e4m3(float a, float b, float c, float d) {
    int v = 0;
    v = cvt_pk_e4m3<false>(a, b, v);
    v = cvt_pk_e4m3<true>(c, d, v);
    return (uint32_t)v;
}

// 1 / (1 + e^-x) with the hardware exponential and reciprocal (v_exp_f32, v_rcp_f32: 1 ulp each).
// Every SwiGLU in the library goes through this one function, so a fused epilogue and the
// stand-alone quantizer of the same values agree bit for bit.  Written as a division the
// compiler emitted the IEEE sequence (v_div_scale x2, v_rcp, four v_fma, v_div_fmas,
// v_div_fixup): ten instructions per value, a sixth of the expert GEMM2-dgrad epilogue.
__device__ __forceinline__ float sigmoid_f32(float x) { return __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }

// Element loaders: 8 consecutive elements starting at p (16-byte aligned for 16-bit types).
template <int DT>
struct Elem;

// Bulk loads and stores of the streaming kernels, with or without the non-temporal hint.  The hint pays for data that is
// read once or written for a consumer far away (measured inside a feed-forward step: the SwiGLU' quantizer 148 -> 131 us
// with hinted loads) and costs where the next kernel would have found the lines in the last-level cache (codes of a 48 MB
// activation written with the hint: the GEMM that reads them next 186 -> 191 us), so each kernel chooses.
template <bool NT, typename V>
__device__ __forceinline__ V stream_load(const V *p) {
    if (NT) return __builtin_nontemporal_load(p);
    return *p;
}
template <bool NT, typename V>
__device__ __forceinline__ void stream_store(V *p, V v) {
    if (NT) __builtin_nontemporal_store(v, p);
    else *p = v;
}

template <>
struct Elem<MX_BF16> {
    typedef uint16_t type;
    static __device__ __forceinline__ void load8(const void *p, float v[8]) {
        v4i r = *(const v4i *)p;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            v[2 * i] = bits2f((uint32_t)r[i] << 16);
            v[2 * i + 1] = bits2f((uint32_t)r[i] & 0xFFFF0000u);
        }
    }
    static __device__ __forceinline__ float load1(const void *p) { return bits2f((uint32_t)(*(const uint16_t *)p) << 16); }
    // The same load in two halves, so that a kernel can put many of them in flight before it converts any.
    typedef v4i raw;
    template <bool NT = false>
    static __device__ __forceinline__ raw load_raw(const void *p) { return stream_load<NT>((const v4i *)p); }
    // value c (0..7) of a raw row chunk, converted where it is used: a kernel that keeps its tile raw holds half the registers
    static __device__ __forceinline__ float elem(const raw &r, int c) {
        const uint32_t w = (uint32_t)r[c >> 1];
        return bits2f((c & 1) ? (w & 0xFFFF0000u) : (w << 16));
    }
    static __device__ __forceinline__ void unpack(const raw &r, float v[8]) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            v[2 * i] = bits2f((uint32_t)r[i] << 16);
            v[2 * i + 1] = bits2f((uint32_t)r[i] & 0xFFFF0000u);
        }
    }
};

template <>
struct Elem<MX_FP16> {
    typedef uint16_t type;
    static __device__ __forceinline__ void load8(const void *p, float v[8]) {
        typedef _Float16 h8 __attribute__((ext_vector_type(8)));
        h8 r = *(const h8 *)p;
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = (float)r[i];
    }
    static __device__ __forceinline__ float load1(const void *p) { return (float)(*(const _Float16 *)p); }
    typedef _Float16 raw __attribute__((ext_vector_type(8)));
    template <bool NT = false>
    static __device__ __forceinline__ raw load_raw(const void *p) { return stream_load<NT>((const raw *)p); }
    static __device__ __forceinline__ float elem(const raw &r, int c) { return (float)r[c]; }
    static __device__ __forceinline__ void unpack(const raw &r, float v[8]) {
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = (float)r[i];
    }
};

template <>
struct Elem<MX_FP32> {
    typedef float type;
    static __device__ __forceinline__ void load8(const void *p, float v[8]) {
        v4f a = ((const v4f *)p)[0], b = ((const v4f *)p)[1];
#pragma unroll
        for (int i = 0; i < 4; i++) {
            v[i] = a[i];
            v[4 + i] = b[i];
        }
    }
    static __device__ __forceinline__ float load1(const void *p) { return *(const float *)p; }
    struct raw {
        v4f a, b;
    };
    template <bool NT = false>
    static __device__ __forceinline__ raw load_raw(const void *p) {
        return raw{stream_load<NT>((const v4f *)p), stream_load<NT>((const v4f *)p + 1)};
    }
    static __device__ __forceinline__ void unpack(const raw &r, float v[8]) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            v[i] = r.a[i];
            v[4 + i] = r.b[i];
        }
    }
};

__device__ __forceinline__ float amax8(const float v[8]) {
    float a = fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fabsf(v[2]));
    float b = fmaxf(fmaxf(fabsf(v[3]), fabsf(v[4])), fabsf(v[5]));
    return fmaxf(fmaxf(a, b), fmaxf(fabsf(v[6]), fabsf(v[7])));
}

// max over the 4 lanes of a quad (DPP quad_perm butterflies); all four lanes get the result.
__device__ __forceinline__ float quad_max(float a) {
    int x = __builtin_amdgcn_mov_dpp((int)f2bits(a), 0xB1, 0xF, 0xF, true);  // lane ^ 1
    a = fmaxf(a, bits2f((uint32_t)x));
    x = __builtin_amdgcn_mov_dpp((int)f2bits(a), 0x4E, 0xF, 0xF, true);  // lane ^ 2
    return fmaxf(a, bits2f((uint32_t)x));
}

// fp32 -> bf16 bits, round to nearest even (finite inputs; NaN keeps a quiet payload).
__device__ __forceinline__ uint32_t f2bf16(float f) {
    uint32_t u = f2bits(f);
    uint32_t r = u + 0x7FFFu + ((u >> 16) & 1u);
    r = (u & 0x7FFFFFFFu) > 0x7F800000u ? (u | 0x00400000u) : r;
    return r >> 16;
}

// Two fp32 -> packed bf16 pair with the hardware v_cvt_pk_bf16_f32 (round to nearest even).
// The software form above costs ~7 VALU ops per element, which made the GEMM epilogue
// (128 values per lane) longer than three K stages.
__device__ __forceinline__ uint32_t pack2_bf16(float lo, float hi) {
    typedef float f2 __attribute__((ext_vector_type(2)));
    typedef __bf16 b2 __attribute__((ext_vector_type(2)));
    f2 v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, b2));
}

// Inclusive prefix sum over the 64 lanes of a wave.
__device__ __forceinline__ int wave_incl_scan(int v, int lane) {
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const int up = __shfl_up(v, off, 64);
        if (lane >= off) v += up;
    }
    return v;
}

}  // namespace mx
