/*
 * CPU oracle for the MXFP8 linear path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, the arithmetic of the reference's MXFP8
 * quantizer, dequantizer and dequantize-then-matmul definitions.  It is the
 * checker the HIP kernels are compared against.  Nothing in the product
 * package links, imports or calls it: only tests/, the smoke entry and the
 * cpu_baseline leg of bench.py may.
 *
 * Reference lines followed (paths relative to the reference tree):
 *   quantizer per-32 block ....... src/kohakuwullm/kernels/mxfp8/quantize.py:39-56
 *   row quantizer layout ......... src/kohakuwullm/kernels/mxfp8/quantize.py:106-137
 *   torch restatement ............ scripts/bench/moe/kernel_ladder.py:184-188
 *   dequantizer .................. src/kohakuwullm/kernels/mxfp8/grouped.py:51-62
 *   dequant -> fp64 matmul ....... src/kohakuwullm/kernels/mxfp8/grouped.py:330-350
 *   SwiGLU -> quantize ........... src/kohakuwullm/kernels/mxfp8/fused_act.py:37-66
 *   cuBLAS scale swizzle ......... src/kohakuwullm/kernels/mxfp8/interop.py:24-41
 *                                  src/kohakuwullm/kernels/mxfp8/quantize.py:175-180
 *
 * Pinning status of each function (what independent check fixes it):
 *   ora_e4m3_from_f32 ...... exhaustive against torch's CPU float8_e4m3fn cast
 *                            over every bf16 and fp16 value below the
 *                            saturation point, plus the 256-entry decode table
 *                            round trip (tests/test_oracle_quantize.py).
 *   ora_scale_byte ......... closed form vs the literal ceil(log2(a/448))
 *                            formula evaluated with libm and with torch, over
 *                            every finite non-negative bf16/fp16 amax; known
 *                            answers (1.0 -> 119, 448 -> 127, 450 -> 128,
 *                            0 -> 19, 3e38 -> 247).
 *   ora_quantize_rows/cols . against the torch restatement above on seeded
 *                            tiles; invariants (gather commutes, zero padding,
 *                            cols == rows of the transpose, |deq| <= 448*2^e).
 *   ora_gemm_nt ............ textbook: equals numpy fp64 matmul of dequantized
 *                            operands; exact-integer special cases.
 *   fp32 inputs within a few ulp of 448*2^j, and Inf/NaN inputs: PARITY
 *   UNPINNED (the reference's result depends on the GPU's approximate
 *   log2/exp2/divide; nothing in its tree fixes it).  The oracle defines the
 *   exact-math result.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define MX_BLOCK 32

enum { ORA_BF16 = 0, ORA_FP16 = 1, ORA_FP32 = 2 };

static inline float bits_to_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_to_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static inline float bf16_to_f32(uint16_t h) { return bits_to_f32((uint32_t)h << 16); }

static float fp16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0) {
        if (man == 0) return bits_to_f32(sign);
        /* subnormal: man * 2^-24 */
        float v = (float)man * 5.9604644775390625e-8f;
        return sign ? -v : v;
    }
    if (exp == 31) return bits_to_f32(sign | 0x7F800000u | (man << 13));
    return bits_to_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* fp32 -> bf16 bits, round to nearest even (what torch's .to(bfloat16) does). */
uint16_t ora_bf16_from_f32(float f) {
    uint32_t u = f32_to_bits(f);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);
    uint32_t lsb = (u >> 16) & 1u;
    u += 0x7FFFu + lsb;
    return (uint16_t)(u >> 16);
}

static float load_elem(const void *x, int dtype, int64_t idx) {
    switch (dtype) {
    case ORA_BF16: return bf16_to_f32(((const uint16_t *)x)[idx]);
    case ORA_FP16: return fp16_to_f32(((const uint16_t *)x)[idx]);
    default: return ((const float *)x)[idx];
    }
}

/*
 * Saturating round-to-nearest-even cast fp32 -> OCP e4m3fn (bias 7, 3 mantissa
 * bits, max 448, subnormal step 2^-9, NaN = 0x7F/0xFF, no infinity).
 * quantize.py:55 (`.to(tl.float8e4nv)`).
 */
uint8_t ora_e4m3_from_f32(float f) {
    uint32_t u = f32_to_bits(f);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    uint32_t a = u & 0x7FFFFFFFu;
    if (a > 0x7F800000u) return (uint8_t)(sign | 0x7Fu);       /* NaN */
    float af = bits_to_f32(a);
    if (af >= 448.0f) return (uint8_t)(sign | 0x7Eu);          /* saturate (and Inf) */
    if (af < 0.015625f) {
        /* below the smallest normal 2^-6: fixed-point with step 2^-9.
         * af * 512 is exact in fp32 (or underflows to < 0.5 -> 0). */
        float scaled = af * 512.0f;
        float r = nearbyintf(scaled);                           /* ties to even */
        return (uint8_t)(sign | (uint8_t)r);                    /* r in 0..8; 8 == 0x08 = 2^-6 */
    }
    /* normal: keep 3 mantissa bits of the fp32 mantissa, RTNE on the dropped 20. */
    uint32_t exp = a >> 23;                                     /* biased 127 */
    uint32_t man = a & 0x7FFFFFu;
    uint32_t keep = man >> 20;
    uint32_t rest = man & 0xFFFFFu;
    uint32_t half = 0x80000u;
    if (rest > half || (rest == half && (keep & 1u))) keep++;
    uint32_t e8 = exp - 127u + 7u;                              /* e4m3 biased exponent, >= 1 here */
    uint32_t code = (e8 << 3) + keep;                           /* mantissa carry bumps exponent */
    if (code > 0x7Eu) code = 0x7Eu;
    return (uint8_t)(sign | code);
}

/* e4m3fn byte -> fp32 (exact).  grouped.py:51-62 reads codes with `.to(float32)`. */
float ora_e4m3_to_f32(uint8_t c) {
    uint32_t e = (c >> 3) & 0xFu, m = c & 7u;
    float v;
    if (e == 15 && m == 7) return bits_to_f32(((uint32_t)(c & 0x80u) << 24) | 0x7FC00000u);
    if (e == 0) v = (float)m * 0.001953125f;                    /* m * 2^-9 */
    else v = ldexpf(1.0f + (float)m * 0.125f, (int)e - 7);
    return (c & 0x80u) ? -v : v;
}

/*
 * UE8M0 scale byte of one block from its amax (fp32, non-negative).
 * quantize.py:53-56: e = max(ceil(log2(max(amax, 1e-30) / 448)), -127); byte = e + 127.
 * Closed form: 448 = 1.75 * 2^8, so with a = (1 + m) * 2^(E - 127),
 * ceil(log2(a / 448)) = E - 135 + (m > 0.75), i.e. byte = E - 8 + (M > 0x600000).
 */
uint8_t ora_scale_byte(float amax) {
    float a = amax > 1e-30f ? amax : 1e-30f;                    /* NaN amax -> 1e-30 like max() */
    uint32_t u = f32_to_bits(a);
    int32_t E = (int32_t)(u >> 23) & 0xFF;
    uint32_t M = u & 0x7FFFFFu;
    int32_t b = E - 8 + (M > 0x600000u ? 1 : 0);
    if (E == 0xFF) b = 255;                                     /* Inf: unpinned; mirror uint8(inf)->saturate */
    if (b < 0) b = 0;                                           /* the -127 floor (unreachable after the clamp) */
    return (uint8_t)b;
}

/* The literal formula, libm arithmetic in fp32 as the reference writes it. */
uint8_t ora_scale_byte_literal(float amax) {
    float a = fmaxf(amax, 1e-30f);
    float e = ceilf(log2f(a / 448.0f));
    if (e < -127.0f) e = -127.0f;
    return (uint8_t)(int)(e + 127.0f);
}

/* 2^(byte-127) as fp32 (byte 0 -> 2^-127 is subnormal but exact). */
static inline float scale_to_f32(uint8_t b) { return ldexpf(1.0f, (int)b - 127); }

/* Quantize one block of 32 fp32 values (quantize.py:49-56). */
static uint8_t quantize_block(const float *v, uint8_t *codes, int64_t code_stride) {
    float amax = 0.0f;
    for (int i = 0; i < MX_BLOCK; i++) {
        float a = fabsf(v[i]);
        if (a > amax) amax = a;                                 /* NaN never wins, like tl.max */
    }
    uint8_t b = ora_scale_byte(amax);
    /* x / 2^e: exact unless the quotient underflows fp32, where e4m3 gives +-0 anyway. */
    float inv = ldexpf(1.0f, 127 - (int)b);
    for (int i = 0; i < MX_BLOCK; i++) codes[i * code_stride] = ora_e4m3_from_f32(v[i] * inv);
    return b;
}

/*
 * Row-axis quantizer: blocks of 32 along the last axis of x (M,K).
 * q (M,K) row pitch ldq, s (M,K/32) row pitch lds.  quantize.py:106-137.
 * Returns 0, or -1 when K is not a multiple of 32 (the reference raises ValueError).
 */
int ora_quantize_rows(const void *x, int dtype, int64_t M, int64_t K, int64_t sx_row, int64_t sx_col,
                      uint8_t *q, int64_t ldq, uint8_t *s, int64_t lds) {
    if (K % MX_BLOCK) return -1;
    float v[MX_BLOCK];
    for (int64_t m = 0; m < M; m++)
        for (int64_t kb = 0; kb < K / MX_BLOCK; kb++) {
            for (int i = 0; i < MX_BLOCK; i++) v[i] = load_elem(x, dtype, m * sx_row + (kb * MX_BLOCK + i) * sx_col);
            s[m * lds + kb] = quantize_block(v, q + m * ldq + kb * MX_BLOCK, 1);
        }
    return 0;
}

/*
 * Column-axis quantizer: blocks of 32 along the FIRST axis of x (M,K); outputs are
 * those of the row quantizer applied to the transpose: qT (K,M), sT (K,M/32).
 * linear.py:111 and moe.py:58-61 realise it as quantize(x.t()).
 */
int ora_quantize_cols(const void *x, int dtype, int64_t M, int64_t K, int64_t sx_row, int64_t sx_col,
                      uint8_t *qT, int64_t ldqT, uint8_t *sT, int64_t ldsT) {
    if (M % MX_BLOCK) return -1;
    float v[MX_BLOCK];
    for (int64_t k = 0; k < K; k++)
        for (int64_t mb = 0; mb < M / MX_BLOCK; mb++) {
            for (int i = 0; i < MX_BLOCK; i++) v[i] = load_elem(x, dtype, (mb * MX_BLOCK + i) * sx_row + k * sx_col);
            sT[k * ldsT + mb] = quantize_block(v, qT + k * ldqT + mb * MX_BLOCK, 1);
        }
    return 0;
}

/* silu(g) * u kept in fp32, then the row quantizer.  fused_act.py:44-56. */
int ora_swiglu_quantize_rows(const void *g, const void *u, int dtype, int64_t M, int64_t K, int64_t ldg, int64_t ldu,
                             uint8_t *q, int64_t ldq, uint8_t *s, int64_t lds) {
    if (K % MX_BLOCK) return -1;
    float v[MX_BLOCK];
    for (int64_t m = 0; m < M; m++)
        for (int64_t kb = 0; kb < K / MX_BLOCK; kb++) {
            for (int i = 0; i < MX_BLOCK; i++) {
                float gv = load_elem(g, dtype, m * ldg + kb * MX_BLOCK + i);
                float uv = load_elem(u, dtype, m * ldu + kb * MX_BLOCK + i);
                float sig = 1.0f / (1.0f + expf(-gv));
                v[i] = gv * sig * uv;
            }
            s[m * lds + kb] = quantize_block(v, q + m * ldq + kb * MX_BLOCK, 1);
        }
    return 0;
}

/* Dequantize to fp32: q * 2^(s-127) broadcast over each block of 32.  grouped.py:51-62. */
void ora_dequant(const uint8_t *q, int64_t ldq, const uint8_t *s, int64_t lds, int64_t M, int64_t K, float *out, int64_t ldo) {
    for (int64_t m = 0; m < M; m++)
        for (int64_t k = 0; k < K; k++)
            out[m * ldo + k] = ora_e4m3_to_f32(q[m * ldq + k]) * scale_to_f32(s[m * lds + k / MX_BLOCK]);
}

/*
 * C = deq(A) * deq(B)^T with fp64 accumulation, A (M,K), B (N,K), both K-minor.
 * grouped.py:330-350 (the precision oracle) for a single group.  Small sizes only.
 */
void ora_gemm_nt_f64(const uint8_t *aq, int64_t lda, const uint8_t *as, int64_t ldas,
                     const uint8_t *bq, int64_t ldb, const uint8_t *bs, int64_t ldbs,
                     int64_t M, int64_t N, int64_t K, double *c, int64_t ldc) {
    double *ad = (double *)malloc((size_t)K * sizeof(double));
    for (int64_t m = 0; m < M; m++) {
        for (int64_t k = 0; k < K; k++)
            ad[k] = (double)ora_e4m3_to_f32(aq[m * lda + k]) * ldexp(1.0, (int)as[m * ldas + k / MX_BLOCK] - 127);
        for (int64_t n = 0; n < N; n++) {
            double acc = 0.0;
            for (int64_t kb = 0; kb < K / MX_BLOCK; kb++) {
                double part = 0.0;
                for (int i = 0; i < MX_BLOCK; i++)
                    part += ad[kb * MX_BLOCK + i] * (double)ora_e4m3_to_f32(bq[n * ldb + kb * MX_BLOCK + i]);
                acc += part * ldexp(1.0, (int)bs[n * ldbs + kb] - 127);
            }
            c[m * ldc + n] = acc;
        }
    }
    free(ad);
}

/*
 * cuBLAS SWIZZLE_32_4_4 placement of a natural (rows, cols) scale matrix:
 * 128-row x 4-col tiles of 512 bytes, in-tile offset (r%32)*16 + (r/32)*4 + c,
 * tiles ordered row-tile major; zero padded.  interop.py:24-41, quantize.py:175-180.
 * out must hold ceil(rows/128)*128 * ceil(cols/4)*4 bytes.
 */
void ora_swizzle_32_4_4(const uint8_t *s, int64_t rows, int64_t cols, int64_t lds, uint8_t *out) {
    int64_t row_tiles = (rows + 127) / 128, col_tiles = (cols + 3) / 4;
    memset(out, 0, (size_t)(row_tiles * col_tiles * 512));
    for (int64_t r = 0; r < rows; r++)
        for (int64_t c = 0; c < cols; c++) {
            int64_t tile = (r / 128) * col_tiles + c / 4;
            int64_t rr = r % 128;
            out[tile * 512 + (rr % 32) * 16 + (rr / 32) * 4 + c % 4] = s[r * lds + c];
        }
}
