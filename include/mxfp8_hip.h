/*
 * libmxfp8_hip -- MXFP8 (e4m3 + UE8M0 per-32) linear path for AMD MI355X (gfx950).
 *
 * C ABI.  Every entry point
 *   - takes raw DEVICE pointers, sizes and strides; never synchronises or frees;
 *     launches on the stream the caller passes (a hipStream_t travelling as
 *     void*; NULL = the default stream);
 *   - returns MX_OK or a negative MX_E* code and never throws;
 *   - allocates nothing: outputs, index scratch and the GEMMs' K-split workspace
 *     all come from the caller (mx_gemm_workspace_bytes, mx_expert_sort_workspace);
 *   - is re-entrant and thread-safe: no state is kept between calls besides two
 *     write-once caches (the CU count per device ordinal, and "the large-LDS
 *     attribute of this kernel is set" per kernel and device);
 *   - refuses with MX_ECAPTURE, before launching anything, when the stream is
 *     being captured into a HIP graph: recording this library's launches ended a
 *     process inside graph instantiation and stays switched off until the cause
 *     is known.
 *
 * The reference (KohakUwULLM) has no FFI; each function cites the reference
 * Python/Triton interface it stands in for (paths relative to the reference tree).
 *
 * Formats.  Codes are OCP float8_e4m3fn bytes.  A scale byte b means 2^(b-127).
 * A "row-quantized" matrix (R,K) has 32-element blocks along K: codes (R,K) and
 * scales (R,K/32), both K-minor ("natural" layout of quantize.py:106-137).
 */
#ifndef MXFP8_HIP_H
#define MXFP8_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MX_ABI_VERSION 2

enum mx_status {
    MX_OK = 0,
    MX_EINVAL = -1,      /* a size/stride/alignment contract is violated (ValueError upstream) */
    MX_EUNSUPPORTED = -2, /* well-formed request this build has no kernel for */
    MX_ELAUNCH = -3,     /* the HIP runtime refused the launch */
    MX_ENODEV = -4,      /* the current device is not gfx950 */
    MX_ECAPTURE = -5,    /* the stream is being captured into a graph: nothing was launched */
    MX_ETOOBIG = -6      /* the request exceeds the fixed capacity of an entry point that allocates nothing */
};

enum mx_dtype { MX_BF16 = 0, MX_FP16 = 1, MX_FP32 = 2 };

/* Epilogues of the GEMM entry points. */
enum mx_epilogue {
    MX_EPI_NONE = 0,      /* C = A B^T, cast to c_dtype */
    MX_EPI_ACCUMULATE = 1 /* C += A B^T with fp32 atomic adds; c_dtype must be MX_FP32 */
};
/* Bits 4-7 of `epilogue` select nothing in this library: mx_gemm_nt answers MX_EUNSUPPORTED when one is set. */
/* OR into `epilogue` to cut K into n slices that run as independent tiles (needs
 * MX_EPI_ACCUMULATE and a caller-zeroed C): fills the GPU when M*N alone gives too few tiles. */
#define MX_EPI_SPLIT_K(n) ((n) << 8)

int mx_abi_version(void);
const char *mx_strerror(int status);
/* 0 when device `dev` is a gfx950 part this library's kernels can run on. */
int mx_device_supported(int dev);

/*
 * Row-axis quantizer.  x (M,K) with element strides (sx_row, sx_col) -> q (M,K)
 * e4m3 with row pitch ldq, s (M,K/32) UE8M0 with row pitch lds.  K % 32 == 0.
 * Per block: amax in fp32, e = ceil(log2(max(amax,1e-30)/448)), code =
 * rtne_sat(x / 2^e), byte = e + 127.
 * Replaces quantize_mx / _quantize_mx_kernel / _quantize_block
 * (src/kohakuwullm/kernels/mxfp8/quantize.py:39-56,65-137).  A singly-strided
 * (transposed) input is taken without a copy, as quantize_mx_vendor does
 * (quantize.py:190-193).
 */
int mx_quantize_rows(const void *x, int x_dtype, int64_t M, int64_t K, int64_t sx_row, int64_t sx_col,
                     uint8_t *q, int64_t ldq, uint8_t *s, int64_t lds, void *stream);

/*
 * Column-axis quantizer.  x (M,K) row-major with row pitch ldx -> qT (K,M), sT
 * (K,M/32): 32-element blocks run along M, outputs are laid out as the row
 * quantizer's outputs for x^T.  M % 32 == 0.
 * Replaces quantize_mx(x.t().contiguous()) / quantize_mx_vendor(pad(W.t()))
 * (src/kohakuwullm/kernels/mxfp8/linear.py:111, moe.py:58-61) without the
 * transposed copy.
 */
int mx_quantize_cols(const void *x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                     uint8_t *qT, int64_t ldqT, uint8_t *sT, int64_t ldsT, void *stream);

/*
 * Both at once, reading x a single time: (q,s) as mx_quantize_rows and (qT,sT)
 * as mx_quantize_cols.  M % 32 == 0 and K % 32 == 0.
 * Replaces the pair of quantize calls an activation needs when it feeds both a
 * forward/dgrad GEMM (blocks along its K) and a wgrad GEMM (blocks along tokens).
 *
 * Stage-major codes.  A code matrix of R rows and C > 128 columns whose leading dimension is
 * given as exactly 128 is stored as C/128 panels: panel p (columns 128 p .. 128 p + 127) at byte
 * offset p * R * 128, row r of it at r * 128.  C % 128 == 0.  A K stage of a GEMM tile (256
 * rows x 128 bytes) is then one contiguous run instead of 256 rows a pitch apart, which DRAM
 * serves 3-4 % faster on long contractions.  Accepted for qT here and in
 * mx_swiglu_quantize_dual, for q and qT in mx_swiglu_bwd_quantize_dual, and for the A and B
 * codes of mx_gemm_nt / mx_gemm_nt_batch.  Scale bytes keep their row-major layout.  The
 * layout has no counterpart in the reference; the public (rows, K) layouts are the default.
 */
int mx_quantize_dual(const void *x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                     uint8_t *q, int64_t ldq, uint8_t *s, int64_t lds,
                     uint8_t *qT, int64_t ldqT, uint8_t *sT, int64_t ldsT, void *stream);

/*
 * (T, H, D) attention operand -> e4m3 codes (T, H, D) and UE8M0 bytes (T, H, D/32), both
 * contiguous, blocks of 32 along D (the contraction axis of QK^T).  x has unit stride along D,
 * stride_h between heads and stride_t between tokens (elements): a slice of a fused projection
 * output is quantized where it lies.  mu: optional (H, D) fp32 mean, subtracted in fp32 before
 * the block maximum is taken (NULL: none).  D % 32 == 0.
 * Replaces _quant_heads_kernel / quantize_heads
 * (src/kohakuwullm/kernels/mxfp8/attention_quant.py:17-118).
 */
int mx_quantize_heads(const void *x, int x_dtype, int64_t T, int64_t H, int64_t D, int64_t stride_t, int64_t stride_h,
                      const float *mu, uint8_t *q, uint8_t *s, void *stream);

/*
 * mx_quantize_dual of `count` matrices behind one launch (one per 24 of them): the
 * once-per-optimizer-step requantization of every weight matrix of a model, which the
 * reference performs as one launch per matrix and axis from refresh_mxfp8_weights
 * (src/kohakuwullm/models/mxfp8_swap.py:331-343; MXFP8Linear.refresh_quantized_weight,
 * src/kohakuwullm/kernels/mxfp8/linear.py:98-108; MXFP8ExpertWeights.refresh,
 * src/kohakuwullm/kernels/mxfp8/moe.py:34-61).  Every problem has the arguments of
 * mx_quantize_dual and gets the same bytes; all are validated before anything is launched.
 */
typedef struct {
    const void *x;      /* (M,K), row pitch ldx elements, dtype x_dtype */
    uint8_t *q, *s;     /* (M,K) codes and (M,K/32) scale bytes, blocks along K */
    uint8_t *qT, *sT;   /* (K,M) codes and (K,M/32) scale bytes, blocks along M */
    int64_t M, K, ldx, ldq, lds, ldqT, ldsT;
} mx_quant_problem;
int mx_quantize_dual_batch(const mx_quant_problem *problems, int count, int x_dtype, void *stream);

/*
 * q,s = quantize_rows(silu(gate) * up) with the product kept in fp32.
 * gate, up (M,K) unit inner stride, row pitches ldg, ldu.  K % 32 == 0.
 * Replaces swiglu_mx / _swiglu_mx_kernel (src/kohakuwullm/kernels/mxfp8/fused_act.py:17-101).
 */
int mx_swiglu_quantize_rows(const void *gate, const void *up, int dtype, int64_t M, int64_t K, int64_t ldg,
                            int64_t ldu, uint8_t *q, int64_t ldq, uint8_t *s, int64_t lds, void *stream);

/*
 * h = silu(gate) * up taken from the fused input-projection output gu (M,2H), gate half
 * first, row pitch ldgu; h is quantized along both axes in one pass: (q,s) (M,H) blocks
 * along H for the output projection's forward, (qT,sT) (H,M) blocks along M for its wgrad.
 * M % 32 == 0, H % 32 == 0.  The dense-MLP form of swiglu_mx (fused_act.py:69-101) for
 * GLUMLP's fused w_in layout (src/kohakuwullm/models/components/mlp.py:61-73).
 */
int mx_swiglu_quantize_dual(const void *gu, int dtype, int64_t M, int64_t H, int64_t ldgu,
                            uint8_t *q, int64_t ldq, uint8_t *s, int64_t lds,
                            uint8_t *qT, int64_t ldqT, uint8_t *sT, int64_t ldsT, void *stream);

/*
 * SwiGLU backward fused with both quantizers: from dh (M,H) and the saved gu (M,2H),
 * dgate = dh * up * sig * (1 + gate * (1 - sig)), dup = dh * gate * sig with sig =
 * sigmoid(gate), all in fp32; dpre = [dgate | dup] (M,2H) is emitted only in MXFP8:
 * (q,s) blocks along 2H for the input projection's dgrad and (qT,sT) (2H,M) blocks along
 * M for its wgrad.  Closed form as src/kohakuwullm/kernels/elementwise/swiglu.py:108-119
 * and experts_bwd.py:145-148.  M % 32 == 0, H % 32 == 0.
 */
int mx_swiglu_bwd_quantize_dual(const void *dh, int64_t lddh, const void *gu, int64_t ldgu, int dtype,
                                int64_t M, int64_t H, uint8_t *q, int64_t ldq, uint8_t *s, int64_t lds,
                                uint8_t *qT, int64_t ldqT, uint8_t *sT, int64_t ldsT, void *stream);

/*
 * RMSNorm as a producer of MXFP8 operands: rstd[m] = 1 / sqrt(mean_k(x[m,k]^2) + eps),
 * y = x * rstd * weight (fp32; weight NULL: 1).  Any of three results, from one pass over x:
 * out (M,K) in x_dtype (NULL: not written), rstd (M) fp32 for the backward (NULL: not
 * written), and (q,s) = y quantized along K from the fp32 values (both NULL: not written;
 * K % 32 == 0 when given).  At least one of the three.  weight is x_dtype or fp32.
 * The sum of squares is accumulated in fp64, the rest is fp32 in the reference's order.
 * Replaces _rmsnorm_fwd with QUANT (src/kohakuwullm/kernels/elementwise/rmsnorm.py:20-84;
 * host side rms_norm_mx :239-246, rms_norm :232-236) and _rmsnorm_mx_kernel / rmsnorm_mx
 * (src/kohakuwullm/kernels/mxfp8/fused_act.py:104-175).  The SWIZZLE branch of the reference
 * is mx_swizzle_scales applied to s.
 */
int mx_rmsnorm_quantize(const void *x, int x_dtype, int64_t M, int64_t K, int64_t ldx,
                        const void *weight, int w_dtype, float eps, void *out, int64_t ldo, float *rstd,
                        uint8_t *q, int64_t ldq, uint8_t *s, int64_t lds, void *stream);

/*
 * RMSNorm as a producer of BOTH MXFP8 operands of the linear layer behind it: y = x * rstd * weight in fp32 as in
 * mx_rmsnorm_quantize, quantized along K into (q,s) (M,K), (M,K/32) -- the layer's forward operand, bit-identical to
 * mx_rmsnorm_quantize's -- and along the tokens into (qT,sT) (K,M), (K,M/32) -- the operand of its weight gradient, the
 * column quantizer applied to the same fp32 y.  Neither the 16-bit normalized activation nor its transpose is written.
 * Two launches: the rows' rstd (M floats, the caller's buffer: also what mx_rmsnorm_backward takes), then 128 x 128
 * tiles of x scaled on the way in.  M % 32 == 0, K % 32 == 0; ldqT == 128 with M > 128 selects the stage-major layout
 * of mx_quantize_dual for qT.  weight: any of the three dtypes, or NULL.
 * No counterpart in the reference, which emits the row-axis pair only (rmsnorm_mx,
 * src/kohakuwullm/kernels/mxfp8/fused_act.py:104-175) and quantizes the activation a second time for WGRAD
 * (src/kohakuwullm/kernels/mxfp8/linear.py:111).
 */
int mx_rmsnorm_quantize_dual(const void *x, int x_dtype, int64_t M, int64_t K, int64_t ldx, const void *weight,
                             int w_dtype, float eps, float *rstd, uint8_t *q, int64_t ldq, uint8_t *s, int64_t lds,
                             uint8_t *qT, int64_t ldqT, uint8_t *sT, int64_t ldsT, void *stream);

/*
 * RMSNorm backward: dx = (dy - xhat * mean_k(dy * xhat)) * rstd with dy = dout * weight and
 * xhat = x * rstd, in dtype (bf16 or fp16); dw_part (parts,K) fp32 (NULL: no weight
 * gradient) receives one partial sum of dout * xhat per workgroup, every row of it written;
 * the caller adds the rows.  1 <= parts <= 65535; K <= 4096.
 * Replaces _rmsnorm_bwd (src/kohakuwullm/kernels/elementwise/rmsnorm.py:87-128, launched
 * from _RMSNorm.backward :196-229 with 512 partial rows).
 */
int mx_rmsnorm_backward(const void *x, int dtype, int64_t M, int64_t K, int64_t ldx, const void *weight,
                        int w_dtype, const void *dout, int64_t lddo, const float *rstd, void *dx, int64_t lddx,
                        float *dw_part, int64_t parts, void *stream);

/*
 * Scale layout interop.  The reference's cuBLAS route keeps UE8M0 scales in the flat
 * SWIZZLE_32_4_4 layout: 128-row x 4-column tiles of 512 bytes, row-tile major, scale
 * (r, c) of a tile at (r % 32) * 16 + (r / 32) * 4 + c, zero padded to whole tiles
 * (ceil(rows/128)*128 * ceil(cols/4)*4 bytes).  The MI355X kernels read the natural
 * (rows, cols) layout; these two convert either way so tensors produced for, or by, the
 * reference's quantize_mx_vendor / mxfp8_mm_swizzled can be exchanged.
 * Replaces swizzle_mx_scales (src/kohakuwullm/kernels/mxfp8/interop.py:24-41) and the
 * swizzled store of _quantize_mx_vendor_kernel (quantize.py:175-180).
 */
int mx_swizzle_scales(const uint8_t *s, int64_t rows, int64_t cols, int64_t lds, uint8_t *swizzled, void *stream);
int mx_unswizzle_scales(const uint8_t *swizzled, int64_t rows, int64_t cols, uint8_t *s, int64_t lds, void *stream);

/*
 * C (M,N) = deq(A) deq(B)^T, fp32 accumulate, cast to c_dtype (round to nearest
 * even).  A: codes (M,K) pitch lda + scales (M,K/32) pitch ldas; B: codes (N,K)
 * pitch ldb + scales (N,K/32) pitch ldbs; both K-minor.  K % 32 == 0.
 * One entry serves forward (X W^T), dgrad (dY (W^T)^T) and wgrad (dY^T (X^T)^T)
 * because the quantizers deliver every operand K-minor.  lda == 128 (ldb == 128) with
 * K > 128 reads A (B) in the stage-major layout described at mx_quantize_dual (K % 128 == 0).
 * workspace: device scratch of workspace_bytes bytes (16-byte aligned) or NULL.  With at least
 * mx_gemm_workspace_bytes() of it, a shape whose last round of tiles leaves most of the GPU idle
 * has the K stages of those tiles dealt over all workgroups (fp32 partial tiles go through the
 * workspace, a second kernel adds them in a fixed order).  With less, every tile is computed
 * whole: same product, fp32 sums in another order, slower on such shapes.  The workspace holds
 * nothing between calls; calls that may overlap in time need separate ones.
 * epilogue: MX_EPI_NONE, or MX_EPI_ACCUMULATE optionally with MX_EPI_SPLIT_K(n); a negative value is
 * MX_EINVAL, any other bit of the low byte MX_EUNSUPPORTED.
 * Replaces mxfp8_matmul_pq / _mxfp8_matmul_pq
 * (src/kohakuwullm/kernels/mxfp8/quantize.py:242-371) and the cuBLAS route
 * mxfp8_mm_swizzled (src/kohakuwullm/kernels/mxfp8/interop.py:51-122); the reference's
 * wrapper allocates what its kernel writes through torch (quantize.py:328-371), which is what
 * the workspace argument leaves to this library's caller.
 */
int mx_gemm_nt(const uint8_t *aq, const uint8_t *as, const uint8_t *bq, const uint8_t *bs,
               void *c, int c_dtype, int64_t M, int64_t N, int64_t K,
               int64_t lda, int64_t ldas, int64_t ldb, int64_t ldbs, int64_t ldc,
               int epilogue, void *workspace, int64_t workspace_bytes, void *stream);

/*
 * Bytes of workspace that let mx_gemm_nt, mx_gemm_nt_batch and mx_grouped_wgrad_nt split K on the
 * current device: two fp32 tiles of 256 x 256 per compute unit (128 MiB on MI355X).  It depends
 * on the device only, never on a shape (the reference's rule for launch plans: a pure function of
 * static properties, never of the token count, src/kohakuwullm/kernels/mxfp8/quantize.py:59-62).
 */
int64_t mx_gemm_workspace_bytes(void);

/*
 * Up to any number of independent products C_j = deq(A_j) deq(B_j)^T behind as few
 * launches as possible (groups of 4 share one launch, the GPU's workgroups divided
 * among them by work).  Meant for products that are ready at the same time and do not
 * fill the GPU one by one: DGRAD with WGRAD of a linear layer, the three products that
 * end a SwiGLU block's backward.  All outputs have dtype c_dtype.  `problems` is a
 * HOST array, read before the call returns.  Results are those of `count` calls of
 * mx_gemm_nt with MX_EPI_NONE.  workspace as in mx_gemm_nt (one for the whole call); without it
 * products are not cut into K slices and a sparse last round is not split.
 * Replaces the back-to-back launches of the reference's backward
 * (src/kohakuwullm/kernels/mxfp8/linear.py:66-74: dx then dw; models/components/mlp.py:68-73
 * under autograd).
 */
typedef struct mx_gemm_problem {
    const uint8_t *aq, *a_scale, *bq, *b_scale;
    void *c;
    int64_t M, N, K, lda, ldas, ldb, ldbs, ldc;
} mx_gemm_problem;
int mx_gemm_nt_batch(const mx_gemm_problem *problems, int count, int c_dtype, void *workspace,
                     int64_t workspace_bytes, void *stream);

/*
 * ---- routed experts -------------------------------------------------------------------
 * Rows are sorted by expert.  `offsets` (E+1) int32 lives on the DEVICE (exclusive prefix sum
 * of per-expert row counts, truncated to the real experts) and is never read on the host: the
 * launch is bounded from M and E alone, so a layer stays graph-capturable
 * (src/kohakuwullm/kernels/mxfp8/grouped.py:3-4,274-275).  Rows outside every expert's range
 * are not written.  Expert weights: codes (E,NB,K) with strides (stride_we, ldw) and scales
 * (E,NB,K/32) with strides (stride_wse, ldws).
 */

/*
 * out[m] = xq[index[m] or m] . wq[e(m)]^T for sorted positions m < offsets[E]; out (M,N).
 * xq has a_rows rows.  Replaces grouped_mxfp8_gemm / _grouped_mxfp8_fwd / tile_owner
 * (src/kohakuwullm/kernels/mxfp8/grouped.py:26-48,65-149,254-327).
 */
int mx_grouped_gemm_nt(const uint8_t *xq, const uint8_t *xs, int64_t a_rows, int64_t ldx, int64_t ldxs,
                       const int32_t *index, const uint8_t *wq, const uint8_t *ws, int64_t stride_we,
                       int64_t ldw, int64_t stride_wse, int64_t ldws, const int32_t *offsets, int64_t E,
                       void *out, int out_dtype, int64_t ldo, int64_t M, int64_t N, int64_t K, void *stream);

/*
 * Expert GEMM1 with its epilogue: rows gathered by token_of, both halves of x . w_in^T
 * (w_in (E,2H,K), gate rows first), accumulators rounded to act_dtype, optional store of
 * pre (M,2H), h = gate * sigmoid(gate) * value quantized per 32 of H into hq (M,H), hs (M,H/32).
 * token_of == NULL gathers nothing (row m is x row m).  With htq/hts != NULL the same h is
 * also quantized along the tokens, into the padded layout of mx_quantize_cols_grouped
 * ((H,Mpad), (H,Mpad/32); with E == 1 and M % 128 == 0 that is plain (H,M)): the operand of
 * GEMM2's WGRAD, bit-identical to mx_quantize_cols_grouped(pre, source = SwiGLU).
 * ldhtq == 128 with more than one 128-position tile in the padded space selects the stage-major
 * form of htq described at mx_quantize_cols_grouped: (Mpad/128, H, 128).
 * With E == 1 this is the dense SwiGLU block's first projection with the activation and both
 * casts in the epilogue (GLUMLP.forward, src/kohakuwullm/models/components/mlp.py:68-73).
 * Replaces _experts_gemm1 / launch_gemm1 (src/kohakuwullm/kernels/mxfp8/experts.py:25-135,225-275).
 */
int mx_experts_gemm1(const uint8_t *xq, const uint8_t *xs, int64_t T, int64_t ldx, int64_t ldxs,
                     const int32_t *token_of, const uint8_t *wq, const uint8_t *ws, int64_t stride_we,
                     int64_t ldw, int64_t stride_wse, int64_t ldws, const int32_t *offsets, int64_t E,
                     uint8_t *hq, int64_t ldhq, uint8_t *hs, int64_t ldhs, void *pre, int64_t ldpre,
                     uint8_t *htq, int64_t ldhtq, uint8_t *hts, int64_t ldhts,
                     int act_dtype, int64_t M, int64_t H, int64_t K, void *stream);

/*
 * out[token_of[m]] += scale(m) * (aq[index[m] or m] . wq[e(m)]^T) with packed 16-bit atomic
 * adds into a caller-zeroed out (T,N); scale(m) = gate[order[m]] when gate != NULL, else 1.
 * With a gate: _experts_gemm2 / launch_gemm2 (experts.py:138-222,278-323).  Without: the
 * GEMM1 dgrad _experts_gemm1_dgrad (src/kohakuwullm/kernels/mxfp8/experts_bwd.py:167-247).
 */
int mx_experts_scatter_gemm(const uint8_t *aq, const uint8_t *as, int64_t a_rows, int64_t lda, int64_t ldas,
                            const int32_t *index, const uint8_t *wq, const uint8_t *ws, int64_t stride_we,
                            int64_t ldw, int64_t stride_wse, int64_t ldws, const int32_t *offsets, int64_t E,
                            const int32_t *token_of, const int32_t *order, const void *gate, int gate_dtype,
                            void *out, int out_dtype, int64_t ldo, int64_t M, int64_t N, int64_t K, void *stream);

/*
 * The same combine without atomics: out (T,N)[t] = sum over k < top_k of
 * scale(t,k) * y[pos(t,k)], where y (M,N) holds one 16-bit row per sorted position (the
 * output of mx_grouped_gemm_nt), pair t*top_k + k sits at the sorted position m with
 * order[m] == t*top_k + k and m < offsets[E] (a pair found nowhere was dropped and adds
 * nothing), and scale = gate[pair] (NULL: 1).  fp32 sum in k order, one rounding: one writer
 * per element, bitwise reproducible.  `inv` is caller-provided scratch of T*top_k int32: the call
 * fills it with pos(t,k) (-1 for a dropped pair).  With order == NULL the call takes inv as filled
 * by an earlier call for the same routing and skips that step (a layer's backward reuses its
 * forward's).
 * Every element of out is written; out need not be zeroed.
 * Stands in for the tl.atomic_add epilogues of _experts_gemm2 (experts.py:138-222) and
 * _experts_gemm1_dgrad (experts_bwd.py:167-247) when order is the reference's pair index
 * (moe.py: token_of = order // top_k).
 */
int mx_experts_combine(const void *y, int64_t ldy, const int32_t *order, const int32_t *offsets, int64_t E,
                       const void *gate, int gate_dtype, int32_t *inv, int64_t T, int64_t top_k,
                       void *out, int dtype, int64_t ldo, int64_t M, int64_t N, void *stream);

/*
 * DGRAD through GEMM2, the combine and SwiGLU at once: acc = dq[token_of[m]] . w_out_dgrad[e]^T
 * (M,H); dgate[order[m]] += <acc, dequant(hq,hs)[m]> (fp32 atomics, caller-zeroed);
 * dh = acc * gate[order[m]]; SwiGLU backward from the stored pre; dpre (M,2H) stored in
 * act_dtype and quantized from the fp32 values into dpq (M,2H), dps (M,2H/32).
 * Optional (both or neither): ptq (2H,Mpad), pts (2H,Mpad/32) receive the stored (rounded)
 * dpre quantized along the tokens in the padded layout of mx_quantize_cols_grouped, bit for
 * bit what that quantizer makes of dpre; dpre itself may then be NULL and is not written.
 * ldptq == 128 selects the stage-major form of ptq, (Mpad/128, 2H, 128), as there.
 * Replaces _experts_gemm2_dgrad (src/kohakuwullm/kernels/mxfp8/experts_bwd.py:29-164); with
 * ptq it also stands in for the pass over the stored dpre that feeds GEMM1's WGRAD
 * (_launch_wgrad(dpre, x, ...), src/kohakuwullm/kernels/mxfp8/moe.py:311-324).
 */
int mx_experts_gemm2_dgrad(const uint8_t *dq, const uint8_t *ds, int64_t T, int64_t lddq, int64_t ldds,
                           const int32_t *token_of, const int32_t *order, const void *gate, int gate_dtype,
                           const uint8_t *wq, const uint8_t *ws, int64_t stride_we, int64_t ldw,
                           int64_t stride_wse, int64_t ldws, const int32_t *offsets, int64_t E,
                           const uint8_t *hq, int64_t ldhq, const uint8_t *hs, int64_t ldhs, const void *pre,
                           void *dpre, int64_t ldpre, uint8_t *dpq, int64_t lddpq, uint8_t *dps, int64_t lddps,
                           uint8_t *ptq, int64_t ldptq, uint8_t *pts, int64_t ldpts,
                           float *dgate, int act_dtype, int64_t M, int64_t H, int64_t K, void *stream);

/*
 * Token-axis quantizer over expert-sorted rows, feeding the experts' MXFP8 WGRAD.  Each
 * expert's rows are laid out from a fresh multiple of 128 in a padded position space of
 * Mpad = (ceil(M/128) + E) * 128 positions (rows past an expert's end are zero), so no 32-row
 * block straddles two experts.  Output qT (C,Mpad), sT (C,Mpad/32).
 * source 0: x[index[m] or m][0:C], optionally times row_scale[scale_index[m] or m] in fp32 --
 *           the gathered, gate-scaled dout rows and the gathered x rows of
 *           grouped_mxfp8_wgrad_kernel (src/kohakuwullm/kernels/mxfp8/grouped.py:152-247);
 * source 1: silu(x[m][c]) * x[m][C + c] from the stored pre-activation (M,2C) -- the h the
 *           reference rebuilds in src/kohakuwullm/kernels/mxfp8/moe.py:288-290.
 * Stage-major codes: ldqT == 128 (with Mpad > 128, always the case for M > 0) stores qT as
 * (Mpad/128, C, 128) -- byte (c, pos) at (pos/128) * C * 128 + c * 128 + pos % 128 -- so that a K stage
 * of a WGRAD tile is one contiguous run; the same bytes, sT unchanged.  mx_grouped_wgrad_nt takes
 * either form per operand.
 */
int mx_quantize_cols_grouped(const void *x, int dtype, int64_t ldx, int64_t C, int source,
                             const int32_t *index, const void *row_scale, int row_scale_dtype,
                             const int32_t *scale_index, const int32_t *offsets, int64_t E, int64_t M,
                             uint8_t *qT, int64_t ldqT, uint8_t *sT, int64_t ldsT, void *stream);

/*
 * dW[e] (N,Kout) = AT[:, seg(e)] . BT[:, seg(e)]^T over the padded positions expert e owns,
 * AT (N,Mpad), BT (Kout,Mpad) from mx_quantize_cols_grouped; dW (E,N,Kout) with strides
 * (stride_dwe, lddw) in elements.  An expert without rows gets zeros.  The MXFP8 form of
 * grouped_mxfp8_wgrad_kernel / _launch_wgrad (grouped.py:152-247, moe.py:64-99), which
 * multiply in 16 bits.
 * lda == 128 / ldb == 128: that operand's codes are stage-major, (Mpad/128, N, 128) / (Mpad/128, Kout, 128),
 * as mx_quantize_cols_grouped, mx_experts_gemm1 and mx_experts_gemm2_dgrad write them on request.
 * When both scale pitches leave 12 readable bytes behind a row's last stage (ldas, ldbs >=
 * mpad/32 + 12) the kernel fetches a row's scale bytes 16 at a time instead of 4.
 * workspace as in mx_gemm_nt: with mx_gemm_workspace_bytes() of it the K stages of the experts that
 * have rows are dealt evenly over the workgroups when their tiles alone would leave CUs idle.
 */
int mx_grouped_wgrad_nt(const uint8_t *aq, const uint8_t *as, int64_t lda, int64_t ldas, const uint8_t *bq,
                        const uint8_t *bs, int64_t ldb, int64_t ldbs, const int32_t *offsets, int64_t E,
                        int64_t M, void *dw, int dw_dtype, int64_t stride_dwe, int64_t lddw, int64_t N,
                        int64_t Kout, void *workspace, int64_t workspace_bytes, void *stream);

/* ---- expert dispatch either side of the routed-expert GEMMs ------------------------------ */

/*
 * counts (num_buckets,) int32 [b] = number of i < n with flat_idx[i] == b.  flat_idx holds n
 * indices of idx_bytes (4: int32, 8: int64) each; values outside [0, num_buckets) are not
 * counted.  counts is overwritten (it need not be zeroed).  num_buckets <= 8192.
 * Replaces expert_counts (src/kohakuwullm/models/components/moe.py:38-46), a scatter_add of
 * ones.
 */
int mx_expert_counts(const void *flat_idx, int idx_bytes, int64_t n, int64_t num_buckets, int32_t *counts,
                     void *stream);

/*
 * Group the n = T * top_k (token, slot) pairs by expert, given their histogram `counts`
 * (what mx_expert_counts returns for flat_expert):
 *   offsets (num_buckets + 1,) = [0, cumsum(counts)];
 *   order (n,): sorted position -> pair index;  token_of (n,) = order / top_k;
 *   max_rows (1,) = max(counts) (a diagnostic; may be NULL).
 * Pairs of one expert keep their input order (a stable sort), so the result is the one of the
 * reference's sort-based form expert_sort_reference (moe_dispatch.py:264-282) bit for bit and
 * does not change from run to run; the reference's device path (_expert_offsets :14-37,
 * _place_pairs :40-57, expert_sort :223-261) leaves the order inside an expert to an atomic
 * cursor.  Pairs whose expert is outside [0, num_buckets) are left out; positions that a
 * histogram inconsistent with flat_expert would put outside [0, n) are not written.
 * workspace: int32 scratch of at least mx_expert_sort_workspace(n, num_buckets) elements,
 * provided by the caller (nothing is allocated here).  num_buckets <= 1024.
 */
int64_t mx_expert_sort_workspace(int64_t n, int64_t num_buckets);
int mx_expert_sort(const void *flat_expert, int idx_bytes, int64_t n, const int32_t *counts, int64_t top_k,
                   int64_t num_buckets, int32_t *offsets, int32_t *order, int32_t *token_of, int32_t *max_rows,
                   int32_t *workspace, int64_t workspace_len, void *stream);

/*
 * mx_expert_sort for callers that can bring no workspace and must not allocate one: a tight serving loop
 * whose buffers were sized once, a harness that forbids hipMalloc.  It has no counterpart in the reference
 * (there, torch allocates inside expert_sort).  Same arguments without the workspace, same results bit for
 * bit; the scratch is a fixed array of MX_EXPERT_SORT_STATIC_WORDS int32 (4 MiB) inside the library's code
 * object, resident on every GPU the library is used on until the process ends.  The call performs no
 * hipMalloc / hipFree and no allocating library call.  A request that needs more than the array holds
 * (mx_expert_sort_workspace(n, num_buckets) > MX_EXPERT_SORT_STATIC_WORDS; never the case for
 * num_buckets <= 256) returns MX_ETOOBIG and launches nothing.  All calls on one GPU share that GPU's
 * array: calls that may overlap in time on one GPU (different streams, different threads) race and must be
 * serialised by the caller; calls in one stream are safe.
 */
#define MX_EXPERT_SORT_STATIC_WORDS (1 << 20)
int mx_expert_sort_static(const void *flat_expert, int idx_bytes, int64_t n, const int32_t *counts, int64_t top_k,
                          int64_t num_buckets, int32_t *offsets, int32_t *order, int32_t *token_of, int32_t *max_rows,
                          void *stream);

/*
 * out (num_tokens, d)[t] = sum over the sorted positions p < valid_rows[0] with
 * order[p] / top_k == t of round(rows[p] * weight[order[p]]): the gated combine of the expert
 * outputs.  rows (n, d) and out have `dtype` (MX_BF16 / MX_FP16 / MX_FP32), weight
 * (num_tokens * top_k,) has w_dtype and is indexed by pair; order (n,) holds distinct pair
 * indices token * top_k + slot (what mx_expert_sort writes; n <= num_tokens * top_k, a pair
 * that appears nowhere adds nothing).  valid_rows
 * is a one-element device int32 or NULL (every row counts).  The product is rounded to
 * `dtype`, the rows of a token are added in ascending sorted position and the sum is rounded
 * to `dtype` after every addition: the arithmetic of an index_add over the sorted rows
 * (combine_routed_reference, moe_dispatch.py:203-220), which the reference's device path
 * (_combine_fwd :60-90, _Combine.forward :134-146) performs with atomic adds in an order that
 * changes from run to run.  One writer per output element, every element written (out need
 * not be zeroed).  inv: caller-provided scratch of num_tokens * top_k int32.  d % 8 == 0,
 * 16-byte aligned rows.
 */
int mx_combine_routed(const void *rows, int dtype, int64_t ld, const void *weight, int w_dtype,
                      const int32_t *order, const int32_t *valid_rows, int32_t *inv, int64_t n, int64_t d,
                      int64_t num_tokens, int64_t top_k, void *out, int64_t ldo, void *stream);

/*
 * Both gradients of the combine: for p < valid_rows[0]
 *   grad_rows[p] = round(grad_out[token_of[p]] * weight[order[p]])       (dtype)
 *   grad_weight[order[p]] = grad_out[token_of[p]] . rows[p]              (fp32)
 * and grad_rows[p] = 0 for the other rows; grad_weight (pairs,) fp32 is zeroed first.
 * Replaces _combine_bwd / _Combine.backward (moe_dispatch.py:93-131, 148-168); the dot
 * product is one fixed-order fp32 reduction per row instead of atomics over column blocks.
 */
int mx_combine_routed_backward(const void *grad_out, int64_t ldg, const void *rows, int64_t ld, int dtype,
                               const void *weight, int w_dtype, const int32_t *order, const int32_t *token_of,
                               const int32_t *valid_rows, int64_t n, int64_t d, int64_t num_tokens, int64_t pairs,
                               void *grad_rows, int64_t ldgr, float *grad_weight, void *stream);

/* ---- measured denominators ---------------------------------------------------------------- */

/*
 * One streaming pass over device buffers, for the bandwidth the quantizers are priced against:
 *   kind 0  read:  reads out_bytes of a (c receives 4 bytes per launched thread, at most 16 MiB);
 *   kind 1  copy:  c = a, out_bytes each way;
 *   kind 2  triad: c = a + 2 b on fp32, out_bytes per operand;
 *   kind 3  2:1:   reads 2 * out_bytes of a, writes out_bytes of c (a 16-bit -> 8-bit cast's traffic).
 * out_bytes % 16 == 0, 16-byte aligned pointers.  The reference measures the same trio on its device
 * and takes the best as its denominator (src/kohakuwullm/bench/core/timing.py:231-268).
 */
int mx_ubench_stream(int kind, const void *a, const void *b, void *c, int64_t out_bytes, void *stream);

/*
 * The same streaming kernels with their launch shape as arguments, so that the ceiling a quantizer is priced against is
 * the best of a sweep and not one fixed point: threads per workgroup (a multiple of 64, at most 1024), 16-byte accesses
 * of every stream in flight per lane (unroll: 1, 2, 4 or 8), workgroups per compute unit of the grid-stride grid (0: one
 * chunk per workgroup, no loop), nontemporal bit 0: loads carry the non-temporal hint, bit 1: stores do.  Two more
 * traffic mixes beside kinds 0-3 of mx_ubench_stream: kind 4 reads a[i] and a[n + i] and writes c[i] (2 : 1 from two
 * input streams; a holds 2 x out_bytes), kind 5 reads a[i], a[n + i], a[2n + i] and writes c[i], c[n + i] (3 : 2, the
 * SwiGLU' quantizer's mix; a holds 3 x out_bytes, c 2 x out_bytes; n = out_bytes / 16).  mx_ubench_stream(kind, ...) is
 * (256 threads, unroll 4, 16 workgroups per CU, both hints).  Same rule of the reference as above
 * (src/kohakuwullm/bench/core/timing.py:231-268).
 */
int mx_ubench_stream_cfg(int kind, int threads, int unroll, int wgs_per_cu, int nontemporal, const void *a,
                         const void *b, void *c, int64_t out_bytes, void *stream);

/*
 * The memory access pattern of the 128 x 128 tile quantizers without their arithmetic, as a second, tighter ceiling
 * for them: every 256-thread workgroup reads a tile of `inputs` 16-bit matrices the way those kernels do (1: x (M,K),
 * pitch ldx; 2: the halves x[:, :K] and x[:, K:2K] of a (M,2K) matrix; 3: those and y (M,K)), writes 8 bytes per
 * 16 read into q (M,K) bytes and, with transposed != 0, the transposed byte tile into qT (K,M) (inputs == 3: a
 * second pair q2, qT2, as the SwiGLU' quantizer has two output halves).  panels != 0: q and qT in the stage-major
 * layout of mx_quantize_dual.  nontemporal as in mx_ubench_stream_cfg.  M % 128 == 0, K % 128 == 0.  The values
 * written are a fold of the values read, nothing more.
 * Same rule of the reference as mx_ubench_stream (src/kohakuwullm/bench/core/timing.py:231-268).
 */
int mx_ubench_tile_pattern(int inputs, int transposed, int nontemporal, int panels, const void *x, int64_t ldx,
                           const void *y, int64_t M, int64_t K, uint8_t *q, uint8_t *qT, uint8_t *q2, uint8_t *qT2,
                           void *stream);

/*
 * Register-resident loop of the block-scaled fp8 MFMA (bit 0 of wide clear: v_mfma_scale_f32_16x16x128_f8f6f4
 * with 8 independent accumulator tiles per wave, set: ..._32x32x64_... with 4), 8 waves on every CU (bit 1 of
 * wide set: 4 waves, one per SIMD; bit 2 set, 16x16x128 form only: scale bytes come from vector registers instead
 * of an inline constant), `iters` rounds; operands zero or (random != 0) a per-lane hash.  Returns the number of MFMA
 * instructions the launch issues (each 2 * 16*16*128 = 65536 or 2 * 32*32*64 = 131072 FLOP) or a
 * negative mx_status.  out: one float per launched thread (512 x CUs).  The reference's rule for a
 * compute ceiling: measured from registers with independent accumulators
 * (docs/internals/kernel-convention.md:14-33).
 */
int64_t mx_ubench_mfma(int wide, int iters, int random, float *out, int64_t out_floats, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* MXFP8_HIP_H */
