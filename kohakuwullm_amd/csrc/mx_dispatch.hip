// Expert dispatch either side of the routed-expert GEMMs, for gfx950: the histogram of the
// router's picks, the grouping of (token, slot) pairs by expert, and the gated combine of the
// expert outputs with its backward.  Semantics follow expert_counts
// (src/kohakuwullm/models/components/moe.py:38-46) and expert_sort / combine_routed
// (src/kohakuwullm/kernels/moe/moe_dispatch.py:14-57, 60-131, 223-261).
//
// The reference places pairs through an atomic cursor (order inside an expert changes from
// run to run) and combines through 16-bit atomic adds (order of the top_k additions changes
// from run to run).  Both are made deterministic here and equal to the reference's own
// sort-based CPU forms (expert_sort_reference :264-282, combine_routed_reference :203-220):
// the sort is a stable counting sort in three small launches, the combine is a gather in
// which each output element has one writer that adds its rows in sorted-position order with
// the rounding of a 16-bit accumulator after every addition.
//
// All of it is index and byte traffic: the combine streams top_k rows per token at HBM rate,
// the sort moves 12 bytes per pair.
#include <atomic>

#include "mx_common.h"

namespace mx {

template <bool WIDE>
__device__ __forceinline__ int64_t load_index(const void *p, int64_t i) {
    return WIDE ? ((const int64_t *)p)[i] : (int64_t)((const int32_t *)p)[i];
}

__device__ __forceinline__ int wave_sum_i32(int v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

__device__ __forceinline__ int wave_max_i32(int v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        int o = __shfl_xor(v, off, 64);
        v = o > v ? o : v;
    }
    return v;
}

__global__ __launch_bounds__(256) void dispatch_fill_kernel(int32_t *dst, int64_t n, int32_t value) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) dst[i] = value;
}

// ---- expert_counts ---------------------------------------------------------------------------
// A workgroup counts `per_block` consecutive picks in LDS and adds its non-zero bins to the
// (zeroed) global histogram.  Picks outside [0, buckets) are not counted.
template <bool WIDE>
__global__ __launch_bounds__(256) void expert_counts_kernel(const void *__restrict__ idx, int64_t n, int buckets,
                                                             int32_t *__restrict__ counts, int64_t per_block) {
    extern __shared__ int32_t bins[];
    for (int b = threadIdx.x; b < buckets; b += 256) bins[b] = 0;
    __syncthreads();
    const int64_t lo = (int64_t)blockIdx.x * per_block;
    const int64_t hi = lo + per_block < n ? lo + per_block : n;
    for (int64_t i = lo + threadIdx.x; i < hi; i += 256) {
        const int64_t e = load_index<WIDE>(idx, i);
        if (e >= 0 && e < buckets) atomicAdd(&bins[e], 1);
    }
    __syncthreads();
    for (int b = threadIdx.x; b < buckets; b += 256)
        if (bins[b]) atomicAdd(&counts[b], bins[b]);
}

// ---- expert_sort -----------------------------------------------------------------------------
// Stable counting sort.  The pairs are cut into `chunks` runs of 64 * rounds consecutive
// pairs, one wave each:
//   1. sort_hist_kernel: per-chunk histogram -> ws[e * chunks + c];
//   2. sort_scan_kernel: wave e turns row e of ws into the first sorted position of every
//      chunk's pairs of expert e (offsets[e] + pairs of e in earlier chunks), and writes
//      offsets = cumsum(counts) and max(counts);
//   3. sort_place_kernel: each wave walks its chunk again, 64 pairs at a time; a pair's
//      position is its chunk's base + the pairs of its expert earlier in the chunk (a running
//      count in LDS) + those on lower lanes of the same 64 (ballot).
template <bool WIDE>
__global__ __launch_bounds__(64) void sort_hist_kernel(const void *__restrict__ expert, int64_t n, int buckets,
                                                        int rounds, int chunks, int32_t *__restrict__ ws) {
    extern __shared__ int32_t bins[];
    const int lane = threadIdx.x, c = blockIdx.x;
    for (int b = lane; b < buckets; b += 64) bins[b] = 0;
    __syncthreads();
    const int64_t lo = (int64_t)c * rounds * 64;
    for (int r = 0; r < rounds; r++) {
        const int64_t i = lo + r * 64 + lane;
        if (i < n) {
            const int64_t e = load_index<WIDE>(expert, i);
            if (e >= 0 && e < buckets) atomicAdd(&bins[e], 1);
        }
    }
    __syncthreads();
    for (int b = lane; b < buckets; b += 64) ws[(int64_t)b * chunks + c] = bins[b];
}

__global__ __launch_bounds__(64) void sort_scan_kernel(const int32_t *__restrict__ counts, int buckets, int chunks,
                                                        int32_t *__restrict__ ws, int32_t *__restrict__ offsets,
                                                        int32_t *__restrict__ max_rows) {
    const int lane = threadIdx.x, e = blockIdx.x;
    int before = 0;
    for (int j = lane; j < e; j += 64) before += counts[j];
    before = wave_sum_i32(before);
    if (lane == 0) {
        offsets[e + 1] = before + counts[e];
        if (e == 0) offsets[0] = 0;
    }
    if (e == 0 && max_rows) {
        int most = 0;
        for (int j = lane; j < buckets; j += 64) most = counts[j] > most ? counts[j] : most;
        most = wave_max_i32(most);
        if (lane == 0) max_rows[0] = most;
    }
    int32_t *row = ws + (int64_t)e * chunks;
    int carry = before;
    for (int c0 = 0; c0 < chunks; c0 += 64) {
        const int c = c0 + lane;
        const int v = c < chunks ? row[c] : 0;
        int incl = v;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int up = __shfl_up(incl, off, 64);
            if (lane >= off) incl += up;
        }
        if (c < chunks) row[c] = carry + incl - v;
        carry += __shfl(incl, 63, 64);
    }
}

template <bool WIDE>
__global__ __launch_bounds__(64) void sort_place_kernel(const void *__restrict__ expert, int64_t n, int buckets,
                                                         int rounds, int chunks, int top_k,
                                                         const int32_t *__restrict__ ws, int32_t *__restrict__ order,
                                                         int32_t *__restrict__ token_of) {
    extern __shared__ int32_t seen[];  // pairs of each expert met so far in this chunk
    const int lane = threadIdx.x, c = blockIdx.x;
    for (int b = lane; b < buckets; b += 64) seen[b] = 0;
    __syncthreads();
    const int64_t lo = (int64_t)c * rounds * 64;
    const uint64_t below = lane ? ~0ull >> (64 - lane) : 0ull;
    for (int r = 0; r < rounds; r++) {
        const int64_t i = lo + r * 64 + lane;
        int e = -1;
        if (i < n) {
            const int64_t v = load_index<WIDE>(expert, i);
            e = v >= 0 && v < buckets ? (int)v : -1;
        }
        const bool live = e >= 0;
        // lanes holding the same expert: rank among them in lane order, and how many they are
        uint64_t todo = __ballot(live);
        int rank = 0, same = 0;
        while (todo) {
            const int leader = __builtin_ctzll(todo);
            const int v = __shfl(e, leader, 64);
            const uint64_t m = __ballot(live && e == v);
            if (live && e == v) {
                rank = __builtin_popcountll(m & below);
                same = __builtin_popcountll(m);
            }
            todo &= ~m;
        }
        int met = 0;
        if (live) {
            met = seen[e];
            const int64_t pos = (int64_t)ws[(int64_t)e * chunks + c] + met + rank;
            if (pos >= 0 && pos < n) {  // only counts that disagree with the picks can fail this
                order[pos] = (int32_t)i;
                token_of[pos] = (int32_t)(i / top_k);
            }
        }
        __syncthreads();
        if (live && rank == 0) seen[e] = met + same;
        __syncthreads();
    }
}

// ---- combine_routed --------------------------------------------------------------------------
// inv[pair] = sorted position of the pair, for positions below the valid bound; -1 elsewhere.
__global__ __launch_bounds__(256) void combine_invert_kernel(const int32_t *__restrict__ order,
                                                              const int32_t *__restrict__ valid_rows, int64_t n,
                                                              int64_t pairs, int32_t *__restrict__ inv) {
    const int64_t p = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (p >= n || (valid_rows && p >= valid_rows[0])) return;
    const int64_t pair = order[p];
    if (pair >= 0 && pair < pairs) inv[pair] = (int32_t)p;
}

// v is an fp32 result that is rounded again when it is stored as 16 bits.  The empty asm keeps
// the compiler from folding the operation that made v and the conversion into one
// v_fma_mix* instruction, which rounds the exact result once and so differs in the last place
// of an fp16 from "fp32 operation, then convert".
__device__ __forceinline__ float settled(float v) {
    asm volatile("" : "+v"(v));
    return v;
}

template <int DT>
__device__ __forceinline__ float round_to(float v) {
    v = settled(v);
    if (DT == MX_BF16) return bits2f(f2bf16(v) << 16);
    if (DT == MX_FP16) return (float)(_Float16)v;
    return v;
}

// Two values at once: bf16 goes through the hardware pair conversion (round to nearest even).
template <int DT>
__device__ __forceinline__ void round_pair_to(float &a, float &b) {
    if (DT == MX_BF16) {
        const uint32_t w = pack2_bf16(settled(a), settled(b));
        a = bits2f(w << 16);
        b = bits2f(w & 0xFFFF0000u);
    } else {
        a = round_to<DT>(a);
        b = round_to<DT>(b);
    }
}

template <int DT>
__device__ __forceinline__ void store_row8(void *p, const float (&y)[8]) {
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

template <int WDT>
__device__ __forceinline__ float load_weight(const void *w, int64_t i) {
    return Elem<WDT>::load1((const typename Elem<WDT>::type *)w + i);
}

// One thread per token: its top_k entries of inv in ascending order, absent pairs (-1) last.
__global__ __launch_bounds__(256) void combine_sort_kernel(int32_t *__restrict__ inv, int top_k, int64_t tokens) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= tokens) return;
    int32_t *mine = inv + t * top_k;
    for (int i = 1; i < top_k; i++) {
        const int32_t v = mine[i];
        const uint32_t key = (uint32_t)v;  // -1 compares as the largest
        int j = i - 1;
        while (j >= 0 && (uint32_t)mine[j] > key) {
            mine[j + 1] = mine[j];
            j--;
        }
        mine[j + 1] = v;
    }
}

// One thread per 8 columns of a token.  The token's rows are added in ascending sorted position
// (the order of an index_add over the sorted rows; `sorted` holds them in that order); the
// product and every partial sum are rounded to the row type, as a 16-bit accumulator in memory
// would.  Rows are fetched four at a time so that their loads overlap.
template <int DT, int WDT>
__global__ __launch_bounds__(256) void combine_routed_kernel(const void *__restrict__ rows, int64_t ld,
                                                              const void *__restrict__ weight,
                                                              const int32_t *__restrict__ order,
                                                              const int32_t *__restrict__ sorted, int top_k,
                                                              void *__restrict__ out, int64_t ldo, int64_t tokens,
                                                              int d8) {
#pragma clang fp contract(off)  // fp32 rows: the product is rounded before it is added, never fused
    typedef typename Elem<DT>::type T;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t t = idx / d8;
    const int col = (int)(idx - t * d8) * 8;
    if (t >= tokens) return;
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; e++) acc[e] = 0.0f;
    const int32_t *mine = sorted + t * top_k;
    for (int k0 = 0; k0 < top_k; k0 += 4) {
        int pos[4];
        float scale[4], v[4][8];
#pragma unroll
        for (int u = 0; u < 4; u++) pos[u] = k0 + u < top_k ? mine[k0 + u] : -1;
#pragma unroll
        for (int u = 0; u < 4; u++) {
            if (pos[u] < 0) continue;
            scale[u] = load_weight<WDT>(weight, order[pos[u]]);
            Elem<DT>::load8((const T *)rows + (int64_t)pos[u] * ld + col, v[u]);
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
            if (pos[u] < 0) continue;
#pragma unroll
            for (int e = 0; e < 8; e += 2) {
                float a = v[u][e] * scale[u], b = v[u][e + 1] * scale[u];
                round_pair_to<DT>(a, b);
                a += acc[e], b += acc[e + 1];
                round_pair_to<DT>(a, b);
                acc[e] = a, acc[e + 1] = b;
            }
        }
    }
    store_row8<DT>((T *)out + t * ldo + col, acc);
}

// One wave per sorted row: grad_rows[p] = grad_out[token_of[p]] * weight[order[p]] rounded to
// the row type, grad_weight[order[p]] = grad_out[token_of[p]] . rows[p] in fp32.  Rows at or
// past the valid bound get a zero gradient and leave grad_weight (zeroed beforehand) alone.
template <int DT, int WDT>
__global__ __launch_bounds__(256) void combine_routed_bwd_kernel(const void *__restrict__ grad_out, int64_t ldg,
                                                                  const void *__restrict__ rows, int64_t ld,
                                                                  const void *__restrict__ weight,
                                                                  const int32_t *__restrict__ order,
                                                                  const int32_t *__restrict__ token_of,
                                                                  const int32_t *__restrict__ valid_rows, int64_t n,
                                                                  int64_t pairs, int64_t tokens, int d,
                                                                  void *__restrict__ grad_rows,
                                                                  int64_t ldgr, float *__restrict__ grad_weight) {
    typedef typename Elem<DT>::type T;
    const int lane = threadIdx.x & 63;
    const int64_t p = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (p >= n) return;
    const int64_t pair = order[p], token = token_of[p];
    const bool live = (!valid_rows || p < valid_rows[0]) && pair >= 0 && pair < pairs && token >= 0 && token < tokens;
    T *dst = (T *)grad_rows + p * ldgr;
    if (!live) {
        const float zero[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int col = lane * 8; col < d; col += 512) store_row8<DT>(dst + col, zero);
        return;
    }
    const float scale = load_weight<WDT>(weight, pair);
    const T *g = (const T *)grad_out + token * ldg, *y = (const T *)rows + p * ld;
    float dot = 0.0f;
    for (int col = lane * 8; col < d; col += 512) {
        float gv[8], yv[8], o[8];
        Elem<DT>::load8(g + col, gv);
        Elem<DT>::load8(y + col, yv);
#pragma unroll
        for (int e = 0; e < 8; e++) {
            o[e] = settled(gv[e] * scale);
            dot += gv[e] * yv[e];
        }
        store_row8<DT>(dst + col, o);
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) dot += __shfl_xor(dot, off, 64);
    if (lane == 0) grad_weight[pair] = dot;
}

static bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }

// Pairs per wave of the sort: at least 4 rounds of 64, more when that keeps the number of
// chunks (and with it the workspace, chunks * buckets int32) at or below 4096.
static int sort_rounds(int64_t n) {
    int64_t rounds = (n + 64 * 4096 - 1) / (64 * 4096);
    return (int)(rounds < 4 ? 4 : rounds);
}

template <int DT>
static int launch_combine(int w_dtype, const void *rows, int64_t ld, const void *weight, const int32_t *order,
                          const int32_t *inv, int top_k, void *out, int64_t ldo, int64_t tokens, int d8, unsigned blocks,
                          hipStream_t st) {
    switch (w_dtype) {
    case MX_BF16: combine_routed_kernel<DT, MX_BF16><<<dim3(blocks), dim3(256), 0, st>>>(rows, ld, weight, order, inv, top_k, out, ldo, tokens, d8); break;
    case MX_FP16: combine_routed_kernel<DT, MX_FP16><<<dim3(blocks), dim3(256), 0, st>>>(rows, ld, weight, order, inv, top_k, out, ldo, tokens, d8); break;
    default: combine_routed_kernel<DT, MX_FP32><<<dim3(blocks), dim3(256), 0, st>>>(rows, ld, weight, order, inv, top_k, out, ldo, tokens, d8); break;
    }
    return hipGetLastError() == hipSuccess ? MX_OK : MX_ELAUNCH;
}

template <int DT>
static int launch_combine_bwd(int w_dtype, const void *grad_out, int64_t ldg, const void *rows, int64_t ld,
                              const void *weight, const int32_t *order, const int32_t *token_of,
                              const int32_t *valid_rows, int64_t n, int64_t pairs, int64_t tokens, int d, void *grad_rows,
                              int64_t ldgr, float *grad_weight, hipStream_t st) {
    const dim3 grid((unsigned)((n + 3) / 4)), block(256);
    switch (w_dtype) {
    case MX_BF16: combine_routed_bwd_kernel<DT, MX_BF16><<<grid, block, 0, st>>>(grad_out, ldg, rows, ld, weight, order, token_of, valid_rows, n, pairs, tokens, d, grad_rows, ldgr, grad_weight); break;
    case MX_FP16: combine_routed_bwd_kernel<DT, MX_FP16><<<grid, block, 0, st>>>(grad_out, ldg, rows, ld, weight, order, token_of, valid_rows, n, pairs, tokens, d, grad_rows, ldgr, grad_weight); break;
    default: combine_routed_bwd_kernel<DT, MX_FP32><<<grid, block, 0, st>>>(grad_out, ldg, rows, ld, weight, order, token_of, valid_rows, n, pairs, tokens, d, grad_rows, ldgr, grad_weight); break;
    }
    return hipGetLastError() == hipSuccess ? MX_OK : MX_ELAUNCH;
}
}  // namespace mx

using namespace mx;

static const int64_t MAX_COUNT_BUCKETS = 8192, MAX_SORT_BUCKETS = 1024;

static bool dtype_ok(int dt) { return dt == MX_BF16 || dt == MX_FP16 || dt == MX_FP32; }

extern "C" int mx_expert_counts(const void *flat_idx, int idx_bytes, int64_t n, int64_t num_buckets, int32_t *counts,
                                void *stream) {
    if (n < 0 || num_buckets <= 0 || (idx_bytes != 4 && idx_bytes != 8) || !counts || (n > 0 && !flat_idx) ||
        n >= 0x7FFFFFFF)
        return MX_EINVAL;
    if (num_buckets > MAX_COUNT_BUCKETS) return MX_EUNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    if (mx::stream_is_capturing(st)) return MX_ECAPTURE;
    dispatch_fill_kernel<<<dim3((unsigned)((num_buckets + 255) / 256)), dim3(256), 0, st>>>(counts, num_buckets, 0);
    if (n) {
        const int64_t per_block = 1024;
        const dim3 grid((unsigned)((n + per_block - 1) / per_block)), block(256);
        const size_t lds = (size_t)num_buckets * sizeof(int32_t);
        if (idx_bytes == 8)
            expert_counts_kernel<true><<<grid, block, lds, st>>>(flat_idx, n, (int)num_buckets, counts, per_block);
        else
            expert_counts_kernel<false><<<grid, block, lds, st>>>(flat_idx, n, (int)num_buckets, counts, per_block);
    }
    return hipGetLastError() == hipSuccess ? MX_OK : MX_ELAUNCH;
}

extern "C" int64_t mx_expert_sort_workspace(int64_t n, int64_t num_buckets) {
    if (n < 0 || num_buckets <= 0 || n >= 0x7FFFFFFF) return -1;
    const int64_t per_chunk = 64 * (int64_t)sort_rounds(n);
    const int64_t chunks = n ? (n + per_chunk - 1) / per_chunk : 1;
    return chunks * num_buckets;
}

// The three launches of the sort on a workspace of `need` = chunks * num_buckets words that the caller of this
// function vouches for (the public entry points check where it comes from and how large it is).
static int sort_launch(const void *flat_expert, int idx_bytes, int64_t n, const int32_t *counts, int64_t top_k,
                       int64_t num_buckets, int32_t *offsets, int32_t *order, int32_t *token_of, int32_t *max_rows,
                       int32_t *workspace, int64_t need, hipStream_t st) {
    const int rounds = sort_rounds(n), buckets = (int)num_buckets;
    const int chunks = (int)(need / num_buckets);
    const size_t lds = (size_t)buckets * sizeof(int32_t);
    const dim3 wave(64);
    // every word of workspace[0, need) is written before it is read: by the fill when there are no pairs, else by
    // the histogram pass (each chunk writes its count for every bucket), so nothing of an earlier call survives
    if (n == 0) dispatch_fill_kernel<<<dim3((unsigned)((need + 255) / 256)), dim3(256), 0, st>>>(workspace, need, 0);
    if (n && idx_bytes == 8) sort_hist_kernel<true><<<dim3((unsigned)chunks), wave, lds, st>>>(flat_expert, n, buckets, rounds, chunks, workspace);
    if (n && idx_bytes == 4) sort_hist_kernel<false><<<dim3((unsigned)chunks), wave, lds, st>>>(flat_expert, n, buckets, rounds, chunks, workspace);
    sort_scan_kernel<<<dim3((unsigned)buckets), wave, 0, st>>>(counts, buckets, chunks, workspace, offsets, max_rows);
    if (n && idx_bytes == 8) sort_place_kernel<true><<<dim3((unsigned)chunks), wave, lds, st>>>(flat_expert, n, buckets, rounds, chunks, (int)top_k, workspace, order, token_of);
    if (n && idx_bytes == 4) sort_place_kernel<false><<<dim3((unsigned)chunks), wave, lds, st>>>(flat_expert, n, buckets, rounds, chunks, (int)top_k, workspace, order, token_of);
    return hipGetLastError() == hipSuccess ? MX_OK : MX_ELAUNCH;
}

static int sort_args_ok(const void *flat_expert, int idx_bytes, int64_t n, const int32_t *counts, int64_t top_k,
                        int64_t num_buckets, const int32_t *offsets, const int32_t *order, const int32_t *token_of) {
    if (n < 0 || n >= 0x7FFFFFFF || num_buckets <= 0 || top_k <= 0 || (idx_bytes != 4 && idx_bytes != 8) || !counts ||
        !offsets || (n > 0 && (!flat_expert || !order || !token_of)))
        return MX_EINVAL;
    return num_buckets > MAX_SORT_BUCKETS ? MX_EUNSUPPORTED : MX_OK;
}

extern "C" int mx_expert_sort(const void *flat_expert, int idx_bytes, int64_t n, const int32_t *counts, int64_t top_k,
                              int64_t num_buckets, int32_t *offsets, int32_t *order, int32_t *token_of,
                              int32_t *max_rows, int32_t *workspace, int64_t workspace_len, void *stream) {
    const int rc = sort_args_ok(flat_expert, idx_bytes, n, counts, top_k, num_buckets, offsets, order, token_of);
    if (rc != MX_OK) return rc;
    const int64_t need = mx_expert_sort_workspace(n, num_buckets);
    if (!workspace || workspace_len < need) return MX_EINVAL;
    hipStream_t st = (hipStream_t)stream;
    if (mx::stream_is_capturing(st)) return MX_ECAPTURE;
    return sort_launch(flat_expert, idx_bytes, n, counts, top_k, num_buckets, offsets, order, token_of, max_rows, workspace,
                       need, st);
}

// Scratch of mx_expert_sort_static: a fixed array in the code object, so the entry point has nothing to allocate.
// Every device the library runs on holds its own copy at its own address for the life of the process.  In host
// code the name below is only a handle for hipGetSymbolAddress; the address kernels may use is what that call
// returns on the device that is current, kept per device ordinal in sort_scratch_of().
static __device__ __align__(256) int32_t scratch[MX_EXPERT_SORT_STATIC_WORDS];

static int32_t *sort_scratch_of_current_device() {
    static std::atomic<int32_t *> known[64];  // by device ordinal; written once with the only value it can hold
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
    int32_t *ptr = known[dev].load(std::memory_order_acquire);
    if (ptr) return ptr;
    if (hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) {
        (void)hipGetLastError();
        return nullptr;
    }
    known[dev].store(ptr, std::memory_order_release);
    return ptr;
}

extern "C" int mx_expert_sort_static(const void *flat_expert, int idx_bytes, int64_t n, const int32_t *counts,
                                     int64_t top_k, int64_t num_buckets, int32_t *offsets, int32_t *order,
                                     int32_t *token_of, int32_t *max_rows, void *stream) {
    const int rc = sort_args_ok(flat_expert, idx_bytes, n, counts, top_k, num_buckets, offsets, order, token_of);
    if (rc != MX_OK) return rc;
    const int64_t need = mx_expert_sort_workspace(n, num_buckets);
    if (need > MX_EXPERT_SORT_STATIC_WORDS) return MX_ETOOBIG;
    hipStream_t st = (hipStream_t)stream;
    if (mx::stream_is_capturing(st)) return MX_ECAPTURE;
    int32_t *const ws = sort_scratch_of_current_device();
    if (!ws) return MX_ELAUNCH;
    return sort_launch(flat_expert, idx_bytes, n, counts, top_k, num_buckets, offsets, order, token_of, max_rows, ws, need, st);
}

extern "C" int mx_combine_routed(const void *rows, int dtype, int64_t ld, const void *weight, int w_dtype,
                                 const int32_t *order, const int32_t *valid_rows, int32_t *inv, int64_t n, int64_t d,
                                 int64_t num_tokens, int64_t top_k, void *out, int64_t ldo, void *stream) {
    if (n < 0 || d < 0 || num_tokens < 0 || top_k <= 0 || top_k > 0x7FFF || n >= 0x7FFFFFFF || !dtype_ok(dtype) ||
        !dtype_ok(w_dtype) || num_tokens * top_k >= 0x7FFFFFFF || n > num_tokens * top_k || ld < d || ldo < d)
        return MX_EINVAL;
    if (num_tokens == 0 || d == 0) return MX_OK;
    const int64_t pairs = num_tokens * top_k;
    if ((n > 0 && (!rows || !order)) || !weight || !inv || !out) return MX_EINVAL;
    const int esz = dtype == MX_FP32 ? 4 : 2;
    if (d % 8 || !aligned16(rows) || !aligned16(out) || (ld * esz) % 16 || (ldo * esz) % 16) return MX_EUNSUPPORTED;
    const int64_t blocks = (num_tokens * (d / 8) + 255) / 256;
    if (blocks > 0x7FFFFFFF) return MX_EUNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    if (mx::stream_is_capturing(st)) return MX_ECAPTURE;
    dispatch_fill_kernel<<<dim3((unsigned)((pairs + 255) / 256)), dim3(256), 0, st>>>(inv, pairs, -1);
    if (n) combine_invert_kernel<<<dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st>>>(order, valid_rows, n, pairs, inv);
    if (n && top_k > 1) combine_sort_kernel<<<dim3((unsigned)((num_tokens + 255) / 256)), dim3(256), 0, st>>>(inv, (int)top_k, num_tokens);
    switch (dtype) {
    case MX_BF16: return launch_combine<MX_BF16>(w_dtype, rows, ld, weight, order, inv, (int)top_k, out, ldo, num_tokens, (int)(d / 8), (unsigned)blocks, st);
    case MX_FP16: return launch_combine<MX_FP16>(w_dtype, rows, ld, weight, order, inv, (int)top_k, out, ldo, num_tokens, (int)(d / 8), (unsigned)blocks, st);
    default: return launch_combine<MX_FP32>(w_dtype, rows, ld, weight, order, inv, (int)top_k, out, ldo, num_tokens, (int)(d / 8), (unsigned)blocks, st);
    }
}

extern "C" int mx_combine_routed_backward(const void *grad_out, int64_t ldg, const void *rows, int64_t ld, int dtype,
                                          const void *weight, int w_dtype, const int32_t *order,
                                          const int32_t *token_of, const int32_t *valid_rows, int64_t n, int64_t d,
                                          int64_t num_tokens, int64_t pairs, void *grad_rows, int64_t ldgr,
                                          float *grad_weight, void *stream) {
    if (n < 0 || d < 0 || num_tokens < 0 || pairs < 0 || n >= 0x7FFFFFFF || pairs >= 0x7FFFFFFF || d >= 0x7FFFFFFF ||
        !dtype_ok(dtype) || !dtype_ok(w_dtype) || ldg < d || ld < d || ldgr < d)
        return MX_EINVAL;
    if (pairs > 0 && !grad_weight) return MX_EINVAL;
    if (n > 0 && (!grad_out || !rows || !weight || !order || !token_of || !grad_rows)) return MX_EINVAL;
    if (pairs == 0 && (n == 0 || d == 0)) return MX_OK;
    const int esz = dtype == MX_FP32 ? 4 : 2;
    if (d % 8 || !aligned16(grad_out) || !aligned16(rows) || !aligned16(grad_rows) || (ldg * esz) % 16 ||
        (ld * esz) % 16 || (ldgr * esz) % 16)
        return MX_EUNSUPPORTED;
    hipStream_t st = (hipStream_t)stream;
    if (mx::stream_is_capturing(st)) return MX_ECAPTURE;
    if (pairs) dispatch_fill_kernel<<<dim3((unsigned)((pairs + 255) / 256)), dim3(256), 0, st>>>((int32_t *)grad_weight, pairs, 0);
    if (n == 0 || d == 0) return hipGetLastError() == hipSuccess ? MX_OK : MX_ELAUNCH;
    switch (dtype) {
    case MX_BF16: return launch_combine_bwd<MX_BF16>(w_dtype, grad_out, ldg, rows, ld, weight, order, token_of, valid_rows, n, pairs, num_tokens, (int)d, grad_rows, ldgr, grad_weight, st);
    case MX_FP16: return launch_combine_bwd<MX_FP16>(w_dtype, grad_out, ldg, rows, ld, weight, order, token_of, valid_rows, n, pairs, num_tokens, (int)d, grad_rows, ldgr, grad_weight, st);
    default: return launch_combine_bwd<MX_FP32>(w_dtype, grad_out, ldg, rows, ld, weight, order, token_of, valid_rows, n, pairs, num_tokens, (int)d, grad_rows, ldgr, grad_weight, st);
    }
}
