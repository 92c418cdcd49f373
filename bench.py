"""Benchmark of the MXFP8 linear path on one MI355X.

Workload (the configuration the headline metric is quoted on): the dense 546M-class
SwiGLU feed-forward, forward and backward -- X bf16 [16384, 1536] ~ N(0,1); W_gate, W_up
[4096, 1536] and W_down [1536, 4096] ~ N(0, 0.02); dY [16384, 1536] ~ N(0, 1e-2); MXFP8
blocks of 32 along every GEMM's contraction axis, token-axis requantization for wgrad.
One step = quantize X (row+token axis) -> GEMM -> SwiGLU+quantize -> GEMM; quantize dY ->
dgrad GEMM -> SwiGLU'+quantize -> dgrad GEMM; two wgrad GEMMs.  Six products, 1855.4 GFLOP.
Weights are quantized once before the timed region (they change once per optimizer step,
not per micro-batch) and that cost is reported separately.

Prints ONE JSON line.  `value` is the whole step's TFLOP/s (quantizers included), inputs
resident in HBM.  `roofline` prices the dominant kernel (the block-scaled MFMA GEMM) from
HIP events recorded around every launch in a second, instrumented run of the same steps;
`quantizer` does the same for the HBM-bound quantizer launches.  `cpu_baseline` times the
CPU oracle (dequantize-then-matmul in fp32 + the torch statement of the quantizer) on a
token subsample of the same workload.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

SEED = 20090220
TOKENS, DIM, FFN = 16384, 1536, 4096
MFMA_PEAK_TFLOPS = 5000.0  # MI355X dense fp8 / MXFP8
HBM_PEAK_GBS = 8000.0


def step_flops(tokens: int) -> float:
    return 3 * (2.0 * tokens * 2 * FFN * DIM + 2.0 * tokens * DIM * FFN)


def make_inputs(tokens: int):
    import torch

    g = torch.Generator().manual_seed(SEED)
    x = torch.randn(tokens, DIM, generator=g).bfloat16()
    w_gate = (torch.randn(FFN, DIM, generator=g) * 0.02).bfloat16()
    w_up = (torch.randn(FFN, DIM, generator=g) * 0.02).bfloat16()
    w_down = (torch.randn(DIM, FFN, generator=g) * 0.02).bfloat16()
    dy = (torch.randn(tokens, DIM, generator=g) * 1e-2).bfloat16()
    return x, torch.cat([w_gate, w_up], 0), w_down, dy


def make_attention_inputs(tokens: int = 32768, dim: int = 2048, heads: int = 16, kv_heads: int = 4, head_dim: int = 128):
    """BASELINE configs[2]: GQA attention projections.  Hidden N(0,1); W_qkv [(heads+2*kv)*hd, dim], W_o [dim, dim] N(0,0.02)."""
    import torch

    g = torch.Generator().manual_seed(SEED)
    hid = torch.randn(tokens, dim, generator=g).bfloat16()
    w_qkv = (torch.randn((heads + 2 * kv_heads) * head_dim, dim, generator=g) * 0.02).bfloat16()
    w_o = (torch.randn(dim, heads * head_dim, generator=g) * 0.02).bfloat16()
    d_qkv = (torch.randn(tokens, w_qkv.shape[0], generator=g) * 1e-2).bfloat16()
    d_o = (torch.randn(tokens, dim, generator=g) * 1e-2).bfloat16()
    return hid, w_qkv, w_o, d_qkv, d_o


def zipf_counts(num_experts: int = 64, total: int = 98304, cap: int = 16384, s: float = 1.1):
    """Per-expert row counts ~ Zipf(s), summing to `total`, each <= cap, at least one expert empty."""
    import numpy as np

    z = np.random.Generator(np.random.PCG64(SEED)).zipf(s, num_experts).astype(np.float64)
    c = np.floor(total * z / z.sum()).astype(np.int64)
    c = np.minimum(c, cap)
    order = np.argsort(-c, kind="stable")
    rem = total - int(c.sum())
    i = 0
    while rem > 0:  # push the remainder / overflow to the next-largest experts
        e = order[i % num_experts]
        add = min(cap - int(c[e]), rem)
        c[e] += add
        rem -= add
        i += 1
    if (c == 0).sum() == 0:
        small, big = int(np.argmin(c)), int(np.argmax(np.where(c < cap, c, -1)))
        c[big] += c[small]
        c[small] = 0
    assert int(c.sum()) == total and (c <= cap).all() and (c == 0).any()
    return [int(v) for v in c]


def ranked_counts(num_experts: int = 64, total: int = 98304, cap: int = 16384, s: float = 1.1, empty: int = 5):
    """Zipf(s) loads by rank instead of by draw: expert of rank r gets ~ r^-s of the rows (capped), `empty` experts none.

    The seeded draws of `zipf_counts` happen to give six full experts and 58 empty ones; this routing keeps
    59 experts alive with loads from 16384 rows down to a few dozen, so ragged tiles are what gets measured.
    """
    import torch

    live = num_experts - empty
    p = torch.arange(1, live + 1, dtype=torch.float64) ** -s
    c = torch.floor(p / p.sum() * total).long().clamp(max=cap)
    i = 0
    while int(c.sum()) < total:
        add = min(cap - int(c[i]), total - int(c.sum()))
        c[i] += add
        i += 1
    perm = torch.randperm(num_experts, generator=torch.Generator().manual_seed(SEED))
    out = torch.zeros(num_experts, dtype=torch.long)
    out[perm[:live]] = c
    return out.tolist()


def make_moe_inputs(tokens: int = 16384, dim: int = 1024, hidden: int = 512, num_experts: int = 64, top_k: int = 6,
                    routing: str = "draws"):
    """BASELINE configs[3]: routed experts with Zipf(1.1) loads; sorted position m -> token m mod T, slot m div T.

    routing "draws": per-expert loads drawn i.i.d. Zipf as the configuration says; "ranked": `ranked_counts`.
    """
    import torch

    g = torch.Generator().manual_seed(SEED)
    x = torch.randn(tokens, dim, generator=g).bfloat16()
    w_in = (torch.randn(num_experts, 2 * hidden, dim, generator=g) * 0.02).bfloat16()
    w_out = (torch.randn(num_experts, dim, hidden, generator=g) * 0.02).bfloat16()
    gate = (torch.rand(tokens * top_k, generator=g) * 0.5 + 0.5).bfloat16()
    dout = (torch.randn(tokens, dim, generator=g) * 1e-2).bfloat16()
    counts = (zipf_counts if routing == "draws" else ranked_counts)(num_experts, tokens * top_k, tokens)
    offsets = torch.zeros(num_experts + 1, dtype=torch.int32)
    offsets[1:] = torch.tensor(counts).cumsum(0)
    m = torch.arange(tokens * top_k)
    token_of = (m % tokens).int()
    order = (token_of.long() * top_k + m // tokens).int()
    return x, w_in, w_out, gate, dout, offsets, order, token_of, counts


def make_outlier_inputs(n: int = 8192):
    """BASELINE configs[4]: Student-t(3) activations with 0.1% of channels x200 and injected special blocks."""
    import torch

    g = torch.Generator().manual_seed(SEED)
    z = torch.randn(n, n, generator=g)
    chi = (torch.randn(n, n, 3, generator=g) ** 2).sum(-1) / 3
    x = z / chi.sqrt()
    cols = torch.randperm(n, generator=g)[: max(1, n // 1000)]
    x[:, cols] *= 200.0
    x = x.bfloat16()
    blocks = x.view(n, n // 32, 32)
    nb = n * (n // 32)
    pick = torch.randperm(nb, generator=g)
    zero, tiny, big, tie = pick[: nb // 1000], pick[nb // 1000 : nb // 1000 + 64], pick[-128:-64], pick[-64:]
    flat = blocks.view(nb, 32)
    flat[zero] = 0.0
    flat[tiny] = 1e-35
    flat[big, 0] = 3.0e38
    flat[big, 1] = -3.0e38
    j = torch.randint(-20, 20, (64,), generator=g).float()
    flat[tie] = flat[tie].clamp(-1, 1)
    flat[tie, 7] = (448.0 * torch.exp2(j)).bfloat16()
    flat[tie] = torch.minimum(flat[tie].float().abs(), (448.0 * torch.exp2(j))[:, None]).bfloat16() * torch.sign(flat[tie].float()).bfloat16()
    flat[tie, 7] = (448.0 * torch.exp2(j)).bfloat16()
    w = (torch.randn(n, n, generator=g) * 0.02).bfloat16()
    dy = (torch.randn(n, n, generator=g) * 1e-2).bfloat16()
    special = dict(zero=zero, tiny=tiny, big=big, tie=tie)
    return x, w, dy, special


def cpu_baseline(sample_tokens: int = TOKENS, device_rows=None) -> dict:
    """The oracle's formulas with PyTorch CPU ops on the first `sample_tokens` tokens.

    `device_rows` = (row indices, the device's output rows for them): the same leg, being the checker, also states
    how far the measured path's forward output is from the oracle's chain on those rows (relative Frobenius error)."""
    import torch

    from oracle import mx_oracle as ora

    x_all, w_in, w_out, dy = make_inputs(TOKENS)
    x, dy = x_all[:sample_tokens].contiguous(), dy[:sample_tokens].contiguous()
    f32 = torch.float32

    def q_rows(t):
        return ora.quantize_rows_torch(t)

    def q_cols(t):
        return ora.quantize_rows_torch(t.t().contiguous())

    t0 = time.perf_counter()
    win_f, win_d, wout_f, wout_d = q_rows(w_in), q_cols(w_in), q_rows(w_out), q_cols(w_out)
    t_weights = time.perf_counter() - t0
    def one_step():
        xq, xt = q_rows(x), q_cols(x)
        gu = ora.gemm_nt(*xq, *win_f, dtype=f32).bfloat16()
        g, u = gu.float().chunk(2, dim=-1)
        h = g * torch.sigmoid(g) * u
        hq, ht = q_rows(h), q_cols(h)
        ora.gemm_nt(*hq, *wout_f, dtype=f32).bfloat16()
        dq, dt = q_rows(dy), q_cols(dy)
        dh = ora.gemm_nt(*dq, *wout_d, dtype=f32).bfloat16().float()
        sg = torch.sigmoid(g)
        dpre = torch.cat([dh * u * sg * (1 + g * (1 - sg)), dh * g * sg], dim=-1)
        pq, pt = q_rows(dpre), q_cols(dpre)
        ora.gemm_nt(*pq, *win_d, dtype=f32).bfloat16()
        ora.gemm_nt(*pt, *xt, dtype=f32).bfloat16()
        ora.gemm_nt(*dt, *ht, dtype=f32).bfloat16()

    # whole steps until about ten seconds of CPU work have been timed (at least one, at most eight)
    steps, t0 = 0, time.perf_counter()
    while steps < 1 or (time.perf_counter() - t0 < 10.0 and steps < 8):
        one_step()
        steps += 1
    dt_step = (time.perf_counter() - t0) / steps
    accuracy = {}
    if device_rows is not None:
        rows, y_dev = device_rows
        gu = ora.gemm_nt(*ora.quantize_rows(x_all[rows]), *win_f).bfloat16().float()
        g, u = gu.chunk(2, dim=-1)
        y_ref = ora.gemm_nt(*ora.quantize_rows(g * torch.sigmoid(g) * u), *wout_f)
        accuracy = {"rel_error": float(f"{ora.rel_error(y_dev, y_ref):.3e}"),
                    "rel_error_of": f"forward output of {len(rows)} sampled tokens against the oracle's dequantize-then-matmul chain in fp64"}
    return {
        **accuracy,
        "value": step_flops(sample_tokens) / dt_step / 1e12,
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{sample_tokens} of {TOKENS} tokens of the same workload, {steps} whole steps, all six products "
        f"(fp32 torch.matmul on dequantized operands) and all quantizers (torch statement); "
        f"{dt_step:.2f} s per step; weights quantized outside ({t_weights:.2f} s); host cpu_count={os.cpu_count()}",
    }



def _event_times(fn, iters: int, warm: int = 3):
    """Device times (ms) of `iters` calls of fn, each bracketed by events on the current stream."""
    import torch

    for _ in range(warm):
        fn()
    pairs = []
    for _ in range(iters):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        pairs.append((a, b))
    torch.cuda.synchronize()
    return sorted(a.elapsed_time(b) for a, b in pairs)


STREAM_KINDS = (("read", 0, 1), ("copy", 1, 2), ("triad", 2, 3), ("read2_write1", 3, 3), ("read2_write1_two_streams", 4, 3),
                ("read3_write2", 5, 5))  # name, kind of mx_ubench_stream_cfg, bytes moved per output byte
# launch shapes swept per mix: (threads, unroll, workgroups per CU [0: one chunk each], non-temporal bits [1 loads, 2 stores])
STREAM_SWEEP_FULL = tuple((t, u, w, nt) for t in (256, 512, 1024) for u in (1, 2, 4, 8) for w in (0, 8, 16, 32) for nt in (0, 1, 2, 3))
# the shapes that won a mix in full sweeps (one chunk per workgroup, one or two accesses in flight), and two persistent ones
STREAM_SWEEP_SHORT = tuple((t, u, 0, nt) for t in (256, 512, 1024) for u in (1, 2) for nt in (0, 3)) + ((256, 4, 16, 3), (512, 4, 32, 3))
STREAM_DEFAULT_POINT = (256, 4, 16, 3)  # what mx_ubench_stream runs


def measure_stream(dev, out_bytes: int = 1 << 29, iters: int = 10, sweep=STREAM_SWEEP_SHORT) -> dict:
    """Streaming bandwidth of this device in GB/s per traffic mix: read, copy, triad, the 2 : 1 mix of a 16-bit -> 8-bit
    cast (from one and from two input streams) and the 3 : 2 mix of the SwiGLU' quantizer.  Every mix is run under every
    launch shape of `sweep` (best of 3 launches each), then `iters` more launches of the best shape give best and
    median; `fixed_point` is the one shape mx_ubench_stream itself runs.  A ceiling is the best of the sweep: a product
    kernel that beats it says the sweep is too narrow."""
    import torch

    from kohakuwullm_amd import _lib

    lib = _lib.load()
    a = torch.empty(3 * out_bytes, dtype=torch.uint8, device=dev).random_(0, 255)  # kind 5 reads three streams
    b = torch.empty(out_bytes, dtype=torch.uint8, device=dev).random_(0, 255)
    c = torch.empty(2 * out_bytes, dtype=torch.uint8, device=dev)                  # ... and writes two
    st = torch.cuda.current_stream(dev).cuda_stream
    out = {}

    def timed(kind, shape, n):
        t, u, w, nt = shape
        return _event_times(lambda: _lib.check(lib.mx_ubench_stream_cfg(kind, t, u, w, nt, a.data_ptr(), b.data_ptr(), c.data_ptr(),
                                                                        out_bytes, st), "mx_ubench_stream_cfg"), n, warm=1)

    for name, kind, factor in STREAM_KINDS:
        moved = factor * out_bytes
        best_shape = min(sweep, key=lambda shape: timed(kind, shape, 3)[0])
        ts, fixed = timed(kind, best_shape, iters), timed(kind, STREAM_DEFAULT_POINT, 3)
        out[name] = {"best": round(moved / ts[0] / 1e6, 1), "median": round(moved / ts[len(ts) // 2] / 1e6, 1),
                     "shape": dict(zip(("threads", "unroll", "wgs_per_cu", "nontemporal"), best_shape)),
                     "fixed_point": round(moved / fixed[0] / 1e6, 1)}
    del a, b, c
    return out


def measure_tile_patterns(dev, iters: int = 12) -> dict:
    """Microseconds the access pattern of the 128 x 128 tile quantizers takes WITHOUT their arithmetic
    (mx_ubench_tile_pattern), at the shapes of the feed-forward step's three bandwidth kernels: the same bytes read
    from and written to the same places, on inputs that rotate through more than the last-level cache holds; best
    over the hint and layout choices.  A kernel cannot be faster than its own pattern."""
    import torch

    from kohakuwullm_amd import _lib

    lib = _lib.load()
    st = torch.cuda.current_stream(dev).cuda_stream
    sets = 3
    out = {}
    for entry, inputs, cols in (("mx_quantize_dual", 1, DIM), ("mx_swiglu_quantize_dual", 2, FFN), ("mx_swiglu_bwd_quantize_dual", 3, FFN)):
        width = cols * (2 if inputs >= 2 else 1)
        xs = [torch.empty(TOKENS, width, dtype=torch.bfloat16, device=dev).normal_() for _ in range(sets)]
        ys = [torch.empty(TOKENS, cols, dtype=torch.bfloat16, device=dev).normal_() for _ in range(sets)] if inputs == 3 else None
        outs = [[torch.empty(TOKENS * cols, dtype=torch.uint8, device=dev) for _ in range(4 if inputs == 3 else 2)] for _ in range(sets)]
        best = None
        for nt in (0, 1, 3):
            for panels in (0, 1):
                state = {"i": 0}

                def call():
                    i = state["i"] % sets
                    state["i"] += 1
                    o = outs[i]
                    _lib.check(lib.mx_ubench_tile_pattern(inputs, 1, nt, panels, xs[i].data_ptr(), width, ys[i].data_ptr() if ys else None,
                                                          TOKENS, cols, o[0].data_ptr(), o[1].data_ptr(),
                                                          o[2].data_ptr() if inputs == 3 else None, o[3].data_ptr() if inputs == 3 else None,
                                                          st), "mx_ubench_tile_pattern")

                ts = _event_times(call, iters, warm=sets)
                med = ts[len(ts) // 2] * 1e3
                if best is None or med < best["us_median"]:
                    best = {"us_median": round(med, 1), "nontemporal": nt, "stage_major": bool(panels),
                            "gbs": round(TOKENS * cols * (2 * inputs + (4 if inputs == 3 else 2)) / med / 1e3, 1)}
        out[entry] = best
        del xs, ys, outs
    return out


def measure_mfma(dev, iters: int = 4000, repeats: int = 5) -> dict:
    """Issue rate of the block-scaled fp8 MFMA from registers in TFLOP/s: both tile shapes, zero and hashed operands."""
    import torch

    from kohakuwullm_amd import _lib

    lib = _lib.load()
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    sink = torch.empty(cus * 512, dtype=torch.float32, device=dev)
    st = torch.cuda.current_stream(dev).cuda_stream
    out = {}
    for wide, shape, flop in ((0, "16x16x128", 2.0 * 16 * 16 * 128), (1, "32x32x64", 2.0 * 32 * 32 * 64),
                              (2, "16x16x128_one_wave_per_simd", 2.0 * 16 * 16 * 128),
                              (4, "16x16x128_scales_in_registers", 2.0 * 16 * 16 * 128),
                              (6, "16x16x128_scales_in_registers_one_wave_per_simd", 2.0 * 16 * 16 * 128)):
        for random, label in ((1, "hashed"), (0, "zeros")):
            count = []

            def launch():
                n = lib.mx_ubench_mfma(wide, iters, random, sink.data_ptr(), sink.numel(), st)
                if n < 0:
                    _lib.check(int(n), "mx_ubench_mfma")
                count.append(n)

            ts = _event_times(launch, repeats)
            out[f"{shape}_{label}"] = {"best": round(count[0] * flop / ts[0] / 1e9, 1),
                                       "median": round(count[0] * flop / ts[len(ts) // 2] / 1e9, 1)}
    return out


def measure_mfma_sustained(dev, iters: int = 4000, launches: int = 240, timed: int = 60) -> float:
    """TFLOP/s of the 16x16x128 MFMA loop on hashed operands once the clock has settled: `launches` launches back to
    back (about 0.1 s of MFMA work), one pair of events around the last `timed` of them."""
    import torch

    from kohakuwullm_amd import _lib

    lib = _lib.load()
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    sink = torch.empty(cus * 512, dtype=torch.float32, device=dev)
    st = torch.cuda.current_stream(dev).cuda_stream
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    n = 0
    for i in range(launches):
        if i == launches - timed:
            a.record()
        n = lib.mx_ubench_mfma(0, iters, 1, sink.data_ptr(), sink.numel(), st)
        if n < 0:
            _lib.check(int(n), "mx_ubench_mfma")
    b.record()
    torch.cuda.synchronize()
    return round(timed * n * 2.0 * 16 * 16 * 128 / a.elapsed_time(b) / 1e9, 1)


def measured_peaks(dev) -> dict:
    """The denominators measured on this device, beside the nominal ones: the best streaming pattern (GB/s) and the
    MFMA loop on hashed operands (TFLOP/s), in single launches from an idle clock and sustained; the kernels are
    priced against the larger of the two (zero operands clock higher still and are reported by --workload peak)."""
    stream, mfma = measure_stream(dev, iters=5), measure_mfma(dev, iters=2000, repeats=3)
    two_to_one = max(stream["read2_write1"]["best"], stream["read2_write1_two_streams"]["best"])
    short = max(v["best"] for k, v in mfma.items() if k.endswith("hashed"))
    sustained = measure_mfma_sustained(dev)
    return {
        "hbm_gbs": max(v["best"] for v in stream.values()),
        "hbm_read2_write1_gbs": two_to_one,
        "hbm_read3_write2_gbs": stream["read3_write2"]["best"],
        "hbm_copy_gbs": stream["copy"]["best"],
        "mfma_tflops": max(short, sustained),
        "mfma_tflops_single_launch": short,
        "mfma_tflops_sustained": sustained,
        "how": "mx_ubench_stream_cfg on 512 MiB per stream, every mix under 14 launch shapes (threads, loads in flight, grid, "
               "non-temporal hints), best launch of the best shape; mx_ubench_mfma from registers, best single launch and the "
               "last 60 of 240 back-to-back launches; all in this run",
    }

# Bytes the GEMM launches of one step move between the L2s and the fabric, per launch, from the
# FETCH_SIZE and WRITE_SIZE counter runs summarised under profiles/ (each scaled by what the
# counter reads for a device copy of known size): 2049 MiB over 4 launches.
GEMM_TRAFFIC_PER_LAUNCH = {"ffn": 512 * 2**20}
TRAFFIC_SOURCE = ("a constant, not measured in this run: the rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs summarised in "
                  "profiles/gemm_nt_kernel_dense_ffn_fwd_bwd.md")

GEMM_ENTRIES = ("mx_gemm_nt", "mx_gemm_nt_batch", "mx_grouped_gemm_nt", "mx_experts_gemm1", "mx_experts_scatter_gemm",
                "mx_experts_gemm2_dgrad", "mx_grouped_wgrad_nt")


def build_workload(name: str, dev, routing: str = "draws"):
    """Returns (step(i), gflop per step, description, refresh())."""
    import torch

    from kohakuwullm_amd.kernels.mxfp8.linear import MXFP8Linear
    from kohakuwullm_amd.kernels.mxfp8.mlp import mxfp8_swiglu_mlp
    from kohakuwullm_amd.kernels.mxfp8.moe import MXFP8ExpertWeights, mxfp8_moe_experts
    from kohakuwullm_amd.kernels.mxfp8.quantize import mxfp8_matmul_pq, quantize_mx, quantize_mx_cols

    ncopies = 4  # rotating activation copies: a step does not find its inputs in the 256 MB last-level cache
    if name == "ffn":
        x_h, w_in_h, w_out_h, dy_h = make_inputs(TOKENS)
        xs = [x_h.to(dev).requires_grad_(True) for _ in range(ncopies)]
        dys = [dy_h.to(dev) for _ in range(ncopies)]
        w_in = w_in_h.to(dev).requires_grad_(True)
        w_out = w_out_h.to(dev).requires_grad_(True)
        state = {}

        def refresh():
            state["packed"] = (quantize_mx(w_in.detach()), quantize_mx_cols(w_in.detach()),
                               quantize_mx(w_out.detach()), quantize_mx_cols(w_out.detach()))

        def step(i):
            x = xs[i % ncopies]
            mxfp8_swiglu_mlp(x, w_in, w_out, state["packed"]).backward(dys[i % ncopies])
            x.grad = w_in.grad = w_out.grad = None

        def sample_rows(n=64):
            """(row indices, the measured path's forward output on those rows) for the accuracy figure."""
            rows = torch.randperm(TOKENS, generator=torch.Generator().manual_seed(SEED))[:n]
            with torch.no_grad():
                y = mxfp8_swiglu_mlp(xs[0].detach(), w_in.detach(), w_out.detach(), state["packed"])
            return rows, y[rows.to(dev)].cpu()

        step.sample_rows = sample_rows
        desc = "dense 546M-class SwiGLU FFN fwd+bwd: tokens 16384, dim 1536, ffn 4096 (BASELINE configs[1])"
        return step, step_flops(TOKENS) / 1e9, desc, refresh
    if name == "attn":
        hid_h, w_qkv_h, w_o_h, d_qkv_h, d_o_h = make_attention_inputs()
        qkv = MXFP8Linear(w_qkv_h.shape[1], w_qkv_h.shape[0]).to(dev)
        proj = MXFP8Linear(w_o_h.shape[1], w_o_h.shape[0]).to(dev)
        with torch.no_grad():
            qkv.weight.copy_(w_qkv_h.to(dev))
            proj.weight.copy_(w_o_h.to(dev))
        xs = [hid_h.to(dev).requires_grad_(True) for _ in range(ncopies)]
        d_qkv, d_o = d_qkv_h.to(dev), d_o_h.to(dev)

        def refresh():
            qkv.refresh_quantized_weight()
            proj.refresh_quantized_weight()

        def step(i):
            # the attention core is not run: o_proj sees another activation of the same shape (its own
            # tensor, as in a block, so autograd has no second dX to add into the first)
            x, a = xs[i % ncopies], xs[(i + 2) % ncopies]
            qkv(x).backward(d_qkv)
            proj(a).backward(d_o)
            x.grad = a.grad = qkv.weight.grad = proj.weight.grad = None

        t, d = hid_h.shape
        gflop = 3 * (2.0 * t * w_qkv_h.shape[0] * d + 2.0 * t * d * d) / 1e9
        return step, gflop, "GQA attention projections fwd+dgrad+wgrad: tokens 32768, dim 2048, W_qkv 3072x2048, W_o 2048x2048 (BASELINE configs[2])", refresh
    if name == "moe":
        x_h, w_in_h, w_out_h, gate_h, dout_h, offsets, order, token_of, counts = make_moe_inputs(routing=routing)
        xs = [x_h.to(dev).requires_grad_(True) for _ in range(ncopies)]
        w_in, w_out = w_in_h.to(dev).requires_grad_(True), w_out_h.to(dev).requires_grad_(True)
        gate = gate_h.to(dev).requires_grad_(True)
        dout, offsets, order, token_of = dout_h.to(dev), offsets.to(dev), order.to(dev), token_of.to(dev)
        state = {}

        def refresh():
            state["packed"] = MXFP8ExpertWeights(w_in.detach(), w_out.detach())

        def step(i):
            x = xs[i % ncopies]
            mxfp8_moe_experts(x, w_in, w_out, gate, token_of, order, offsets, state["packed"]).backward(dout)
            x.grad = w_in.grad = w_out.grad = gate.grad = None

        m, dim, hid = int(sum(counts)), x_h.shape[1], w_out_h.shape[2]
        live = sum(1 for c in counts if c)
        how = "Zipf 1.1 draws" if routing == "draws" else "Zipf 1.1 by rank"
        return step, 3 * 6.0 * m * dim * hid / 1e9, (f"routed experts fwd+bwd: 64 experts ({how}: {live} with rows, {64 - live} empty, largest "
                                                     f"{max(counts)} rows), top-6, tokens 16384, dim 1024, hidden 512 (BASELINE configs[3])"), refresh
    if name == "outlier":
        x_h, w_h, dy_h, _ = make_outlier_inputs()
        x, w, dy = x_h.to(dev), w_h.to(dev), dy_h.to(dev)
        state = {}

        def refresh():
            state["w"] = quantize_mx(w)

        def step(i):
            xq, xs_ = quantize_mx(x)
            mxfp8_matmul_pq(xq, xs_, *state["w"])
            mxfp8_matmul_pq(*quantize_mx_cols(dy), *quantize_mx_cols(x))

        n = x_h.shape[0]
        return step, 2 * 2.0 * n**3 / 1e9, "outlier-stress 8192^3 GEMM, fwd + wgrad, quantizers included (BASELINE configs[4])", refresh
    if name == "norm":
        from kohakuwullm_amd.kernels.elementwise import rms_norm_mx

        g = torch.Generator().manual_seed(SEED)
        tokens, dim = 32768, 2048  # the hidden-state matrix of BASELINE configs[2]
        x_h = torch.randn(tokens, dim, generator=g).bfloat16()
        w_h = (1.0 + 0.1 * torch.randn(dim, generator=g)).bfloat16()
        dy_h = (torch.randn(tokens, dim, generator=g) * 1e-2).bfloat16()
        xs = [x_h.to(dev).requires_grad_(True) for _ in range(ncopies)]
        dys = [dy_h.to(dev) for _ in range(ncopies)]
        w = w_h.to(dev).requires_grad_(True)

        def step(i):
            x = xs[i % ncopies]
            out, q, s = rms_norm_mx(x, w, 1e-6)
            out.backward(dys[i % ncopies])
            x.grad = w.grad = None

        # beside the step: the norm as producer of BOTH operands of the linear layer behind it, against the launches it
        # replaces (norm with its 16-bit output and row-axis pair, then the column quantizer on that output)
        from kohakuwullm_amd.kernels.mxfp8.fused_act import rmsnorm_mx_dual
        from kohakuwullm_amd.kernels.mxfp8.quantize import quantize_mx_cols as cols

        def dual(i=[0]):
            i[0] += 1
            rmsnorm_mx_dual(xs[i[0] % ncopies].detach(), w.detach(), 1e-6)

        def unfused(i=[0]):
            i[0] += 1
            with torch.no_grad():
                out, q, s = rms_norm_mx(xs[i[0] % ncopies].detach(), w.detach(), 1e-6)
                cols(out)

        step.compare = {"rmsnorm_mx_dual": dual, "rms_norm_mx_then_quantize_mx_cols": unfused}
        return step, 0.0, "RMSNorm -> (bf16 out, MXFP8 pair) fwd + bwd on the 32768 x 2048 hidden states of BASELINE configs[2]", lambda: None
    if name == "dispatch":
        from kohakuwullm_amd.kernels.moe import combine_routed, expert_counts, expert_sort

        tokens, dim, experts, top_k = 16384, 1024, 64, 6  # the routing of BASELINE configs[3]
        _, _, _, gate_h, dout_h, offsets_h, order_h, _, _ = make_moe_inputs(tokens, dim, 512, experts, top_k)
        expert_of_position = torch.repeat_interleave(torch.arange(experts), (offsets_h[1:] - offsets_h[:-1]).long())
        flat_h = torch.empty(tokens * top_k, dtype=torch.int64)
        flat_h[order_h.long()] = expert_of_position  # the router's pick of every (token, slot) pair
        g = torch.Generator().manual_seed(SEED)
        rows_h = torch.randn(tokens * top_k, dim, generator=g).bfloat16()
        flat = flat_h.to(dev)
        rows = [rows_h.to(dev).requires_grad_(True) for _ in range(ncopies)]
        douts = [dout_h.to(dev) for _ in range(ncopies)]
        gate = gate_h.float().to(dev).requires_grad_(True)

        def step(i):
            r = rows[i % ncopies]
            offsets, order, token_of, _ = expert_sort(flat, expert_counts(flat, experts), top_k, experts)
            out = combine_routed(r, gate, order, token_of, tokens)
            out.backward(douts[i % ncopies])
            r.grad = gate.grad = None

        return step, 0.0, ("expert dispatch of BASELINE configs[3] (16384 tokens, top-6 of 64 experts, 1024 wide): "
                           "counts + sort + gated combine fwd + bwd"), lambda: None
    if name == "heads":
        from kohakuwullm_amd.kernels.mxfp8.attention_quant import column_mean, quantize_heads

        # q and k of the fused projection output of BASELINE configs[2]: 32768 tokens, 16 query and 4 KV heads of 128
        tokens, hq, hkv, d = 32768, 16, 4, 128
        g = torch.Generator().manual_seed(SEED)
        qkv_h = torch.randn(tokens, (hq + 2 * hkv) * d, generator=g).bfloat16()
        qkvs = [qkv_h.to(dev) for _ in range(ncopies)]
        mus = [column_mean(qkvs[0][:, lo : lo + n * d].view(tokens, n, d)) for lo, n in ((0, hq), (hq * d, hkv))]

        def step(i):
            qkv = qkvs[i % ncopies]
            quantize_heads(qkv[:, : hq * d].view(tokens, hq, d), mus[0])
            quantize_heads(qkv[:, hq * d : (hq + hkv) * d].view(tokens, hkv, d), mus[1])

        return step, 0.0, ("MXFP8 QK^T operands: q (16 heads) and k (4 heads) of 128 channels, 32768 tokens, read in place from the "
                           "fused projection output of BASELINE configs[2], per-channel mean subtracted, blocks along the head dimension"), lambda: None
    if name == "refresh":
        from kohakuwullm_amd.models.mlp import MXFP8SwiGLU
        from kohakuwullm_amd.models.mxfp8_swap import refresh_mxfp8_weights

        # every linear weight of a 546M-class dense model: 20 blocks of the feed-forward pair of
        # BASELINE configs[1] (dim 1536, ffn 4096) and GQA projections of the same width (12 query and
        # 4 KV heads of 128): 80 matrices, 503 M parameters
        dim, ffn, blocks = 1536, 4096, 20
        torch.manual_seed(SEED)
        model = torch.nn.ModuleList()
        for _ in range(blocks):
            model.append(MXFP8Linear(dim, dim + 2 * 512))
            model.append(MXFP8Linear(dim, dim))
            model.append(MXFP8SwiGLU(dim, hidden=ffn))
        model.to(dev)
        params = sum(p.numel() for p in model.parameters())

        def step(i):
            refresh_mxfp8_weights(model)

        def one_by_one():
            for module in model:
                module.refresh_quantized_weight()

        step.alternative = ("ms_per_step_one_module_at_a_time", one_by_one)
        return step, 0.0, (f"requantization of all {4 * blocks} linear weights ({params / 1e6:.0f} M parameters, bf16 masters) of a "
                           "546M-class dense model along both axes: refresh_mxfp8_weights, once per optimizer step"), lambda: None
    raise SystemExit(f"unknown workload {name!r}")


# metric and arithmetic type of the workloads that launch streaming kernels only
STREAM_METRICS = {
    "norm": ("RMSNorm -> MXFP8 producer fwd+bwd GB/s", "f32 arithmetic on bf16, fp64 sum of squares"),
    "dispatch": ("expert dispatch (counts, sort, combine fwd+bwd) GB/s", "int32 indices, f32 arithmetic on bf16 rows"),
    "heads": ("MXFP8 attention-operand quantizer GB/s", "bf16 - f32 mean -> e4m3 + ue8m0"),
    "refresh": ("MXFP8 weight requantization (row + column axis) GB/s", "bf16 -> e4m3 + ue8m0"),
}


QUANT_SHAPES = ((16384, 1536), (16384, 4096), (32768, 2048), (8192, 8192))  # activations of BASELINE configs[1], [1], [2], [4]


def _dequant(q, s):
    """fp32 values of an MXFP8 pair (codes (R, K), scale bytes (R, K/32)) with torch ops on the tensors' device."""
    import torch

    scale = torch.exp2(s.to(torch.float32) - 127.0).repeat_interleave(32, dim=1)
    return q.to(torch.float32) * scale


def _rel_error(got, want) -> float:
    """Relative Frobenius distance, accumulated in fp64 (the reference's accuracy figure, bench/core/timing.py:201-206)."""
    d = (got.double() - want.double()).norm()
    return float(d / want.double().norm())


def run_quant(dev, iters: int) -> dict:
    """The stand-alone quantizers (rows, columns, both) on the activation shapes, cold: every launch reads a copy of
    the input that left the 256 MB last-level cache several launches ago.  Per kernel and shape: algorithmic bytes
    (3.03125 B/element for one axis, 4.0625 for both) / device time from events around each launch."""
    import torch

    from kohakuwullm_amd.kernels.mxfp8.quantize import quantize_mx, quantize_mx_cols, quantize_mx_dual

    g = torch.Generator().manual_seed(SEED)
    rows_out, total_bytes, total_ms = [], 0.0, 0.0
    for m, k in QUANT_SHAPES:
        copies = max(3, -(-(768 << 20) // (m * k * 2)))  # at least 768 MB of distinct inputs in rotation
        base = torch.randn(m, k, generator=g).bfloat16()
        xs = [base.to(dev).add_(0) for _ in range(copies)]
        for name, fn, per_elem in (("rows", quantize_mx, 3.03125), ("cols", quantize_mx_cols, 3.03125),
                                   ("dual", quantize_mx_dual, 4.0625)):
            state = {"i": 0}

            def call():
                fn(xs[state["i"] % copies])
                state["i"] += 1

            ts = _event_times(call, iters, warm=copies)
            nbytes = m * k * per_elem
            med, best = ts[len(ts) // 2], ts[0]
            # accuracy in the same row: what the cast loses, dequantized on the device against the 16-bit input
            out = fn(xs[0])
            loss = _rel_error(_dequant(out[0], out[1]) if name != "cols" else _dequant(out[0], out[1]).t(), xs[0])
            del out
            rows_out.append({"kernel": f"quantize_mx_{name}", "shape": [m, k], "us_median": round(med * 1e3, 2),
                             "us_best": round(best * 1e3, 2), "gbs_median": round(nbytes / med / 1e6, 1),
                             "gbs_best": round(nbytes / best / 1e6, 1), "rel_error_of_cast": round(loss, 5)})
            total_bytes += nbytes * len(ts)
            total_ms += sum(ts)
        del xs
    return {"kernels": rows_out, "gbs": total_bytes / total_ms / 1e6, "launches": len(rows_out) * iters,
            "avg_us": total_ms / (len(rows_out) * iters) * 1e3}


GEMM_SHAPES = ((16384, 8192, 1536), (16384, 1536, 4096), (16384, 4096, 1536), (16384, 1536, 8192), (8192, 1536, 16384),
               (1536, 4096, 16384), (8192, 8192, 8192))  # the six products of BASELINE configs[1], and configs[4]'s
GEMM_VARIANTS = (("tile256_lockstep", 0), ("tile256_phased", 0x20), ("tile128_pair", 0x10),
                 ("tile256_wide_waves", 0x40))  # MX_EPI_PHASED, MX_EPI_TILE_128, MX_EPI_WIDE_WAVES


def run_gemm_variants(dev, iters: int) -> dict:
    """mx_gemm_nt alone on the benchmark's products, cold operands (rotating copies), in the shipped tiling/schedule and in
    the three alternatives of the variants library (csrc/mx_gemm_variants.h): same product bit for bit, timed against each other."""
    import torch

    from kohakuwullm_amd import _lib
    from kohakuwullm_amd.kernels.mxfp8.quantize import quantize_mx

    g = torch.Generator().manual_seed(SEED)
    rows = []
    for m, n, k in GEMM_SHAPES:
        copies = max(2, min(8, (600 << 20) // ((m + n) * k)))
        ops = []
        for _ in range(copies):
            a = torch.randn(m, k, generator=g).bfloat16().to(dev)
            b = (torch.randn(n, k, generator=g) * 0.02).bfloat16().to(dev)
            ops.append((*quantize_mx(a), *quantize_mx(b)))
            del a, b
        ws = _lib.gemm_workspace(ops[0][0])
        c = torch.empty(m, n, device=dev, dtype=torch.bfloat16)
        row = {"shape": [m, n, k]}
        first = None
        for name, flag in GEMM_VARIANTS:
            state = {"i": 0}

            def call():
                aq, sa, bq, sb = ops[state["i"] % copies]
                state["i"] += 1
                fn = (_lib.load_variants() if flag else _lib.load()).mx_gemm_nt
                _lib.check(fn(aq.data_ptr(), sa.data_ptr(), bq.data_ptr(), sb.data_ptr(), c.data_ptr(), 0, m, n, k, k, k // 32,
                              k, k // 32, n, flag, ws.data_ptr(), ws.numel(), _lib.stream_of(aq)), "mx_gemm_nt")

            ts = _event_times(call, iters, warm=copies)
            state["i"] = 0
            call()
            torch.cuda.synchronize()
            if first is None:
                first = c.clone()
                # accuracy in the same row: against torch's fp32 matmul of the dequantized operands, on the device
                aq, sa, bq, sb = ops[0]
                row["rel_error"] = round(_rel_error(first, _dequant(aq, sa) @ _dequant(bq, sb).t()), 6)
            row[name] = {"us_median": round(ts[len(ts) // 2] * 1e3, 1), "tflops_median": round(2.0 * m * n * k / ts[len(ts) // 2] / 1e9, 1),
                         "tflops_best": round(2.0 * m * n * k / ts[0] / 1e9, 1), "equal_to_shipped": bool(torch.equal(c, first))}
        row["vendor_library"] = _vendor_scaled_mm(ops, first, iters)
        rows.append(row)
        del ops
    return {"shapes": rows}


def _vendor_scaled_mm(ops, ours, iters: int) -> dict:
    """The same product through the vendor's GEMM library as PyTorch reaches it (torch._scaled_mm with one ue8m0 scale per 32
    of K in the natural (rows, K/32) layout), on the same rotating operands: a yardstick beside the shipped kernel, as the
    reference keeps its cuBLAS route beside its own kernel.  Nothing in the package calls it; a PyTorch build without the
    block-scaled form reports the error text instead of a time."""
    import torch

    e8 = getattr(torch, "float8_e8m0fnu", None)
    if e8 is None or not hasattr(torch, "_scaled_mm"):
        return {"error": "this PyTorch has no block-scaled _scaled_mm"}
    state = {"i": 0}
    out = {}

    def call():
        aq, sa, bq, sb = ops[state["i"] % len(ops)]
        state["i"] += 1
        out["c"] = torch._scaled_mm(aq, bq.t(), scale_a=sa.view(e8), scale_b=sb.view(e8), out_dtype=torch.bfloat16)

    try:
        ts = _event_times(call, iters, warm=len(ops))
        state["i"] = 0
        call()
        torch.cuda.synchronize()
    except Exception as ex:  # noqa: BLE001 - whatever the library or the binding refuses
        return {"error": f"{type(ex).__name__}: {str(ex)[:200]}"}
    m, k = ops[0][0].shape
    n = ops[0][2].shape[0]
    return {"us_median": round(ts[len(ts) // 2] * 1e3, 1), "tflops_median": round(2.0 * m * n * k / ts[len(ts) // 2] / 1e9, 1),
            "rel_error_to_shipped": round(_rel_error(out["c"], ours.float()), 6)}


def standalone_line(args, dev) -> dict:
    """--workload stream | peak | quant: one JSON line each, the same schema as the step workloads."""
    common = {"n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "higher_is_better": True, "scaling": "weak",
              "vs_baseline": None, "data": "synthetic"}
    if args.workload == "gemm":
        res = run_gemm_variants(dev, max(args.steps, 20))
        flops = sum(2.0 * m * n * k for m, n, k in GEMM_SHAPES)
        secs = sum(r["tile256_lockstep"]["us_median"] for r in res["shapes"]) * 1e-6
        peaks = measured_peaks(dev)
        val = flops / secs / 1e12
        return {"metric": "MXFP8 GEMM TFLOP/s (mx_gemm_nt alone, cold operands, shipped tiling)", "value": round(val, 1), "unit": "TFLOP/s",
                "ms_per_step": round(secs * 1e3, 4), "dtype": "e4m3 x e4m3, ue8m0 scales, fp32 accumulate, bf16 out", **common,
                "config": {"workload": "the six products of BASELINE configs[1] and the 8192^3 of configs[4], each alone; the shipped 256x256 "
                                       "lockstep kernel of the product library against the three kernels of the variants library and, as a yardstick, the "
                                       "vendor library's block-scaled GEMM as torch._scaled_mm reaches it", **res},
                "roofline": {"kernel": "gemm_nt_kernel", "bound": "mfma", "achieved": round(val, 1), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                             "frac": round(val / MFMA_PEAK_TFLOPS, 4), "traffic": None, "peak_measured": peaks["mfma_tflops"],
                             "frac_of_measured": round(val / peaks["mfma_tflops"], 4)}}
    if args.workload == "stream":
        bw = measure_stream(dev, iters=max(args.steps, 10), sweep=STREAM_SWEEP_FULL)
        best = max(v["best"] for v in bw.values())
        return {"metric": "device streaming bandwidth GB/s (best of read / copy / triad / 2:1 / 3:2 mixes)", "value": best, "unit": "GB/s",
                "ms_per_step": None, "dtype": "bytes", **common,
                "config": {"workload": f"512 MiB per stream, 16-byte accesses, every mix under {len(STREAM_SWEEP_FULL)} launch shapes "
                                       "(threads 256-1024, 2-8 accesses in flight, one chunk per workgroup or 8-32 workgroups per CU, "
                                       "temporal or non-temporal loads and stores): mx_ubench_stream_cfg", "patterns": bw},
                "roofline": {"kernel": "stream_kernel", "bound": "hbm", "achieved": best, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                             "frac": round(best / HBM_PEAK_GBS, 4), "traffic": None}}
    if args.workload == "peak":
        mf = measure_mfma(dev, repeats=max(args.steps // 4, 5))
        mf["16x16x128_hashed_sustained"] = measure_mfma_sustained(dev)
        best = max(mf["16x16x128_hashed_sustained"], *(v["best"] for k, v in mf.items() if k.endswith("hashed")))
        return {"metric": "block-scaled fp8 MFMA issue rate from registers TFLOP/s (hashed operands)", "value": best, "unit": "TFLOP/s",
                "ms_per_step": None, "dtype": "e4m3 x e4m3, ue8m0 scales, fp32 accumulate", **common,
                "config": {"workload": "8 waves per CU, 8 (16x16x128) or 4 (32x32x64) independent accumulator tiles per wave, "
                                       "4000 rounds, no memory traffic (mx_ubench_mfma)", "variants": mf},
                "roofline": {"kernel": "mfma_peak_kernel", "bound": "mfma", "achieved": best, "peak": MFMA_PEAK_TFLOPS,
                             "unit": "TFLOP/s", "frac": round(best / MFMA_PEAK_TFLOPS, 4), "traffic": None}}
    q = run_quant(dev, max(args.steps, 20))
    peaks = measured_peaks(dev)
    # every kernel against the best streaming rate measured for its own read : write mix (2 : 1 for one axis, 1 : 1 for both)
    for row in q["kernels"]:
        ceiling = peaks["hbm_copy_gbs"] if row["kernel"].endswith("dual") else peaks["hbm_read2_write1_gbs"]
        row["mix_ceiling_gbs"] = ceiling
        row["frac_of_mix_ceiling"] = round(row["gbs_median"] / ceiling, 4)
    return {"metric": "MXFP8 quantizer GB/s (rows, columns, both; activation shapes, cold inputs)", "value": round(q["gbs"], 1),
            "unit": "GB/s", "ms_per_step": None, "dtype": "bf16 -> e4m3 + ue8m0", **common,
            "config": {"workload": "quantize_mx / quantize_mx_cols / quantize_mx_dual on 16384x1536, 16384x4096, 32768x2048, "
                                   "8192x8192 bf16; inputs rotate through >= 768 MB of copies", "kernels": q["kernels"]},
            "roofline": {"kernel": "quant_rows_kernel, quant_cols_kernel<false>, quant_cols_kernel<true>", "bound": "hbm",
                         "achieved": round(q["gbs"], 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(q["gbs"] / HBM_PEAK_GBS, 4),
                         "traffic": None, "launches": q["launches"], "avg_launch_us": round(q["avg_us"], 2),
                         "peak_measured": peaks["hbm_gbs"], "frac_of_measured": round(q["gbs"] / peaks["hbm_gbs"], 4),
                         "peak_measured_read2_write1": peaks["hbm_read2_write1_gbs"]}}


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="ffn",
                    choices=("ffn", "attn", "moe", "outlier", "norm", "dispatch", "refresh", "heads", "quant", "gemm", "stream", "peak"),
                    help="ffn (default) is the configuration the headline metric is quoted on; quant: the stand-alone "
                         "quantizers; gemm: mx_gemm_nt alone in its three tilings/schedules; stream / peak: the device's "
                         "measured bandwidth and MFMA rate")
    ap.add_argument("--routing", default="draws", choices=("draws", "ranked"),
                    help="moe: per-expert loads drawn i.i.d. Zipf (six full experts with the fixed seed) or Zipf by rank (59 live experts)")
    ap.add_argument("--samples", type=int, default=100,
                    help="after the timed region, time this many further steps one by one (events around each) and report "
                         "their median and best beside the K-step mean (the reference's protocol, bench/core/timing.py:35-63: "
                         "100 or more samples, median and best); 0 switches it off")
    ap.add_argument("--settle-ms", type=float, default=150.0,
                    help="milliseconds of untimed steps between a first timed region (reported as ms_per_step_from_cold_start) "
                         "and the one the line's value comes from; 0: one timed region, straight after the warmup")
    ap.add_argument("--variants-library", action="store_true",
                    help="run the workload on libmxfp8_hip_variants.so instead of the product library: for moe, the two fused "
                         "expert kernels on 128 x 128 tiles with two workgroups per CU (measured slower; kept as evidence)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--breakdown", action="store_true",
                    help="also print the per-entry-point launch times of a step (the line's launch_breakdown) on stderr")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="after the timed region, run one device copy of 256 MiB: a kernel of known traffic "
                         "against which a counter run (FETCH_SIZE / WRITE_SIZE) is scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one MI355X: this path is built and run on a single GPU (--gpus 1)")

    import torch

    from kohakuwullm_amd import _lib

    dev = torch.device("cuda:0")
    if args.variants_library:
        _lib.variants_library().__enter__()  # for the rest of the process
    _lib.check(_lib.load().mx_device_supported(0), "mx_device_supported")
    if args.workload in ("quant", "gemm", "stream", "peak"):
        print(json.dumps(standalone_line(args, dev)))
        return
    step, gflop, desc, refresh = build_workload(args.workload, dev, args.routing)

    refresh()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(5):
        refresh()
    torch.cuda.synchronize()
    weight_refresh_ms = (time.perf_counter() - t0) / 5 * 1e3

    def timed_region():
        """W untimed warmup steps, then exactly K steps between two synchronizations; returns ms per step."""
        for i in range(args.warmup):
            step(i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(args.steps):
            step(i)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / args.steps * 1e3

    # A process's first steps run under a transient of the part's power management: the GEMM launches (not the
    # bandwidth kernels) take 15 % longer in steps 3-6 than they do from step ~30 on, falling all the while.  The
    # timed region is therefore run twice, before and after `--settle-ms` of the same steps untimed: the first
    # result is reported as it is (`ms_per_step_from_cold_start`), the second is the line's `ms_per_step` / `value`.
    cold_ms = timed_region() if args.settle_ms > 0 else None
    settle_steps = 0
    t_end = time.perf_counter() + args.settle_ms * 1e-3
    while args.settle_ms > 0 and time.perf_counter() < t_end:
        for i in range(10):
            step(settle_steps + i)
        torch.cuda.synchronize()
        settle_steps += 10
    ms_per_step = timed_region()
    tflops = gflop / ms_per_step
    settled = {} if cold_ms is None else {"ms_per_step_from_cold_start": round(cold_ms, 4), "settle_steps": settle_steps,
                                          "settle_ms": args.settle_ms}

    sampled = {}
    if args.samples > 0:
        counter = {"i": 0}

        def one():
            step(counter["i"])
            counter["i"] += 1

        ts = _event_times(one, args.samples, warm=0)
        sampled = {"ms_per_step_median": round(ts[len(ts) // 2], 4), "ms_per_step_best": round(ts[0], 4), "samples": len(ts)}
        if gflop:
            sampled["value_at_median"] = round(gflop / ts[len(ts) // 2], 2)
    sampled.update(settled)
    # device memory held at the high-water mark of the steps so far (inputs, weights, caches, one step's activations and
    # the K-split workspace of the GEMM wrappers), before the microbenchmarks below allocate their own buffers
    sampled["peak_memory_mib"] = round(torch.cuda.max_memory_allocated(dev) / 2**20, 1)

    if args.calibrate_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # Instrumented pass: the same steps with events around every kernel launch.
    _lib.TIMER = []
    for i in range(args.steps):
        step(i)
    torch.cuda.synchronize()
    records, _lib.TIMER = _lib.TIMER, None
    # per entry-point call of a step, in launch order: median device time over the steps and the rate it gives
    launches = []
    per_step = len(records) // args.steps if args.steps and len(records) % args.steps == 0 else 0
    for j in range(per_step):
        ts = sorted(records[i * per_step + j][2].elapsed_time(records[i * per_step + j][3]) for i in range(args.steps))
        name, work = records[j][0], records[j][1]
        rate = work / (ts[len(ts) // 2] * 1e-3)
        is_gemm = name in GEMM_ENTRIES
        launches.append({"entry": name, "us_median": round(ts[len(ts) // 2] * 1e3, 1), "us_best": round(ts[0] * 1e3, 1),
                         "rate_median": round(rate / (1e12 if is_gemm else 1e9), 1), "unit": "TFLOP/s" if is_gemm else "GB/s"})
        if args.breakdown:
            print(f"  {j:2d} {name:28s} median {ts[len(ts) // 2] * 1e3:8.1f} us   "
                  + (f"{rate / 1e12:7.1f} TFLOP/s" if is_gemm else f"{rate / 1e9:7.0f} GB/s"), file=sys.stderr)
    gemm = [(n, w, a.elapsed_time(b)) for n, w, a, b in records if n in GEMM_ENTRIES]
    quant = [(n, w, a.elapsed_time(b)) for n, w, a, b in records if n not in GEMM_ENTRIES]
    gemm_flops, gemm_ms = sum(w for _, w, _ in gemm), sum(t for _, _, t in gemm)
    quant_bytes, quant_ms = sum(w for _, w, _ in quant), sum(t for _, _, t in quant)
    quant_gbs = quant_bytes / (quant_ms * 1e-3) / 1e9
    if not gemm:
        # a workload of streaming kernels only: the figure of merit is bytes per second against HBM
        step_bytes = quant_bytes / args.steps
        stream_peak = max(v["best"] for v in measure_stream(dev, iters=5).values())
        extra = {}
        if hasattr(step, "alternative"):  # the same work done another way, timed the same way, for comparison
            key, other = step.alternative
            for _ in range(args.warmup):
                other()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                other()
            torch.cuda.synchronize()
            extra[key] = round((time.perf_counter() - t0) / args.steps * 1e3, 4)
        if hasattr(step, "compare"):  # named alternatives, each timed with events around every call: median microseconds
            extra["compare_us_median"] = {}
            for key, fn in step.compare.items():
                ts = _event_times(fn, max(args.steps, 20), warm=4)
                extra["compare_us_median"][key] = round(ts[len(ts) // 2] * 1e3, 1)
        print(json.dumps({
            "metric": STREAM_METRICS[args.workload][0], "value": round(step_bytes / (ms_per_step * 1e-3) / 1e9, 1),
            "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": STREAM_METRICS[args.workload][1],
            "data": "synthetic", "config": {"workload": desc, "bytes_per_step": int(step_bytes)},
            "roofline": {"kernel": ", ".join(sorted({n for n, _, _ in quant})), "bound": "hbm", "achieved": round(quant_gbs, 1),
                         "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(quant_gbs / HBM_PEAK_GBS, 4), "traffic": None,
                         "peak_measured": stream_peak, "frac_of_measured": round(quant_gbs / stream_peak, 4),
                         "launches": len(quant), "avg_launch_us": round(quant_ms / len(quant) * 1e3, 2)},
            **sampled, **extra, "launch_breakdown": launches,
        }))
        return
    gemm_tflops = gemm_flops / (gemm_ms * 1e-3) / 1e12
    peaks = measured_peaks(dev)
    # every bandwidth launch against the best streaming rate measured for its own read : write mix
    mix_of = {"mx_quantize_dual": "hbm_copy_gbs", "mx_swiglu_bwd_quantize_dual": "hbm_read3_write2_gbs"}
    patterns = measure_tile_patterns(dev) if args.workload == "ffn" else {}
    for row in launches:
        if row["unit"] == "GB/s":
            row["mix_ceiling"] = peaks[mix_of.get(row["entry"], "hbm_read2_write1_gbs")]
            row["frac_of_mix_ceiling"] = round(row["rate_median"] / row["mix_ceiling"], 4)
            if row["entry"] in patterns:  # the kernel's own access pattern without arithmetic: a tighter bound
                row["access_pattern_us"] = patterns[row["entry"]]["us_median"]
                row["frac_of_access_pattern"] = round(row["access_pattern_us"] / row["us_median"], 4)

    out = {
        "metric": "MXFP8 linear fwd+bwd TFLOP/s (quantizers included)",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        **sampled,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "mxfp8 (e4m3 x e4m3 with ue8m0 per-32 scales, fp32 accumulate, bf16 out)",
        "data": "synthetic",
        "config": {
            "workload": desc,
            "gflop_per_step": round(gflop, 1),
            "products": "fwd, dgrad and wgrad all in MXFP8 (wgrad on token-axis blocks)",
        },
        "frac_of_mfma_peak": round(tflops / MFMA_PEAK_TFLOPS, 4),
        "roofline": {
            "kernel": "block-scaled MFMA GEMM kernels (" + ", ".join(sorted({n for n, _, _ in gemm})) + ")",
            "bound": "mfma",
            "achieved": round(gemm_tflops, 2),
            "peak": MFMA_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(gemm_tflops / MFMA_PEAK_TFLOPS, 4),
            "traffic": GEMM_TRAFFIC_PER_LAUNCH.get(args.workload),
            "traffic_source": TRAFFIC_SOURCE if args.workload in GEMM_TRAFFIC_PER_LAUNCH else None,
            "peak_measured": peaks["mfma_tflops"],
            "frac_of_measured": round(gemm_tflops / peaks["mfma_tflops"], 4),
            "launches": len(gemm),
            "avg_launch_us": round(gemm_ms / len(gemm) * 1e3, 2),
            "gflop_per_launch": round(gemm_flops / len(gemm) / 1e9, 2),
        },
        "quantizer": {
            "kernels": ", ".join(sorted({n for n, _, _ in quant})),
            "bound": "hbm",
            "achieved": round(quant_gbs, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(quant_gbs / HBM_PEAK_GBS, 4),
            "peak_measured": peaks["hbm_gbs"],
            "frac_of_measured": round(quant_gbs / peaks["hbm_gbs"], 4),
            "launches": len(quant),
            "avg_launch_us": round(quant_ms / len(quant) * 1e3, 2),
            "share_of_step": round(quant_ms / (quant_ms + gemm_ms), 4),
        },
        "peaks_measured": peaks,
        "tile_access_patterns": patterns,
        "weight_refresh_ms": round(weight_refresh_ms, 4),
        "launch_breakdown": launches,
    }
    if not args.no_cpu_baseline and args.workload == "ffn":
        out["cpu_baseline"] = cpu_baseline(device_rows=step.sample_rows())
    print(json.dumps(out))


if __name__ == "__main__":
    main()
