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


def cpu_baseline(sample_tokens: int = TOKENS) -> dict:
    """The oracle's formulas with PyTorch CPU ops on the first `sample_tokens` tokens."""
    import torch

    from oracle import mx_oracle as ora

    x, w_in, w_out, dy = make_inputs(TOKENS)
    x, dy = x[:sample_tokens].contiguous(), dy[:sample_tokens].contiguous()
    f32 = torch.float32

    def q_rows(t):
        return ora.quantize_rows_torch(t)

    def q_cols(t):
        return ora.quantize_rows_torch(t.t().contiguous())

    t0 = time.perf_counter()
    win_f, win_d, wout_f, wout_d = q_rows(w_in), q_cols(w_in), q_rows(w_out), q_cols(w_out)
    t_weights = time.perf_counter() - t0
    t0 = time.perf_counter()
    xq, xt = q_rows(x), q_cols(x)
    gu = ora.gemm_nt(*xq, *win_f, dtype=f32).bfloat16()
    g, u = gu.float().chunk(2, dim=-1)
    h = g * torch.sigmoid(g) * u
    hq, ht = q_rows(h), q_cols(h)
    y = ora.gemm_nt(*hq, *wout_f, dtype=f32).bfloat16()
    dq, dt = q_rows(dy), q_cols(dy)
    dh = ora.gemm_nt(*dq, *wout_d, dtype=f32).bfloat16().float()
    sg = torch.sigmoid(g)
    dpre = torch.cat([dh * u * sg * (1 + g * (1 - sg)), dh * g * sg], dim=-1)
    pq, pt = q_rows(dpre), q_cols(dpre)
    dx = ora.gemm_nt(*pq, *win_d, dtype=f32).bfloat16()
    dw_in = ora.gemm_nt(*pt, *xt, dtype=f32).bfloat16()
    dw_out = ora.gemm_nt(*dt, *ht, dtype=f32).bfloat16()
    dt_step = time.perf_counter() - t0
    del y, dx, dw_in, dw_out
    return {
        "value": step_flops(sample_tokens) / dt_step / 1e12,
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"{sample_tokens} of {TOKENS} tokens of the same workload, one step, all six products "
        f"(fp32 torch.matmul on dequantized operands) and all quantizers (torch statement); "
        f"{dt_step:.2f} s; weights quantized outside ({t_weights:.2f} s); host cpu_count={os.cpu_count()}",
    }


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one MI355X: this path is built and run on a single GPU (--gpus 1)")

    import torch

    from kohakuwullm_amd import _lib
    from kohakuwullm_amd.kernels.mxfp8.mlp import mxfp8_swiglu_mlp
    from kohakuwullm_amd.kernels.mxfp8.quantize import quantize_mx, quantize_mx_cols

    dev = torch.device("cuda:0")
    _lib.check(_lib.load().mx_device_supported(0), "mx_device_supported")
    x_h, w_in_h, w_out_h, dy_h = make_inputs(TOKENS)
    # Several copies of the activations so consecutive steps do not find their inputs in the
    # 256 MB last-level cache.
    ncopies = 4
    xs = [x_h.to(dev).requires_grad_(True) for _ in range(ncopies)]
    dys = [dy_h.to(dev) for _ in range(ncopies)]
    w_in = w_in_h.to(dev).requires_grad_(True)
    w_out = w_out_h.to(dev).requires_grad_(True)

    def refresh():
        return (quantize_mx(w_in.detach()), quantize_mx_cols(w_in.detach()),
                quantize_mx(w_out.detach()), quantize_mx_cols(w_out.detach()))

    packed = refresh()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(10):
        packed = refresh()
    torch.cuda.synchronize()
    weight_refresh_ms = (time.perf_counter() - t0) / 10 * 1e3

    def step(i: int) -> None:
        x = xs[i % ncopies]
        y = mxfp8_swiglu_mlp(x, w_in, w_out, packed)
        y.backward(dys[i % ncopies])
        x.grad = None
        w_in.grad = None
        w_out.grad = None

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(i)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    tflops = step_flops(TOKENS) / (ms_per_step * 1e-3) / 1e12

    # Instrumented pass: the same steps with events around every kernel launch.
    _lib.TIMER = []
    for i in range(args.steps):
        step(i)
    torch.cuda.synchronize()
    records, _lib.TIMER = _lib.TIMER, None
    gemm = [(w, a.elapsed_time(b)) for n, w, a, b in records if n == "mx_gemm_nt"]
    quant = [(w, a.elapsed_time(b)) for n, w, a, b in records if n != "mx_gemm_nt"]
    gemm_flops, gemm_ms = sum(w for w, _ in gemm), sum(t for _, t in gemm)
    quant_bytes, quant_ms = sum(w for w, _ in quant), sum(t for _, t in quant)
    gemm_tflops = gemm_flops / (gemm_ms * 1e-3) / 1e12
    quant_gbs = quant_bytes / (quant_ms * 1e-3) / 1e9

    out = {
        "metric": "MXFP8 linear fwd+bwd TFLOP/s (dense SwiGLU FFN, quantizers included)",
        "value": round(tflops, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "mxfp8 (e4m3 x e4m3 with ue8m0 per-32 scales, fp32 accumulate, bf16 out)",
        "data": "synthetic",
        "config": {
            "workload": "dense 546M-class SwiGLU FFN fwd+bwd: tokens 16384, dim 1536, ffn 4096 (BASELINE configs[1])",
            "gflop_per_step": round(step_flops(TOKENS) / 1e9, 1),
            "products": "fwd 2, dgrad 2, wgrad 2 (all MXFP8, wgrad on token-axis blocks)",
        },
        "frac_of_mfma_peak": round(tflops / MFMA_PEAK_TFLOPS, 4),
        "roofline": {
            "kernel": "gemm_nt_kernel (mx_gemm_nt)",
            "bound": "mfma",
            "achieved": round(gemm_tflops, 2),
            "peak": MFMA_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(gemm_tflops / MFMA_PEAK_TFLOPS, 4),
            "traffic": None,
            "launches": len(gemm),
            "avg_launch_us": round(gemm_ms / len(gemm) * 1e3, 2),
            "gflop_per_launch": round(gemm_flops / len(gemm) / 1e9, 2),
        },
        "quantizer": {
            "kernels": "mx_quantize_dual, mx_swiglu_quantize_dual, mx_swiglu_bwd_quantize_dual",
            "bound": "hbm",
            "achieved": round(quant_gbs, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(quant_gbs / HBM_PEAK_GBS, 4),
            "launches": len(quant),
            "avg_launch_us": round(quant_ms / len(quant) * 1e3, 2),
            "share_of_step": round(quant_ms / (quant_ms + gemm_ms), 4),
        },
        "weight_refresh_ms": round(weight_refresh_ms, 4),
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
