"""The benchmark configurations at their full sizes: dense feed-forward, attention projections, routed experts, outlier stress.

The CPU oracle cannot redo a whole 8192^3 product in seconds, so each case checks
  * quantizers bit for bit on the whole tensor (the C oracle quantizes 67M elements in about a second),
  * GEMM outputs on sampled rows (forward, dgrad) and sampled columns (wgrad) against the fp64 oracle,
  * size-independent properties: a fused QKV product equals its three slices bit for bit, empty
    experts get exactly zero weight gradients, a problem restricted to a token subset or to whole
    32-blocks of hidden channels reproduces the matching slices of the full problem.
Inputs come from bench.py's generators so the tested data is the measured data.
"""

import sys
from pathlib import Path

import pytest
import torch

sys.path.insert(0, str(Path(__file__).resolve().parent.parent))

import bench  # noqa: E402
from conftest import SEED  # noqa: E402
from mx_checks import assert_codes_equal_up_to_ties  # noqa: E402
from test_gpu_moe import _expert_oracle  # noqa: E402

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL = 1e-2
F8 = torch.float8_e4m3fn


def _u8(t):
    return t.view(torch.uint8).cpu()


# ----------------------------------------------------------------------------- dense SwiGLU feed-forward


def test_dense_ffn_full_size(oracle):
    """The benchmarked step (tokens 16384, dim 1536, ffn 4096) through ``mxfp8_swiglu_mlp``, on the benchmark's data.

    The fused function is first shown equal, bit for bit, to its launches issued one by one (which exposes
    the intermediates: the launch plan is the measured one, stage-major operands, the three backward products
    in one batched launch).  Then every stage is held to the oracle on samples: quantizers on the whole
    tensors, GEMM rows and columns against the fp64 dequantize-then-matmul on the operands the device used,
    the SwiGLU casts against the oracle's evaluation up to rounding ties.
    """
    from kohakuwullm_amd.kernels.mxfp8.mlp import mxfp8_swiglu_mlp, swiglu_bwd_mx_dual, swiglu_mx_dual
    from kohakuwullm_amd.kernels.mxfp8.quantize import (
        mxfp8_matmul_pq, mxfp8_matmul_pq_batch, quantize_mx, quantize_mx_cols, quantize_mx_dual, rows_of_stage_major)

    x, w_in, w_out, dy = bench.make_inputs(bench.TOKENS)
    tokens, dim = x.shape
    hid = w_out.shape[1]
    xd, wi, wo = (t.to(DEV).requires_grad_(True) for t in (x, w_in, w_out))
    dyd = dy.to(DEV)
    packed = (quantize_mx(wi.detach()), quantize_mx_cols(wi.detach()), quantize_mx(wo.detach()), quantize_mx_cols(wo.detach()))
    y = mxfp8_swiglu_mlp(xd, wi, wo, packed)
    y.backward(dyd)
    y, dx, dw_in, dw_out = y.detach(), xd.grad, wi.grad, wo.grad

    # the same launches one by one
    xq, xs, xtq, xts = quantize_mx_dual(xd.detach(), stage_major_t=True)
    gu = mxfp8_matmul_pq(xq, xs, *packed[0])
    hq, hs, htq, hts = swiglu_mx_dual(gu, stage_major_t=True)
    assert torch.equal(mxfp8_matmul_pq(hq, hs, *packed[2]), y)
    dq, ds, dtq, dts = quantize_mx_dual(dyd, stage_major_t=True)
    dh = mxfp8_matmul_pq(dq, ds, *packed[3])
    pq, ps, ptq, pts = swiglu_bwd_mx_dual(dh, gu, stage_major=True)
    products = [(pq, ps, *packed[1]), (ptq, pts, xtq, xts), (dtq, dts, htq, hts)]
    together = mxfp8_matmul_pq_batch(products)
    for got, want in zip(together, (dx, dw_in, dw_out)):
        assert torch.equal(got, want)
    # the batched launch against each product launched alone: the same fp32 sums up to the order of their
    # K pieces, then one bf16 rounding
    for got, prob in zip(together, products):
        alone = mxfp8_matmul_pq(*prob)
        assert oracle.rel_error(got.cpu(), alone.double().cpu()) < 2e-3

    # quantizers, whole tensors, bit for bit (stage-major codes read back as rows)
    for t, (q, s, qt, st) in ((x, (xq, xs, xtq, xts)), (dy, (dq, ds, dtq, dts))):
        rq, rs = oracle.quantize_rows(t)
        cq, cs = oracle.quantize_cols(t)
        assert torch.equal(_u8(q), rq) and torch.equal(s.cpu(), rs)
        assert torch.equal(_u8(rows_of_stage_major(qt)), cq) and torch.equal(st.cpu(), cs)
    win_f, win_d = oracle.quantize_rows(w_in), oracle.quantize_cols(w_in)
    wout_f, wout_d = oracle.quantize_rows(w_out), oracle.quantize_cols(w_out)
    for dev_pair, ref_pair in zip(packed, (win_f, win_d, wout_f, wout_d)):
        assert torch.equal(_u8(dev_pair[0]), ref_pair[0]) and torch.equal(dev_pair[1].cpu(), ref_pair[1])

    g = torch.Generator().manual_seed(SEED)
    rows = torch.randperm(tokens, generator=g)[:192].sort().values
    rd = rows.to(DEV)
    # forward, sampled token rows
    gu_rows = gu[rd].cpu()
    assert oracle.rel_error(gu_rows, oracle.gemm_nt(_u8(xq[rd]), xs[rd].cpu(), *win_f)) < TOL
    gate, up = gu_rows.float().chunk(2, dim=-1)
    h_rows = gate * torch.sigmoid(gate) * up
    ties = assert_codes_equal_up_to_ties(oracle, hq[rd], hs[rd], h_rows, what="h along H")
    assert ties[0] < 5e-3 * h_rows.numel()
    assert oracle.rel_error(y[rd].cpu(), oracle.gemm_nt(_u8(hq[rd]), hs[rd].cpu(), *wout_f)) < TOL
    # backward, the same rows
    dh_rows = dh[rd].cpu()
    assert oracle.rel_error(dh_rows, oracle.gemm_nt(_u8(dq[rd]), ds[rd].cpu(), *wout_d)) < TOL
    sg = torch.sigmoid(gate)
    dpre_rows = torch.cat([dh_rows.float() * up * sg * (1 + gate * (1 - sg)), dh_rows.float() * gate * sg], dim=-1)
    pq_rows = rows_of_stage_major(pq[:, rd])
    terms = torch.cat([(dh_rows.float() * up * sg).abs() * (1 + gate.abs() * (1 - sg)), (dh_rows.float() * gate * sg).abs()], dim=-1)
    ties = assert_codes_equal_up_to_ties(oracle, pq_rows, ps[rd], dpre_rows, ulps=8, what="dpre along 2H", magnitude=terms)
    assert ties[0] < 5e-3 * dpre_rows.numel()
    assert oracle.rel_error(dx[rd].cpu(), oracle.gemm_nt(_u8(pq_rows), ps[rd].cpu(), *win_d)) < TOL

    # token-axis casts of h and dpre: four sampled panels of 128 tokens, every channel
    for panel in torch.randperm(tokens // 128, generator=g)[:4].tolist():
        tok = slice(panel * 128, panel * 128 + 128)
        gate, up = gu[tok].cpu().float().chunk(2, dim=-1)
        sg = torch.sigmoid(gate)
        h_t = (gate * sg * up).t().contiguous()
        assert_codes_equal_up_to_ties(oracle, htq[panel], hts[:, panel * 4 : panel * 4 + 4], h_t, what="h along tokens")
        dh_p = dh[tok].cpu().float()
        dpre_t = torch.cat([dh_p * up * sg * (1 + gate * (1 - sg)), dh_p * gate * sg], dim=-1).t().contiguous()
        terms = torch.cat([(dh_p * up * sg).abs() * (1 + gate.abs() * (1 - sg)), (dh_p * gate * sg).abs()], dim=-1).t().contiguous()
        assert_codes_equal_up_to_ties(oracle, ptq[panel], pts[:, panel * 4 : panel * 4 + 4], dpre_t, ulps=8, what="dpre along tokens",
                                      magnitude=terms)

    # weight gradients: sampled output rows against all input channels, and sampled input channels against
    # all output rows, contracting all 16384 tokens on the device's own token-axis operands
    xt_cpu, ht_cpu = (_u8(rows_of_stage_major(xtq)), xts.cpu()), (_u8(rows_of_stage_major(htq)), hts.cpu())
    pt_cpu, dt_cpu = (_u8(rows_of_stage_major(ptq)), pts.cpu()), (_u8(rows_of_stage_major(dtq)), dts.cpu())
    for dw, a, b in ((dw_in, pt_cpu, xt_cpu), (dw_out, dt_cpu, ht_cpu)):
        pick = torch.randperm(a[0].shape[0], generator=g)[:48].sort().values
        assert oracle.rel_error(dw[pick.to(DEV)].cpu(), oracle.gemm_nt(a[0][pick], a[1][pick], *b)) < TOL
        pick = torch.randperm(b[0].shape[0], generator=g)[:32].sort().values
        assert oracle.rel_error(dw[:, pick.to(DEV)].cpu(), oracle.gemm_nt(*a, b[0][pick], b[1][pick])) < TOL
    assert hid * 2 == w_in.shape[0] and dw_in.shape == w_in.shape and dw_out.shape == w_out.shape


# ----------------------------------------------------------------------------- attention projections


@pytest.fixture(scope="module")
def attn():
    return bench.make_attention_inputs()


def test_attention_fused_qkv_equals_slices(oracle, attn):
    from kohakuwullm_amd.kernels.mxfp8.linear import MXFP8Linear

    hid, w_qkv, w_o, d_qkv, _ = attn
    tokens, dim = hid.shape
    n_q, n_kv = 2048, 512
    fused = MXFP8Linear(dim, w_qkv.shape[0]).to(DEV)
    with torch.no_grad():
        fused.weight.copy_(w_qkv.to(DEV))
    x = hid.to(DEV).requires_grad_(True)
    y = fused(x)
    y.backward(d_qkv.to(DEV))
    bounds = [(0, n_q), (n_q, n_q + n_kv), (n_q + n_kv, n_q + 2 * n_kv)]
    dx_sum = torch.zeros(tokens, dim, dtype=torch.float32, device=DEV)
    for lo, hi in bounds:
        part = MXFP8Linear(dim, hi - lo).to(DEV)
        with torch.no_grad():
            part.weight.copy_(w_qkv[lo:hi].to(DEV))
        xp = hid.to(DEV).requires_grad_(True)
        yp = part(xp)
        # every output element contracts the same K sequence in the same order: identical bits
        assert torch.equal(yp, y[:, lo:hi])
        yp.backward(d_qkv[:, lo:hi].to(DEV))
        # dW may be cut into a different number of K slices per launch plan: the same fp32 sum up to
        # its order, then one bf16 rounding
        assert oracle.rel_error(part.weight.grad.cpu(), fused.weight.grad[lo:hi].double().cpu()) < 2e-3
        dx_sum += xp.grad.float()
    # dX of the fused product contracts all 3072 output features at once; the three partial
    # dgrads are rounded to bf16 separately, so this one is a norm comparison
    assert oracle.rel_error(x.grad.float().cpu(), dx_sum.cpu()) < TOL


def test_attention_projections_sampled_oracle(oracle, attn):
    from kohakuwullm_amd.kernels.mxfp8.linear import MXFP8Linear

    hid, w_qkv, w_o, d_qkv, d_o = attn
    g = torch.Generator().manual_seed(SEED)
    rows = torch.randperm(hid.shape[0], generator=g)[:256]
    xq, xs = oracle.quantize_rows(hid)
    xtq, xts = oracle.quantize_cols(hid)
    for w, dy in ((w_qkv, d_qkv), (w_o, d_o)):
        lin = MXFP8Linear(w.shape[1], w.shape[0]).to(DEV)
        with torch.no_grad():
            lin.weight.copy_(w.to(DEV))
        x = hid.to(DEV).requires_grad_(True)
        y = lin(x)
        y.backward(dy.to(DEV))
        wq, ws = oracle.quantize_rows(w)
        assert oracle.rel_error(y[rows.to(DEV)].cpu(), oracle.gemm_nt(xq[rows], xs[rows], wq, ws)) < TOL
        dq, ds = oracle.quantize_rows(dy[rows].contiguous())
        wtq, wts = oracle.quantize_cols(w)
        assert oracle.rel_error(x.grad[rows.to(DEV)].cpu(), oracle.gemm_nt(dq, ds, wtq, wts)) < TOL
        feat = torch.randperm(w.shape[0], generator=g)[:64]
        dtq, dts = oracle.quantize_cols(dy[:, feat].contiguous())
        assert oracle.rel_error(lin.weight.grad[feat.to(DEV)].cpu(), oracle.gemm_nt(dtq, dts, xtq, xts)) < TOL


# ----------------------------------------------------------------------------- routed experts


def _moe_problem(kind):
    return bench.make_moe_inputs(routing="ranked" if kind == "ranked" else "draws")


@pytest.mark.parametrize("kind", ["zipf_draws", "ranked"])
def test_experts_full_size(oracle, kind):
    from kohakuwullm_amd.kernels.mxfp8.moe import MXFP8ExpertWeights, mxfp8_moe_experts

    x, w_in, w_out, gate, dout, offsets, order, token_of, counts = _moe_problem(kind)
    tokens, dim = x.shape
    hid = w_out.shape[2]
    top_k = gate.numel() // tokens
    assert sum(counts) == tokens * top_k and min(counts) == 0 and max(counts) <= tokens
    xd, wi, wo, gd = (t.to(DEV).requires_grad_(True) for t in (x, w_in, w_out, gate))
    packed = MXFP8ExpertWeights(wi.detach(), wo.detach())
    out = mxfp8_moe_experts(xd, wi, wo, gd, token_of.to(DEV), order.to(DEV), offsets.to(DEV), packed)
    out.backward(dout.to(DEV))
    out, dx, dw_in, dw_out, dgate = out.detach().cpu(), xd.grad.cpu(), wi.grad.cpu(), wo.grad.cpu(), gd.grad.cpu()
    for e, c in enumerate(counts):
        if c == 0:
            assert not dw_in[e].any() and not dw_out[e].any()
    assert torch.isfinite(out.float()).all() and torch.isfinite(dx.float()).all()

    # (1) token subset: out, dx and dgate of a token depend on that token's routed rows only
    g = torch.Generator().manual_seed(SEED)
    keep = torch.zeros(tokens, dtype=torch.bool)
    keep[torch.randperm(tokens, generator=g)[:384]] = True
    sel = keep[token_of.long()]
    new_id = torch.cumsum(keep, 0) - 1
    sub_counts = [int(sel[offsets[e] : offsets[e + 1]].sum()) for e in range(len(counts))]
    sub_off = torch.zeros(len(counts) + 1, dtype=torch.int32)
    sub_off[1:] = torch.tensor(sub_counts).cumsum(0)
    sub_tok = new_id[token_of.long()[sel]].int()
    sub_order = (sub_tok.long() * top_k + order.long()[sel] % top_k).int()
    sub_gate = gate.view(tokens, top_k)[keep].reshape(-1)
    ref = _expert_oracle(oracle, x[keep], w_in, w_out, sub_gate, sub_tok, sub_order, sub_off, dout[keep])
    assert oracle.rel_error(out[keep], ref["out"]) < TOL
    assert oracle.rel_error(dx[keep], ref["dx"]) < TOL
    assert oracle.rel_error(dgate.view(tokens, top_k)[keep].reshape(-1), ref["dgate"]) < TOL

    # (2) two whole 32-blocks of hidden channels: the weight-gradient slices that touch them
    blocks = torch.randperm(hid // 32, generator=g)[:2].sort().values
    ch = (blocks[:, None] * 32 + torch.arange(32)).reshape(-1)
    ch2 = torch.cat([ch, hid + ch])
    ref = _expert_oracle(oracle, x, w_in[:, ch2].contiguous(), w_out[:, :, ch].contiguous(), gate, token_of, order,
                         offsets, dout)
    live = [e for e, c in enumerate(counts) if c > 0]
    probe = live if len(live) <= 8 else [live[i] for i in torch.randperm(len(live), generator=g)[:8].tolist()]
    # experts with a handful of rows have tiny gradients whose error is all in the last e4m3 bit
    for e in probe:
        tol = TOL if counts[e] >= 32 else 0.05
        assert oracle.rel_error(dw_in[e][ch2], ref["dw_in"][e]) < tol, (e, counts[e])
        assert oracle.rel_error(dw_out[e][:, ch], ref["dw_out"][e]) < tol, (e, counts[e])


# ----------------------------------------------------------------------------- outlier stress


@pytest.fixture(scope="module")
def outlier():
    return bench.make_outlier_inputs()


def test_outlier_quantizers_bit_exact(oracle, outlier):
    from kohakuwullm_amd.kernels.mxfp8.quantize import quantize_mx, quantize_mx_cols, quantize_mx_dual

    x, _, _, special = outlier
    n = x.shape[0]
    rq, rs = oracle.quantize_rows(x)
    q, s = quantize_mx(x.to(DEV))
    assert torch.equal(_u8(q), rq) and torch.equal(s.cpu(), rs)
    cq, cs = oracle.quantize_cols(x)
    qt, st = quantize_mx_cols(x.to(DEV))
    assert torch.equal(_u8(qt), cq) and torch.equal(st.cpu(), cs)
    q2, s2, qt2, st2 = quantize_mx_dual(x.to(DEV))
    assert torch.equal(_u8(q2), rq) and torch.equal(s2.cpu(), rs) and torch.equal(_u8(qt2), cq) and torch.equal(st2.cpu(), cs)
    # the injected blocks hit the special cases they were made for
    flat_s, flat_q = rs.view(-1), rq.view(n * n // 32, 32)
    assert (flat_s[special["zero"]] == 19).all() and not flat_q[special["zero"]].any()
    assert (flat_s[special["tiny"]] == 19).all()
    assert (flat_s[special["big"]] == 247).all()  # 3e38 = 1.41 * 2^127 -> 127 - 8 + 127 + 1
    tie = flat_q[special["tie"]]
    assert (tie[:, 7] == 0x7E).all()  # amax / 2^(e-8) == 448 exactly: the top code, not past it
    assert ((rq & 0x7F) != 0x7F).all() and ((cq & 0x7F) != 0x7F).all()  # no NaN code anywhere


def test_outlier_gemm_sampled(oracle, outlier):
    from kohakuwullm_amd.kernels.mxfp8.quantize import mxfp8_matmul_pq, quantize_mx, quantize_mx_cols

    x, w, dy, special = outlier
    n = x.shape[0]
    g = torch.Generator().manual_seed(SEED)
    xq, xs = quantize_mx(x.to(DEV))
    wq, ws = quantize_mx(w.to(DEV))
    y = mxfp8_matmul_pq(xq, xs, wq, ws)
    assert torch.isfinite(y.float()).all()
    big_rows = torch.unique(special["big"] // (n // 32))
    typical = torch.ones(n, dtype=torch.bool)
    typical[big_rows] = False
    rows = torch.cat([typical.nonzero().flatten()[torch.randperm(int(typical.sum()), generator=g)[:192]], big_rows[:32]])
    ref = oracle.gemm_nt(_u8(xq)[rows], xs.cpu()[rows], _u8(wq), ws.cpu())
    got = y[rows.to(DEV)].cpu()
    assert oracle.rel_error(got[:192], ref[:192]) < TOL  # rows without the 3e38 entries
    assert oracle.rel_error(got, ref) < TOL  # and with them (they dominate the norm)
    per_row = (got.double() - ref).norm(dim=1) / ref.norm(dim=1)
    assert per_row.max() < TOL
    # WGRAD dy^T x on token-axis blocks: sampled output features, all 8192 input channels
    feat = torch.randperm(n, generator=g)[:128]
    dtq, dts = quantize_mx_cols(dy.to(DEV))
    xtq, xts = quantize_mx_cols(x.to(DEV))
    dw = mxfp8_matmul_pq(dtq, dts, xtq, xts)
    ref = oracle.gemm_nt(_u8(dtq)[feat], dts.cpu()[feat], _u8(xtq), xts.cpu())
    got = dw[feat.to(DEV)].cpu()
    per_col = (got.double() - ref).norm(dim=0) / ref.norm(dim=0).clamp_min(1e-300)
    assert oracle.rel_error(got, ref) < TOL and per_col.max() < TOL
    # what the quantization itself costs on this data, against the unquantized product (reported, loosely bounded)
    exact = x[rows[:192]].double() @ w.double().T
    assert oracle.rel_error(y[rows[:192].to(DEV)].cpu(), exact) < 0.1
