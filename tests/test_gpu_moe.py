"""Routed experts in MXFP8 against the CPU oracle: grouped GEMM, the fused expert kernels, WGRAD.

Oracle = per-expert loop over the offset table of dequantize-then-matmul in fp64 on operands
quantized by the oracle; 1e-2 relative Frobenius for 16-bit outputs.  Outputs accumulated with
atomics (out, dx, dgate) are compared by norm, never bitwise: their summation order is free.
"""

import pytest
import torch

from conftest import SEED

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL = 1e-2
F8 = torch.float8_e4m3fn


def _dev(q, s):
    return q.to(DEV).view(F8), s.to(DEV)


def _routing(counts, top_k, tokens, seed=SEED):
    """offsets/order/token_of for given per-expert counts: position m of expert e takes distinct tokens."""
    g = torch.Generator().manual_seed(seed)
    offsets = torch.zeros(len(counts) + 1, dtype=torch.int32)
    offsets[1:] = torch.tensor(counts).cumsum(0)
    m = int(offsets[-1])
    token_of = torch.empty(m, dtype=torch.int32)
    slot = torch.zeros(tokens, dtype=torch.int64)  # how many experts each token already has
    order = torch.empty(m, dtype=torch.int32)
    for e, c in enumerate(counts):
        free = (slot < top_k).nonzero().flatten()
        pick = free[torch.randperm(free.numel(), generator=g)[:c]]
        assert pick.numel() == c
        lo = int(offsets[e])
        token_of[lo : lo + c] = pick.int()
        order[lo : lo + c] = (pick * top_k + slot[pick]).int()
        slot[pick] += 1
    return offsets, order, token_of


COUNT_CASES = [
    [300, 0, 1, 257, 0, 130],  # empty, single-row, just over a tile
    [64, 64, 64, 64],
    [0, 0, 5, 0],
    [700],
    # many experts, most of them empty, the busy ones behind long runs of empties: the owner of a
    # tile is found through the per-workgroup expert tables (more than one 64-expert chunk)
    [0] * 70 + [200] + [0] * 130 + [129, 1] + [0] * 50,
    # more experts than the expert dW kernel's smaller table beside its scale staging area holds (760), fewer than
    # the full table (1024): the dW kernel with scale bytes in registers
    [0] * 780 + [150, 40] + [0] * 20,
    # more experts than the tables hold: the kernels fall back to walking `offsets`
    [0] * 1040 + [90, 0, 33] + [0] * 20,
]


@pytest.mark.parametrize("counts", COUNT_CASES)
@pytest.mark.parametrize("use_index", [False, True])
def test_grouped_gemm(oracle, counts, use_index):
    from kohakuwullm_amd.kernels.mxfp8.grouped import grouped_mxfp8_gemm, grouped_mxfp8_reference

    g = torch.Generator().manual_seed(SEED)
    e, n, k = len(counts), 320, 256
    m = sum(counts)
    tokens = max(m, 8) if not use_index else 200
    x = torch.randn(tokens, k, generator=g).bfloat16()
    w = (torch.randn(e, n, k, generator=g) * 0.05).bfloat16()
    xq, xs = oracle.quantize_rows(x)
    wq, ws = oracle.quantize_rows(w.reshape(e * n, k))
    wq, ws = wq.view(e, n, k), ws.view(e, n, k // 32)
    offsets = torch.zeros(e + 1, dtype=torch.int32)
    offsets[1:] = torch.tensor(counts).cumsum(0)
    index = torch.randint(0, tokens, (m,), generator=g).int() if use_index else None
    ref = oracle.grouped_gemm_nt(xq, xs, wq, ws, offsets, index)
    got = grouped_mxfp8_gemm(*_dev(xq, xs), *_dev(wq, ws), offsets.to(DEV), None if index is None else index.to(DEV),
                             rows=m)
    assert got.shape == (m, n) and got.dtype == torch.bfloat16
    assert oracle.rel_error(got.cpu(), ref) < TOL
    # the reference's own precision oracle, run on the device tensors, agrees with ours
    ref2 = grouped_mxfp8_reference(*_dev(xq, xs), *_dev(wq, ws), offsets.to(DEV), None if index is None else index.to(DEV))
    assert oracle.rel_error(ref2.cpu(), ref) < 1e-12
    # fp32 output: nothing but the MFMA's internal adder between us and fp64
    got32 = grouped_mxfp8_gemm(*_dev(xq, xs), *_dev(wq, ws), offsets.to(DEV), None if index is None else index.to(DEV),
                               out_dtype=torch.float32, rows=m)
    assert oracle.rel_error(got32.cpu(), ref) < 1e-4


@pytest.mark.parametrize("k", [512, 1024])
@pytest.mark.parametrize("use_index", [False, True])
@pytest.mark.parametrize("counts,n", [([3000, 0, 2500, 1, 4100, 700], 1792), ([5, 0, 130], 264), ([0, 0, 1], 8), ([257] * 9, 512)])
def test_grouped_gemm_look_ahead_schedule(oracle, k, use_index, counts, n):
    """K a multiple of 512 with 16-byte aligned scale rows takes the schedule that fetches the A operand two K stages
    ahead and its scale bytes through the copy engine.  More tiles than workgroups, so every workgroup crosses tile
    boundaries (ragged last tiles, an empty and a one-row expert among them), and launches of one or a few tiles; with
    and without gathered rows.  Against
    the fp64 oracle, and bit for bit against the one-stage schedule, which scale rows of another pitch select."""
    from kohakuwullm_amd.kernels.mxfp8.grouped import grouped_mxfp8_gemm
    from kohakuwullm_amd.kernels.mxfp8.quantize import quantize_mx

    g = torch.Generator().manual_seed(SEED + 21)
    e, m = len(counts), sum(counts)  # the first case: 43 row tiles x 7 column tiles; the others: at most a tile per workgroup
    tokens = max(m // 3, 8) if use_index else m
    x = torch.randn(tokens, k, generator=g).bfloat16()
    w = (torch.randn(e * n, k, generator=g) * 0.05).bfloat16()
    xq, xs = quantize_mx(x.to(DEV))
    wq, ws = quantize_mx(w.to(DEV))
    wq, ws = wq.view(e, n, k), ws.view(e, n, k // 32)
    offsets = torch.zeros(e + 1, dtype=torch.int32)
    offsets[1:] = torch.tensor(counts).cumsum(0)
    index = torch.randint(0, tokens, (m,), generator=g).int().to(DEV) if use_index else None
    got = grouped_mxfp8_gemm(xq, xs, wq, ws, offsets.to(DEV), index, rows=m)
    ref = oracle.grouped_gemm_nt(xq.view(torch.uint8).cpu(), xs.cpu(), wq.view(torch.uint8).cpu(), ws.cpu(), offsets,
                                 None if index is None else index.cpu())
    assert oracle.rel_error(got.cpu(), ref) < TOL
    xs_other = torch.empty(tokens, k // 32 + 4, device=DEV, dtype=torch.uint8)[:, : k // 32]  # pitch not a multiple of 16
    xs_other.copy_(xs)
    assert torch.equal(got, grouped_mxfp8_gemm(xq, xs_other, wq, ws, offsets.to(DEV), index, rows=m))
    got32 = grouped_mxfp8_gemm(xq, xs, wq, ws, offsets.to(DEV), index, out_dtype=torch.float32, rows=m)
    assert oracle.rel_error(got32.cpu(), ref) < 1e-4


def test_grouped_gemm_sentinel_rows_untouched_and_errors(oracle):
    from kohakuwullm_amd.kernels.mxfp8.grouped import grouped_mxfp8_gemm

    g = torch.Generator().manual_seed(SEED)
    e, n, k, m = 3, 128, 128, 100
    x = torch.randn(m, k, generator=g).bfloat16()
    w = (torch.randn(e, n, k, generator=g) * 0.05).bfloat16()
    xq, xs = oracle.quantize_rows(x)
    wq, ws = oracle.quantize_rows(w.reshape(e * n, k))
    wq, ws = wq.view(e, n, k), ws.view(e, n, k // 32)
    offsets = torch.tensor([0, 30, 30, 70], dtype=torch.int32)  # rows 70..99 belong to no real expert
    out = torch.full((m, n), 7.0, dtype=torch.bfloat16, device=DEV)
    grouped_mxfp8_gemm(*_dev(xq, xs), *_dev(wq, ws), offsets.to(DEV), out=out)
    ref = oracle.grouped_gemm_nt(xq, xs, wq, ws, offsets)
    assert oracle.rel_error(out[:70].cpu(), ref) < TOL
    assert (out[70:] == 7.0).all()
    # K not a multiple of 128: the generic kernel
    xq2, xs2, wq2, ws2 = xq[:, :96].contiguous(), xs[:, :3].contiguous(), wq[:, :, :96].contiguous(), ws[:, :, :3].contiguous()
    got = grouped_mxfp8_gemm(*_dev(xq2, xs2), *_dev(wq2, ws2), offsets.to(DEV), rows=70)
    assert oracle.rel_error(got.cpu(), oracle.grouped_gemm_nt(xq2, xs2, wq2, ws2, offsets)) < TOL
    with pytest.raises(ValueError):
        grouped_mxfp8_gemm(*_dev(xq[:, :64], xs[:, :2]), *_dev(wq, ws), offsets.to(DEV))
    with pytest.raises(ValueError):
        grouped_mxfp8_gemm(*_dev(xq, xs), *_dev(wq, ws[:, :, :2]), offsets.to(DEV))
    with pytest.raises(ValueError):
        grouped_mxfp8_gemm(*_dev(xq, xs), *_dev(wq, ws), offsets.to(DEV), out=torch.empty(3, 3, device=DEV))


def _padded_cols_ref(oracle, rows_fp32, offsets, dtype=torch.bfloat16):
    """Oracle for the grouped token-axis quantizer: each expert's rows padded to a multiple of 128, then quantize_cols."""
    off = offsets.tolist()
    e = len(off) - 1
    mpad = (-(-rows_fp32.shape[0] // 128) + e) * 128
    c = rows_fp32.shape[1]
    q = torch.zeros(c, mpad, dtype=torch.uint8)
    s = torch.zeros(c, mpad // 32, dtype=torch.uint8)
    valid = torch.zeros(mpad, dtype=torch.bool)
    pos = 0
    for i in range(e):
        cnt = off[i + 1] - off[i]
        tiles = -(-cnt // 128)
        if tiles == 0:
            continue
        block = torch.zeros(tiles * 128, c)
        block[:cnt] = rows_fp32[off[i] : off[i + 1]]
        bq, bs = oracle.quantize_cols(block)
        q[:, pos : pos + tiles * 128] = bq
        s[:, pos // 32 : (pos + tiles * 128) // 32] = bs
        valid[pos : pos + tiles * 128] = True
        pos += tiles * 128
    return q, s, valid


@pytest.mark.parametrize("counts", COUNT_CASES[:3] + COUNT_CASES[4:])
def test_grouped_token_axis_quantizer_and_wgrad(oracle, counts):
    from kohakuwullm_amd.kernels.mxfp8.grouped import grouped_mxfp8_wgrad, quantize_mx_cols_grouped

    g = torch.Generator().manual_seed(SEED)
    e, m = len(counts), sum(counts)
    tokens, n, k = 400, 256, 192
    offsets = torch.zeros(e + 1, dtype=torch.int32)
    offsets[1:] = torch.tensor(counts).cumsum(0)
    a = (torch.randn(m, n, generator=g) * 1e-2).bfloat16()
    x = torch.randn(tokens, k, generator=g).bfloat16()
    index = torch.randint(0, tokens, (m,), generator=g).int()
    scale = (torch.rand(m * 2, generator=g) + 0.5).bfloat16()
    sidx = torch.randperm(m * 2, generator=g)[:m].int()
    # plain
    atq, ats = quantize_mx_cols_grouped(a.to(DEV), offsets.to(DEV), m)
    rq, rs, valid = _padded_cols_ref(oracle, a.float(), offsets)
    vs = valid.view(-1, 32)[:, 0]
    assert torch.equal(atq.view(torch.uint8).cpu()[:, valid], rq[:, valid])
    assert torch.equal(ats.cpu()[:, vs], rs[:, vs])
    # gathered rows times a gathered row scale (fp32 product, then quantized)
    btq, bts = quantize_mx_cols_grouped(x.to(DEV), offsets.to(DEV), m, index=index.to(DEV), row_scale=scale.to(DEV),
                                        scale_index=sidx.to(DEV))
    rows = x[index.long()].float() * scale[sidx.long()].float()[:, None]
    bq_ref, bs_ref, _ = _padded_cols_ref(oracle, rows, offsets)
    assert torch.equal(btq.view(torch.uint8).cpu()[:, valid], bq_ref[:, valid])
    assert torch.equal(bts.cpu()[:, vs], bs_ref[:, vs])
    # swiglu source
    pre = torch.randn(m, 2 * 128, generator=g).bfloat16()
    htq, hts = quantize_mx_cols_grouped(pre.to(DEV), offsets.to(DEV), m, swiglu=True)
    gg, vv = pre.float().chunk(2, dim=-1)
    hq_ref, hs_ref, _ = _padded_cols_ref(oracle, gg * torch.sigmoid(gg) * vv, offsets)
    assert (htq.view(torch.uint8).cpu()[:, valid] != hq_ref[:, valid]).float().mean() < 5e-3
    # WGRAD on the token-axis operands: per-expert A^T B of the dequantized padded blocks
    dw = grouped_mxfp8_wgrad(atq, ats, btq, bts, offsets.to(DEV), m)
    assert dw.shape == (e, n, k)
    # the quantizer leaves spare bytes behind every scale row and the kernel then fetches scales 16 bytes
    # at a time; scale rows packed end to end take the dword-per-stage path: same result, bit for bit
    assert ats.stride(0) > ats.shape[1] and bts.stride(0) > bts.shape[1]
    dw_packed = grouped_mxfp8_wgrad(atq, ats.contiguous(), btq, bts.contiguous(), offsets.to(DEV), m)
    assert torch.equal(dw, dw_packed)
    ad = oracle.dequant(rq.T.contiguous().T, rs)  # (n, mpad)
    bd = oracle.dequant(bq_ref, bs_ref)  # (k, mpad)
    pos = 0
    for i, cnt in enumerate(counts):
        tiles = -(-cnt // 128)
        ref = ad[:, pos : pos + tiles * 128] @ bd[:, pos : pos + tiles * 128].T
        pos += tiles * 128
        if cnt == 0:
            assert (dw[i] == 0).all()
        else:
            assert oracle.rel_error(dw[i].cpu(), ref) < TOL, (i, cnt)


@pytest.mark.parametrize("with_scale", [False, True])
def test_grouped_token_axis_quantizer_many_rows(oracle, with_scale):
    """Enough routed rows and columns that a workgroup walks four column tiles of its 128 rows
    (the launch picks that for 512 or more row tiles of 4 or more column tiles): bit-exact."""
    from kohakuwullm_amd.kernels.mxfp8.grouped import quantize_mx_cols_grouped

    g = torch.Generator().manual_seed(SEED + 11)
    counts = [30000, 0, 20001, 17000, 130]
    e, m = len(counts), sum(counts)
    tokens, c = 4096, 640  # five column tiles: one workgroup of four, one of one
    offsets = torch.zeros(e + 1, dtype=torch.int32)
    offsets[1:] = torch.tensor(counts).cumsum(0)
    x = torch.randn(tokens, c, generator=g).bfloat16()
    index = torch.randint(0, tokens, (m,), generator=g).int()
    scale = (torch.rand(m, generator=g) + 0.5).bfloat16()
    sidx = torch.randperm(m, generator=g).int()
    kw = dict(row_scale=scale.to(DEV), scale_index=sidx.to(DEV)) if with_scale else {}
    tq, ts = quantize_mx_cols_grouped(x.to(DEV), offsets.to(DEV), m, index=index.to(DEV), **kw)
    rows = x[index.long()].float()
    if with_scale:
        rows = rows * scale[sidx.long()].float()[:, None]
    rq, rs, valid = _padded_cols_ref(oracle, rows, offsets)
    vs = valid.view(-1, 32)[:, 0]
    assert torch.equal(tq.view(torch.uint8).cpu()[:, valid], rq[:, valid])
    assert torch.equal(ts.cpu()[:, vs], rs[:, vs])


@pytest.mark.parametrize("counts", [[2400, 0, 700, 2900], [5000, 1], [130, 0, 0, 4000, 0, 1500]])
def test_wgrad_even_k_split_ranges_straddle_experts(oracle, counts):
    """Few busy experts with several output tiles each: the K stages of all experts are cut into equal
    ranges, one per group of workgroups, and ranges end inside an expert and straddle two of them
    (19 + 6 + 23 stages in ranges of 2, for the first case).  Every expert against the fp64 oracle."""
    from kohakuwullm_amd.kernels.mxfp8.grouped import grouped_mxfp8_wgrad, quantize_mx_cols_grouped

    g = torch.Generator().manual_seed(SEED + 7)
    e, m = len(counts), sum(counts)
    n, k = 512, 384  # 2 x 2 output tiles per expert
    offsets = torch.zeros(e + 1, dtype=torch.int32)
    offsets[1:] = torch.tensor(counts).cumsum(0)
    a = (torch.randn(m, n, generator=g) * 1e-2).bfloat16()
    b = torch.randn(m, k, generator=g).bfloat16()
    atq, ats = quantize_mx_cols_grouped(a.to(DEV), offsets.to(DEV), m)
    btq, bts = quantize_mx_cols_grouped(b.to(DEV), offsets.to(DEV), m)
    dw = grouped_mxfp8_wgrad(atq, ats, btq, bts, offsets.to(DEV), m)
    assert torch.equal(dw, grouped_mxfp8_wgrad(atq, ats, btq, bts, offsets.to(DEV), m))  # deterministic
    aq_ref, as_ref, _ = _padded_cols_ref(oracle, a.float(), offsets)
    bq_ref, bs_ref, _ = _padded_cols_ref(oracle, b.float(), offsets)
    ad, bd = oracle.dequant(aq_ref, as_ref), oracle.dequant(bq_ref, bs_ref)
    pos = 0
    for i, cnt in enumerate(counts):
        tiles = -(-cnt // 128)
        ref = ad[:, pos : pos + tiles * 128] @ bd[:, pos : pos + tiles * 128].T
        pos += tiles * 128
        if cnt == 0:
            assert (dw[i] == 0).all()
        else:
            assert oracle.rel_error(dw[i].cpu(), ref) < TOL, (i, cnt)


@pytest.mark.parametrize("counts,n,k", [([50] * 300, 256, 256), ([50, 300, 1, 129, 128, 5, 0, 257] * 45, 512, 256),
                                        ([128] * 130 + [4000] + [1] * 140, 256, 512)])
def test_wgrad_runs_of_single_stage_tiles(oracle, counts, n, k):
    """More (expert, tile) units than workgroups, most of them a single K stage (experts of up to 128 rows), in runs and
    mixed with longer ones: the expert dW kernel fetches its A operand two stages ahead, and a stage that lies two tiles
    on is fetched one stage ahead instead.  Every expert against the fp64 oracle."""
    from kohakuwullm_amd.kernels.mxfp8.grouped import grouped_mxfp8_wgrad, quantize_mx_cols_grouped

    g = torch.Generator().manual_seed(SEED + 8)
    e, m = len(counts), sum(counts)
    offsets = torch.zeros(e + 1, dtype=torch.int32)
    offsets[1:] = torch.tensor(counts).cumsum(0)
    a = (torch.randn(m, n, generator=g) * 1e-2).bfloat16()
    b = torch.randn(m, k, generator=g).bfloat16()
    atq, ats = quantize_mx_cols_grouped(a.to(DEV), offsets.to(DEV), m, stage_major=True)
    btq, bts = quantize_mx_cols_grouped(b.to(DEV), offsets.to(DEV), m)
    dw = grouped_mxfp8_wgrad(atq, ats, btq, bts, offsets.to(DEV), m)
    assert torch.equal(dw, grouped_mxfp8_wgrad(atq, ats, btq, bts, offsets.to(DEV), m))  # deterministic
    aq_ref, as_ref, _ = _padded_cols_ref(oracle, a.float(), offsets)
    bq_ref, bs_ref, _ = _padded_cols_ref(oracle, b.float(), offsets)
    ad, bd = oracle.dequant(aq_ref, as_ref), oracle.dequant(bq_ref, bs_ref)
    dw = dw.cpu()
    pos = 0
    for i, cnt in enumerate(counts):
        tiles = -(-cnt // 128)
        ref = ad[:, pos : pos + tiles * 128] @ bd[:, pos : pos + tiles * 128].T
        pos += tiles * 128
        if cnt == 0:
            assert (dw[i] == 0).all()
        else:
            assert oracle.rel_error(dw[i], ref) < TOL, (i, cnt)


def _expert_oracle(ora, x, w_in, w_out, gate, token_of, order, offsets, dout):
    """The fused path's arithmetic restated with oracle primitives, stage by stage."""
    e, two_h, dim = w_in.shape
    hid = two_h // 2
    off = offsets.tolist()
    m = off[-1]
    t_idx, p_idx = token_of.long()[:m], order.long()[:m]

    def stacked(w):
        q, s = ora.quantize_rows(w.reshape(-1, w.shape[-1]))
        return q.view(*w.shape), s.view(*w.shape[:-1], w.shape[-1] // 32)

    in_f, out_f = stacked(w_in), stacked(w_out)
    in_d, out_d = stacked(w_in.transpose(1, 2).contiguous()), stacked(w_out.transpose(1, 2).contiguous())
    xq, xs = ora.quantize_rows(x)
    pre = ora.grouped_gemm_nt(xq, xs, *in_f, offsets, t_idx).bfloat16()
    g, v = pre.float().chunk(2, dim=-1)
    h = g * torch.sigmoid(g) * v
    hq, hs = ora.quantize_rows(h)
    y = ora.grouped_gemm_nt(hq, hs, *out_f, offsets)
    gate_m = gate.float()[p_idx].double()
    out = torch.zeros(x.shape[0], dim, dtype=torch.float64).index_add_(0, t_idx, y * gate_m[:, None])
    # backward
    dq, ds = ora.quantize_rows(dout)
    acc = ora.grouped_gemm_nt(dq, ds, *out_d, offsets, t_idx)  # (m, hid)
    dgate = torch.zeros(gate.numel(), dtype=torch.float64).index_add_(0, p_idx, (acc * ora.dequant(hq, hs)).sum(-1))
    dh = (acc * gate_m[:, None]).float()
    sg = torch.sigmoid(g)
    dpre = torch.cat([dh * v * sg * (1 + g * (1 - sg)), dh * g * sg], dim=-1)
    pq, ps = ora.quantize_rows(dpre)
    dx = torch.zeros(x.shape[0], dim, dtype=torch.float64).index_add_(0, t_idx, ora.grouped_gemm_nt(pq, ps, *in_d, offsets))
    # WGRAD on token-axis blocks inside each expert's segment
    a_out = dout.float()[t_idx] * gate.float()[p_idx][:, None]
    dw_out = torch.zeros(e, dim, hid, dtype=torch.float64)
    dw_in = torch.zeros(e, two_h, dim, dtype=torch.float64)
    dpre16 = dpre.bfloat16().float()
    xg = x.float()[t_idx]
    for i in range(e):
        lo, hi = off[i], off[i + 1]
        if hi == lo:
            continue
        pad = -(hi - lo) % 32

        def qc(rows):
            rows = torch.nn.functional.pad(rows, (0, 0, 0, pad))
            return ora.quantize_cols(rows)

        dw_out[i] = ora.gemm_nt(*qc(a_out[lo:hi]), *qc(h[lo:hi]))
        dw_in[i] = ora.gemm_nt(*qc(dpre16[lo:hi]), *qc(xg[lo:hi]))
    # The reference's own expert dW (kernels/mxfp8/grouped.py:152-247 called from moe.py:284-325) multiplies 16-bit
    # operands: gate * dout[token] rounded to the activation dtype against h rebuilt from the stored pre with PyTorch's
    # 16-bit operators, and dpre against x[token]; fp32 accumulation.  Restated here in fp64 on those 16-bit operands.
    act = x.dtype
    a16 = a_out.to(act).double()
    pre16 = pre.to(act)
    h16 = (torch.nn.functional.silu(pre16[:, :hid]) * pre16[:, hid:]).double()
    dw_out16 = torch.zeros_like(dw_out)
    dw_in16 = torch.zeros_like(dw_in)
    for i in range(e):
        lo, hi = off[i], off[i + 1]
        dw_out16[i] = a16[lo:hi].T @ h16[lo:hi]
        dw_in16[i] = dpre16[lo:hi].double().T @ xg[lo:hi].double()
    return dict(out=out, pre=pre, hq=hq, hs=hs, dx=dx, dgate=dgate, dw_in=dw_in, dw_out=dw_out, dw_in16=dw_in16,
                dw_out16=dw_out16)


def _unfused_oracle(ora, x, w_in, w_out, gate, token_of, order, offsets, dout):
    """The unfused path's own arithmetic (src/kohakuwullm/kernels/mxfp8/moe_unfused.py:25-158) restated with oracle
    primitives.  Its casts sit elsewhere than the fused graph's: `pre`, `h`, the combine's rows, `dh` and `dpre` all make
    a 16-bit round trip between launches, SwiGLU and its derivative are PyTorch's 16-bit elementwise operators (taken
    here from PyTorch on the CPU, autograd included), and the gate is applied to the upstream rows BEFORE the dgrad
    quantizer (the combine's backward), not to the accumulator behind it.  WGRAD is this build's: MXFP8 on token-axis
    blocks inside each expert's segment."""
    e, two_h, dim = w_in.shape
    off = offsets.tolist()
    m = off[-1]
    t_idx, p_idx = token_of.long()[:m], order.long()[:m]

    def stacked(w):
        q, s = ora.quantize_rows(w.reshape(-1, w.shape[-1]))
        return q.view(*w.shape), s.view(*w.shape[:-1], w.shape[-1] // 32)

    in_f, out_f = stacked(w_in), stacked(w_out)
    in_d, out_d = stacked(w_in.transpose(1, 2).contiguous()), stacked(w_out.transpose(1, 2).contiguous())
    act = x.dtype
    pre = ora.grouped_gemm_nt(*ora.quantize_rows(x), *in_f, offsets, t_idx).to(act).requires_grad_(True)
    gate_h, value = pre.chunk(2, dim=-1)
    h = torch.nn.functional.silu(gate_h) * value  # 16-bit operators: silu rounds, the product rounds again
    y = ora.grouped_gemm_nt(*ora.quantize_rows(h.detach()), *out_f, offsets).to(act)
    out = ora.combine_routed(y, gate, order[:m], token_of[:m], x.shape[0])
    # backward: combine, second product, SwiGLU (autograd of the 16-bit operators), first product
    grad_rows, dgate = ora.combine_routed_grads(dout, y, gate, order[:m], token_of[:m])
    dh = ora.grouped_gemm_nt(*ora.quantize_rows(grad_rows), *out_d, offsets).to(act)
    (dpre,) = torch.autograd.grad(h, pre, dh)
    dx_sorted = ora.grouped_gemm_nt(*ora.quantize_rows(dpre), *in_d, offsets).to(act)
    dx = torch.zeros(x.shape[0], dim, dtype=torch.float64).index_add_(0, t_idx, dx_sorted.double())
    dw_out = torch.zeros(e, dim, two_h // 2, dtype=torch.float64)
    dw_in = torch.zeros(e, two_h, dim, dtype=torch.float64)
    xg, h16 = x.float()[t_idx], h.detach().float()
    for i in range(e):
        lo, hi = off[i], off[i + 1]
        if hi == lo:
            continue
        pad = -(hi - lo) % 32

        def qc(rows):
            return ora.quantize_cols(torch.nn.functional.pad(rows, (0, 0, 0, pad)))

        dw_out[i] = ora.gemm_nt(*qc(grad_rows.float()[lo:hi]), *qc(h16[lo:hi]))
        dw_in[i] = ora.gemm_nt(*qc(dpre.float()[lo:hi]), *qc(xg[lo:hi]))
    return dict(out=out, dx=dx, dgate=dgate, dw_in=dw_in, dw_out=dw_out)


@pytest.mark.parametrize("counts,top_k", [([300, 0, 1, 257, 0, 130], 2), ([256, 256], 1),
                                          ([0] * 70 + [200] + [0] * 130 + [129, 1] + [0] * 50, 1)])
@pytest.mark.parametrize("dout_scale", [1.0, 2.0**-20])
def test_fused_experts_fwd_bwd(oracle, counts, top_k, dout_scale):
    from kohakuwullm_amd.kernels.mxfp8.moe import (
        MXFP8ExpertWeights,
        mxfp8_moe_experts,
        mxfp8_moe_experts_reference,
        mxfp8_moe_experts_unfused,
    )

    g = torch.Generator().manual_seed(SEED)
    e, tokens, dim, hid = len(counts), 512, 256, 128
    offsets, order, token_of = _routing(counts, top_k, tokens)
    x = torch.randn(tokens, dim, generator=g).bfloat16()
    w_in = (torch.randn(e, 2 * hid, dim, generator=g) * 0.06).bfloat16()
    w_out = (torch.randn(e, dim, hid, generator=g) * 0.06).bfloat16()
    gate = (torch.rand(tokens * top_k, generator=g) * 0.5 + 0.5).bfloat16()
    dout = (torch.randn(tokens, dim, generator=g) * dout_scale).bfloat16()
    ref = _expert_oracle(oracle, x, w_in, w_out, gate, token_of, order, offsets, dout)

    def run(fn):
        xd, wi, wo, gd = (t.to(DEV).requires_grad_(True) for t in (x, w_in, w_out, gate))
        packed = MXFP8ExpertWeights(wi.detach(), wo.detach())
        out = fn(xd, wi, wo, gd, token_of.to(DEV), order.to(DEV), offsets.to(DEV), packed)
        assert out.grad_fn is not None and out.shape == (tokens, dim) and out.dtype == torch.bfloat16
        out.backward(dout.to(DEV))
        return out.detach().cpu(), xd.grad.cpu(), wi.grad.cpu(), wo.grad.cpu(), gd.grad.cpu()

    out, dx, dw_in, dw_out, dgate = run(mxfp8_moe_experts)
    assert oracle.rel_error(out, ref["out"]) < TOL
    assert oracle.rel_error(dx, ref["dx"]) < TOL
    assert oracle.rel_error(dgate, ref["dgate"]) < TOL
    assert oracle.rel_error(dw_out, ref["dw_out"]) < TOL
    assert oracle.rel_error(dw_in, ref["dw_in"]) < TOL
    for i, c in enumerate(counts):
        if c == 0:
            assert (dw_in[i] == 0).all() and (dw_out[i] == 0).all()
    assert dgate.dtype == gate.dtype and dw_in.dtype == torch.bfloat16
    # Distance to the reference's 16-bit expert dW: this build quantizes both operands of the product to e4m3 along the
    # tokens, each cast 2.7e-2 away from its operand in relative Frobenius norm, so the product is sqrt(2) x 2.7e-2 =
    # 3.8e-2 away in expectation.  Held at 5e-2: the quantization and nothing else.
    assert oracle.rel_error(dw_out, ref["dw_out16"]) < 5e-2
    assert oracle.rel_error(dw_in, ref["dw_in16"]) < 5e-2

    # structural reference without quantization (autograd in fp32): the gap is the e4m3 error of the chain
    xf, wif, wof, gf = (t.float().requires_grad_(True) for t in (x, w_in, w_out, gate))
    yf = mxfp8_moe_experts_reference(xf, wif, wof, gf, token_of, order, offsets)
    yf.backward(dout.float())
    assert oracle.rel_error(out, yf) < 0.08
    assert oracle.rel_error(dx, xf.grad) < 0.12
    assert oracle.rel_error(dw_in, wif.grad) < 0.12
    assert oracle.rel_error(dw_out, wof.grad) < 0.12
    assert oracle.rel_error(dgate, gf.grad) < 0.12

    # the unfused twin computes the same function through differently placed casts (16-bit h and
    # dh round trips, the gate applied before the dgrad quantizer): held to an oracle chain of ITS cast
    # placement at the same 1e-2 as the fused graph, forward and every gradient
    out_u, dx_u, dw_in_u, dw_out_u, dgate_u = run(mxfp8_moe_experts_unfused)
    ref_u = _unfused_oracle(oracle, x, w_in, w_out, gate, token_of, order, offsets, dout)
    assert oracle.rel_error(out_u, ref_u["out"].double()) < TOL
    assert oracle.rel_error(dx_u, ref_u["dx"]) < TOL
    assert oracle.rel_error(dgate_u, ref_u["dgate"]) < TOL
    assert oracle.rel_error(dw_out_u, ref_u["dw_out"]) < TOL
    assert oracle.rel_error(dw_in_u, ref_u["dw_in"]) < TOL
    assert oracle.rel_error(out_u, ref["out"]) < 2e-2  # and within the 16-bit round trips of the fused oracle


@pytest.mark.parametrize("counts,top_k", [([300, 0, 1, 257, 0, 130], 2), ([0, 511], 1)])
def test_fused_experts_scatter_route(oracle, counts, top_k):
    """The atomic route of GEMM2 and GEMM1-dgrad (the reference's own: tl.atomic_add epilogues, experts.py:138-222,
    experts_bwd.py:167-247).  The fused graph takes it when `order` is not known to be the pair index token * top_k +
    slot -- here: a gate vector one element longer than tokens * top_k, whose last element no pair uses -- and the
    scatter GEMM is also called on its own, with 16-bit and fp32 outputs, with and without a gate and a row index.
    Sums of atomics: compared by norm, never bitwise."""
    from kohakuwullm_amd.kernels.mxfp8.moe import MXFP8ExpertWeights, launch_scatter_gemm, mxfp8_moe_experts
    from kohakuwullm_amd.kernels.mxfp8.quantize import quantize_mx

    g = torch.Generator().manual_seed(SEED + 3)
    e, tokens, dim, hid = len(counts), 512, 256, 128
    offsets, order, token_of = _routing(counts, top_k, tokens)
    x = torch.randn(tokens, dim, generator=g).bfloat16()
    w_in = (torch.randn(e, 2 * hid, dim, generator=g) * 0.06).bfloat16()
    w_out = (torch.randn(e, dim, hid, generator=g) * 0.06).bfloat16()
    gate = (torch.rand(tokens * top_k + 1, generator=g) * 0.5 + 0.5).bfloat16()
    dout = torch.randn(tokens, dim, generator=g).bfloat16()
    ref = _expert_oracle(oracle, x, w_in, w_out, gate, token_of, order, offsets, dout)

    xd, wi, wo, gd = (t.to(DEV).requires_grad_(True) for t in (x, w_in, w_out, gate))
    packed = MXFP8ExpertWeights(wi.detach(), wo.detach())
    from kohakuwullm_amd import _lib

    _lib.TIMER = []  # records the entry points the call goes through
    try:
        out = mxfp8_moe_experts(xd, wi, wo, gd, token_of.to(DEV), order.to(DEV), offsets.to(DEV), packed)
        out.backward(dout.to(DEV))
        torch.cuda.synchronize()
        called = [name for name, *_ in _lib.TIMER]
    finally:
        _lib.TIMER = None
    assert called.count("mx_experts_scatter_gemm") == 2 and "mx_experts_combine" not in called
    assert oracle.rel_error(out.detach().cpu(), ref["out"]) < TOL
    assert oracle.rel_error(xd.grad.cpu(), ref["dx"]) < TOL
    assert oracle.rel_error(gd.grad.cpu(), ref["dgate"]) < TOL and gd.grad[-1] == 0
    assert oracle.rel_error(wi.grad.cpu(), ref["dw_in"]) < TOL and oracle.rel_error(wo.grad.cpu(), ref["dw_out"]) < TOL

    # the entry point on its own: out[token_of[m]] += scale(m) * (a[index[m] or m] . w[e(m)]^T)
    m = sum(counts)
    hq, hs = ref["hq"], ref["hs"]  # the oracle's h codes: sorted rows, K = hid
    wq, ws = oracle.quantize_rows(w_out.reshape(-1, hid))
    wq, ws = wq.view(e, dim, hid), ws.view(e, dim, hid // 32)
    y = oracle.grouped_gemm_nt(hq, hs, wq, ws, offsets)  # (m, dim) fp64
    t_idx, p_idx = token_of.long()[:m], order.long()[:m]
    dev = lambda t: t.to(DEV)  # noqa: E731
    # (16-bit outputs only: the adds are packed 16-bit atomics; the gate in the output's type or in fp32)
    for out_dtype, gate_dtype in ((torch.bfloat16, torch.bfloat16), (torch.float16, torch.float32), (torch.float16, None)):
        gate_t = gate.to(gate_dtype) if gate_dtype else None
        scale = gate_t.double()[p_idx] if gate_dtype else torch.ones(m, dtype=torch.float64)
        want = torch.zeros(tokens, dim, dtype=torch.float64).index_add_(0, t_idx, y * scale[:, None])
        got = torch.zeros(tokens, dim, device=DEV, dtype=out_dtype)
        launch_scatter_gemm(*_dev(hq, hs), *_dev(wq, ws), got, dev(token_of), dev(order) if gate_dtype else None,
                            dev(gate_t) if gate_dtype else None, dev(offsets))
        assert oracle.rel_error(got.cpu(), want) < TOL, (out_dtype, gate_dtype)
    with pytest.raises(ValueError):  # an fp32 output is refused, not mis-added
        launch_scatter_gemm(*_dev(hq, hs), *_dev(wq, ws), torch.zeros(tokens, dim, device=DEV), dev(token_of), None, None,
                            dev(offsets))
    # with a row index: a[index[m]] in place of a[m] (the quantized token rows gathered inside the kernel)
    xq, xs = oracle.quantize_rows(x)
    wq1, ws1 = oracle.quantize_rows(w_in.reshape(-1, dim))
    wq1, ws1 = wq1.view(e, 2 * hid, dim), ws1.view(e, 2 * hid, dim // 32)
    want = torch.zeros(tokens, 2 * hid, dtype=torch.float64).index_add_(
        0, t_idx, oracle.grouped_gemm_nt(xq, xs, wq1, ws1, offsets, t_idx))
    got = torch.zeros(tokens, 2 * hid, device=DEV, dtype=torch.bfloat16)
    launch_scatter_gemm(*_dev(xq, xs), *_dev(wq1, ws1), got, dev(token_of), None, None, dev(offsets), index=dev(token_of))
    assert oracle.rel_error(got.cpu(), want) < TOL


def test_gemm1_intermediates(oracle):
    """GEMM1's three outputs against the oracle: pre is the rounded accumulator, h is quantized from fp32."""
    from kohakuwullm_amd.kernels.mxfp8.moe import MXFP8ExpertWeights, launch_gemm1
    from kohakuwullm_amd.kernels.mxfp8.quantize import quantize_mx

    g = torch.Generator().manual_seed(SEED)
    counts, top_k = [200, 0, 56], 1
    e, tokens, dim, hid = len(counts), 256, 128, 160
    offsets, order, token_of = _routing(counts, top_k, tokens)
    x = torch.randn(tokens, dim, generator=g).bfloat16()
    w_in = (torch.randn(e, 2 * hid, dim, generator=g) * 0.08).bfloat16()
    w_out = (torch.randn(e, dim, hid, generator=g) * 0.08).bfloat16()
    gate = torch.ones(tokens, dtype=torch.bfloat16)
    ref = _expert_oracle(oracle, x, w_in, w_out, gate, token_of, order, offsets, torch.zeros(tokens, dim).bfloat16())
    packed = MXFP8ExpertWeights(w_in.to(DEV), w_out.to(DEV))
    m = sum(counts)
    xq, xs = quantize_mx(x.to(DEV))
    hq = torch.zeros(m, hid, device=DEV, dtype=F8)
    hs = torch.zeros(m, hid // 32, device=DEV, dtype=torch.uint8)
    pre = torch.zeros(m, 2 * hid, device=DEV, dtype=torch.bfloat16)
    from kohakuwullm_amd.kernels.mxfp8.grouped import padded_rows, quantize_mx_cols_grouped

    mpad = padded_rows(m, e)
    htq = torch.zeros(hid, mpad, device=DEV, dtype=F8)
    hts = torch.zeros(hid, mpad // 32, device=DEV, dtype=torch.uint8)
    launch_gemm1(xq, xs, token_of.to(DEV), *packed.in_fwd, hq, hs, pre, offsets.to(DEV), hid, dim, torch.bfloat16, htq, hts)
    # the token-axis copy written by the epilogue is the grouped quantizer's result on the stored pre, bit for bit
    rq, rs = quantize_mx_cols_grouped(pre, offsets.to(DEV), m, swiglu=True)
    valid = torch.zeros(mpad, dtype=torch.bool)
    pos = 0
    for c in counts:
        tiles = -(-c // 128)
        valid[pos : pos + tiles * 128] = True
        pos += tiles * 128
    assert torch.equal(htq.view(torch.uint8).cpu()[:, valid], rq.view(torch.uint8).cpu()[:, valid])
    assert torch.equal(hts.cpu()[:, valid.view(-1, 32)[:, 0]], rs.cpu()[:, valid.view(-1, 32)[:, 0]])
    assert not htq.view(torch.uint8).cpu()[:, ~valid].any()  # nothing is written past the experts' tiles
    assert oracle.rel_error(pre.cpu(), ref["pre"].double()) < 2e-3  # same bf16 values up to accumulation-order ulps
    hd = oracle.dequant(hq.view(torch.uint8).cpu(), hs.cpu())
    assert oracle.rel_error(hd, oracle.dequant(ref["hq"], ref["hs"])) < 2e-2
    assert (hs.cpu() != ref["hs"]).float().mean() < 0.02


def test_gemm2_dgrad_token_axis(oracle):
    """The dgrad epilogue's token-axis copy of dpre is the grouped column quantizer's result on the stored dpre, bit for
    bit, and asking for it changes none of the other outputs (dpre itself becomes optional)."""
    from kohakuwullm_amd.kernels.mxfp8.grouped import padded_rows, quantize_mx_cols_grouped
    from kohakuwullm_amd.kernels.mxfp8.moe import MXFP8ExpertWeights, launch_gemm1, launch_gemm2_dgrad
    from kohakuwullm_amd.kernels.mxfp8.quantize import quantize_mx

    g = torch.Generator().manual_seed(SEED + 7)
    for counts, hid in (([200, 0, 56, 300], 160), ([256, 256], 256), ([1, 700], 544)):
        top_k = 1
        e, dim = len(counts), 128
        tokens = sum(counts)
        offsets, order, token_of = _routing(counts, top_k, tokens)
        x = torch.randn(tokens, dim, generator=g).bfloat16()
        w_in = (torch.randn(e, 2 * hid, dim, generator=g) * 0.08).bfloat16()
        w_out = (torch.randn(e, dim, hid, generator=g) * 0.08).bfloat16()
        gate = (torch.rand(tokens, generator=g) * 0.5 + 0.5).bfloat16().to(DEV)
        dout = torch.randn(tokens, dim, generator=g).bfloat16().to(DEV)
        packed = MXFP8ExpertWeights(w_in.to(DEV), w_out.to(DEV))
        m = sum(counts)
        off_d, tok_d, ord_d = offsets.to(DEV), token_of.to(DEV), order.to(DEV)
        xq, xs = quantize_mx(x.to(DEV))
        hq = torch.zeros(m, hid, device=DEV, dtype=F8)
        hs = torch.zeros(m, hid // 32, device=DEV, dtype=torch.uint8)
        pre = torch.zeros(m, 2 * hid, device=DEV, dtype=torch.bfloat16)
        launch_gemm1(xq, xs, tok_d, *packed.in_fwd, hq, hs, pre, off_d, hid, dim, torch.bfloat16)
        dq, ds = quantize_mx(dout)
        mpad = padded_rows(m, e)

        def run(with_dpre, with_tok):
            dpre = torch.zeros(m, 2 * hid, device=DEV, dtype=torch.bfloat16) if with_dpre else None
            dpq = torch.zeros(m, 2 * hid, device=DEV, dtype=F8)
            dps = torch.zeros(m, 2 * hid // 32, device=DEV, dtype=torch.uint8)
            dgate = torch.zeros(tokens, device=DEV, dtype=torch.float32)
            ptq = torch.zeros(2 * hid, mpad, device=DEV, dtype=F8) if with_tok else None
            pts = torch.zeros(2 * hid, mpad // 32, device=DEV, dtype=torch.uint8) if with_tok else None
            launch_gemm2_dgrad(dq, ds, tok_d, ord_d, gate, *packed.out_dgrad, hq, hs, pre, dpre, dpq, dps, dgate, off_d,
                               ptq, pts)
            return dpre, dpq, dps, dgate, ptq, pts

        dpre0, dpq0, dps0, dgate0, _, _ = run(True, False)
        dpre1, dpq1, dps1, dgate1, ptq1, pts1 = run(True, True)
        _, dpq2, dps2, dgate2, ptq2, pts2 = run(False, True)
        for a, b in ((dpre0, dpre1), (dpq0, dpq1), (dps0, dps1), (dpq0, dpq2), (dps0, dps2), (ptq1, ptq2), (pts1, pts2)):
            assert torch.equal(a.view(torch.uint8) if a.dtype == F8 else a, b.view(torch.uint8) if b.dtype == F8 else b)
        # dgate is an fp32 atomic sum: order-dependent in the last bits
        assert torch.allclose(dgate0, dgate1, rtol=1e-4, atol=1e-6) and torch.allclose(dgate0, dgate2, rtol=1e-4, atol=1e-6)
        rq, rs = quantize_mx_cols_grouped(dpre0, off_d, m)
        valid = torch.zeros(mpad, dtype=torch.bool)
        pos = 0
        for c in counts:
            tiles = -(-c // 128)
            valid[pos : pos + tiles * 128] = True
            pos += tiles * 128
        assert torch.equal(ptq1.view(torch.uint8).cpu()[:, valid], rq.view(torch.uint8).cpu()[:, valid])
        assert torch.equal(pts1.cpu()[:, valid.view(-1, 32)[:, 0]], rs.cpu()[:, valid.view(-1, 32)[:, 0]])
        assert not ptq1.view(torch.uint8).cpu()[:, ~valid].any()  # nothing is written past the experts' tiles
        with pytest.raises(Exception):
            run(False, False)  # neither output asked for


@pytest.mark.parametrize("counts,hid", [([200, 0, 56, 300], 160), ([1, 700], 544), ([130] * 5, 256)])
def test_expert_kernels_on_small_tiles_agree(counts, hid):
    """The variants library runs the two fused expert kernels on 128 x 128 tiles, two workgroups per CU: every element
    contracts the same K sequence and goes through the same epilogue arithmetic, so every output of GEMM1 and of
    GEMM2-dgrad equals the shipped kernels' bit for bit (dgate, a sum of atomics, by norm)."""
    from kohakuwullm_amd import _lib
    from kohakuwullm_amd.kernels.mxfp8.grouped import padded_rows
    from kohakuwullm_amd.kernels.mxfp8.moe import MXFP8ExpertWeights, launch_gemm1, launch_gemm2_dgrad
    from kohakuwullm_amd.kernels.mxfp8.quantize import quantize_mx

    g = torch.Generator().manual_seed(SEED + 11)
    e, dim, top_k = len(counts), 256, 1
    tokens = sum(counts) + 40
    offsets, order, token_of = (t.to(DEV) for t in _routing(counts, top_k, tokens))
    m = sum(counts)
    mpad = padded_rows(m, e)
    x = torch.randn(tokens, dim, generator=g).bfloat16().to(DEV)
    dout = torch.randn(tokens, dim, generator=g).bfloat16().to(DEV)
    gate = (torch.rand(tokens, generator=g) * 0.5 + 0.5).bfloat16().to(DEV)
    packed = MXFP8ExpertWeights((torch.randn(e, 2 * hid, dim, generator=g) * 0.06).bfloat16().to(DEV),
                                (torch.randn(e, dim, hid, generator=g) * 0.06).bfloat16().to(DEV))
    xq, xs = quantize_mx(x)
    dq, ds = quantize_mx(dout)

    def run():
        z = lambda *shape, dtype=torch.uint8: torch.zeros(*shape, device=DEV, dtype=dtype)  # noqa: E731
        hq, hs, pre = z(m, hid, dtype=F8), z(m, hid // 32), z(m, 2 * hid, dtype=torch.bfloat16)
        htq, hts = z(hid, mpad, dtype=F8), z(hid, mpad // 32)
        launch_gemm1(xq, xs, token_of, *packed.in_fwd, hq, hs, pre, offsets, hid, dim, torch.bfloat16, htq, hts)
        dpre, dpq, dps = z(m, 2 * hid, dtype=torch.bfloat16), z(m, 2 * hid, dtype=F8), z(m, 2 * hid // 32)
        ptq, pts, dgate = z(2 * hid, mpad, dtype=F8), z(2 * hid, mpad // 32), z(tokens, dtype=torch.float32)
        launch_gemm2_dgrad(dq, ds, token_of, order, gate, *packed.out_dgrad, hq, hs, pre, dpre, dpq, dps, dgate, offsets, ptq, pts)
        torch.cuda.synchronize()
        return [t.view(torch.uint8) if t.dtype == F8 else t for t in (hq, hs, pre, htq, hts, dpre, dpq, dps, ptq, pts)], dgate

    shipped, dgate = run()
    with _lib.variants_library():
        small, dgate_small = run()
    for name, a, b in zip("hq hs pre htq hts dpre dpq dps ptq pts".split(), shipped, small):
        assert torch.equal(a, b), name
    assert float((dgate - dgate_small).norm() / dgate.norm()) < 1e-5


def test_expert_call_contract():
    from kohakuwullm_amd.kernels.mxfp8.moe import MXFP8ExpertWeights, mxfp8_moe_experts

    e, tokens, dim, hid = 2, 64, 128, 128
    x = torch.randn(tokens, dim, device=DEV, dtype=torch.bfloat16)
    w_in = torch.randn(e, 2 * hid, dim, device=DEV, dtype=torch.bfloat16)
    w_out = torch.randn(e, dim, hid, device=DEV, dtype=torch.bfloat16)
    packed = MXFP8ExpertWeights(w_in, w_out)
    assert packed.in_fwd[0].shape == (e, 2 * hid, dim) and packed.in_dgrad[0].shape == (e, dim, 2 * hid)
    assert packed.out_fwd[0].shape == (e, dim, hid) and packed.out_dgrad[0].shape == (e, hid, dim)
    assert packed.in_fwd[0].dtype == F8 and packed.in_fwd[1].dtype == torch.uint8
    tok = torch.arange(tokens, device=DEV, dtype=torch.int32)
    off = torch.tensor([0, 32, 64], device=DEV, dtype=torch.int32)
    gate = torch.ones(tokens, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        mxfp8_moe_experts(x.float(), w_in, w_out, gate, tok, tok, off, packed)
    with pytest.raises(ValueError):
        mxfp8_moe_experts(x.t().contiguous().t(), w_in[:, :, :64], w_out, gate, tok, tok, off, packed)
    with pytest.raises(ValueError):
        mxfp8_moe_experts(torch.randn(dim, tokens, device=DEV, dtype=torch.bfloat16).t(), w_in, w_out, gate, tok, tok, off, packed)
    with pytest.raises(ValueError):
        mxfp8_moe_experts(x, w_in, w_out, gate, tok, tok[:10], off, packed)
    y = mxfp8_moe_experts(x, w_in, w_out, gate, tok, tok, off, packed)  # no grad needed: inference path
    assert y.grad_fn is None and y.shape == (tokens, dim)


def test_moe_module_swap_and_train_step(oracle):
    """MoEMLP built from a reference-style spec, through swap_mxfp8: declaration protocol, MXFP8 vs 16-bit outputs, refresh contract."""
    from kohakuwullm_amd.models.moe import MoEMLP, expert_sort
    from kohakuwullm_amd.models.mxfp8_swap import refresh_mxfp8_weights, swap_mxfp8
    from kohakuwullm_amd.registry import MLP, build

    torch.manual_seed(0)
    spec = {"name": "moe", "hidden": 128, "num_experts": 8, "top_k": 2, "num_shared": 0, "score_func": "softmax",
            "bias_update_rate": 0.0}
    moe = build(spec, MLP, dim=256).to(DEV, torch.bfloat16)
    x = torch.randn(4, 96, 256, device=DEV, dtype=torch.bfloat16)
    y_eager = moe(x)
    report = swap_mxfp8(moe)
    assert not report.blocking, report.summary()
    assert sorted(report.swapped) == ["w_in", "w_out"] and report.by_design == ["router.weight"]
    assert report.mac["fp8"] == 2 * (2 * 128 * 256 + 256 * 128)
    assert refresh_mxfp8_weights(moe) == 1
    assert list(moe.state_dict()) == ["w_in", "w_out", "router.weight"]
    xg = x.clone().requires_grad_(True)
    y = moe(xg)
    assert y.shape == x.shape and oracle.rel_error(y.float().cpu(), y_eager.float().cpu()) < 0.08
    y.float().square().mean().backward()
    for name in ("w_in", "w_out"):
        grad = getattr(moe, name).grad
        assert grad is not None and grad.abs().sum() > 0
    assert moe.router.weight.grad is not None and xg.grad.abs().sum() > 0
    moe.float()
    assert moe._packed is None
    # the unfused path is selected before conversion
    moe2 = MoEMLP(256, hidden=128, num_experts=8, top_k=2, num_shared=0).to(DEV, torch.bfloat16)
    moe2.mxfp8_expert_path = "unfused"
    swap_mxfp8(moe2)
    assert moe2._routed == moe2._routed_mxfp8_unfused and moe2(x).shape == x.shape
    bad = MoEMLP(256, hidden=48, num_experts=4, top_k=2, num_shared=0).to(DEV)
    assert swap_mxfp8(bad).blocking
    # dispatch format: stable order inside an expert, offsets = cumsum(counts)
    idx = torch.tensor([2, 0, 2, 1, 0, 2], device=DEV)
    counts = torch.tensor([2, 1, 3], device=DEV, dtype=torch.int32)
    offsets, order, token_of, _ = expert_sort(idx, counts, 2, 3)
    assert offsets.tolist() == [0, 2, 3, 6] and order.tolist() == [1, 4, 3, 0, 2, 5] and token_of.tolist() == [0, 2, 1, 0, 1, 2]


def test_moe_module_reference_defaults(oracle):
    """The reference's defaults: one shared expert (a GLUMLP the swap converts too), sigmoid scores with the balancing
    bias, master weights in fp32 under bf16 autocast, a router that reads another tensor, both MXFP8 paths."""
    from kohakuwullm_amd.kernels.mxfp8.linear import MXFP8Linear
    from kohakuwullm_amd.models.moe import MoEMLP
    from kohakuwullm_amd.models.mxfp8_swap import refresh_mxfp8_weights, swap_mxfp8

    torch.manual_seed(1)
    moe = MoEMLP(256, hidden=128, num_experts=16, top_k=4, aux_loss_weight=0.01, z_loss_weight=1e-3).to(DEV)
    assert moe.shared is not None and moe.shared.hidden == 128 and moe.num_buckets == 16 and not moe._has_sentinel
    assert list(moe.state_dict()) == ["w_in", "w_out", "router.weight", "router.expert_bias", "router.load_accum",
                                      "shared.w_in.weight", "shared.w_out.weight"]
    assert moe.emits_router_loss and moe.active_parameters() == 4 * 3 * 128 * 256 + 16 * 256 + 3 * 128 * 256
    x = torch.randn(200, 256, device=DEV)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y16 = moe(x)
    report = swap_mxfp8(moe)
    assert not report.blocking, report.summary()
    assert isinstance(moe.shared.w_in, MXFP8Linear) and isinstance(moe.shared.w_out, MXFP8Linear)
    assert refresh_mxfp8_weights(moe) == 3  # the routed experts and the two shared projections
    for path in ("fused", "unfused"):
        moe.mxfp8_expert_path = path
        moe.enable_mxfp8()
        xg = x.clone().requires_grad_(True)
        with torch.autocast("cuda", dtype=torch.bfloat16):
            y = moe(xg)
            aux = moe.router_losses()
        assert y.dtype == torch.bfloat16 and oracle.rel_error(y.float().cpu(), y16.float().cpu()) < 0.08, path
        assert aux is not None and aux.requires_grad
        (y.float().square().mean() + aux).backward()
        assert moe.w_in.grad.dtype == torch.float32 and moe.w_in.grad.abs().sum() > 0 and xg.grad.abs().sum() > 0
        assert moe.router.weight.grad.abs().sum() > 0 and moe.shared.w_in.weight.grad.abs().sum() > 0
        moe.zero_grad()
    # the balancing bias moves once per optimizer step and the load counter is cleared
    stats = moe.router.update_bias()
    assert stats.shape == (3,) and moe.router.load_accum.sum() == 0 and moe.router.expert_bias.abs().max() > 0
    # the router may read another tensor than the experts do
    route_on = torch.randn(200, 256, device=DEV)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        assert not torch.equal(moe(x, route_on=route_on), moe(x))
    # outside autocast the sum of the routed and the shared branch takes the promoted dtype, as in the reference's
    # forward: fp32 activations through the 16-bit arm stay fp32; the MXFP8 arm refuses them (the compute dtype is the
    # caller's to choose) and answers 16-bit activations of a 16-bit module in kind
    plain = MoEMLP(256, hidden=128, num_experts=16, top_k=4).to(DEV)
    assert plain(x).dtype == torch.float32
    plain.enable_mxfp8()
    with pytest.raises(ValueError, match="compute dtype"):
        plain(x)
    assert plain.to(torch.bfloat16)(x.bfloat16()).dtype == torch.bfloat16
    # the per-expert loop is the eager test arm: the swap refuses it and says why
    loop = MoEMLP(256, hidden=128, num_experts=4, top_k=2, num_shared=0, dense_fallback=True).to(DEV)
    rep = swap_mxfp8(loop)
    assert rep.blocking and any("dense_fallback" in why for _, why in rep.skipped)


@pytest.mark.parametrize("counts,hid", [([200, 0, 56, 300], 160), ([1, 700], 544), ([130] * 5, 256), ([90], 64)])
def test_token_axis_operands_stage_major_are_the_same_bytes(counts, hid):
    """Every writer of a token-axis code matrix (the grouped quantizer with its three sources, GEMM1's and GEMM2-dgrad's
    epilogues) can lay it out stage-major, (Mpad // 128, rows, 128), and the expert WGRAD reads either layout per
    operand: the panels hold the row-major bytes, nothing is written past the experts' tiles, scales are untouched and
    dW is bit-identical whichever way each operand is stored."""
    from kohakuwullm_amd.kernels.mxfp8.grouped import (
        grouped_mxfp8_wgrad, padded_rows, quantize_mx_cols_grouped, token_axis_buffers)
    from kohakuwullm_amd.kernels.mxfp8.moe import MXFP8ExpertWeights, launch_gemm1, launch_gemm2_dgrad
    from kohakuwullm_amd.kernels.mxfp8.quantize import quantize_mx, rows_of_stage_major

    g = torch.Generator().manual_seed(SEED + 12)
    e, dim, top_k = len(counts), 256, 1
    tokens = sum(counts) + 24
    offsets, order, token_of = (t.to(DEV) for t in _routing(counts, top_k, tokens))
    m = sum(counts)
    mpad = padded_rows(m, e)
    x = torch.randn(tokens, dim, generator=g).bfloat16().to(DEV)
    dout = torch.randn(tokens, dim, generator=g).bfloat16().to(DEV)
    gate = (torch.rand(tokens, generator=g) * 0.5 + 0.5).bfloat16().to(DEV)
    packed = MXFP8ExpertWeights((torch.randn(e, 2 * hid, dim, generator=g) * 0.06).bfloat16().to(DEV),
                                (torch.randn(e, dim, hid, generator=g) * 0.06).bfloat16().to(DEV))
    xq, xs = quantize_mx(x)
    dq, ds = quantize_mx(dout)

    def run(stage_major):
        z = lambda *shape, dtype=torch.uint8: torch.zeros(*shape, device=DEV, dtype=dtype)  # noqa: E731

        def zeroed(rows):
            q, s = token_axis_buffers(rows, mpad, DEV, stage_major)
            q.view(torch.uint8).zero_()
            s.zero_()
            return q, s

        hq, hs, pre = z(m, hid, dtype=F8), z(m, hid // 32), z(m, 2 * hid, dtype=torch.bfloat16)
        htq, hts = zeroed(hid)
        launch_gemm1(xq, xs, token_of, *packed.in_fwd, hq, hs, pre, offsets, hid, dim, torch.bfloat16, htq, hts)
        dpre, dpq, dps = z(m, 2 * hid, dtype=torch.bfloat16), z(m, 2 * hid, dtype=F8), z(m, 2 * hid // 32)
        ptq, pts = zeroed(2 * hid)
        dgate = z(tokens, dtype=torch.float32)
        launch_gemm2_dgrad(dq, ds, token_of, order, gate, *packed.out_dgrad, hq, hs, pre, dpre, dpq, dps, dgate, offsets, ptq, pts)
        dtq, dts = quantize_mx_cols_grouped(dout, offsets, m, index=token_of, row_scale=gate, scale_index=order,
                                            stage_major=stage_major)
        xtq, xts = quantize_mx_cols_grouped(x, offsets, m, index=token_of, stage_major=stage_major)
        rtq, rts = quantize_mx_cols_grouped(pre, offsets, m, swiglu=True, stage_major=stage_major)
        torch.cuda.synchronize()
        return {"h": (htq, hts), "dpre": (ptq, pts), "dout": (dtq, dts), "x": (xtq, xts), "h from pre": (rtq, rts)}

    rows, panels = run(False), run(True)
    valid = torch.zeros(mpad, dtype=torch.bool)
    pos = 0
    for c in counts:
        tiles = -(-c // 128)
        valid[pos : pos + tiles * 128] = True
        pos += tiles * 128
    for name in rows:
        (rq, rs), (pq, ps) = rows[name], panels[name]
        assert pq.dim() == 3 and pq.shape == (mpad // 128, rq.shape[0], 128), name
        flat = rows_of_stage_major(pq).view(torch.uint8).cpu()
        assert torch.equal(flat[:, valid], rq.view(torch.uint8).cpu()[:, valid]), name
        assert torch.equal(ps.cpu()[:, valid.view(-1, 32)[:, 0]], rs.cpu()[:, valid.view(-1, 32)[:, 0]]), name
        if name in ("h", "dpre"):  # these buffers were zeroed: nothing lands past the experts' tiles
            assert not flat[:, ~valid].any(), name
    # dW_out = dout^T h and dW_in = dpre^T x with each operand in either layout
    for a, b in (("dout", "h"), ("dpre", "x")):
        want = grouped_mxfp8_wgrad(*rows[a], *rows[b], offsets, m)
        for la, lb in ((panels, panels), (panels, rows), (rows, panels)):
            assert torch.equal(grouped_mxfp8_wgrad(*la[a], *lb[b], offsets, m), want), (a, b)
