"""MXFP8Linear, the fused SwiGLU feed-forward and the swap, against the CPU oracle.

Every product is compared with dequantize-then-matmul (fp64) on operands the ORACLE
quantized from the same bf16 inputs; tolerance 1e-2 relative Frobenius, bf16 outputs.
"""

import copy
import pickle

import pytest
import torch
import torch.nn as nn

from conftest import SEED
from mx_checks import assert_codes_equal_up_to_ties

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL = 1e-2


def _draw(*shapes_scales, seed=SEED):
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(*shape, generator=g) * scale).bfloat16() for shape, scale in shapes_scales]


def _linear_refs(ora, x2d, w, dy2d, pad=0):
    """fwd, dgrad, wgrad of one linear by the oracle (K-blocked operands for each product)."""
    xq, xs = ora.quantize_rows(x2d)
    wq, ws = ora.quantize_rows(w)
    y = ora.gemm_nt(xq, xs, wq, ws)
    dyp = torch.nn.functional.pad(dy2d, (0, pad))
    wtp = torch.nn.functional.pad(w.t(), (0, pad)).contiguous()
    dq, ds = ora.quantize_rows(dyp)
    wtq, wts = ora.quantize_rows(wtp)
    dx = ora.gemm_nt(dq, ds, wtq, wts)
    # token blocks of 32: a ragged last block is completed with zero rows, which add nothing to dW
    extra = -x2d.shape[0] % 32
    dtq, dts = ora.quantize_cols(torch.nn.functional.pad(dy2d, (0, 0, 0, extra)))
    xtq, xts = ora.quantize_cols(torch.nn.functional.pad(x2d, (0, 0, 0, extra)))
    dw = ora.gemm_nt(dtq, dts, xtq, xts)
    return y, dx, dw


@pytest.mark.parametrize("tokens,in_f,out_f", [(256, 512, 384), (96, 128, 200), (1000, 256, 128), (50, 128, 64)])
def test_linear_fwd_bwd(oracle, tokens, in_f, out_f):
    from kohakuwullm_amd.kernels.mxfp8.linear import MXFP8Linear

    x, w, dy = _draw(((tokens, in_f), 1.0), ((out_f, in_f), 0.02), ((tokens, out_f), 1e-2))
    lin = MXFP8Linear(in_f, out_f).to(DEV)
    assert lin.padded_out_features == -(-out_f // 128) * 128
    with torch.no_grad():
        lin.weight.copy_(w.to(DEV))
    xd = x.to(DEV).requires_grad_(True)
    out = lin(xd)
    assert out.dtype == torch.bfloat16 and out.shape == (tokens, out_f) and out.grad_fn is not None
    out.backward(dy.to(DEV))
    y, dx, dw = _linear_refs(oracle, x, w, dy, pad=lin.padded_out_features - out_f)
    assert oracle.rel_error(out.detach().cpu(), y) < TOL
    assert oracle.rel_error(xd.grad.cpu(), dx) < TOL
    assert lin.weight.grad.shape == (out_f, in_f) and lin.weight.grad.abs().sum() > 0
    assert oracle.rel_error(lin.weight.grad.cpu(), dw) < TOL


def test_linear_leading_dims_and_training_scale_grads(oracle):
    from kohakuwullm_amd.kernels.mxfp8.linear import MXFP8Linear

    x, w, dy = _draw(((4, 64, 256), 1.0), ((128, 256), 0.02), ((4, 64, 128), 2.0**-20))
    lin = MXFP8Linear(256, 128).to(DEV)
    with torch.no_grad():
        lin.weight.copy_(w.to(DEV))
    xd = x.to(DEV).requires_grad_(True)
    out = lin(xd)
    assert out.shape == (4, 64, 128)
    out.backward(dy.to(DEV))
    y, dx, dw = _linear_refs(oracle, x.reshape(-1, 256), w, dy.reshape(-1, 128))
    assert oracle.rel_error(out.detach().cpu().reshape(-1, 128), y) < TOL
    assert oracle.rel_error(xd.grad.cpu().reshape(-1, 256), dx) < TOL
    assert oracle.rel_error(lin.weight.grad.cpu(), dw) < TOL


def test_linear_module_contract():
    from kohakuwullm_amd.kernels.mxfp8.linear import MXFP8Linear

    with pytest.raises(ValueError):
        MXFP8Linear(100, 128)
    lin = MXFP8Linear(128, 256)
    assert list(lin.state_dict()) == ["weight"] and lin.weight.dtype == torch.bfloat16
    assert abs(lin.weight.float().std().item() - 128**-0.5) < 0.01
    lin = lin.to(DEV)
    x = torch.randn(32, 128, device=DEV, dtype=torch.bfloat16)
    y0 = lin(x)
    assert lin._cache is not None and len(lin._cache) == 4
    assert lin._cache[0].dtype == torch.float8_e4m3fn and lin._cache[1].dtype == torch.uint8
    assert list(lin.state_dict()) == ["weight"]  # caches are not buffers
    # a stale cache is what the module computes with until refreshed
    with torch.no_grad():
        lin.weight.mul_(2.0)
    assert torch.equal(lin(x), y0)
    lin.refresh_quantized_weight()
    assert not torch.equal(lin(x), y0)
    lin.float()  # any _apply drops the cache
    assert lin._cache is None
    lin.bfloat16()
    clone = pickle.loads(pickle.dumps(copy.deepcopy(lin)))
    assert torch.equal(clone(x), lin(x))
    # autocast decides the compute dtype, not the weight
    with torch.autocast("cuda", dtype=torch.float16):
        assert lin(x.float()).dtype == torch.float16
    # inference without grad
    with torch.no_grad():
        assert lin(x).grad_fn is None


def test_swap_and_refresh(oracle):
    from kohakuwullm_amd.kernels.mxfp8.linear import MXFP8Linear
    from kohakuwullm_amd.models.mlp import AttentionProjections, MXFP8SwiGLU, SwiGLU
    from kohakuwullm_amd.models.mxfp8_swap import refresh_mxfp8_weights, swap_mxfp8
    from kohakuwullm_amd.registry import MLP, build

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.attn = AttentionProjections(256, num_heads=4, num_kv_heads=2, head_dim=64)
            self.mlp = build("swiglu", MLP, dim=256, hidden=512)
            self.fused = build({"name": "swiglu_mxfp8", "hidden": 256}, MLP, dim=256)
            self.embed = nn.Embedding(64, 256)

    torch.manual_seed(0)
    model = Block().to(DEV).bfloat16()
    before = {k: v.clone() for k, v in model.state_dict().items()}
    report = swap_mxfp8(model)
    assert not report.blocking, report.summary()
    assert isinstance(model.mlp.w_in, MXFP8Linear) and isinstance(model.attn.k_proj, MXFP8Linear)
    assert len(report.swapped) == 8 and len(report.modules) == 7
    assert report.mac["fp8"] == 256 * (256 + 128 + 128 + 256) + 3 * 256 * 512 + 3 * 256 * 256
    after = model.state_dict()
    assert set(after) == set(before) and all(torch.equal(after[k], before[k]) for k in before)
    assert refresh_mxfp8_weights(model) == len(report.modules)
    again = swap_mxfp8(model)  # idempotent
    assert len(again.swapped) == 8 and not again.blocking
    x = torch.randn(64, 256, device=DEV, dtype=torch.bfloat16, requires_grad=True)
    q, k, v = model.attn.project(x)
    assert q.shape == (64, 4, 64) and k.shape == (64, 2, 64)
    y = model.attn.merge(q) + model.mlp(x) + model.fused(x) + k.sum() + v.sum()
    y.float().square().mean().backward()
    for name, p in model.named_parameters():
        if "embed" not in name:
            assert p.grad is not None and p.grad.abs().sum() > 0, name
    # a biased or misaligned linear is refused and blocks
    bad = SwiGLU(192, hidden=256).to(DEV).bfloat16()
    rep = swap_mxfp8(bad)
    assert rep.blocking and any("in_features=192" in why for _, why in rep.skipped)


@pytest.mark.parametrize("tokens,dim,hidden", [(256, 256, 512), (128, 128, 96), (77, 128, 64)])
def test_fused_swiglu_mlp(oracle, tokens, dim, hidden):
    from kohakuwullm_amd.kernels.mxfp8.mlp import mxfp8_swiglu_mlp
    from kohakuwullm_amd.kernels.mxfp8.quantize import quantize_mx, quantize_mx_cols

    ora = oracle
    x, w_in, w_out, dy = _draw(((tokens, dim), 1.0), ((2 * hidden, dim), 0.05), ((dim, hidden), 0.05), ((tokens, dim), 1e-2))
    xd = x.to(DEV).requires_grad_(True)
    wi = w_in.to(DEV).requires_grad_(True)
    wo = w_out.to(DEV).requires_grad_(True)
    packed = (quantize_mx(wi.detach()), quantize_mx_cols(wi.detach()), quantize_mx(wo.detach()), quantize_mx_cols(wo.detach()))
    y = mxfp8_swiglu_mlp(xd, wi, wo, packed)
    y.backward(dy.to(DEV))

    # the oracle's chain, rounding to bf16 where the device path stores bf16
    gu = ora.gemm_nt(*ora.quantize_rows(x), *ora.quantize_rows(w_in)).bfloat16()
    g, u = gu.float().chunk(2, dim=-1)
    h = g * torch.sigmoid(g) * u
    y_ref = ora.gemm_nt(*ora.quantize_rows(h), *ora.quantize_rows(w_out))
    dh = ora.gemm_nt(*ora.quantize_rows(dy), *ora.quantize_cols(w_out)).bfloat16().float()
    sg = torch.sigmoid(g)
    dpre = torch.cat([dh * u * sg * (1 + g * (1 - sg)), dh * g * sg], dim=-1)
    dx_ref = ora.gemm_nt(*ora.quantize_rows(dpre), *ora.quantize_cols(w_in))

    def tok(t):  # the token axis in whole blocks of 32: zero rows complete a ragged last block
        return torch.nn.functional.pad(t, (0, 0, 0, -t.shape[0] % 32))

    dwin_ref = ora.gemm_nt(*ora.quantize_cols(tok(dpre)), *ora.quantize_cols(tok(x)))
    dwout_ref = ora.gemm_nt(*ora.quantize_cols(tok(dy)), *ora.quantize_cols(tok(h)))
    assert ora.rel_error(y.detach().cpu(), y_ref) < TOL
    assert ora.rel_error(xd.grad.cpu(), dx_ref) < TOL
    assert ora.rel_error(wi.grad.cpu(), dwin_ref) < TOL
    assert ora.rel_error(wo.grad.cpu(), dwout_ref) < TOL

    # structural check against plain autograd in fp32 on the unquantized operands: the gap is
    # the accumulated e4m3 error of a chain of products, far below any wiring mistake
    xf, wif, wof = (t.float().requires_grad_(True) for t in (x, w_in, w_out))
    gg, uu = (xf @ wif.T).chunk(2, dim=-1)
    yf = (torch.nn.functional.silu(gg) * uu) @ wof.T
    yf.backward(dy.float())
    assert ora.rel_error(y.detach().cpu(), yf) < 0.08
    assert ora.rel_error(xd.grad.cpu(), xf.grad) < 0.12
    assert ora.rel_error(wi.grad.cpu(), wif.grad) < 0.12
    assert ora.rel_error(wo.grad.cpu(), wof.grad) < 0.12


@pytest.mark.parametrize("tokens,dim,hidden", [(384, 256, 160), (128, 128, 32), (512, 384, 256)])
def test_fused_swiglu_projection_equals_gemm_then_quantizer(tokens, dim, hidden):
    """The first projection with SwiGLU and both casts in its epilogue == GEMM, then the fused quantizer."""
    from kohakuwullm_amd.kernels.mxfp8.mlp import fused_swiglu_projection, swiglu_mx_dual
    from kohakuwullm_amd.kernels.mxfp8.quantize import mxfp8_matmul_pq, quantize_mx

    x, w_in = _draw(((tokens, dim), 1.0), ((2 * hidden, dim), 0.05))
    xq, xs = quantize_mx(x.to(DEV))
    wq, ws = quantize_mx(w_in.to(DEV))
    gu, hq, hs, htq, hts = fused_swiglu_projection(xq, xs, wq, ws, torch.bfloat16)
    gu_ref = mxfp8_matmul_pq(xq, xs, wq, ws)
    assert torch.equal(gu, gu_ref)
    for got, ref in zip((hq, hs, htq, hts), swiglu_mx_dual(gu_ref)):
        assert got.shape == ref.shape and torch.equal(got.view(torch.uint8), ref.view(torch.uint8))


def test_swiglu_dual_kernels_bitwise_vs_composition(oracle):
    """The fused SwiGLU quantizers equal quantizing the separately computed activation."""
    from kohakuwullm_amd.kernels.mxfp8.mlp import swiglu_bwd_mx_dual, swiglu_mx_dual

    (gu, dh) = _draw(((256, 512), 1.5), ((256, 256), 1e-2))
    q, s, qt, st = swiglu_mx_dual(gu.to(DEV))
    g, u = gu.float().chunk(2, dim=-1)
    h = g * torch.sigmoid(g) * u
    # hardware exp/rcp vs torch.sigmoid: only values within a few ulp of a rounding boundary may differ
    for codes, scales, vals in ((q, s, h), (qt, st, h.t().contiguous())):
        n_q, n_s = assert_codes_equal_up_to_ties(oracle, codes, scales, vals, what="swiglu dual")
        assert n_q < 5e-3 * codes.numel() and n_s < 1e-3 * scales.numel() + 1
    assert oracle.rel_error(oracle.dequant(q.view(torch.uint8).cpu(), s.cpu()), h) < 0.04
    assert oracle.rel_error(oracle.dequant(qt.view(torch.uint8).cpu(), st.cpu()), h.T) < 0.04

    pq, ps, ptq, pts = swiglu_bwd_mx_dual(dh.to(DEV), gu.to(DEV))
    sg = torch.sigmoid(g)
    dpre = torch.cat([dh.float() * u * sg * (1 + g * (1 - sg)), dh.float() * g * sg], dim=-1)
    terms = torch.cat([(dh.float() * u * sg).abs() * (1 + g.abs() * (1 - sg)), (dh.float() * g * sg).abs()], dim=-1)
    assert pq.shape == (256, 512) and ptq.shape == (512, 256)
    for codes, scales, vals, mag in ((pq, ps, dpre, terms), (ptq, pts, dpre.t().contiguous(), terms.t().contiguous())):
        n_q, n_s = assert_codes_equal_up_to_ties(oracle, codes, scales, vals, ulps=8, what="swiglu' dual", magnitude=mag)
        assert n_q < 5e-3 * codes.numel() and n_s < 1e-3 * scales.numel() + 1
    assert oracle.rel_error(oracle.dequant(pq.view(torch.uint8).cpu(), ps.cpu()), dpre) < 0.04
    assert oracle.rel_error(oracle.dequant(ptq.view(torch.uint8).cpu(), pts.cpu()), dpre.T) < 0.04


@pytest.mark.skip(
    reason="ending the capture of this step (torch.cuda.graphs capture_end -> graph instantiation) ended the process "
    "with a segmentation fault inside the HIP runtime on the test box, twice, the second time after the library "
    "stopped making any HIP call besides kernel launches on the per-launch path; cause not established, so the "
    "case stays off the GPU"
)
def test_mlp_step_under_hip_graph(oracle):
    """The fused MLP forward+backward captured in a HIP graph replays to the eager result.

    The graph is replayed several times with eager work and synchronisations in between, and
    every replay is compared: the library records no memset nodes on this path and allocates
    nothing while the stream is being captured.
    """
    from kohakuwullm_amd.kernels.mxfp8.mlp import mxfp8_swiglu_mlp
    from kohakuwullm_amd.kernels.mxfp8.quantize import quantize_mx, quantize_mx_cols

    tokens, dim, hidden = 512, 256, 384
    x, w_in, w_out, dy = _draw(((tokens, dim), 1.0), ((2 * hidden, dim), 0.05), ((dim, hidden), 0.05), ((tokens, dim), 1e-2))
    xd = x.to(DEV).requires_grad_(True)
    wi = w_in.to(DEV).requires_grad_(True)
    wo = w_out.to(DEV).requires_grad_(True)
    dyd = dy.to(DEV)
    packed = (quantize_mx(wi.detach()), quantize_mx_cols(wi.detach()), quantize_mx(wo.detach()), quantize_mx_cols(wo.detach()))

    def step():
        y = mxfp8_swiglu_mlp(xd, wi, wo, packed)
        gx, gwi, gwo = torch.autograd.grad(y, (xd, wi, wo), dyd)
        return y, gx, gwi, gwo

    eager = [t.clone() for t in step()]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):  # warm-up on the capture stream: scratch buffers are created here, not under capture
            step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        captured = step()
    for replay in range(4):
        for t in captured:
            t.fill_(float("nan")) if t.dtype != torch.uint8 else None
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(captured, eager):
            assert torch.equal(got, want), replay
        _ = [t.clone() for t in step()]  # eager work between replays
        torch.cuda.synchronize()
