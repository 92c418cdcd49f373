"""Host-side logic that needs no GPU: registry, swap accounting, module contracts, error behaviour, oracle GEMMs."""

import pytest
import torch
import torch.nn as nn

from conftest import SEED


def test_registry_build_forms():
    from kohakuwullm_amd.registry import MLP, Registry, build, import_class, resolve

    reg = Registry("thing")

    @reg.register("a")
    class A:
        def __init__(self, x=1, y=2):
            self.x, self.y = x, y

    with pytest.raises(KeyError):
        reg.register("a")(A)
    with pytest.raises(KeyError):
        reg.get("missing")
    assert build(None, reg) is None
    assert build("a", reg, x=5).x == 5
    assert build({"name": "a", "y": 7}, reg, x=3).y == 7
    assert build(A, reg, x=9).x == 9
    inst = A()
    assert build(inst, reg) is inst
    assert isinstance(build("torch.nn.Identity", None), nn.Identity)
    with pytest.raises(ValueError):
        resolve("a", None)
    assert import_class("torch.nn.Linear") is nn.Linear and import_class(3) == 3
    assert "swiglu" in __import__("kohakuwullm_amd.models.mlp", fromlist=["x"]).MLP and "swiglu" in MLP.keys()

    class Spec:
        def build(self):
            return "built"

    assert build(Spec(), reg) == "built"


class _StubLinear(nn.Linear):
    """Stands in for MXFP8Linear so the surgery runs on the CPU."""

    def __init__(self, in_features, out_features, dtype=None):
        super().__init__(in_features, out_features, bias=False, dtype=dtype)
        self.refreshed = 0

    def refresh_quantized_weight(self):
        self.refreshed += 1


def test_swap_accounting_on_cpu():
    from kohakuwullm_amd.models.mlp import AttentionProjections, SwiGLU
    from kohakuwullm_amd.models.mxfp8_swap import Matmul, refresh_mxfp8_weights, swap_mxfp8

    class Declares(nn.Module):
        def __init__(self, refusal=None, convert=True):
            super().__init__()
            self.w = nn.Parameter(torch.zeros(8, 8))
            self.r = nn.Parameter(torch.zeros(4, 8))
            self._refusal = refusal
            self.enabled = False
            if convert:
                self.enable_mxfp8 = self._enable

        def mxfp8_matmul(self):
            return {"w": Matmul(64, self._refusal), "r": Matmul(32, "router", never=True)}

        def _enable(self):
            self.enabled = True
            self.refresh_quantized_weight = lambda: None

    class Model(nn.Module):
        def __init__(self):
            super().__init__()
            self.attn = AttentionProjections(128, 2, 1, 64)
            self.mlp = SwiGLU(128, hidden=256)
            self.biased = SwiGLU(128, hidden=128, bias=True)
            self.ok = Declares()
            self.refused = Declares(refusal="shape")
            self.unreached = Declares(convert=False)
            self.emb = nn.Embedding(10, 128)
            self.stray = nn.Parameter(torch.zeros(3, 3))

    model = Model()
    report = swap_mxfp8(model, linear_cls=_StubLinear)
    assert isinstance(model.mlp.w_in, _StubLinear) and isinstance(model.attn.q_proj, _StubLinear)
    assert isinstance(model.biased.w_in, nn.Linear) and not isinstance(model.biased.w_in, _StubLinear)
    assert {n for n, _ in report.skipped} == {"biased.w_in", "biased.w_out", "refused.w"}
    assert [n for n, _ in report.unreached] == ["unreached.w"]
    assert report.unaccounted == ["stray(3, 3)"]
    assert model.ok.enabled and "ok" in report.modules and "ok.w" in report.swapped
    assert set(report.by_design) == {"ok.r", "refused.r", "unreached.r", "emb.weight"}
    assert report.blocking
    assert report.mac["fp8"] == 128 * 128 + 2 * 128 * 64 + 128 * 128 + 3 * 128 * 256 + 64
    assert report.mac["skipped"] == 3 * 128 * 128 + 64 and report.mac["unreached"] == 64 and report.mac["never"] == 96
    assert abs(sum(report.share(b) for b in ("fp8", "skipped", "unreached", "never")) - 1.0) < 1e-9
    assert "[skipped] biased.w_in: has a bias" in report.summary() and "[unaccounted] stray(3, 3)" in report.summary()
    # 6 swapped linears + the declaring module that converted
    assert refresh_mxfp8_weights(model) == 7 and model.mlp.w_in.refreshed == 1
    # scope: everything outside is reported, left alone, and does not block
    m2 = Model()
    r2 = swap_mxfp8(m2, linear_cls=_StubLinear, scope=("attn.",))
    assert isinstance(m2.attn.k_proj, _StubLinear) and not isinstance(m2.mlp.w_in, _StubLinear)
    assert "mlp.w_in" in r2.out_of_scope and "ok.w" in r2.out_of_scope
    r3 = swap_mxfp8(Model(), linear_cls=_StubLinear, convert_declared=False)
    assert {"ok.w", "unreached.w"} <= {n for n, _ in r3.unreached}


def test_swap_leaves_the_lm_head_alone():
    """A backbone with an LM head (a bare (vocab, dim) ``projection`` on a module whose class is called LMHead, as the
    reference's): the head is 16-bit by design, charged to `never`, and does not block the swap."""
    from kohakuwullm_amd.models.mlp import SwiGLU
    from kohakuwullm_amd.models.mxfp8_swap import swap_mxfp8

    class LMHead(nn.Module):
        def __init__(self, vocab, dim):
            super().__init__()
            self.projection = nn.Parameter(torch.zeros(vocab, dim))

    class NotAHead(nn.Module):  # the same tensor under another class name is nobody's: it blocks
        def __init__(self):
            super().__init__()
            self.projection = nn.Parameter(torch.zeros(5, 128))

    class Backbone(nn.Module):
        def __init__(self, head):
            super().__init__()
            self.mlp = SwiGLU(128, hidden=256)
            self.head = head

    report = swap_mxfp8(Backbone(LMHead(1000, 128)), linear_cls=_StubLinear)
    assert not report.blocking and report.by_design == ["head.projection"] and report.mac["never"] == 1000 * 128
    other = swap_mxfp8(Backbone(NotAHead()), linear_cls=_StubLinear)
    assert other.blocking and other.unaccounted == ["head.projection(5, 128)"]


def test_module_contracts_without_gpu():
    from kohakuwullm_amd._lib import MXFP8LibraryError
    from kohakuwullm_amd.kernels.mxfp8 import mxfp8_matmul_pq, quantize_mx
    from kohakuwullm_amd.kernels.mxfp8.linear import MXFP8Linear, _PadLastAxis
    from kohakuwullm_amd.kernels.mxfp8.moe import _validate_expert_call
    from kohakuwullm_amd.models.mlp import MXFP8SwiGLU, resolve_hidden

    with pytest.raises(ValueError, match="multiple of 128"):
        MXFP8Linear(96, 128)
    lin = MXFP8Linear(128, 200)
    assert lin.padded_out_features == 256 and lin._pad_k.width == 56 and lin.weight.shape == (200, 128)
    assert _PadLastAxis(0)(lin.weight) is lin.weight and _PadLastAxis(3)(torch.zeros(2, 5)).shape == (2, 8)
    assert list(lin.state_dict()) == ["weight"]
    with pytest.raises(MXFP8LibraryError, match="no CPU path"):
        lin(torch.zeros(4, 128, dtype=torch.bfloat16))
    with pytest.raises(ValueError):
        quantize_mx(torch.zeros(4, 48, dtype=torch.bfloat16))
    with pytest.raises(MXFP8LibraryError):
        quantize_mx(torch.zeros(4, 64, dtype=torch.bfloat16))
    with pytest.raises(ValueError):
        mxfp8_matmul_pq(torch.zeros(4, 64, dtype=torch.uint8), torch.zeros(4, 2, dtype=torch.uint8),
                        torch.zeros(4, 32, dtype=torch.uint8), torch.zeros(4, 1, dtype=torch.uint8))
    assert resolve_hidden(1536, 4.0) == 4096 and resolve_hidden(100, 4.0, hidden=77) == 77
    mlp = MXFP8SwiGLU(256, hidden=96)
    assert set(mlp.mxfp8_matmul()) == {"w_in", "w_out"} and mlp.mxfp8_matmul()["w_in"].refusal is None
    assert MXFP8SwiGLU(256, hidden=40).mxfp8_matmul()["w_in"].refusal is not None
    x = torch.zeros(8, 64, dtype=torch.bfloat16)
    w_in, w_out = torch.zeros(2, 128, 64), torch.zeros(2, 64, 64)
    tok = torch.zeros(8, dtype=torch.int32)
    assert _validate_expert_call(x, w_in, w_out, tok, tok) == 64
    for bad in ((x.float(), w_in, w_out, tok, tok), (x, w_in[:, :100], w_out, tok, tok), (x, w_in, w_out, tok, tok[:3]),
                (x[:, :32], w_in, w_out, tok, tok), (torch.zeros(64, 8, dtype=torch.bfloat16).t(), w_in, w_out, tok, tok)):
        with pytest.raises(ValueError):
            _validate_expert_call(*bad)


def test_oracle_gemm_matches_scalar_and_grouped_loop(oracle):
    g = torch.Generator().manual_seed(SEED)
    a = torch.randn(24, 96, generator=g).bfloat16()
    b = (torch.randn(3 * 16, 96, generator=g) * 0.1).bfloat16()
    aq, as_ = oracle.quantize_rows(a)
    bq, bs = oracle.quantize_rows(b)
    full = oracle.gemm_nt(aq, as_, bq, bs)
    assert oracle.rel_error(full, oracle.gemm_nt_scalar(aq, as_, bq, bs)) < 1e-14
    # exact special case: codes 1.0 and power-of-two scales give integer sums
    ones = torch.full((4, 64), 0x38, dtype=torch.uint8)
    s = torch.tensor([[127, 128]] * 4, dtype=torch.uint8)
    assert torch.equal(oracle.gemm_nt(ones, s, ones, s), torch.full((4, 4), 32.0 + 32 * 4, dtype=torch.float64))
    # grouped = loop of dense products over the offset table, ragged and empty experts, with a gather
    offsets = torch.tensor([0, 5, 5, 24], dtype=torch.int32)
    wq, ws = bq.view(3, 16, 96), bs.view(3, 16, 3)
    idx = torch.randperm(24, generator=g).int()
    got = oracle.grouped_gemm_nt(aq, as_, wq, ws, offsets, idx)
    ad = oracle.dequant(aq, as_)[idx.long()]
    ref = torch.cat([ad[0:5] @ oracle.dequant(wq[0], ws[0]).T, ad[5:24] @ oracle.dequant(wq[2], ws[2]).T])
    assert torch.equal(got, ref)
    # quantization error of a randn x randn/10 product is the e4m3 figure the reference reports (~3.75e-2)
    exact = a.double() @ b.double().T
    assert 0.02 < oracle.rel_error(full, exact) < 0.06
    dw = oracle.grouped_wgrad(a, a, offsets)
    assert dw.shape == (3, 96, 96) and (dw[1] == 0).all()
    assert torch.allclose(dw[0], a[:5].double().T @ a[:5].double())


def test_moe_block_builds_from_a_reference_spec():
    """``build({"name": "moe", ...}, MLP, dim=...)`` with the reference's keywords; ``swap_mxfp8`` converts the result.

    Nothing here runs a kernel: building, declaring and converting are host logic.
    """
    from kohakuwullm_amd.models.mlp import GLUMLP
    from kohakuwullm_amd.models.moe import MoEMLP, TopKRouter
    from kohakuwullm_amd.models.mxfp8_swap import swap_mxfp8
    from kohakuwullm_amd.registry import MLP, ROUTER, build

    assert "moe" in MLP and "swiglu" in MLP and "topk" in ROUTER
    spec = {"name": "moe", "hidden": 512, "num_experts": 64, "top_k": 6, "num_shared": 0}
    moe = build(spec, MLP, dim=1024)
    assert isinstance(moe, MoEMLP) and isinstance(moe.router, TopKRouter)
    assert moe.w_in.shape == (64, 1024, 1024) and moe.w_out.shape == (64, 1024, 512) and moe.shared is None
    assert moe.router.weight.shape == (64, 1024) and moe.router.top_k == 6 and moe.num_buckets == 64
    report = swap_mxfp8(moe, linear_cls=_StubLinear)
    assert not report.blocking and sorted(report.swapped) == ["w_in", "w_out"] and report.modules == [""]
    assert moe._routed == moe._routed_mxfp8 and callable(moe.refresh_quantized_weight)
    assert report.mac["fp8"] == 6 * 3 * 512 * 1024 and report.mac["never"] == 64 * 1024

    # every keyword of the reference's constructor, a router given as a spec with its own keywords
    full = build({"name": "moe", "ratio": 2.0, "multiple_of": 64, "num_experts": 8, "top_k": 2, "num_shared": 2, "bias": False,
                  "router": {"name": "topk", "score_func": "softmax"}, "router_dim": 96, "dense_fallback": False,
                  "expert_path": "eager", "n_groups": 2, "topk_groups": 1, "bias_update_rate": 0.0}, MLP, dim=256)
    assert full.hidden == 384 and isinstance(full.shared, GLUMLP) and full.shared.hidden == 768
    assert full.router.weight.shape == (8, 96) and full.router.n_groups == 2 and full.router.expert_bias is None
    assert full.expert_path == "eager" and not full.emits_router_loss and full.router_losses() is None
    idx, weight, counts = full.router.route(torch.randn(50, 96))
    assert idx.shape == (50, 2) and int(counts.sum()) == 100
    assert torch.allclose(weight.sum(-1), torch.ones(50), atol=1e-5)
    assert ((idx[:, 0] // 4) == (idx[:, 1] // 4)).all()  # one group of four experts per token
    report = swap_mxfp8(full, linear_cls=_StubLinear)
    assert not report.blocking and {"w_in", "w_out", "shared.w_in", "shared.w_out"} == set(report.swapped)
    with pytest.raises(ValueError, match="expert_path"):
        build({"name": "moe", "expert_path": "triton"}, MLP, dim=128)
    with pytest.raises(ValueError, match="score_func"):
        build({"name": "moe", "score_func": "relu"}, MLP, dim=128)
    loop = build({"name": "moe", "hidden": 128, "num_experts": 4, "top_k": 2, "dense_fallback": True}, MLP, dim=128)
    assert "dense_fallback" in loop.mxfp8_matmul()["w_in"].refusal
