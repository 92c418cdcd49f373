"""The opaque custom operators: fake kernels (shapes, dtypes, devices) without a GPU, schema and
fake-vs-real agreement plus equality with the eager functions on the GPU."""

import pytest
import torch
from torch._subclasses.fake_tensor import FakeTensorMode

F8 = torch.float8_e4m3fn
NAMES = ["combine_routed", "expert_sort", "grouped_mxfp8_gemm", "mxfp8_matmul_pq", "quantize_mx", "quantize_mx_cols",
         "quantize_mx_dual", "rms_norm_mx", "swiglu_mx"]


def _meta(t):
    return tuple(t.shape), t.dtype, t.device.type


def test_every_operator_is_registered_with_a_fake_kernel():
    import kohakuwullm_amd.ops as ops

    assert sorted(ops.__all__) == NAMES
    ns = torch.ops.kohakuwullm_amd
    with FakeTensorMode():
        x = torch.empty(64, 256, dtype=torch.bfloat16, device="cuda")
        w = torch.empty(256, dtype=torch.bfloat16, device="cuda")
        q, s = ns.quantize_mx(x)
        assert _meta(q) == ((64, 256), F8, "cuda") and _meta(s) == ((64, 8), torch.uint8, "cuda")
        qt, st = ns.quantize_mx_cols(x)
        assert _meta(qt) == ((256, 64), F8, "cuda") and _meta(st) == ((256, 2), torch.uint8, "cuda")
        assert [_meta(t) for t in ns.quantize_mx_dual(x)] == [_meta(q), _meta(s), _meta(qt), _meta(st)]
        assert _meta(ns.mxfp8_matmul_pq(q, s, q, s)) == ((64, 64), torch.bfloat16, "cuda")
        assert _meta(ns.mxfp8_matmul_pq(q, s, q, s, torch.float32)) == ((64, 64), torch.float32, "cuda")
        assert [_meta(t) for t in ns.swiglu_mx(x, x)] == [_meta(q), _meta(s)]
        out, nq, ns_ = ns.rms_norm_mx(x, w)
        assert _meta(out) == ((64, 256), torch.bfloat16, "cuda") and _meta(nq) == _meta(q) and _meta(ns_) == _meta(s)
        wq = torch.empty(4, 128, 256, dtype=F8, device="cuda")
        ws = torch.empty(4, 128, 8, dtype=torch.uint8, device="cuda")
        offsets = torch.empty(5, dtype=torch.int32, device="cuda")
        index = torch.empty(96, dtype=torch.int32, device="cuda")
        assert _meta(ns.grouped_mxfp8_gemm(q, s, wq, ws, offsets)) == ((64, 128), torch.bfloat16, "cuda")
        assert _meta(ns.grouped_mxfp8_gemm(q, s, wq, ws, offsets, index)) == ((96, 128), torch.bfloat16, "cuda")
        flat = torch.empty(192, dtype=torch.int64, device="cuda")
        counts = torch.empty(4, dtype=torch.int32, device="cuda")
        offs, order, token_of, most = ns.expert_sort(flat, counts, 3, 4)
        assert [_meta(t) for t in (offs, order, token_of, most)] == [((n,), torch.int32, "cuda") for n in (5, 192, 192, 1)]
        rows = torch.empty(192, 256, dtype=torch.bfloat16, device="cuda")
        gate = torch.empty(192, dtype=torch.float32, device="cuda")
        assert _meta(ns.combine_routed(rows, gate, order, token_of, 64)) == ((64, 256), torch.bfloat16, "cuda")


@pytest.mark.gpu
def test_operators_agree_with_the_eager_functions():
    import kohakuwullm_amd.ops  # noqa: F401  (registers the operators)
    from kohakuwullm_amd.kernels.elementwise import rms_norm_mx
    from kohakuwullm_amd.kernels.moe import combine_routed, expert_counts, expert_sort
    from kohakuwullm_amd.kernels.mxfp8 import mxfp8_matmul_pq, quantize_mx, quantize_mx_cols, quantize_mx_dual
    from kohakuwullm_amd.kernels.mxfp8.fused_act import swiglu_mx
    from kohakuwullm_amd.kernels.mxfp8.grouped import grouped_mxfp8_gemm

    dev = "cuda:0"
    ns = torch.ops.kohakuwullm_amd
    g = torch.Generator(device=dev).manual_seed(7)
    x = torch.randn(128, 256, device=dev, generator=g).bfloat16()
    w = torch.randn(256, device=dev, generator=g).bfloat16()
    # the schema check hashes every tensor with arithmetic that fp8 tensors do not support: operators
    # that take or return e4m3 get the fake-vs-real comparison only
    checks = ("test_faketensor",)
    plain = ("test_schema", "test_faketensor")

    def same(a, b):
        a, b = (a, b) if isinstance(a, (tuple, list)) else ((a,), (b,))
        assert len(a) == len(b)
        for s, t in zip(a, b):
            assert s.dtype == t.dtype and torch.equal(s.view(torch.uint8) if s.dtype == F8 else s, t.view(torch.uint8) if t.dtype == F8 else t)

    for op, fn, args in (
        (ns.quantize_mx, quantize_mx, (x,)),
        (ns.quantize_mx_cols, quantize_mx_cols, (x,)),
        (ns.quantize_mx_dual, quantize_mx_dual, (x,)),
        (ns.swiglu_mx, swiglu_mx, (x, x.flip(0))),
        (ns.rms_norm_mx, rms_norm_mx, (x, w, 1e-6)),
    ):
        same(op(*args), fn(*args))
        torch.library.opcheck(op, args, test_utils=checks)
    q, s = quantize_mx(x)
    same(ns.mxfp8_matmul_pq(q, s, q, s), mxfp8_matmul_pq(q, s, q, s))
    torch.library.opcheck(ns.mxfp8_matmul_pq, (q, s, q, s, torch.float32), test_utils=checks)
    wq, ws = quantize_mx(torch.randn(4 * 128, 256, device=dev, generator=g).bfloat16())
    wq, ws = wq.view(4, 128, 256), ws.view(4, 128, 8)
    offsets = torch.tensor([0, 40, 40, 100, 128], dtype=torch.int32, device=dev)
    same(ns.grouped_mxfp8_gemm(q, s, wq, ws, offsets), grouped_mxfp8_gemm(q, s, wq, ws, offsets))
    torch.library.opcheck(ns.grouped_mxfp8_gemm, (q, s, wq, ws, offsets), test_utils=checks)
    flat = torch.randint(0, 4, (128 * 3,), device=dev, generator=g)
    counts = expert_counts(flat, 4)
    same(ns.expert_sort(flat, counts, 3, 4), expert_sort(flat, counts, 3, 4))
    torch.library.opcheck(ns.expert_sort, (flat, counts, 3, 4), test_utils=plain)
    _, order, token_of, _ = expert_sort(flat, counts, 3, 4)
    rows = torch.randn(384, 256, device=dev, generator=g).bfloat16()
    gate = torch.rand(384, device=dev, generator=g)
    same(ns.combine_routed(rows, gate, order, token_of, 128), combine_routed(rows, gate, order, token_of, 128))
    torch.library.opcheck(ns.combine_routed, (rows, gate, order, token_of, 128), test_utils=plain)
