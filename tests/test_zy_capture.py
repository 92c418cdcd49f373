"""Work on a stream that is being captured into a HIP graph is refused, not recorded.

Recording this library's launches ended the process inside graph instantiation (cause not established), so
every entry point asks the runtime whether its stream is capturing and returns MX_ECAPTURE before it launches
anything.  What is captured here is therefore an EMPTY graph: the test checks the refusal and that the library
works as before afterwards.  The file sorts behind the other tests on purpose.
"""

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def test_entry_points_refuse_a_capturing_stream():
    from kohakuwullm_amd import _lib
    from kohakuwullm_amd.kernels.elementwise import rms_norm_mx
    from kohakuwullm_amd.kernels.moe import expert_counts
    from kohakuwullm_amd.kernels.mxfp8.fused_act import swiglu_mx
    from kohakuwullm_amd.kernels.mxfp8.quantize import mxfp8_matmul_pq, mxfp8_matmul_pq_batch, quantize_mx, quantize_mx_dual

    torch.manual_seed(0)
    x = torch.randn(256, 256, device=DEV, dtype=torch.bfloat16)
    w = torch.ones(256, device=DEV, dtype=torch.bfloat16)
    picks = torch.randint(0, 8, (512,), device=DEV)
    q, s = quantize_mx(x)
    before = mxfp8_matmul_pq(q, s, q, s)
    calls = {
        "quantize_mx": lambda: quantize_mx(x),
        "quantize_mx_dual": lambda: quantize_mx_dual(x),
        "swiglu_mx": lambda: swiglu_mx(x, x),
        "mxfp8_matmul_pq": lambda: mxfp8_matmul_pq(q, s, q, s),
        "mxfp8_matmul_pq_batch": lambda: mxfp8_matmul_pq_batch([(q, s, q, s), (q, s, q, s)]),
        "rms_norm_mx": lambda: rms_norm_mx(x, w, 1e-6),
        "expert_counts": lambda: expert_counts(picks, 8),
    }
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    refused = []
    with torch.cuda.graph(graph):
        for name, call in calls.items():
            with pytest.raises(_lib.MXFP8LibraryError, match="captured"):
                call()
            refused.append(name)
    torch.cuda.synchronize()
    assert refused == list(calls)
    after = mxfp8_matmul_pq(*quantize_mx(x), q, s)
    assert torch.equal(after, before)
