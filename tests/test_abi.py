"""The C ABI: every function include/mxfp8_hip.h declares is exported, typed in the binding, and arity-checked.

No kernel runs here (no GPU needed); the library only has to load.
"""

import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "mxfp8_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    decls = {}
    for m in re.finditer(r"\b(?:int|int64_t|const char \*)\s*(mx_\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.S):
        params = m.group(2).strip()
        decls[m.group(1)] = 0 if params in ("", "void") else params.count(",") + 1
    return decls


def test_header_parses_to_the_expected_surface():
    names = set(_declared())
    assert {"mx_quantize_rows", "mx_quantize_cols", "mx_quantize_dual", "mx_gemm_nt", "mx_grouped_gemm_nt",
            "mx_experts_gemm1", "mx_experts_scatter_gemm", "mx_experts_gemm2_dgrad", "mx_grouped_wgrad_nt",
            "mx_quantize_cols_grouped", "mx_swiglu_quantize_rows", "mx_swiglu_quantize_dual",
            "mx_swiglu_bwd_quantize_dual", "mx_abi_version", "mx_strerror", "mx_device_supported",
            "mx_rmsnorm_quantize", "mx_rmsnorm_backward", "mx_expert_counts", "mx_expert_sort_workspace",
            "mx_expert_sort", "mx_combine_routed", "mx_combine_routed_backward", "mx_gemm_workspace_bytes", "mx_gemm_nt_batch"} <= names


def test_library_exports_every_declared_symbol():
    from kohakuwullm_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        pytest.fail(f"{_lib.LIB_PATH} is not built: run __graft_entry__.build()")
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in _declared():
        assert hasattr(lib, name), f"{name} is declared in the header but not exported"


def test_binding_matches_header():
    from kohakuwullm_amd import _lib

    declared = _declared()
    assert set(_lib.SIGNATURES) == set(declared)
    for name, (restype, argtypes) in _lib.SIGNATURES.items():
        assert len(argtypes) == declared[name], f"{name}: binding has {len(argtypes)} args, header {declared[name]}"
    lib = _lib.load()
    assert lib.mx_abi_version() == _lib.MX_ABI_VERSION == 2
    assert b"invalid" in lib.mx_strerror(-1) and lib.mx_strerror(0) == b"ok"
    assert b"captured" in lib.mx_strerror(_lib.MX_ECAPTURE)


def test_entry_points_validate_before_launch():
    """Contract violations are refused with MX_EINVAL before any kernel is launched (null pointers are never touched)."""
    from kohakuwullm_amd import _lib

    lib = _lib.load()
    assert lib.mx_quantize_rows(None, 0, 4, 48, 48, 1, None, 48, None, 1, None) == _lib.MX_EINVAL  # K % 32
    assert lib.mx_quantize_cols(None, 0, 48, 64, 64, None, 48, None, 1, None) == _lib.MX_EINVAL  # M % 32
    assert lib.mx_quantize_rows(None, 0, 0, 64, 64, 1, None, 64, None, 2, None) == _lib.MX_OK  # empty
    assert lib.mx_gemm_nt(None, None, None, None, None, 0, 4, 4, 48, 48, 1, 48, 1, 4, 0, None, 0, None) == _lib.MX_EINVAL
    assert lib.mx_gemm_nt(None, None, None, None, None, 0, 4, 4, 64, 32, 2, 64, 2, 4, 0, None, 0, None) == _lib.MX_EINVAL  # lda < K
    assert lib.mx_gemm_nt(None, None, None, None, None, 0, 0, 4, 64, 64, 2, 64, 2, 4, 0, None, 0, None) == _lib.MX_OK
    assert lib.mx_gemm_nt(None, None, None, None, None, 0, 4, 4, 64, 64, 2, 64, 2, 4, 1, None, 0, None) == _lib.MX_EINVAL  # accumulate needs fp32
    assert lib.mx_gemm_nt(None, None, None, None, None, 0, 4, 4, 64, 64, 2, 64, 2, 4, 0, None, -1, None) == _lib.MX_EINVAL  # workspace size
    assert lib.mx_gemm_nt_batch(None, 0, 0, None, 0, None) == _lib.MX_OK and lib.mx_gemm_nt_batch(None, 1, 0, None, 0, None) == _lib.MX_EINVAL
    assert lib.mx_grouped_wgrad_nt(None, None, 256, 8, None, None, 256, 8, None, 1, 128, None, 0, 0, 64, 64, 64, None, -1, None) == _lib.MX_EINVAL
    # expert dispatch: sizes, index widths and the workspace are checked before anything is launched
    assert lib.mx_expert_counts(None, 3, 8, 4, None, None) == _lib.MX_EINVAL  # idx_bytes
    assert lib.mx_expert_counts(None, 8, 8, 4, None, None) == _lib.MX_EINVAL  # null pointers
    assert lib.mx_expert_sort_workspace(98304, 64) == 384 * 64 and lib.mx_expert_sort_workspace(0, 5) == 5
    assert lib.mx_expert_sort_workspace(64 * 4096 * 5, 2) == 4096 * 2 and lib.mx_expert_sort_workspace(-1, 4) == -1
    assert lib.mx_expert_sort(None, 8, 16, None, 2, 4, None, None, None, None, None, 0, None) == _lib.MX_EINVAL
    assert lib.mx_combine_routed(None, 0, 16, None, 2, None, None, None, 12, 16, 5, 2, None, 16, None) == _lib.MX_EINVAL  # 12 rows > 5 * 2 pairs
    assert lib.mx_combine_routed(None, 0, 8, None, 2, None, None, None, 12, 16, 6, 2, None, 16, None) == _lib.MX_EINVAL  # ld < d
    assert lib.mx_combine_routed(None, 0, 16, None, 2, None, None, None, 0, 16, 0, 2, None, 16, None) == _lib.MX_OK  # empty
    assert lib.mx_combine_routed_backward(None, 16, None, 16, 3, None, 2, None, None, None, 4, 16, 2, 4, None, 16, None, None) == _lib.MX_EINVAL
    assert lib.mx_combine_routed_backward(None, 16, None, 16, 0, None, 2, None, None, None, 0, 16, 2, 0, None, 16, None, None) == _lib.MX_OK
    # the batched quantizer validates every problem before it launches anything
    probs = (_lib.QuantProblem * 2)()
    probs[0] = _lib.QuantProblem(None, None, None, None, None, 0, 64, 64, 64, 2, 0, 0)
    probs[1] = _lib.QuantProblem(None, None, None, None, None, 48, 64, 64, 64, 2, 48, 1)  # M % 32
    assert lib.mx_quantize_dual_batch(ctypes.byref(probs), 1, 0, None) == _lib.MX_OK  # an empty matrix
    assert lib.mx_quantize_dual_batch(ctypes.byref(probs), 2, 0, None) == _lib.MX_EINVAL
    assert lib.mx_quantize_dual_batch(None, 1, 0, None) == _lib.MX_EINVAL
    assert lib.mx_quantize_dual_batch(ctypes.byref(probs), 1, 7, None) == _lib.MX_EINVAL  # dtype
    probs[1] = _lib.QuantProblem(None, None, None, None, None, 64, 64, 64, 64, 2, 64, 2)  # null operands
    assert lib.mx_quantize_dual_batch(ctypes.byref(probs), 2, 0, None) == _lib.MX_EINVAL
    assert lib.mx_quantize_heads(None, 0, 8, 4, 48, 192, 48, None, None, None, None) == _lib.MX_EINVAL  # D % 32
    assert lib.mx_quantize_heads(None, 0, 8, 4, 64, 256, 32, None, None, None, None) == _lib.MX_EINVAL  # heads overlap
    assert lib.mx_quantize_heads(None, 0, 0, 4, 64, 256, 64, None, None, None, None) == _lib.MX_OK
    assert lib.mx_quantize_heads(None, 0, 8, 4, 64, 256, 64, None, None, None, None) == _lib.MX_EINVAL  # null operands
    # a leading dimension of exactly 128 on a wider code matrix selects the stage-major layout: K % 128 then
    assert lib.mx_gemm_nt(None, None, None, None, None, 0, 0, 4, 256, 128, 8, 256, 8, 4, 0, None, 0, None) == _lib.MX_OK  # A panels, empty
    assert lib.mx_gemm_nt(None, None, None, None, None, 0, 4, 4, 160, 128, 5, 160, 5, 4, 0, None, 0, None) == _lib.MX_EINVAL  # K % 128
    assert lib.mx_gemm_nt(None, None, None, None, None, 0, 4, 4, 256, 64, 8, 256, 8, 4, 0, None, 0, None) == _lib.MX_EINVAL  # lda < K, not 128
    assert lib.mx_quantize_dual(None, 0, 0, 64, 64, None, 64, None, 2, None, 128, None, 0, None) == _lib.MX_OK
    assert lib.mx_quantize_dual(None, 0, 160, 64, 64, None, 64, None, 2, None, 128, None, 5, None) == _lib.MX_EINVAL  # panels need M % 128
