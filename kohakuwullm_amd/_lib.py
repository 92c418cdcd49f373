"""ctypes binding of ``libmxfp8_hip.so`` -- the only door from Python to the HIP kernels.

The library is built in-tree by ``csrc/Makefile`` (``__graft_entry__.build()``).  It is
loaded after ``import torch`` so that its ``libamdhip64.so.7`` dependency resolves to the
HIP runtime PyTorch already mapped, which makes PyTorch's streams and device pointers
valid inside the library.  A missing library or a non-zero status raises: nothing falls
back to another implementation.
"""

from __future__ import annotations

import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmxfp8_hip.so")

MX_OK, MX_EINVAL, MX_EUNSUPPORTED, MX_ELAUNCH, MX_ENODEV, MX_ECAPTURE, MX_ETOOBIG = 0, -1, -2, -3, -4, -5, -6
MX_ABI_VERSION = 2
MX_DTYPE = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}

_i64, _p, _ci = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int

# name -> (restype, argtypes); mirrors include/mxfp8_hip.h declaration by declaration.
SIGNATURES = {
    "mx_abi_version": (_ci, []),
    "mx_strerror": (ctypes.c_char_p, [_ci]),
    "mx_device_supported": (_ci, [_ci]),
    "mx_quantize_rows": (_ci, [_p, _ci, _i64, _i64, _i64, _i64, _p, _i64, _p, _i64, _p]),
    "mx_quantize_cols": (_ci, [_p, _ci, _i64, _i64, _i64, _p, _i64, _p, _i64, _p]),
    "mx_quantize_dual": (_ci, [_p, _ci, _i64, _i64, _i64, _p, _i64, _p, _i64, _p, _i64, _p, _i64, _p]),
    "mx_quantize_heads": (_ci, [_p, _ci, _i64, _i64, _i64, _i64, _i64, _p, _p, _p, _p]),
    "mx_quantize_dual_batch": (_ci, [_p, _ci, _ci, _p]),
    "mx_swiglu_quantize_rows": (_ci, [_p, _p, _ci, _i64, _i64, _i64, _i64, _p, _i64, _p, _i64, _p]),
    "mx_swiglu_quantize_dual": (_ci, [_p, _ci, _i64, _i64, _i64, _p, _i64, _p, _i64, _p, _i64, _p, _i64, _p]),
    "mx_swiglu_bwd_quantize_dual": (
        _ci, [_p, _i64, _p, _i64, _ci, _i64, _i64, _p, _i64, _p, _i64, _p, _i64, _p, _i64, _p]),
    "mx_grouped_gemm_nt": (
        _ci, [_p, _p, _i64, _i64, _i64, _p, _p, _p, _i64, _i64, _i64, _i64, _p, _i64, _p, _ci, _i64, _i64, _i64, _i64, _p]),
    "mx_experts_gemm1": (
        _ci, [_p, _p, _i64, _i64, _i64, _p, _p, _p, _i64, _i64, _i64, _i64, _p, _i64, _p, _i64, _p, _i64, _p, _i64,
              _p, _i64, _p, _i64, _ci, _i64, _i64, _i64, _p]),
    "mx_experts_scatter_gemm": (
        _ci, [_p, _p, _i64, _i64, _i64, _p, _p, _p, _i64, _i64, _i64, _i64, _p, _i64, _p, _p, _p, _ci, _p, _ci, _i64,
              _i64, _i64, _i64, _p]),
    "mx_experts_gemm2_dgrad": (
        _ci, [_p, _p, _i64, _i64, _i64, _p, _p, _p, _ci, _p, _p, _i64, _i64, _i64, _i64, _p, _i64, _p, _i64, _p, _i64,
              _p, _p, _i64, _p, _i64, _p, _i64, _p, _i64, _p, _i64, _p, _ci, _i64, _i64, _i64, _p]),
    "mx_experts_combine": (_ci, [_p, _i64, _p, _p, _i64, _p, _ci, _p, _i64, _i64, _p, _ci, _i64, _i64, _i64, _p]),
    "mx_quantize_cols_grouped": (
        _ci, [_p, _ci, _i64, _i64, _ci, _p, _p, _ci, _p, _p, _i64, _i64, _p, _i64, _p, _i64, _p]),
    "mx_grouped_wgrad_nt": (
        _ci, [_p, _p, _i64, _i64, _p, _p, _i64, _i64, _p, _i64, _i64, _p, _ci, _i64, _i64, _i64, _i64, _p, _i64, _p]),
    "mx_rmsnorm_quantize": (
        _ci, [_p, _ci, _i64, _i64, _i64, _p, _ci, ctypes.c_float, _p, _i64, _p, _p, _i64, _p, _i64, _p]),
    "mx_rmsnorm_quantize_dual": (
        _ci, [_p, _ci, _i64, _i64, _i64, _p, _ci, ctypes.c_float, _p, _p, _i64, _p, _i64, _p, _i64, _p, _i64, _p]),
    "mx_rmsnorm_backward": (
        _ci, [_p, _ci, _i64, _i64, _i64, _p, _ci, _p, _i64, _p, _p, _i64, _p, _i64, _p]),
    "mx_expert_counts": (_ci, [_p, _ci, _i64, _i64, _p, _p]),
    "mx_expert_sort_workspace": (_i64, [_i64, _i64]),
    "mx_expert_sort": (_ci, [_p, _ci, _i64, _p, _i64, _i64, _p, _p, _p, _p, _p, _i64, _p]),
    "mx_expert_sort_static": (_ci, [_p, _ci, _i64, _p, _i64, _i64, _p, _p, _p, _p, _p]),
    "mx_combine_routed": (_ci, [_p, _ci, _i64, _p, _ci, _p, _p, _p, _i64, _i64, _i64, _i64, _p, _i64, _p]),
    "mx_combine_routed_backward": (
        _ci, [_p, _i64, _p, _i64, _ci, _p, _ci, _p, _p, _p, _i64, _i64, _i64, _i64, _p, _i64, _p, _p]),
    "mx_swizzle_scales": (_ci, [_p, _i64, _i64, _i64, _p, _p]),
    "mx_unswizzle_scales": (_ci, [_p, _i64, _i64, _p, _i64, _p]),
    "mx_gemm_nt": (_ci, [_p, _p, _p, _p, _p, _ci, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _ci, _p, _i64, _p]),
    "mx_gemm_workspace_bytes": (_i64, []),
    "mx_gemm_nt_batch": (_ci, [_p, _ci, _ci, _p, _i64, _p]),
    "mx_ubench_stream": (_ci, [_ci, _p, _p, _p, _i64, _p]),
    "mx_ubench_stream_cfg": (_ci, [_ci, _ci, _ci, _ci, _ci, _p, _p, _p, _i64, _p]),
    "mx_ubench_tile_pattern": (_ci, [_ci, _ci, _ci, _ci, _p, _i64, _p, _i64, _i64, _p, _p, _p, _p, _p]),
    "mx_ubench_mfma": (_i64, [_ci, _ci, _ci, _p, _i64, _p]),
}


class GemmProblem(ctypes.Structure):
    """``mx_gemm_problem`` of the C header."""

    _fields_ = [(n, _p) for n in ("aq", "a_scale", "bq", "b_scale", "c")] + [
        (n, _i64) for n in ("M", "N", "K", "lda", "ldas", "ldb", "ldbs", "ldc")
    ]



class QuantProblem(ctypes.Structure):
    """``mx_quant_problem`` of the C header."""

    _fields_ = [(n, _p) for n in ("x", "q", "s", "qT", "sT")] + [
        (n, _i64) for n in ("M", "K", "ldx", "ldq", "lds", "ldqT", "ldsT")
    ]


_lib: ctypes.CDLL | None = None


class MXFP8LibraryError(RuntimeError):
    """The HIP library is missing, or one of its entry points returned an error."""


def load() -> ctypes.CDLL:
    """Load (once) and type the library.  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise MXFP8LibraryError(
            f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
            "(or `python -c 'import __graft_entry__ as g; g.build()'`); there is no fallback path"
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError here means the header and the build disagree
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


# Measured-slower alternative kernels live in a library of their own, built from the same sources with
# -DMX_BENCH_VARIANTS: the dense GEMM's three other tilings / schedules behind flags of `epilogue`
# (csrc/mx_gemm_variants.h; the product library answers MX_EUNSUPPORTED to each), and the two fused expert kernels on
# 128 x 128 tiles with two workgroups per CU in place of the shipped 256 x 256 ones (csrc/mx_grouped.hip).  Only the
# benchmark (--variants-library) and the bit-equality tests of the kernels load it.
VARIANTS_PATH = os.path.join(_HERE, "libmxfp8_hip_variants.so")
MX_EPI_TILE_128, MX_EPI_PHASED, MX_EPI_WIDE_WAVES = 0x10, 0x20, 0x40
_variants: ctypes.CDLL | None = None


def load_variants() -> ctypes.CDLL:
    """The variants library, typed like the product library."""
    global _variants
    if _variants is None:
        if not os.path.exists(VARIANTS_PATH):
            raise MXFP8LibraryError(f"{VARIANTS_PATH} is missing: `make -C {os.path.join(_HERE, 'csrc')}` builds it")
        lib = ctypes.CDLL(VARIANTS_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = restype, argtypes
        _variants = lib
    return _variants


class variants_library:
    """``with variants_library():`` every entry point called inside goes to the variants library (benchmarks and tests only)."""

    def __enter__(self):
        global _lib
        load()
        self._saved, _lib = _lib, load_variants()
        return _lib

    def __exit__(self, *exc):
        global _lib
        _lib = self._saved
        return False


def check(status: int, what: str) -> None:
    if status == MX_OK:
        return
    msg = load().mx_strerror(status).decode()
    if status == MX_EINVAL:
        raise ValueError(f"{what}: {msg}")
    if status == MX_ECAPTURE:
        raise MXFP8LibraryError(
            f"{what}: {msg}.  Keep MXFP8 layers out of torch.cuda.graph / hipStreamBeginCapture regions."
        )
    raise MXFP8LibraryError(f"{what}: {msg} (status {status})")


def stream_of(t: torch.Tensor) -> int:
    """The raw hipStream_t PyTorch is currently issuing on for ``t``'s device."""
    return torch.cuda.current_stream(t.device).cuda_stream


_WORKSPACES: dict[tuple[int, int], torch.Tensor] = {}


def gemm_workspace(t: torch.Tensor) -> torch.Tensor:
    """Scratch for the K splits of ``mx_gemm_nt`` / ``mx_gemm_nt_batch`` / ``mx_grouped_wgrad_nt`` on ``t``'s device.

    One tensor per (device, current stream), allocated the first time that stream asks and kept: calls on one
    stream run in order and may share it, work on another stream gets its own, and the hot path never goes
    back to the allocator for a 128 MiB block that smaller tensors may have carved up in the meantime.
    The library itself allocates nothing.
    """
    index = t.device.index if t.device.index is not None else torch.cuda.current_device()
    key = (index, stream_of(t))
    ws = _WORKSPACES.get(key)
    if ws is None:
        with torch.cuda.device(index):
            ws = torch.empty(int(load().mx_gemm_workspace_bytes()), dtype=torch.uint8, device=t.device)
        _WORKSPACES[key] = ws
    return ws


def require_gpu(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise MXFP8LibraryError(
            f"{name} lives on {t.device}: the MXFP8 kernels run on an MI355X (gfx950) only and have no CPU path"
        )


# Optional per-call device timing, used by the benchmark's roofline pass only.  When a list is
# installed here every entry point call is bracketed by two events on the launch stream and
# (name, work, start, end) is appended; `work` is the caller's algorithmic byte/flop count.
TIMER: list | None = None


def invoke(name: str, work: float, tensor: torch.Tensor, *args) -> None:
    """Call entry point ``name`` with ``args`` on ``tensor``'s current stream and check its status."""
    fn = getattr(load(), name)
    if TIMER is None:
        check(fn(*args, stream_of(tensor)), name)
        return
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    status = fn(*args, stream_of(tensor))
    end.record()
    check(status, name)
    TIMER.append((name, work, start, end))
