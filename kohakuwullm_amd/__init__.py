"""MI355X-native MXFP8 linear path behind KohakUwULLM's module and function API.

Only the MXFP8 linear path lives here: the quantizers, the dense and grouped GEMMs,
the ``MXFP8Linear`` module and the routed-expert functions, all calling hand-written
gfx950 HIP kernels through ``libmxfp8_hip.so`` (C ABI, ``include/mxfp8_hip.h``).
There is no CPU fallback: importing works anywhere, calling a kernel without the
built library or without a gfx950 GPU raises.
"""

__version__ = "0.1.0"
