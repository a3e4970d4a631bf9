"""MI355X (gfx950) execution backend for FluidML.

``fluidml_amd.cabi``    ctypes binding of the C ABI (include/fluidml_hip.h) over the HIP kernels
``fluidml_amd.fluidml`` the compiled host module with the reference's Python surface
                        (Executor.make_plain_linear / make_plain_greedy / make_dp_greedy, compile, invoke, ...)

Both are built in-tree by ``fluidml_amd/csrc/Makefile``; neither has a CPU fallback.
"""
from . import cabi  # noqa: F401  (raises ImportError when libfluidml_hip.so is not built)

__all__ = ["cabi"]
