"""AdderNet convolution for AMD MI355X (gfx950): hand-written HIP kernels behind
the operator surface of the CUDA reference.

    from addernetcuda_amd import adder            # adder.adder2d, adder.adder2d_function, adder.adder
    from addernetcuda_amd import adder_cuda       # ADDER_CONV / ADDER_BACKWARD / ADDER_CONV_WEIGHT / ADDER_CONV_INPUT

The compute lives in ``libaddernet_hip.so`` (C ABI, see include/addernet_hip.h);
there is no CPU or PyTorch fallback: a missing library or a non-GPU tensor is an
error.
"""
from . import _lib  # noqa: F401  (loads the shared library eagerly so a missing build fails at import)
from . import adder_cuda  # noqa: F401
from . import adder  # noqa: F401
from .adder import adder2d, adder2d_function  # noqa: F401

__all__ = ["adder", "adder_cuda", "adder2d", "adder2d_function"]
