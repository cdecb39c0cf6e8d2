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

__all__ = ["adder", "adder_cuda", "adder2d", "adder2d_function", "install", "uninstall"]


def install(force=False):
    """Make the reference's own import lines bind to this build: after this call ``import adder`` (resnet20.py:3,
    resnet50.py:5, vgg.py:6, densenet.py:5) and ``import adder_cuda`` (adder.py:15, adder_cuda/test_cuda.py:4)
    return this package's ``adder`` and ``adder_cuda`` modules, so the reference's model files run unedited.

    A module of either name that is already imported from somewhere else is left alone and reported with an
    ImportError unless ``force`` is given.  The same effect without a call: put ``addernetcuda_amd/dropin`` on
    ``PYTHONPATH``.
    """
    import sys
    for name, mod in (("adder_cuda", adder_cuda), ("adder", adder)):
        have = sys.modules.get(name)
        if have is not None and have is not mod and not force:
            raise ImportError(f"a different module named '{name}' is already imported from "
                              f"{getattr(have, '__file__', '?')}; pass force=True to replace it")
        sys.modules[name] = mod


def uninstall():
    """Undo ``install()``: the top-level names ``adder`` / ``adder_cuda`` no longer point at this package."""
    import sys
    for name, mod in (("adder_cuda", adder_cuda), ("adder", adder)):
        if sys.modules.get(name) is mod:
            del sys.modules[name]
