"""``import adder_cuda`` as the reference's adder.py:15 and adder_cuda/test_cuda.py:4 write it.

Put this directory on ``sys.path`` (``PYTHONPATH=.../addernetcuda_amd/dropin``, or ``addernetcuda_amd.install()``)
and the top-level name ``adder_cuda`` is this build's binding of the four entry points of
adder_cuda/adder_cuda.cpp:88-93 (``ADDER_CONV``, ``ADDER_BACKWARD``, ``ADDER_CONV_WEIGHT``, ``ADDER_CONV_INPUT``).
"""
import sys

from addernetcuda_amd import adder_cuda as _impl

sys.modules[__name__] = _impl
