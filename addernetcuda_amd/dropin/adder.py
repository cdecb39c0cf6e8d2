"""``import adder`` as the reference's model files write it (resnet20.py:3, resnet50.py:5, vgg.py:6, densenet.py:5).

Put this directory on ``sys.path`` (``PYTHONPATH=.../addernetcuda_amd/dropin``, or ``addernetcuda_amd.install()``)
and the top-level name ``adder`` is this build's operator module: ``adder.adder2d``, ``adder.adder2d_function``,
``adder.adder`` (adder.py:22-108) on the MI355X kernels.
"""
import sys

from addernetcuda_amd import adder as _impl

sys.modules[__name__] = _impl
