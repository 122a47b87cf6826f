"""The reference's import path rtp/rotated_tensor_parallel.py: RotatedTensorParallel, FlyweightWarpper, split_tensor.

This file is the module `rtp_amd.rotated_tensor_parallel` under the reference's name: after import, `sys.modules` maps this name to
that very module object, so every class and function is identical (not a copy) whichever name it is imported by.
"""
import sys

from rtp_amd import rotated_tensor_parallel as _impl

sys.modules[__name__] = _impl
