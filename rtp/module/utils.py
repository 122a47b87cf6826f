"""The reference's import path rtp/module/utils.py: affine_weight, divide_and_check_no_remainder, ....

This file is the module `rtp_amd.module.utils` under the reference's name: after import, `sys.modules` maps this name to
that very module object, so every class and function is identical (not a copy) whichever name it is imported by.
"""
import sys

from rtp_amd.module import utils as _impl

sys.modules[__name__] = _impl
