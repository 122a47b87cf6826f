"""The reference's import path rtp/module/top2gate.py: top2gating, Top2Gate, WeightTop2Gate.

This file is the module `rtp_amd.module.top2gate` under the reference's name: after import, `sys.modules` maps this name to
that very module object, so every class and function is identical (not a copy) whichever name it is imported by.
"""
import sys

from rtp_amd.module import top2gate as _impl

sys.modules[__name__] = _impl
