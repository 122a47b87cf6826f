"""The reference's import path rtp/module/collectives.py: zero_full_grads and the flat-shard store.

This file is the module `rtp_amd.module.collectives` under the reference's name: after import, `sys.modules` maps this name to
that very module object, so every class and function is identical (not a copy) whichever name it is imported by.
"""
import sys

from rtp_amd.module import collectives as _impl

sys.modules[__name__] = _impl
