"""The reference's import path rtp/module/embedding.py: ParallelEmbedding.

This file is the module `rtp_amd.module.embedding` under the reference's name: after import, `sys.modules` maps this name to
that very module object, so every class and function is identical (not a copy) whichever name it is imported by.
"""
import sys

from rtp_amd.module import embedding as _impl

sys.modules[__name__] = _impl
