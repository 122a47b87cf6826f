"""The reference's import path rtp/models/transformer_lm_rtp.py: TransformerLM and its blocks.

This file is the module `rtp_amd.models.transformer_lm_rtp` under the reference's name: after import, `sys.modules` maps this name to
that very module object, so every class and function is identical (not a copy) whichever name it is imported by.
"""
import sys

from rtp_amd.models import transformer_lm_rtp as _impl

sys.modules[__name__] = _impl
