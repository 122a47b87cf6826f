"""rtp_amd: RTP (rotated tensor parallelism) rotated-shard layer compute for one MI355X (gfx950).

Python host code mirroring the reference's rtp.* API over hand-written HIP kernels reached through the
C ABI of librtp_hip.so.  No kernel has a PyTorch or CPU fallback.
"""
from .module.collectives import emulate_shards, rotated_weight_bytes, zero_full_grads  # noqa: F401
from .ring import rotation_window, set_rotation_window, staging_bytes  # noqa: F401

__all__ = ["emulate_shards", "rotated_weight_bytes", "zero_full_grads", "staging_bytes"]
