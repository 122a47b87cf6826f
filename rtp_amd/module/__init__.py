"""Rotated (RTP) layers: drop-in counterparts of the reference's rtp.module package."""
