"""Forwarder for ``hbsattn.utils.calculate_blocks`` (see :mod:`hbsattn_amd.utils`)."""
from hbsattn_amd.utils import calculate_blocks  # noqa: F401

__all__ = ["calculate_blocks"]
