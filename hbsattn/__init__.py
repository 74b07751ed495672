"""Import-name compatibility: code written against zhengqigao/hbsattn does
``from hbsattn import HBSAttention`` / ``from hbsattn.utils import calculate_blocks``.
Everything lives in :mod:`hbsattn_amd`; this package only forwards the two names."""
from hbsattn_amd import HBSAttention  # noqa: F401

__all__ = ["HBSAttention"]
