"""``hbsattn.benchmark`` import name of the reference, served by :mod:`hbsattn_amd.benchmark`."""
from hbsattn_amd.benchmark import _check_correctness, benchmark  # noqa: F401
