"""``dion.polar_express`` of microsoft/dion (dion/polar_express.py:20-85), served by ``dion_amd``."""
from dion_amd.newton_schulz import polar_express, polar_express_triton  # noqa: F401

__all__ = ["polar_express", "polar_express_triton"]
