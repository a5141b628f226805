"""``dion.normuon`` of microsoft/dion (dion/normuon.py), served by ``dion_amd``."""
from dion_amd.optimizers import NorMuon  # noqa: F401

__all__ = ["NorMuon"]
