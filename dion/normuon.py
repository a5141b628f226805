"""``dion.normuon`` of microsoft/dion (dion/normuon.py), served by ``dion_amd``."""
from dion_amd.functional import normuon_normalization_stacked  # noqa: F401
from dion_amd.optimizers import NorMuon  # noqa: F401

__all__ = ["NorMuon", "normuon_normalization_stacked"]
