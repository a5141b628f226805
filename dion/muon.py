"""``dion.muon`` of microsoft/dion (dion/muon.py), served by ``dion_amd``."""
from dion_amd.functional import muon_update_post_orthogonalize, muon_update_pre_orthogonalize  # noqa: F401
from dion_amd.newton_schulz import zeropower_via_newtonschulz5  # noqa: F401
from dion_amd.optimizers import Muon  # noqa: F401

__all__ = ["Muon", "zeropower_via_newtonschulz5", "muon_update_pre_orthogonalize",
           "muon_update_post_orthogonalize"]
