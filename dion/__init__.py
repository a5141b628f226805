"""``from dion import Muon, Dion2, NorMuon`` -- the import path of microsoft/dion
(dion/__init__.py:5-8), served by the MI355X-native implementation in ``dion_amd``."""
import dion_amd as _impl

Muon = _impl.Muon
NorMuon = _impl.NorMuon
Dion2 = _impl.Dion2

__all__ = ["Muon", "NorMuon", "Dion2"]
