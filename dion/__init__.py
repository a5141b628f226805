"""``from dion import Muon, Dion2, NorMuon`` -- the import path of microsoft/dion
(dion/__init__.py:5-8), served by the MI355X-native implementation in ``dion_amd``."""
import dion_amd as _impl

Muon = _impl.Muon
NorMuon = _impl.NorMuon
Dion2 = _impl.Dion2
NorDion2 = _impl.NorDion2
Dion3 = _impl.Dion3  # alias of NorDion2 (dion/__init__.py:10)

__all__ = ["Muon", "NorMuon", "Dion2", "NorDion2", "Dion3"]
