"""MI355X-native Muon / NorMuon / Dion2 / NorDion2 optimizer-step kernels behind the microsoft/dion API."""
from .newton_schulz import (  # noqa: F401
    gram_newton_schulz,
    newton_schulz_triton,
    ns_line_1,
    ns_line_2,
    ns_line_3,
    polar_express,
    polar_express_triton,
    zeropower_kj,
    zeropower_via_newtonschulz5,
)

from .hip_graph import CudaGraphOptimizer, HipGraphOptimizer  # noqa: E402,F401
from .optimizers import Dion2, Dion3, Muon, NorDion2, NorMuon  # noqa: E402,F401

__all__ = [
    "Muon",
    "NorMuon",
    "Dion2",
    "NorDion2",
    "Dion3",
    "HipGraphOptimizer",
    "CudaGraphOptimizer",
    "gram_newton_schulz",
    "newton_schulz_triton",
    "ns_line_1",
    "ns_line_2",
    "ns_line_3",
    "polar_express",
    "polar_express_triton",
    "zeropower_kj",
    "zeropower_via_newtonschulz5",
]
