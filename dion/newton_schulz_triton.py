"""``dion.newton_schulz_triton`` of microsoft/dion (dion/newton_schulz_triton.py:160-568), served by the
gfx950 kernels of ``dion_amd``."""
from dion_amd.newton_schulz import (  # noqa: F401
    newton_schulz_triton,
    ns_line_1,
    ns_line_2,
    ns_line_3,
    zeropower_via_newtonschulz5,
)

__all__ = ["ns_line_1", "ns_line_2", "ns_line_3", "newton_schulz_triton", "zeropower_via_newtonschulz5"]
