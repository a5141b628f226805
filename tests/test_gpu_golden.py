"""The HIP orthogonalization against the reference's own output vectors (tests/golden/ns_vectors.npz:
the reference's three functions run on the CPU in the build container, each as exported -- through
torch.compile -- and undecorated), through the C ABI.

What the vectors allow and what they do not: the reference's two own paths differ from each other
by 1.7-2.3e-2 (NS5), 3.8-5.8e-2 (Polar-Express) and 3.0-3.6e-2 (KJ) relative Frobenius on these
inputs, so "within 2e-2 of the reference path" is a property the reference itself has only for
NS5.  The bars:
  * every schedule: within 2e-2 of the exact (float64) result of the reference's algorithm on
    the same bf16 input;
  * NS5: within 2e-2 of BOTH reference paths;
  * Polar-Express, KJ: no further from either reference path than REL x the distance between the
    reference's two paths on that input (REL = 1.25 towards the eager path, 1.0 towards the
    compiled one: the compiled path shares some roundings with the eager one, the HIP path none).
The measured distances are printed (pytest -s)."""
import os

import numpy as np
import pytest
import torch

from oracle import dion_oracle as oracle

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ns_vectors.npz")
SHAPES = [(64, 128), (128, 64), (128, 128), (4, 64, 128), (96, 160), (160, 96)]


def _t(a):
    return torch.from_numpy(a.astype(np.int16)).view(torch.bfloat16)


def _rel(a, b) -> float:
    a = a.double() if isinstance(a, torch.Tensor) else torch.from_numpy(np.asarray(a, dtype=np.float64))
    b = b.double() if isinstance(b, torch.Tensor) else torch.from_numpy(np.asarray(b, dtype=np.float64))
    return float((a - b).norm() / b.norm())


def _case(z, name, shape):
    tag = "x".join(str(v) for v in shape)
    return _t(z[f"in_{tag}"]), _t(z[f"{name}_eager_{tag}"]), _t(z[f"{name}_compiled_{tag}"])


def _run(name, G):
    from dion_amd import polar_express, zeropower_kj, zeropower_via_newtonschulz5

    g = G.to("cuda")
    if name == "ns5":
        return zeropower_via_newtonschulz5(g, 1e-7).cpu()
    if name == "pe":
        return polar_express(g, 1e-6).cpu()
    return zeropower_kj(g, steps=5, eps=1e-7).cpu()


SCHEDULES = {"ns5": (oracle.NS5_COEFFS, 1.0, 1e-7), "pe": (oracle.POLAR_EXPRESS_COEFFS, 1.02, 1e-6),
             "kj": (oracle.KJ_COEFFS, 1.0, 1e-7)}


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("name", ["ns5", "pe", "kj"])
def test_hip_against_the_references_own_vectors(name, shape):
    if name == "kj" and len(shape) != 2:
        pytest.skip("muon_reference's function is 2-D only")
    z = np.load(GOLDEN)
    G, eager, comp = _case(z, name, shape)
    out = _run(name, G)
    assert out.dtype == torch.bfloat16 and out.shape == G.shape
    coeffs, scale, eps = SCHEDULES[name]
    x = oracle.ns_fp64(G.float().numpy(), coeffs, scale, eps)
    d_x, d_e, d_c, d_ec = _rel(out, x), _rel(out, eager), _rel(out, comp), _rel(comp, eager)
    print(f"golden {name} {shape}: hip-fp64 {d_x:.2e} hip-eager {d_e:.2e} hip-compiled {d_c:.2e} | "
          f"reference: eager-compiled {d_ec:.2e} eager-fp64 {_rel(eager, x):.2e} compiled-fp64 {_rel(comp, x):.2e}")
    assert d_x <= 2e-2, d_x
    if name == "ns5":
        assert d_e <= 2e-2 and d_c <= 2e-2, (d_e, d_c)
    else:
        assert d_e <= 1.25 * d_ec, (d_e, d_ec)
        assert d_c <= 1.0 * d_ec, (d_c, d_ec)
