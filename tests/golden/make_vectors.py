"""Writes tests/golden/ns_vectors.npz: input / output vectors of the reference's three orthogonalization
functions on the CPU, for the one thing no closed form pins -- the exact bf16 rounding sequence of
the reference's own paths (the functions are decorated with torch.compile, so the compiler decides
which intermediates are rounded).

Run in the build container only, where the reference tree is mounted; the reference never travels,
the vectors do:

    python tests/golden/make_vectors.py [/root/reference]

For every case the file holds the bf16 input bits and two outputs per function: `compiled` (the
function as the reference exports it, i.e. through torch.compile / inductor on the CPU) and `eager`
(the same Python function without the decorator).  Functions:
  ns5  dion/newton_schulz_triton.py:494-522  zeropower_via_newtonschulz5(G, epsilon=1e-7)
  pe   dion/polar_express.py:19-50           polar_express(G, epsilon=1e-6)
  kj   dion/muon_reference.py:10-27          zeropower_via_newtonschulz5(G, steps=5, eps=1e-7)  (2-D only)
Shapes and seed follow the reference's tests/test_polar_express.py:10-42 (seed 42, randn), plus a pair that
is not a multiple of any tile size.
"""
import os
import sys

import numpy as np
import torch

SHAPES = [(64, 128), (128, 64), (128, 128), (4, 64, 128), (96, 160), (160, 96)]
SEED = 42


def _bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().contiguous().to(torch.bfloat16).view(torch.int16).numpy().astype(np.uint16)


def _undecorated(fn):
    orig = getattr(fn, "_torchdynamo_orig_callable", None) or getattr(fn, "__wrapped__", None)
    if orig is None:
        raise RuntimeError(f"cannot find the undecorated function behind {fn!r}")
    return orig


def main() -> None:
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    here = os.path.dirname(os.path.abspath(__file__))
    # the reference's package must win over this repository's dion/ import-path shim
    sys.path[:] = [p for p in sys.path if os.path.abspath(p or ".") != os.path.dirname(os.path.dirname(here))]
    sys.path.insert(0, ref)
    import dion.muon_reference as mr
    import dion.newton_schulz_triton as nst
    import dion.polar_express as pe

    assert os.path.abspath(pe.__file__).startswith(os.path.abspath(ref)), pe.__file__
    funcs = {
        "ns5": (nst.zeropower_via_newtonschulz5, lambda f, g: f(g, 1e-7)),
        "pe": (pe.polar_express, lambda f, g: f(g, 1e-6)),
        "kj": (mr.zeropower_via_newtonschulz5, lambda f, g: f(g, 5, 1e-7)),
    }
    out = {}
    with torch.no_grad():
        for shape in SHAPES:
            torch.manual_seed(SEED)
            G = torch.randn(shape).to(torch.bfloat16)
            tag = "x".join(str(s) for s in shape)
            out[f"in_{tag}"] = _bits(G)
            for name, (fn, call) in funcs.items():
                if name == "kj" and len(shape) != 2:
                    continue
                torch._dynamo.reset()
                out[f"{name}_compiled_{tag}"] = _bits(call(fn, G.clone()))
                out[f"{name}_eager_{tag}"] = _bits(call(_undecorated(fn), G.clone()))
                print(name, tag, "done", flush=True)
    path = os.path.join(here, "ns_vectors.npz")
    np.savez_compressed(path, torch_version=np.array(torch.__version__), **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
