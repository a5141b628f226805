"""The momentum kernel writing the orthogonalization input in the layout the iteration carries
(short side along rows, unnormalised, partial sums of squares alongside) and the orthogonalization
taking it that way, with the Frobenius normalisation of dion/polar_express.py:30-35 /
dion/newton_schulz_triton.py:508-513 folded into the first two GEMMs.

Pinned here: the prepared momentum kernel against the plain one (momentum bit for bit, same bf16
values, transposed for tall matrices; the partial sums against a float64 sum of the values written),
the prepared orthogonalization against the exact (float64) iteration of the reference's algorithm at
the bar of every other orthogonalization test (2e-2 relative Frobenius) and next to the unprepared
call, and whole optimizer steps with the prepared input on and off.
"""
import pytest
import torch

from oracle import dion_oracle as oracle

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _rel(a, b) -> float:
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / b.norm().clamp(min=1e-30))


def _ns_fp64_on_device(G, coeffs, norm_scale, eps):
    """oracle.ns_fp64 with torch float64 matmuls on the device (same statements)."""
    X = G.to(torch.bfloat16).double()
    tall = X.shape[-2] > X.shape[-1]
    if tall:
        X = X.mT
    X = X / (X.pow(2).sum(dim=(-2, -1), keepdim=True).sqrt() * norm_scale + eps)
    for a, b, c in coeffs:
        A = X @ X.mT
        B = b * A + c * (A @ A)
        X = a * X + B @ X
    return X.mT if tall else X


@pytest.mark.parametrize("mdtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("gdtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("mats,rows,cols", [(1, 256, 512), (1, 512, 256), (3, 384, 128), (2, 128, 640), (1, 256, 256)])
def test_prepared_momentum_kernel_vs_plain(mats, rows, cols, gdtype, mdtype):
    from dion_amd import ops

    gen = torch.Generator().manual_seed(rows * 7 + cols + mats)
    n = 3
    G = [(torch.randn(mats, rows, cols, generator=gen) * 0.02).to(gdtype).to(DEV) for _ in range(n)]
    M0 = [(torch.randn(mats, rows, cols, generator=gen) * 0.02).to(mdtype).to(DEV) for _ in range(n)]
    for nesterov in (True, False):
        Ma = [m.clone() for m in M0]
        Mb = [m.clone() for m in M0]
        U_plain = ops.muon_pre(G, Ma, 0.95, nesterov)                      # [n, mats, rows, cols]
        U, sumsq = ops.muon_pre_prepared(G, Mb, 0.95, nesterov, mats, rows, cols)
        torch.cuda.synchronize()
        for a, b in zip(Ma, Mb):
            assert torch.equal(a, b)
        want = U_plain.view(n * mats, rows, cols)
        if rows > cols:
            want = want.mT
        assert U.shape == (n * mats, min(rows, cols), max(rows, cols))
        assert torch.equal(U, want.contiguous())
        assert sumsq.shape == (n * mats, rows * cols // 4096)
        exact = U.double().pow(2).sum(dim=(1, 2))
        assert float(((sumsq.double().sum(dim=1) - exact).abs() / exact).max()) <= 1e-6


@pytest.mark.parametrize("shape", [(4, 256, 1024), (4, 1024, 256), (2, 512, 512), (12, 768, 3072), (12, 3072, 768),
                                   (3, 2048, 512)])
@pytest.mark.parametrize("variant", ["ns5", "polar_express", "gram"])
def test_prepared_orthogonalization_vs_exact_and_unprepared(variant, shape):
    from dion_amd import newton_schulz as ns
    from dion_amd import ops

    batch, rows, cols = shape
    gen = torch.Generator().manual_seed(batch + rows + cols)
    G = (torch.randn(shape, generator=gen) * 0.02).to(torch.bfloat16).to(DEV)
    func = {"ns5": ns.zeropower_via_newtonschulz5, "polar_express": ns.polar_express,
            "gram": ns.gram_newton_schulz}[variant]
    coeffs, scale, eps = {"ns5": (oracle.NS5_COEFFS, 1.0, 1e-8), "polar_express": (oracle.POLAR_EXPRESS_COEFFS, 1.02, 1e-8),
                          "gram": (oracle.POLAR_EXPRESS_COEFFS, 1.02, 0.0)}[variant]
    if not ns.accepts_prepared(func, batch, rows, cols):
        pytest.skip("this shape is padded to the GEMM tile: the unprepared path is the only one")
    U = (G.mT if rows > cols else G).contiguous()
    # the partial sums any producer could hand over: here one block per matrix row
    sumsq = U.float().pow(2).sum(dim=2).contiguous()
    out = ns.orthogonalize_prepared(func, U, sumsq, rows, cols, eps)
    plain = func(G, eps)
    exact = _ns_fp64_on_device(G, coeffs, scale, eps)
    assert out.shape == G.shape and out.dtype == torch.bfloat16
    per = (out.double() - exact).flatten(1).norm(dim=1) / exact.flatten(1).norm(dim=1)
    per_plain = (plain.double() - exact).flatten(1).norm(dim=1) / exact.flatten(1).norm(dim=1)
    print(f"{shape} {variant}: prepared {float(per.max()):.2e}, unprepared {float(per_plain.max()):.2e} from exact; "
          f"prepared vs unprepared {_rel(out, plain):.2e}")
    assert float(per.max()) <= 2e-2
    # not rounding X0 to bf16 once more can only help: no worse than the unprepared call, up to noise
    assert float(per.max()) <= float(per_plain.max()) * 1.15 + 1e-3


def test_prepared_input_is_refused_where_it_does_not_apply():
    from dion_amd import newton_schulz as ns
    from dion_amd import ops

    assert not ops.ns_accepts_prepared(4, 96, 160, 5)        # padded to the tile
    assert not ops.ns_accepts_prepared(4, 64, 768, 5)        # the LDS-resident small-matrix kernel
    assert not ops.ns_accepts_prepared(4, 256, 512, 0)       # nothing to carry the normalisation
    assert ops.ns_accepts_prepared(4, 256, 512, 5)
    U = torch.zeros(4, 128, 160, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ValueError):
        ns.orthogonalize_prepared(ns.polar_express, U, torch.ones(4, 5, device=DEV), 128, 160, 1e-7)


@pytest.mark.parametrize("cls_name", ["Muon", "NorMuon"])
@pytest.mark.parametrize("shape", [(256, 512), (512, 256), (3, 384, 128)])
def test_step_with_and_without_prepared_input(cls_name, shape):
    """The same step with the input handed over prepared and through the arena in the parameters' layout:
    momentum (and the update's inputs) identical, parameters equal up to the last-bit differences of the
    orthogonalized matrices (lr-scaled)."""
    import dion

    cls = getattr(dion, cls_name)
    gen = torch.Generator().manual_seed(11)
    X = [torch.randn(shape, generator=gen) * 0.02 for _ in range(3)]
    G = [(torch.randn(shape, generator=gen) * 0.02).to(torch.bfloat16) for _ in range(3)]

    def run(prepared):
        ps = [torch.nn.Parameter(x.clone().to(DEV)) for x in X]
        for p, g in zip(ps, G):
            p.grad_dtype = None
            p.grad = g.to(DEV)
        opt = cls(ps, lr=0.02, mu=0.95, nesterov=True, weight_decay=0.01)
        opt.prepared_input = prepared
        opt.step()
        opt.step()
        torch.cuda.synchronize()
        return ps, opt

    pa, oa = run(True)
    pb, ob = run(False)
    for a, b, x in zip(pa, pb, X):
        assert torch.equal(oa.state[a]["momentum"], ob.state[b]["momentum"])
        moved = _rel(b.data, x)                      # how far two steps move the parameters
        assert _rel(a.data, b.data) <= 2e-2 * moved  # the two paths agree to a fraction of that
        if cls_name == "NorMuon":
            assert _rel(oa.state[a]["variance_neuron"], ob.state[b]["variance_neuron"]) <= 2e-2


@pytest.mark.parametrize("mdtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,cols,select_dim,k", [(256, 1024, -2, 128), (1024, 256, -1, 128), (384, 256, -1, 256),
                                                    (512, 512, -2, 256), (256, 1024, -2, 64), (130, 520, -2, 33)])
def test_prepared_dion2_gather_vs_plain(rows, cols, select_dim, k, mdtype):
    """dion2_select with prepared=True against the plain call: same indices, same momentum bit for bit, the
    same bf16 block (transposed when it is tall), partial sums = the float64 sum of squares of the block."""
    from dion_amd import ops

    gen = torch.Generator().manual_seed(rows + 3 * cols + k)
    n, mats = 2, 2
    G = [(torch.randn(mats, rows, cols, generator=gen) * 0.02).to(torch.bfloat16).to(DEV) for _ in range(n)]
    M0 = [(torch.randn(mats, rows, cols, generator=gen) * 0.02).to(mdtype).to(DEV) for _ in range(n)]
    assert ops.dion2_prepared_blocks(rows, cols, select_dim, k) > 0
    Ma = [m.clone() for m in M0]
    Mb = [m.clone() for m in M0]
    U_plain, idx_a, map_a = ops.dion2_select(G, Ma, k, select_dim, 0.9)
    U, idx_b, map_b, sumsq = ops.dion2_select(G, Mb, k, select_dim, 0.9, prepared=True)
    torch.cuda.synchronize()
    assert torch.equal(idx_a, idx_b) and torch.equal(map_a, map_b)
    for a, b in zip(Ma, Mb):
        assert torch.equal(a, b)
    sr, sc = (k, cols) if select_dim == -2 else (rows, k)
    want = U_plain.reshape(n * mats, sr, sc)
    if sr > sc:
        want = want.mT
    assert U.shape == (n * mats, min(sr, sc), max(sr, sc))
    assert torch.equal(U, want.contiguous())
    exact = U.double().pow(2).sum(dim=(1, 2))
    assert sumsq.shape == (n * mats, ops.dion2_prepared_blocks(rows, cols, select_dim, k))
    assert float(((sumsq.double().sum(dim=1) - exact).abs() / exact).max()) <= 1e-6


def test_dion2_blocks_without_a_prepared_form():
    from dion_amd import ops

    assert ops.dion2_prepared_blocks(1024, 256, -2, 512) == 0   # rows selected, block taller than wide
    assert ops.dion2_prepared_blocks(1000, 256, -1, 64) == 0    # transposed form needs whole 64 x 64 tiles
    assert ops.dion2_prepared_blocks(1024, 256, -1, 64) == 16 * 1


@pytest.mark.parametrize("cls_name", ["Dion2", "NorDion2"])
@pytest.mark.parametrize("shape", [(512, 1024), (1024, 512), (2, 512, 512)])
def test_dion2_step_with_and_without_prepared_input(cls_name, shape):
    import dion

    cls = getattr(dion, cls_name)
    gen = torch.Generator().manual_seed(12)
    X = [torch.randn(shape, generator=gen) * 0.02 for _ in range(3)]
    G = [(torch.randn(shape, generator=gen) * 0.02).to(torch.bfloat16) for _ in range(3)]

    def run(prepared):
        ps = [torch.nn.Parameter(x.clone().to(DEV)) for x in X]
        for p, g in zip(ps, G):
            p.grad_dtype = None
            p.grad = g.to(DEV)
        opt = cls(ps, lr=0.02, fraction=0.25, weight_decay=0.01)
        opt.prepared_input = prepared
        opt.step()
        opt.step()
        torch.cuda.synchronize()
        return ps, opt

    pa, oa = run(True)
    pb, ob = run(False)
    for a, b, x in zip(pa, pb, X):
        assert torch.equal(oa.state[a]["momentum"], ob.state[b]["momentum"])
        moved = _rel(b.data - x.to(DEV) * (1 - 0.02 * 0.01) ** 2, x)   # what the selected updates add up to
        assert _rel(a.data, b.data) <= 2e-2 * max(moved, 1e-6)
