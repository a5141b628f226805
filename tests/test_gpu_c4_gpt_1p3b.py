"""NorMuon and Dion2 at the GPT-1.3B shapes (d_model 2048, MLP 8192: 6144x2048, 2048x2048, 8192x2048,
2048x8192), as whole optimizer steps and as whole orthogonalizations of the sub-matrices Dion2 selects
at fraction 0.25 -- [24, 6144, 512] (columns of the tall qkv weight), [24, 512, 2048], [24, 8192, 512],
[24, 512, 8192].

The composition under test is the reference's per-shape-group update, dion/normuon.py:222-341
(momentum, orthogonalization, neuron-wise normalization, update) and dion/dion2.py:205-421 (accumulate,
select, orthogonalize the selected slices, error feedback, selective update).  The oracle runs the
element-wise parts on the host; the orthogonalization in between is the exact (float64) iteration of the
reference's algorithm, run with torch float64 matmuls on the device (the same statements as
oracle.ns_fp64, which tests/test_gpu_workload_configs.py::test_fp64_on_device_is_the_oracle pins).
Bars: momentum bit for bit (NorMuon) / 1e-6 (Dion2), the selected index set exactly, the update within
2e-2 relative Frobenius of the exact one, parameters within the lr-scaled equivalent of that, entries Dion2
does not select bit-identical to a * x.
"""
import pytest
import torch

from oracle import dion_oracle as oracle

pytestmark = pytest.mark.gpu
DEV = "cuda"

GPT_1P3B = [(6144, 2048), (2048, 2048), (8192, 2048), (2048, 8192)]
PER_SHAPE = 2
LR, WD = 0.02, 0.01


def _rel(a, b) -> float:
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / b.norm().clamp(min=1e-30))


def _ns_fp64_on_device(G: torch.Tensor, coeffs, norm_scale: float, eps: float) -> torch.Tensor:
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


def _tensors():
    gen = torch.Generator().manual_seed(1300)
    X, G = [], []
    for shape in GPT_1P3B:
        for _ in range(PER_SHAPE):
            X.append(torch.randn(shape, generator=gen) * 0.02)
            G.append((torch.randn(shape, generator=gen) * 0.02).to(torch.bfloat16))
    return X, G


def _params(X, G):
    params = [torch.nn.Parameter(x.clone().to(DEV)) for x in X]
    for p, g in zip(params, G):
        p.grad_dtype = None  # bf16 gradients on fp32 parameters
        p.grad = g.to(DEV)
    return params


def test_normuon_step_at_gpt_1p3b_shapes_vs_oracle_composition():
    from dion import NorMuon

    X, G = _tensors()
    params = _params(X, G)
    opt = NorMuon(params, lr=LR, mu=0.95, muon_beta2=0.95, weight_decay=WD, nesterov=True,
                  use_polar_express=False)
    opt.step()
    torch.cuda.synchronize()
    a = 1 - torch.tensor(LR) * torch.tensor(WD)
    worst = 0.0
    for i, (x, g) in enumerate(zip(X, G)):
        shape = tuple(x.shape)
        m, u = oracle.muon_pre(g, torch.zeros_like(x), 0.95, True)
        assert torch.equal(opt.state[params[i]]["momentum"].cpu(), m), f"momentum of parameter {i} {shape}"
        o = _ns_fp64_on_device(u.to(DEV), oracle.NS5_COEFFS, 1.0, 1e-8).float().cpu()
        nU, V = oracle.normuon_normalize(o, torch.zeros(shape[0], 1), 0.95)
        ratio = oracle.adjust_lr_ratio(shape, "spectral_norm")
        x_want = oracle.muon_post(x, nU, LR, ratio, WD)
        # second moments are squares of the orthogonalized entries: twice their relative error
        assert _rel(opt.state[params[i]]["variance_neuron"], V) <= 3e-2, (i, shape)
        u_gpu = (x * a - params[i].data.cpu()) / (LR * ratio)
        d = _rel(u_gpu, nU)
        worst = max(worst, d)
        assert d <= 2e-2, (i, shape, d)
        assert _rel(params[i].data, x_want) <= 1e-3, (i, shape)
        # Frobenius norm of the normalised update = that of the orthogonalized matrix (dion/normuon.py:395-398)
        assert abs(float(u_gpu.norm() / o.norm()) - 1.0) <= 1e-2
    print(f"NorMuon step at GPT-1.3B shapes: worst update distance to the exact composition {worst:.2e}")


def test_dion2_step_at_gpt_1p3b_shapes_vs_oracle_composition():
    from dion import Dion2

    X, G = _tensors()
    params = _params(X, G)
    opt = Dion2(params, lr=LR, fraction=0.25, ef_decay=0.95, weight_decay=WD, use_polar_express=False)
    opt.step()
    torch.cuda.synchronize()
    a = 1 - torch.tensor(LR) * torch.tensor(WD)
    worst = 0.0
    for i, (x, g) in enumerate(zip(X, G)):
        shape = tuple(x.shape)
        sd = oracle.dion2_select_dim(*shape)
        m, u, idx = oracle.dion2_pre(g, torch.zeros_like(x), 0.25, 0.95, sd)
        assert idx.numel() == oracle.dion2_k(0.25, shape[sd])
        m_gpu = opt.state[params[i]]["momentum"].cpu()
        assert _rel(m_gpu, m) <= 1e-6, (i, shape)
        # the decayed slices are exactly the selected ones: the index set is pinned through the momentum
        mg = torch.zeros_like(x) + g.float()
        decayed = (m_gpu != mg).any(dim=-1 if sd == -2 else -2).nonzero().flatten()
        assert torch.equal(decayed, idx), (i, shape)
        o = _ns_fp64_on_device(u.to(DEV), oracle.NS5_COEFFS, 1.0, 1e-8).float().cpu()
        ratio = oracle.adjust_lr_ratio(shape, "spectral_norm")
        x_gpu = params[i].data.cpu()
        delta = (x * a - x_gpu) / (LR * ratio)
        sel = delta[idx, :] if sd == -2 else delta[:, idx]
        d = _rel(sel, o)
        worst = max(worst, d)
        assert d <= 2e-2, (i, shape, d)
        # outside the selected slices the parameters only see the weight decay, bit for bit
        keep = torch.ones(shape[sd], dtype=torch.bool)
        keep[idx] = False
        if sd == -2:
            assert torch.equal(x_gpu[keep, :], (x * a)[keep, :]), (i, shape)
        else:
            assert torch.equal(x_gpu[:, keep], (x * a)[:, keep]), (i, shape)
        x_want = oracle.dion2_post(x, o.to(torch.bfloat16), idx, LR, ratio, WD, sd)
        assert _rel(x_gpu, x_want) <= 1e-3, (i, shape)
    print(f"Dion2 step at GPT-1.3B shapes: worst selected-update distance to the exact composition {worst:.2e}")


@pytest.mark.parametrize("shape", [(24, 512, 8192), (24, 6144, 512), (24, 8192, 512), (24, 512, 2048)])
@pytest.mark.parametrize("variant", ["ns5", "polar_express"])
def test_dion2_selected_submatrices_whole_orthogonalization(variant, shape):
    from dion_amd import polar_express, zeropower_via_newtonschulz5

    gen = torch.Generator().manual_seed(77)
    G = (torch.randn(shape, generator=gen) * 0.02).to(torch.bfloat16).to(DEV)
    if variant == "ns5":
        out = zeropower_via_newtonschulz5(G, 1e-8)
        exact = _ns_fp64_on_device(G, oracle.NS5_COEFFS, 1.0, 1e-8)
    else:
        out = polar_express(G, 1e-8)
        exact = _ns_fp64_on_device(G, oracle.POLAR_EXPRESS_COEFFS, 1.02, 1e-8)
    assert out.shape == G.shape and out.dtype == torch.bfloat16
    per = (out.double() - exact).flatten(1).norm(dim=1) / exact.flatten(1).norm(dim=1)
    print(f"{shape} {variant}: worst matrix {float(per.max()):.2e} from the exact iteration")
    assert float(per.max()) <= 2e-2, float(per.max())
