"""GPU parity of the memory-bound step kernels against the CPU oracle, through the C ABI.
fp32 state (momentum, variance, parameters): relative error <= 1e-5 (momentum is bit exact);
bf16 outputs: bit exact where the arithmetic is a cast of an fp32 value."""
import pytest
import torch

from oracle import dion_oracle as oracle

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _rel(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / b.norm().clamp(min=1e-30))


@pytest.mark.parametrize("shape", [(64, 128), (7, 13), (3, 40, 24), (768, 768)])
@pytest.mark.parametrize("nesterov", [False, True])
@pytest.mark.parametrize("gdtype", [torch.bfloat16, torch.float32])
def test_muon_pre(shape, nesterov, gdtype):
    from dion_amd import ops

    torch.manual_seed(0)
    n = 3
    G = [(torch.randn(shape) * 0.02).to(gdtype) for _ in range(n)]
    M = [torch.randn(shape) * 0.01 for _ in range(n)]
    Gd = [g.to(DEV) for g in G]
    Md = [m.to(DEV) for m in M]
    for step in range(2):
        U = ops.muon_pre(Gd, Md, 0.95, nesterov)
        assert U.shape == (n, *shape) and U.dtype == torch.bfloat16
        for i in range(n):
            m_ref, u_ref = oracle.muon_pre(G[i], M[i], 0.95, nesterov)
            assert torch.equal(Md[i].cpu(), m_ref), "momentum must be bit exact"
            assert torch.equal(U[i].cpu(), u_ref)
            M[i] = m_ref


def test_muon_pre_first_step_is_gradient():
    from dion_amd import ops

    torch.manual_seed(1)
    G = [torch.randn(32, 64, device=DEV).to(torch.bfloat16)]
    M = [torch.zeros(32, 64, device=DEV)]
    U = ops.muon_pre(G, M, 0.95, True)
    assert torch.equal(M[0], G[0].float())
    assert torch.equal(U[0], (G[0].float() * 0.95 + G[0].float()).to(torch.bfloat16))


@pytest.mark.parametrize("shape", [(64, 128), (7, 13), (3, 40, 24)])
@pytest.mark.parametrize("cautious", [False, True])
@pytest.mark.parametrize("udtype", [torch.bfloat16, torch.float32])
def test_muon_post(shape, cautious, udtype):
    from dion_amd import ops

    torch.manual_seed(2)
    n = 2
    X = [torch.randn(shape) * 0.02 for _ in range(n)]
    U = (torch.randn(n, *shape) * 0.1).to(udtype)
    lr = torch.tensor(0.02, device=DEV)
    Xd = [x.to(DEV) for x in X]
    ops.muon_post(Xd, U.to(DEV), lr, 0.5, 0.01, cautious)
    for i in range(n):
        ref = oracle.muon_post(X[i], U[i], 0.02, 0.5, 0.01, cautious)
        assert _rel(Xd[i], ref) <= 1e-6
        assert float((Xd[i].cpu() - ref).abs().max()) <= 1e-7
    # live weight decay tensor on the device gives the same result
    Xd2 = [x.to(DEV) for x in X]
    ops.muon_post(Xd2, U.to(DEV), lr, 0.5, torch.tensor(0.01, device=DEV), cautious)
    assert all(torch.equal(a, b) for a, b in zip(Xd, Xd2))


def test_muon_post_zero_update_is_pure_decay():
    from dion_amd import ops

    X = [torch.randn(16, 24, device=DEV)]
    x0 = X[0].clone()
    ops.muon_post(X, torch.zeros(1, 16, 24, device=DEV, dtype=torch.bfloat16), torch.tensor(0.1, device=DEV),
                  1.0, 0.5, False)
    a = 1 - torch.tensor(0.1) * torch.tensor(0.5)
    assert torch.equal(X[0].cpu(), x0.cpu() * a)


@pytest.mark.parametrize("shape", [(4, 64, 128), (2, 10, 24), (3, 128, 64), (1, 2, 17, 33)])
def test_normuon_stats_and_post(shape):
    from dion_amd import ops

    torch.manual_seed(3)
    n = shape[0]
    U = (torch.randn(shape) * 0.05).to(torch.bfloat16)
    V = [torch.rand(*shape[1:-1], 1) * 1e-3 for _ in range(n)]
    Vd = [v.to(DEV) for v in V]
    X = [torch.randn(shape[1:]) * 0.02 for _ in range(n)]
    Xd = [x.to(DEV) for x in X]
    Ud = U.to(DEV)
    scale = ops.normuon_stats(Ud, Vd, 0.95)
    ops.muon_post(Xd, Ud, torch.tensor(0.02, device=DEV), 0.5, 0.01, False, row_scale=scale)
    for i in range(n):
        nU, v_ref = oracle.normuon_normalize(U[i], V[i], 0.95)
        assert _rel(Vd[i], v_ref) <= 1e-5
        x_ref = oracle.muon_post(X[i], nU, 0.02, 0.5, 0.01, False)
        assert _rel(Xd[i], x_ref) <= 1e-5
        # the implied normalised update itself
        rows = shape[-2]
        s = scale.view(n, -1, rows)[i].reshape(*shape[1:-1], 1).cpu()
        assert _rel(U[i].float() * s, nU) <= 1e-5


@pytest.mark.parametrize("shape,frac", [((17, 40), 0.35), ((40, 17), 0.35), ((64, 128), 0.25), ((128, 64), 0.25),
                                        ((3, 32, 48), 0.5), ((16, 16), 1.0)])
def test_dion2_select_and_post(shape, frac):
    from dion_amd import ops

    torch.manual_seed(4)
    n = 2
    rows, cols = shape[-2:]
    sd = oracle.dion2_select_dim(rows, cols)
    dim = rows if sd == -2 else cols
    k = min(oracle.dion2_k(frac, dim), dim)
    G = [(torch.randn(shape) * 0.02).to(torch.bfloat16) for _ in range(n)]
    M = [torch.randn(shape) * 0.02 for _ in range(n)]
    X = [torch.randn(shape) * 0.02 for _ in range(n)]
    as3 = lambda t: t.reshape(-1, rows, cols)
    Gd = [as3(g).to(DEV) for g in G]
    Md = [as3(m).to(DEV) for m in M]
    Xd = [as3(x).to(DEV) for x in X]
    U, idx, imap = ops.dion2_select(Gd, Md, k, sd, 0.9)
    mats = Gd[0].shape[0]
    assert idx.shape == (n * mats, k) and imap.shape == (n * mats, dim)
    O = (torch.randn(U.shape) * 0.1).to(torch.bfloat16)  # stand-in for the orthogonalized block
    ops.dion2_post(Xd, O.to(DEV), imap, torch.tensor(0.02, device=DEV), 1.5, 0.1, sd)
    for i in range(n):
        for b in range(mats):
            m_ref, u_ref, idx_ref = oracle.dion2_pre(as3(G[i])[b], as3(M[i])[b], frac, 0.9, sd)
            got_idx = idx[i * mats + b].cpu().long()
            assert torch.equal(got_idx, idx_ref)
            assert torch.equal(U[i, b].cpu(), u_ref)
            assert _rel(Md[i][b], m_ref) <= 1e-6
            mp = imap[i * mats + b].cpu()
            assert int((mp >= 0).sum()) == k and torch.equal(mp[got_idx], torch.arange(k, dtype=torch.int32))
            x_ref = oracle.dion2_post(as3(X[i])[b], O[i, b], idx_ref, 0.02, 1.5, 0.1, sd)
            assert _rel(Xd[i][b], x_ref) <= 1e-6
            # unselected entries are exactly a*x (reference tests/test_dion2_post_ortho_triton.py:253-258)
            a = 1 - torch.tensor(0.02) * torch.tensor(0.1)
            mask = torch.ones(dim, dtype=torch.bool)
            mask[idx_ref] = False
            got = Xd[i][b].cpu()
            exp = as3(X[i])[b] * a
            if sd == -2:
                assert torch.equal(got[mask], exp[mask])
            else:
                assert torch.equal(got[:, mask], exp[:, mask])


def test_dion2_topk_ties_and_padding_rows():
    """Zero (padding) slices are never selected ahead of real ones; ties go to the lower index."""
    from dion_amd import ops

    M = [torch.zeros(1, 20, 8, device=DEV)]
    vals = torch.arange(1, 18, dtype=torch.float32, device=DEV)
    M[0][0, :17, 0] = vals  # 17 real rows, 3 zero rows
    G = [torch.zeros(1, 20, 8, device=DEV)]
    k = 6
    U, idx, imap = ops.dion2_select(G, M, k, -2, 1.0)
    assert idx[0].tolist() == [11, 12, 13, 14, 15, 16]
    M2 = [torch.ones(1, 10, 4, device=DEV)]
    U, idx, imap = ops.dion2_select([torch.zeros(1, 10, 4, device=DEV)], M2, 3, -2, 1.0)
    assert idx[0].tolist() == [0, 1, 2]


def test_select_dim_validation():
    from dion_amd import ops

    t = [torch.zeros(1, 8, 8, device=DEV)]
    with pytest.raises(ValueError, match="select_dim"):
        ops.dion2_select(t, t, 2, 0, 1.0)
    with pytest.raises(ValueError, match="select_dim"):
        ops.dion2_post(t, torch.zeros(1, 1, 2, 8, device=DEV, dtype=torch.bfloat16),
                       torch.zeros(1, 8, dtype=torch.int32, device=DEV), torch.tensor(0.1, device=DEV), 1.0, 0.0, 1)
