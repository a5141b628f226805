"""GPU parity of the reference's list-of-tensors operator functions (same names and call signatures,
import paths dion.dion2 / dion.dion2_triton / dion.scalar_opts) against the CPU oracle.  The cases of
the post-orthogonalization tests follow tests/test_dion2_post_ortho_triton.py:206-303 of the reference
(fp32 parameters): unselected entries are bitwise a*x, selected ones within 1e-6 / 1e-5."""
import math

import pytest
import torch

from oracle import dion_oracle as oracle

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _rel(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / b.norm().clamp(min=1e-30))


def _post_case(shape, k, select_dim, seed, u_dtype):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(shape, generator=g)
    lead = shape[:-2]
    full = shape[select_dim]
    nb = math.prod(lead) if lead else 1
    # unordered, distinct indices per matrix
    idx = torch.stack([torch.randperm(full, generator=g)[:k] for _ in range(nb)]).view(*lead, k)
    ushape = (*lead, k, shape[-1]) if select_dim == -2 else (*lead, shape[-2], k)
    u = torch.randn(ushape, generator=g).to(u_dtype)
    return x, u, idx


def _post_ref(x, u, idx, lr, adj, wd, select_dim):
    rows, cols = x.shape[-2], x.shape[-1]
    xf = x.reshape(-1, rows, cols)
    uf = u.reshape(-1, *u.shape[-2:])
    idf = idx.reshape(-1, idx.shape[-1])
    out = torch.empty_like(xf)
    masks = torch.zeros_like(xf, dtype=torch.bool)
    for b in range(xf.shape[0]):
        order = idf[b].argsort()
        sidx = idf[b][order]
        ub = uf[b][order] if select_dim == -2 else uf[b][:, order]
        out[b] = oracle.dion2_post(xf[b], ub, sidx, lr, adj / lr, wd, select_dim)
        if select_dim == -2:
            masks[b][sidx] = True
        else:
            masks[b][:, sidx] = True
    return out.view(x.shape), masks.view(x.shape)


@pytest.mark.parametrize("shape, select_dim, fraction, weight_decay", [
    ((64, 128), -2, 0.25, 0.01), ((64, 128), -2, 0.5, 0.01), ((128, 64), -2, 0.25, 0.01),
    ((64, 128), -1, 0.25, 0.01), ((128, 64), -1, 0.5, 0.01), ((64, 64), -2, 0.5, 0.01),
    ((4, 32, 128), -2, 0.25, 0.01), ((4, 128, 32), -1, 0.5, 0.01), ((8, 64, 64), -2, 0.5, 0.01),
    ((64, 128), -2, 1.0, 0.01), ((64, 128), -2, 1 / 64, 0.01), ((64, 128), -2, 0.25, 0.0),
    ((7, 13), -2, 0.4, 0.01), ((7, 13), -1, 0.4, 0.01),
])
@pytest.mark.parametrize("u_dtype", [torch.bfloat16, torch.float32])
def test_post_orthogonalize_single_tensor(shape, select_dim, fraction, weight_decay, u_dtype):
    from dion.dion2 import dion2_post_orthogonalize, dion2_post_orthogonalize_fused
    from dion.dion2_triton import TRITON_AVAILABLE, dion2_post_orthogonalize_triton

    assert TRITON_AVAILABLE
    full = shape[select_dim]
    k = max(1, int(math.ceil(fraction * full)))
    x, u, idx = _post_case(shape, k, select_dim, 42, u_dtype)
    ref, sel = _post_ref(x, u, idx, 0.01, 0.005, weight_decay, select_dim)
    kwargs = dict(indices=[idx.to(DEV)], base_lr=torch.tensor(0.01, device=DEV),
                  adjusted_lr=torch.tensor(0.005, device=DEV),
                  weight_decay=torch.tensor(weight_decay, device=DEV), select_dim=select_dim)
    outs = []
    for fn in (dion2_post_orthogonalize_triton, dion2_post_orthogonalize, dion2_post_orthogonalize_fused):
        xd = x.clone().to(DEV)
        fn(X=[xd], U=[u.to(DEV)], **kwargs)
        outs.append(xd.cpu())
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    got = outs[0]
    a = 1 - torch.tensor(0.01) * torch.tensor(weight_decay)
    assert torch.equal(got[~sel], (x * a)[~sel]), "unselected entries must be bitwise a*x"
    assert torch.allclose(got[sel], ref[sel], atol=1e-6, rtol=1e-5)
    assert torch.allclose(got, ref, atol=1e-6, rtol=1e-5)


def test_post_orthogonalize_megabatch_and_errors():
    from dion.dion2_triton import dion2_post_orthogonalize_triton

    shape, k = (64, 128), 16
    cases = [_post_case(shape, k, -2, 42 + i, torch.bfloat16) for i in range(4)]
    Xd = [c[0].clone().to(DEV) for c in cases]
    kwargs = dict(base_lr=torch.tensor(0.01, device=DEV), adjusted_lr=torch.tensor(0.005, device=DEV),
                  weight_decay=torch.tensor(0.01, device=DEV))
    dion2_post_orthogonalize_triton(X=Xd, U=[c[1].to(DEV) for c in cases], indices=[c[2].to(DEV) for c in cases],
                                    select_dim=-2, **kwargs)
    for xd, (x, u, idx) in zip(Xd, cases):
        ref, sel = _post_ref(x, u, idx, 0.01, 0.005, 0.01, -2)
        assert torch.equal(xd.cpu()[~sel], (x * (1 - torch.tensor(0.01) * torch.tensor(0.01)))[~sel])
        assert torch.allclose(xd.cpu(), ref, atol=1e-6, rtol=1e-5)
    x, u, idx = cases[0]
    with pytest.raises(ValueError):
        dion2_post_orthogonalize_triton(X=[x.to(DEV)], U=[u.to(DEV)], indices=[idx.to(DEV)], select_dim=0, **kwargs)
    xt = torch.randn(128, 64, device=DEV).t()  # [64, 128] view, not contiguous
    with pytest.raises(ValueError):
        dion2_post_orthogonalize_triton(X=[xt], U=[u.to(DEV)], indices=[idx.to(DEV)], select_dim=-2, **kwargs)
    # an empty tensor is skipped (dion/dion2_triton.py:206-212)
    dion2_post_orthogonalize_triton(X=[torch.empty(0, 128, device=DEV)],
                                    U=[torch.empty(0, 128, dtype=torch.bfloat16, device=DEV)],
                                    indices=[torch.empty(0, dtype=torch.int64, device=DEV)], select_dim=-2, **kwargs)


def test_build_index_map():
    from dion.dion2_triton import _build_index_map

    g = torch.Generator().manual_seed(3)
    idx = torch.stack([torch.randperm(37, generator=g)[:9] for _ in range(5)])
    imap = _build_index_map(idx.to(DEV), 37).cpu()
    assert imap.shape == (5, 37) and imap.dtype == torch.int32
    for b in range(5):
        ref = torch.full((37,), -1, dtype=torch.int32)
        ref[idx[b]] = torch.arange(9, dtype=torch.int32)
        assert torch.equal(imap[b], ref)
    with pytest.raises(TypeError):
        _build_index_map(idx.to(torch.int32).to(DEV), 37)


@pytest.mark.parametrize("shape,select_dim", [((64, 128), -2), ((128, 64), -1), ((3, 32, 48), -2), ((7, 13), -1)])
@pytest.mark.parametrize("gdtype", [torch.bfloat16, torch.float32])
def test_pre_orthogonalize_lists(shape, select_dim, gdtype):
    """dion2_pre_orthogonalize on a list of parameters: momentum bit exact, selected set and block equal
    to the CPU restatement's, int64 indices; k_override forces (and clamps) the count."""
    from dion.dion2 import dion2_pre_orthogonalize

    torch.manual_seed(5)
    n = 3
    G = [(torch.randn(shape) * 0.02).to(gdtype) for _ in range(n)]
    M = [torch.randn(shape) * 0.01 for _ in range(n)]
    Md = [m.clone().to(DEV) for m in M]
    U, idx = dion2_pre_orthogonalize([g.to(DEV) for g in G], Md, torch.tensor(0.25), torch.tensor(0.9), select_dim)
    rows, cols = shape[-2], shape[-1]
    dim = shape[select_dim]
    k = max(1, math.ceil(0.25 * dim))
    for i in range(n):
        assert idx[i].dtype == torch.int64 and idx[i].shape == (*shape[:-2], k)
        assert U[i].dtype == torch.bfloat16
        gm, mm = G[i].reshape(-1, rows, cols), M[i].reshape(-1, rows, cols)
        for j in range(gm.shape[0]):
            m_ref, u_ref, idx_ref = oracle.dion2_pre(gm[j], mm[j], 0.25, 0.9, select_dim)
            assert torch.equal(idx[i].reshape(-1, k)[j].cpu(), idx_ref)
            assert torch.equal(U[i].reshape(-1, *u_ref.shape)[j].cpu(), u_ref)
            assert torch.equal(Md[i].reshape(-1, rows, cols)[j].cpu(), m_ref)
    M2 = [m.clone().to(DEV) for m in M]
    U2, idx2 = dion2_pre_orthogonalize([g.to(DEV) for g in G], M2, 0.25, 0.9, select_dim, k_override=dim + 5)
    assert idx2[0].shape[-1] == dim and U2[0].shape[select_dim] == dim


def test_pre_orthogonalize_empty_shard():
    from dion.dion2 import dion2_pre_orthogonalize

    U, idx = dion2_pre_orthogonalize([torch.empty(0, 16, dtype=torch.bfloat16, device=DEV)],
                                     [torch.empty(0, 16, device=DEV)], 0.25, 0.9, -2)
    assert U[0].shape == (0, 16) and idx[0].shape == (0,)


@pytest.mark.parametrize("form", ["legacy", "capturable"])
@pytest.mark.parametrize("cautious", [False, True])
def test_adamw_update_foreach(form, cautious):
    """Both forms of the reference's call (python-int step; per-parameter device counters with a tensor
    lr) over a ragged list of more than 48 tensors, against the float64 restatement."""
    from dion.scalar_opts import adamw_update_foreach

    torch.manual_seed(7)
    sizes = [1, 5, 64, 1001] + [9 + i for i in range(50)]
    X = [torch.randn(n) for n in sizes]
    M = [torch.zeros(n) for n in sizes]
    V = [torch.zeros(n) for n in sizes]
    Xd, Md, Vd = ([t.to(DEV) for t in ts] for ts in (X, M, V))
    counters = [torch.zeros((), device=DEV) for _ in sizes]
    for step in range(1, 4):
        G = [torch.randn(n) for n in sizes]
        Gd = [g.to(DEV) for g in G]
        if form == "legacy":
            adamw_update_foreach(Xd, Gd, Md, Vd, 0.01, 0.9, 0.95, 0.1, step, 1e-8, cautious_wd=cautious)
        else:
            adamw_update_foreach(Xd, Gd, Md, Vd, torch.tensor(0.01, device=DEV), torch.tensor(0.9),
                                 torch.tensor(0.95), torch.tensor(0.1, device=DEV), epsilon=1e-8,
                                 cautious_wd=cautious, state_steps=counters)
        for i in range(len(X)):
            x, m, v = oracle.adamw_update(X[i], G[i], M[i], V[i], 0.01, 0.9, 0.95, 0.1, step, 1e-8, cautious)
            assert _rel(Md[i], m) <= 1e-6 and _rel(Vd[i], v) <= 1e-6
            assert float((Xd[i].double().cpu() - x).abs().max()) <= 2e-6
            X[i], M[i], V[i] = Xd[i].double().cpu(), Md[i].double().cpu(), Vd[i].double().cpu()
    if form == "capturable":
        assert all(float(c) == 3.0 for c in counters)
    with pytest.raises(ValueError):
        adamw_update_foreach(Xd, Gd, Md, Vd, 0.01, 0.9, 0.95, 0.1)


def test_lion_update_foreach():
    from dion.scalar_opts import lion_update_foreach

    torch.manual_seed(8)
    sizes = [3, 64, 1001]
    X = [torch.randn(n) for n in sizes]
    M = [torch.randn(n) * 0.1 for n in sizes]
    G = [torch.randn(n) for n in sizes]
    Xd, Md = [x.to(DEV) for x in X], [m.to(DEV) for m in M]
    lion_update_foreach(Xd, [g.to(DEV) for g in G], Md, torch.tensor(0.01, device=DEV), 0.9, 0.99, 0.1)
    for i in range(len(X)):
        x_ref, m_ref = oracle.lion_update(X[i], G[i], M[i], 0.01, 0.9, 0.99, 0.1)
        assert _rel(Md[i], m_ref) <= 1e-6
        bad = (Xd[i].double().cpu() - x_ref).abs() > 1e-6
        assert int(bad.sum()) <= 1  # a blend within rounding of zero may take the other sign


@pytest.mark.parametrize("nesterov", [False, True])
def test_muon_update_pre_and_post_orthogonalize(nesterov):
    """The list-of-tensors forms of dion/muon.py:284-347 against the oracle."""
    from dion.muon import muon_update_post_orthogonalize, muon_update_pre_orthogonalize

    torch.manual_seed(21)
    shape, n = (48, 80), 3
    G = [(torch.randn(shape) * 0.02).to(torch.bfloat16) for _ in range(n)]
    M = [torch.randn(shape) * 0.01 for _ in range(n)]
    X = [torch.randn(shape) * 0.05 for _ in range(n)]
    Md, Xd = [m.to(DEV) for m in M], [x.to(DEV) for x in X]
    U = muon_update_pre_orthogonalize([g.to(DEV) for g in G], Md, torch.tensor(0.95), nesterov)
    assert len(U) == n and all(u.dtype == torch.bfloat16 and u.shape == shape for u in U)
    for i in range(n):
        m_ref, u_ref = oracle.muon_pre(G[i], M[i], 0.95, nesterov)
        assert torch.equal(Md[i].cpu(), m_ref) and torch.equal(U[i].cpu(), u_ref)
    base_lr, adjusted_lr = torch.tensor(0.02, device=DEV), torch.tensor(0.02 * 0.7746, device=DEV)
    for cautious, u_list in ((False, U), (True, [u.float().clone() for u in U])):  # arena views, then loose tensors
        Xc = [x.clone() for x in Xd]
        muon_update_post_orthogonalize(Xc, u_list, base_lr, adjusted_lr, 0.1, cautious_wd=cautious)
        for i in range(n):
            ref = oracle.muon_post(X[i], U[i].cpu(), 0.02, float(adjusted_lr) / 0.02, 0.1, cautious)
            assert float((Xc[i].cpu() - ref).abs().max()) <= 1e-7
    muon_update_post_orthogonalize([], [], base_lr, adjusted_lr, 0.1)
    assert muon_update_pre_orthogonalize([], [], 0.95, nesterov) == []


@pytest.mark.parametrize("vdtype", [torch.float32, torch.bfloat16])
def test_normuon_normalization_stacked(vdtype):
    """dion/normuon.py:344-399 out of place: normalised update and new second moments against the oracle,
    the Frobenius norm is preserved, and split_sizes equals separate calls on the blocks."""
    from dion.normuon import normuon_normalization_stacked

    torch.manual_seed(22)
    n, rows, cols = 4, 24, 40
    U = (torch.randn(n, rows, cols) * 0.05).to(torch.bfloat16)
    V = (torch.rand(n, rows, 1) * 1e-3).to(vdtype)
    Ud, Vd = U.to(DEV), V.to(DEV)
    v_before = Vd.clone()
    nU, nV = normuon_normalization_stacked(Ud, Vd, torch.tensor(0.95))
    assert torch.equal(Vd, v_before), "the call is out of place"
    assert nU.dtype == vdtype and nV.dtype == vdtype and nU.shape == U.shape and nV.shape == V.shape
    tol = 1e-5 if vdtype == torch.float32 else 2.0 ** -7
    for i in range(n):
        u_ref, v_ref = oracle.normuon_normalize(U[i], V[i].float(), 0.95)
        assert _rel(nV[i].float(), v_ref) <= tol and _rel(nU[i].float(), u_ref) <= tol
        assert abs(float(nU[i].float().norm()) / float(U[i].float().norm()) - 1) <= tol
    split = (8, 16)
    sU, sV = normuon_normalization_stacked(Ud, Vd, 0.95, split_sizes=split)
    off = 0
    for sz in split:
        bU, bV = normuon_normalization_stacked(Ud[:, off:off + sz].contiguous(), Vd[:, off:off + sz].contiguous(), 0.95)
        assert torch.equal(sU[:, off:off + sz], bU) and torch.equal(sV[:, off:off + sz], bV)
        off += sz
    with pytest.raises(ValueError):
        normuon_normalization_stacked(Ud, Vd, 0.95, split_sizes=(8, 8))
    with pytest.raises(TypeError):
        normuon_normalization_stacked(Ud.float(), Vd, 0.95)


@pytest.mark.parametrize("vdtype", [torch.float32, torch.bfloat16])
def test_normalize_selected_stacked_matches_unfused(vdtype):
    """The reference's own check (tests/test_optimizers.py:241-277): the selected-rows helper equals gather ->
    normuon_normalization_stacked -> scatter."""
    from dion.nordion2 import nordion2_normalize_selected_stacked
    from dion.normuon import normuon_normalization_stacked

    torch.manual_seed(3)
    n, rows, cols, k = 4, 16, 32, 8
    u = torch.randn(n, k, cols, device=DEV, dtype=torch.bfloat16)
    v_full = torch.rand(n, rows, 1, device=DEV).to(vdtype)
    indices = torch.stack([torch.randperm(rows, device=DEV)[:k] for _ in range(n)], dim=0)
    beta2 = torch.tensor(0.9)
    u_fused, v_fused = nordion2_normalize_selected_stacked(u.clone(), v_full.clone(), indices, beta2)
    assert u_fused.dtype == torch.float32 and v_fused.dtype == vdtype

    idx = indices.unsqueeze(-1)
    v_sel = torch.gather(v_full, dim=-2, index=idx).float()
    u_ref, v_sel_new = normuon_normalization_stacked(u.clone(), v_sel, beta2)
    v_ref = v_full.clone()
    for i in range(n):
        v_ref[i].scatter_(dim=-2, index=idx[i], src=v_sel_new[i].to(v_ref.dtype))
    if vdtype == torch.float32:
        torch.testing.assert_close(u_fused, u_ref, atol=1e-5, rtol=1e-5)
        torch.testing.assert_close(v_fused, v_ref, atol=1e-5, rtol=1e-5)
    else:  # the scale comes from the stored (rounded) second moments
        torch.testing.assert_close(u_fused, u_ref, atol=1e-5, rtol=2.0 ** -8)
        assert torch.equal(v_fused, v_ref)
    unsel = torch.ones(n, rows, dtype=torch.bool, device=DEV).scatter_(1, indices, False)
    assert torch.equal(v_fused.squeeze(-1)[unsel], v_full.squeeze(-1)[unsel])


def test_submodule_import_paths():
    """The names the reference's tests and callers import from its submodules resolve."""
    import dion
    from dion.cuda_graph import CudaGraphOptimizer
    from dion.dion2 import Dion2, _make_select_and_orthogonalize, dion2_post_orthogonalize_masked, dion2_pre_accumulate
    from dion.dion3 import Dion3
    from dion.muon import Muon, muon_update_post_orthogonalize, muon_update_pre_orthogonalize
    from dion.newton_schulz_triton import newton_schulz_triton, ns_line_1, ns_line_2, ns_line_3, zeropower_via_newtonschulz5
    from dion.nordion2 import NorDion2, nordion2_normalize_selected_stacked, nordion2_post_orthogonalize_masked
    from dion.normuon import NorMuon, normuon_normalization_stacked
    from dion.opt_utils import as_scalar_tensor, lm_head_lr_scale
    from dion.polar_express import polar_express, polar_express_triton

    assert Dion3 is NorDion2 is dion.NorDion2 and Dion2 is dion.Dion2 and Muon is dion.Muon and NorMuon is dion.NorMuon
    assert all(callable(f) for f in (CudaGraphOptimizer, _make_select_and_orthogonalize, dion2_pre_accumulate,
                                     dion2_post_orthogonalize_masked, nordion2_post_orthogonalize_masked,
                                     newton_schulz_triton, ns_line_1, ns_line_2, ns_line_3,
                                     zeropower_via_newtonschulz5, polar_express, polar_express_triton,
                                     muon_update_pre_orthogonalize, muon_update_post_orthogonalize,
                                     nordion2_normalize_selected_stacked, normuon_normalization_stacked,
                                     as_scalar_tensor, lm_head_lr_scale))
