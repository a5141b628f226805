"""Pins the CPU oracle (oracle/dion_oracle.py) without running the reference: closed forms,
invariants, brute force on tiny inputs and the bounds the reference's own tests state.  A dropped
term, a wrong sign or a transposed operand in the oracle fails at least one of these."""
import math

import numpy as np
import pytest
import torch

from oracle import dion_oracle as o


def _rand_svd(m, n, s, seed):
    rng = np.random.default_rng(seed)
    U, _ = np.linalg.qr(rng.standard_normal((m, m)))
    V, _ = np.linalg.qr(rng.standard_normal((n, m)))
    return U, V, (U * s) @ V.T


@pytest.mark.parametrize("coeffs,scale", [(o.NS5_COEFFS, 1.0), (o.POLAR_EXPRESS_COEFFS, 1.02), (o.KJ_COEFFS, 1.0)])
def test_fp64_ns_is_the_scalar_map_on_singular_values(coeffs, scale):
    """For G = U diag(s) V^T the iteration returns U diag(phi(s/(scale*||s||))) V^T."""
    m, n = 12, 20
    s = np.linspace(0.2, 1.0, m)
    U, V, G = _rand_svd(m, n, s, 0)
    X = o.ns_fp64(G, coeffs, scale, 0.0, round_input=False)
    phi = o.scalar_map(s / (np.linalg.norm(s) * scale), coeffs)
    np.testing.assert_allclose(X, (U * phi) @ V.T, atol=1e-10)
    # tall input: same map on the transpose
    Xt = o.ns_fp64(G.T, coeffs, scale, 0.0, round_input=False)
    np.testing.assert_allclose(Xt, X.T, atol=1e-10)


def test_scalar_bands_of_the_coefficient_tables():
    """Band each schedule maps the unit interval into (computed from the tables)."""
    x = np.linspace(0.01, 1.0, 20001)
    ns5 = o.scalar_map(x, o.NS5_COEFFS)
    assert 0.97 < ns5.min() and ns5.max() < 1.04
    pe = o.scalar_map(np.linspace(0.001, 1.0, 20001) / 1.02, o.POLAR_EXPRESS_COEFFS)
    assert 0.84 < pe.min() and pe.max() < 1.15
    kj = o.scalar_map(np.linspace(0.005, 1.0, 20001), o.KJ_COEFFS)
    assert 0.68 < kj.min() and kj.max() < 1.16
    # fixed point structure: a + b + c maps 1 close to 1 for the last (polishing) NS5 polynomial
    a, b, c = o.NS5_COEFFS[-1]
    assert abs(a + b + c - 1.0) < 0.02


def test_fp64_invariances():
    rng = np.random.default_rng(1)
    G = o.bf16_round(rng.standard_normal((3, 16, 40)))
    X = o.ns_fp64(G, o.NS5_COEFFS, 1.0, 0.0)
    # positive scaling by a power of two (exact in bf16) does not change the result
    np.testing.assert_allclose(o.ns_fp64(4.0 * G, o.NS5_COEFFS, 1.0, 0.0), X, atol=1e-12)
    # row permutation equivariance
    perm = rng.permutation(16)
    np.testing.assert_allclose(o.ns_fp64(G[:, perm], o.NS5_COEFFS, 1.0, 0.0), X[:, perm], atol=1e-10)
    # zero rows stay zero
    G2 = G.copy()
    G2[:, 3] = 0
    assert np.abs(o.ns_fp64(G2, o.NS5_COEFFS, 1.0, 0.0)[:, 3]).max() == 0.0
    # batching is independent per matrix
    np.testing.assert_allclose(o.ns_fp64(G[1], o.NS5_COEFFS, 1.0, 0.0), X[1], atol=1e-12)


def test_gram_form_equals_standard_form_in_exact_arithmetic():
    rng = np.random.default_rng(2)
    for shape in [(10, 24), (24, 10), (2, 8, 8)]:
        G = rng.standard_normal(shape)
        a = o.gram_ns_fp64(G, o.POLAR_EXPRESS_COEFFS, 1.02, 0.0, reset_iterations=(2,))
        b = o.ns_fp64(G, o.POLAR_EXPRESS_COEFFS, 1.02, 0.0)
        np.testing.assert_allclose(a, b, atol=1e-9)
        c = o.gram_ns_fp64(G, o.POLAR_EXPRESS_COEFFS, 1.02, 0.0, reset_iterations=())
        np.testing.assert_allclose(c, b, atol=1e-8)


@pytest.mark.parametrize("shape", [(64, 128), (128, 64), (128, 128), (4, 64, 128), (4, 128, 64)])
def test_bf16_paths_meet_the_references_orthogonality_bound(shape):
    """max|X X^T - I| < 0.15 on seed 42 (reference tests/test_polar_express.py:10-42, :81-99)."""
    for fn in (lambda g: o.polar_express_bf16(g), lambda g: o.ns_bf16(g), lambda g: o.ns_bf16_fused(g)):
        torch.manual_seed(42)
        G = torch.randn(shape)
        X = fn(G).float()
        P = X @ X.mT if shape[-2] <= shape[-1] else X.mT @ X
        assert float((P - torch.eye(P.shape[-1])).abs().max()) < 0.15


def test_bf16_paths_track_fp64():
    torch.manual_seed(3)
    G = torch.randn(96, 160)
    r64 = o.ns_fp64(G.numpy(), o.NS5_COEFFS, 1.0, 1e-7)
    for X in (o.ns_bf16(G), o.ns_bf16_fused(G)):
        err = np.linalg.norm(X.float().numpy() - r64) / np.linalg.norm(r64)
        assert err < 3e-2
    # polar_express on a tall input equals polar_express on the transpose (up to bf16 noise)
    a = o.polar_express_bf16(G.T.contiguous()).float()
    b = o.polar_express_bf16(G).float().T
    assert float((a - b).norm() / b.norm()) < 6e-2
    # KJ variant normalises before transposing: same Frobenius norm either way
    k1 = o.kj_ns_bf16(G).float()
    k2 = o.kj_ns_bf16(G.T.contiguous()).float().T
    assert float((k1 - k2).norm() / k1.norm()) < 6e-2


def test_muon_pre_first_step_closed_form():
    """Zero momentum: M == G exactly; nesterov U == bf16((1+mu) G) (reference
    tests/test_state_prepopulation.py:110-125)."""
    torch.manual_seed(4)
    G = torch.randn(8, 12).to(torch.bfloat16)
    M0 = torch.zeros(8, 12)
    M1, U = o.muon_pre(G, M0, 0.95, nesterov=True)
    assert torch.equal(M1, G.float())
    expect = (G.float() * torch.tensor(0.95) + G.float()).to(torch.bfloat16)
    assert torch.equal(U, expect)
    M1b, Ub = o.muon_pre(G, M0, 0.95, nesterov=False)
    assert torch.equal(Ub, G)
    # second step: M = mu*M + G
    M2, _ = o.muon_pre(G, M1, 0.5, nesterov=False)
    assert torch.allclose(M2, 1.5 * G.float())


def test_muon_post_closed_forms_and_cautious_mask():
    X = torch.tensor([[1.0, -2.0], [3.0, -4.0]])
    Z = torch.zeros(2, 2)
    out = o.muon_post(X, Z, lr=0.1, adj_ratio=2.0, wd=0.5)
    assert torch.allclose(out, X * 0.95)
    U = torch.tensor([[1.0, 1.0], [-1.0, 0.0]])
    out = o.muon_post(X, U, lr=0.1, adj_ratio=2.0, wd=0.0)
    assert torch.allclose(out, X - 0.2 * U)
    # cautious: decay only where x*u >= 0 (brute force over the four sign cases + zero)
    out = o.muon_post(X, U, lr=0.1, adj_ratio=0.0, wd=0.5, cautious=True)
    expect = torch.tensor([[1.0 * 0.95, -2.0], [3.0, -4.0 * 0.95]])
    assert torch.allclose(out, expect)


def test_adjust_lr_ratio_closed_forms():
    assert o.adjust_lr_ratio((768, 3072), "spectral_norm") == pytest.approx(0.5)
    assert o.adjust_lr_ratio((3072, 768), "spectral_norm") == pytest.approx(2.0)
    assert o.adjust_lr_ratio((768, 3072), "rms_norm") == pytest.approx(0.2 * math.sqrt(3072))
    assert o.adjust_lr_ratio((4, 8, 16), "spectral_norm", flatten=True) == pytest.approx(math.sqrt(4 / 128))
    assert o.adjust_lr_ratio((5, 7), None) == 1.0


def test_normuon_normalize_invariants():
    torch.manual_seed(5)
    U = torch.randn(3, 10, 24)
    V0 = torch.zeros(3, 10, 1)
    N1, V1 = o.normuon_normalize(U, V0, 0.95)
    # Frobenius norm preserved per matrix
    assert torch.allclose(N1.norm(dim=(-2, -1)), U.norm(dim=(-2, -1)), rtol=1e-5)
    # first step: V = (1 - beta2) * mean(U^2)
    assert torch.allclose(V1, 0.05 * (U * U).mean(-1, keepdim=True), rtol=1e-5)
    # rows of equal energy: the normalised update is U itself
    E = torch.randn(1, 6, 16)
    E = E / E.norm(dim=-1, keepdim=True)
    N2, _ = o.normuon_normalize(E, torch.zeros(1, 6, 1), 0.9)
    assert torch.allclose(N2, E, atol=1e-5)
    # a row with twice the amplitude is scaled down relative to the others
    W = E.clone()
    W[0, 0] *= 2
    N3, _ = o.normuon_normalize(W, torch.zeros(1, 6, 1), 0.9)
    assert torch.allclose(N3[0, 0].norm(), N3[0, 1].norm(), rtol=1e-4)


def test_dion2_selection_bruteforce_and_degenerate_cases():
    torch.manual_seed(6)
    G = torch.randn(17, 40)
    M0 = torch.randn(17, 40)
    for frac, sd in [(0.35, -2), (0.25, -1), (1.0, -2)]:
        M1, U, idx = o.dion2_pre(G, M0, frac, 0.9, sd)
        S = M0 + G
        dim = 17 if sd == -2 else 40
        k = max(1, math.ceil(frac * dim))
        assert len(idx) == k  # 17 rows at 0.35 -> 6 (reference tests/test_dion2_selection_scope.py:138-169)
        norms = S.abs().sum(dim=1 if sd == -2 else 0)
        thresh = torch.sort(norms, descending=True).values[k - 1]
        assert bool((norms[idx] >= thresh).all())
        mask = torch.zeros(dim, dtype=torch.bool)
        mask[idx] = True
        assert bool((norms[~mask] <= thresh).all())
        if sd == -2:
            assert torch.equal(U, S[idx].to(torch.bfloat16))
            assert torch.allclose(M1[idx], S[idx] * 0.9) and torch.equal(M1[~mask], S[~mask])
        else:
            assert torch.equal(U, S[:, idx].to(torch.bfloat16))
            assert torch.allclose(M1[:, idx], S[:, idx] * 0.9) and torch.equal(M1[:, ~mask], S[:, ~mask])
    # fraction 1: every slice selected, M = ef_decay * (M + G)
    M1, U, idx = o.dion2_pre(G, M0, 1.0, 0.5, -2)
    assert torch.allclose(M1, 0.5 * (M0 + G)) and len(idx) == 17
    assert o.dion2_k(1, 64) == 64 and o.dion2_k(0.001, 64) == 1
    assert o.dion2_select_dim(32, 128) == -2 and o.dion2_select_dim(128, 32) == -1


def test_dion2_post_unselected_is_exactly_a_times_x():
    torch.manual_seed(7)
    X = torch.randn(9, 14)
    idx = torch.tensor([1, 4, 8])
    U = torch.randn(3, 14).to(torch.bfloat16)
    out = o.dion2_post(X, U, idx, lr=0.02, adj_ratio=1.5, wd=0.1, select_dim=-2)
    a = 1 - torch.tensor(0.02) * torch.tensor(0.1)
    mask = torch.ones(9, dtype=torch.bool)
    mask[idx] = False
    assert torch.equal(out[mask], (a.double() * X[mask].double()).float())
    b = torch.tensor(0.02) * torch.tensor(1.5)
    assert torch.allclose(out[idx], a * X[idx] - b * U.float(), rtol=1e-6)
    # column selection
    Uc = torch.randn(9, 2).to(torch.bfloat16)
    out = o.dion2_post(X, Uc, torch.tensor([0, 13]), 0.02, 1.5, 0.1, -1)
    assert torch.allclose(out[:, [0, 13]], a * X[:, [0, 13]] - b * Uc.float(), rtol=1e-6)
    assert torch.allclose(out[:, 1:13], a * X[:, 1:13])


def test_nordion2_selected_normalisation_reduces_to_normuon():
    """With every row selected, in order, the selected-row normalisation IS NorMuon's; with a subset,
    unselected entries of V are untouched and the update keeps the Frobenius norm of its input."""
    torch.manual_seed(9)
    U = torch.randn(6, 10).to(torch.bfloat16)
    V = torch.rand(6, 1) * 1e-2
    nU_all, V_all = o.nordion2_normalize_selected(U, V, torch.arange(6), 0.9)
    nU_ref, V_ref = o.normuon_normalize(U, V, 0.9)
    assert torch.equal(nU_all, nU_ref) and torch.equal(V_all, V_ref)
    idx = torch.tensor([1, 4, 5])
    nU, V2 = o.nordion2_normalize_selected(U[idx], V, idx, 0.9)
    keep = torch.tensor([0, 2, 3])
    assert torch.equal(V2[keep], V[keep])
    assert not torch.equal(V2[idx], V[idx])
    assert abs(float(nU.norm() / U[idx].float().norm()) - 1.0) < 1e-5


def test_nordion2_step_closed_cases():
    """fraction = 1 selects every row: M_after = mu * (M + G) everywhere, and the update equals a
    NorMuon-normalised orthogonalization of M + G.  First step from zero state: V = (1 - beta2) *
    mean(O^2) on selected rows and 0 elsewhere."""
    torch.manual_seed(10)
    x = torch.randn(8, 16) * 0.02
    g = (torch.randn(8, 16) * 0.02).to(torch.bfloat16)
    m = torch.randn(8, 16) * 0.02
    v = torch.zeros(8, 1)
    ident = lambda u: u  # keeps the case checkable by hand
    x2, m2, v2, idx = o.nordion2_step(x, g, m, v, 0.02, 1.0, 0.95, 0.9, 0.01, None, ns=ident)
    acc = m + g.float()
    assert torch.equal(idx, torch.arange(8))
    assert torch.allclose(m2, acc * 0.95, rtol=0, atol=0)
    u = acc.to(torch.bfloat16)
    nU, v_ref = o.normuon_normalize(u, v, 0.9)
    assert torch.equal(v2, v_ref)
    assert torch.allclose(x2, x * (1 - 0.02 * 0.01) - 0.02 * nU, rtol=1e-6, atol=1e-9)
    # a quarter of the rows: V stays zero off the selection
    x3, m3, v3, idx3 = o.nordion2_step(x, g, m, v, 0.02, 0.25, 0.95, 0.9, 0.01, None, ns=ident)
    assert idx3.numel() == 2
    mask = torch.ones(8, dtype=torch.bool)
    mask[idx3] = False
    assert float(v3[mask].abs().max()) == 0.0 and float(v3[idx3].min()) > 0.0
    assert torch.equal(m3[mask], acc[mask]) and torch.equal(x3[mask], (x * torch.tensor(1 - 0.02 * 0.01))[mask])


def test_adamw_restatement_known_answers():
    """The reference's hand-computed cautious-weight-decay vector (tests/test_adamw_foreach.py:80-112):
    mask [1, 0, 0, 1], two positions decayed, two not.  Plus torch.optim.AdamW as an independent
    implementation of the non-cautious rule over several steps."""
    X = torch.tensor([1.0, 1.0, -1.0, -1.0])
    G = torch.tensor([2.0, -2.0, 2.0, -2.0])
    lr, b1, b2, wd, eps = 0.1, 0.9, 0.999, 0.5, 1e-8
    x2, m2, v2 = o.adamw_update(X, G, torch.zeros(4), torch.zeros(4), lr, b1, b2, wd, 1, eps, cautious=True)
    m_new = (1 - b1) * G.double()
    v_new = (1 - b2) * G.double() ** 2
    update = (lr / (1 - b1)) * m_new / (v_new.sqrt() / math.sqrt(1 - b2) + eps)
    expected = X.double() - lr * wd * X.double() * torch.tensor([1.0, 0.0, 0.0, 1.0]).double() - update
    assert torch.allclose(x2, expected, atol=1e-12, rtol=0)
    assert torch.allclose(m2, m_new) and torch.allclose(v2, v_new)

    torch.manual_seed(21)
    p = torch.nn.Parameter(torch.randn(50, dtype=torch.float64))
    x, m, v = p.data.clone(), torch.zeros(50, dtype=torch.float64), torch.zeros(50, dtype=torch.float64)
    ref = torch.optim.AdamW([p], lr=0.01, betas=(0.9, 0.95), eps=1e-8, weight_decay=0.1)
    for step in range(1, 5):
        g = torch.randn(50, dtype=torch.float64)
        p.grad = g.clone()
        ref.step()
        x, m, v = o.adamw_update(x, g, m, v, 0.01, 0.9, 0.95, 0.1, step, 1e-8)
        assert torch.allclose(x, p.data, rtol=1e-10, atol=1e-12)


def test_lion_restatement_closed_cases():
    """First step from zero momentum: U = sign(G), so X moves by exactly lr against the gradient sign
    after the decay; M = (1-beta2) G.  Cautious decay touches only entries where sign(U) == sign(X)."""
    X = torch.tensor([1.0, 1.0, -1.0, -1.0, 0.5])
    G = torch.tensor([2.0, -2.0, 2.0, -2.0, 0.0])
    x2, m2 = o.lion_update(X, G, torch.zeros(5), 0.1, 0.9, 0.99, 0.5)
    assert torch.allclose(x2, X.double() * 0.95 - 0.1 * torch.sign(G).double(), atol=1e-15)
    assert torch.allclose(m2, 0.01 * G.double(), atol=1e-15)
    x3, _ = o.lion_update(X, G, torch.zeros(5), 0.1, 0.9, 0.99, 0.5, cautious=True)
    mask = torch.tensor([1.0, 0.0, 0.0, 1.0, 1.0]).double()  # U*X >= 0 (U = 0 counts)
    assert torch.allclose(x3, X.double() - 0.05 * X.double() * mask - 0.1 * torch.sign(G).double(), atol=1e-15)
    # second step blends momentum and gradient with beta1 before the sign
    M = torch.tensor([1.0, -1.0, 1.0, -1.0, 0.0])
    G2 = torch.tensor([-5.0, 5.0, -20.0, 20.0, 1.0])
    x4, m4 = o.lion_update(X, G2, M, 0.1, 0.9, 0.99, 0.0)
    blend = 0.9 * M.double() + 0.1 * G2.double()  # [0.4, -0.4, -1.1, 1.1, 0.1]
    assert torch.allclose(x4, X.double() - 0.1 * torch.sign(blend), atol=1e-15)
    assert torch.allclose(m4, 0.99 * M.double() + 0.01 * G2.double(), atol=1e-15)
