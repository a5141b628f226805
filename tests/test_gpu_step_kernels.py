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


@pytest.mark.parametrize("cautious", [False, True])
@pytest.mark.parametrize("gdtype", [torch.bfloat16, torch.float32])
def test_adamw_multi_tensor_vs_oracle(cautious, gdtype):
    """Ragged list (empty, scalar-sized, odd, unaligned view, > 48 tensors, one large) over three
    steps against the float64 restatement of dion/scalar_opts.py:7-65."""
    from dion_amd import ops

    torch.manual_seed(31)
    sizes = [0, 1, 3, 7, 64, 129, 1000, 4096 * 33 + 5] + [17 + i for i in range(50)]
    base = [torch.randn(n + 1) for n in sizes]
    X = [b[1:].clone() if i % 3 else b[:-1].clone() for i, b in enumerate(base)]
    Xd = [x.to(DEV) for x in X]
    # every third tensor is an offset view: 4-byte aligned only
    for i in range(0, len(Xd), 3):
        buf = torch.zeros(sizes[i] + 1, device=DEV)
        buf[1:].copy_(Xd[i])
        Xd[i] = buf[1:]
    M = [torch.zeros_like(x) for x in X]
    V = [torch.zeros_like(x) for x in X]
    Md = [torch.zeros_like(x) for x in Xd]
    Vd = [torch.zeros_like(x) for x in Xd]
    steps = [torch.zeros((), device=DEV) for _ in Xd]
    lr = torch.tensor(0.01, device=DEV)
    for step in range(1, 4):
        G = [torch.randn(n).to(gdtype) for n in sizes]
        ops.adamw_step(Xd, [g.to(DEV) for g in G], Md, Vd, steps, lr, 0.9, 0.95, 0.1, 1e-8, cautious)
        for i in range(len(X)):
            X[i], M[i], V[i] = oracle.adamw_update(X[i], G[i].float(), M[i], V[i], 0.01, 0.9, 0.95, 0.1, step,
                                                   1e-8, cautious)
            if sizes[i] == 0:
                continue
            assert _rel(Md[i], M[i]) <= 1e-6 and _rel(Vd[i], V[i]) <= 1e-6
            # bf16 gradients cancel the momentum exactly now and then (g2 == -0.9 g1): its sign, and
            # with it the cautious mask, is then decided by rounding -- leave those entries out
            clear = M[i].abs() > 1e-6 * G[i].double().abs()
            assert float(((Xd[i].double().cpu() - X[i]).abs() * clear).max()) <= 2e-6
            assert int((~clear).sum()) <= 1 + sizes[i] // 1000
            # keep fp32 rounding from accumulating into a sign flip of the cautious mask
            X[i], M[i], V[i] = Xd[i].double().cpu(), Md[i].double().cpu(), Vd[i].double().cpu()
        assert all(float(s) == float(step) for s in steps)


def test_adamw_known_answer_and_shared_step_counter():
    """The reference's hand-computed cautious case (tests/test_adamw_foreach.py:80-112) and a step
    counter shared by the tensors of one call (advanced once per call)."""
    from dion_amd import ops

    X = [torch.tensor([1.0, 1.0, -1.0, -1.0], device=DEV), torch.tensor([1.0, 1.0, -1.0, -1.0], device=DEV)]
    G = [torch.tensor([2.0, -2.0, 2.0, -2.0], device=DEV) for _ in range(2)]
    M = [torch.zeros(4, device=DEV) for _ in range(2)]
    V = [torch.zeros(4, device=DEV) for _ in range(2)]
    step = torch.zeros((), device=DEV)
    ops.adamw_step(X, G, M, V, [step, step], torch.tensor(0.1, device=DEV), 0.9, 0.999, 0.5, 1e-8, True)
    assert float(step) == 1.0
    g = torch.tensor([2.0, -2.0, 2.0, -2.0])
    x0 = torch.tensor([1.0, 1.0, -1.0, -1.0])
    m_new, v_new = 0.1 * g, 0.001 * g * g
    update = (0.1 / 0.1) * m_new / (v_new.sqrt() / (1 - 0.999) ** 0.5 + 1e-8)
    expected = x0 - 0.1 * 0.5 * x0 * torch.tensor([1.0, 0.0, 0.0, 1.0]) - update
    for x in X:
        assert torch.allclose(x.cpu(), expected, atol=1e-6, rtol=0)


@pytest.mark.parametrize("cautious", [False, True])
@pytest.mark.parametrize("gdtype", [torch.bfloat16, torch.float32])
def test_lion_multi_tensor_vs_oracle(cautious, gdtype):
    from dion_amd import ops

    torch.manual_seed(32)
    sizes = [0, 1, 5, 64, 1001, 4096 * 17 + 3] + [9 + i for i in range(50)]
    X = [torch.randn(n) for n in sizes]
    M = [torch.randn(n) * 0.1 for n in sizes]
    Xd, Md = [x.to(DEV) for x in X], [m.to(DEV) for m in M]
    lr = torch.tensor(0.01, device=DEV)
    for _ in range(2):
        G = [torch.randn(n).to(gdtype) for n in sizes]
        ops.lion_step(Xd, [g.to(DEV) for g in G], Md, lr, 0.9, 0.99, 0.1, cautious)
        for i in range(len(X)):
            x_ref, m_ref = oracle.lion_update(X[i], G[i].float(), M[i], 0.01, 0.9, 0.99, 0.1, cautious)
            if sizes[i]:
                assert _rel(Md[i], m_ref) <= 1e-6
                # a blend within rounding of zero may take the other sign: allow a handful of 2*lr moves
                d = (Xd[i].double().cpu() - x_ref).abs()
                assert int((d > 2e-6).sum()) <= max(1, sizes[i] // 100000)
            X[i], M[i] = Xd[i].cpu(), Md[i].cpu()


def test_scalar_groups_inside_an_optimizer():
    """Mixed param groups through Muon.step(): AdamW and Lion groups follow the restatement while
    the matrix group is orthogonalized; step_dev advances on the device."""
    from dion import Muon

    torch.manual_seed(33)
    w = torch.nn.Parameter(torch.randn(64, 128, device=DEV) * 0.02)
    b = torch.nn.Parameter(torch.randn(300, device=DEV))
    e = torch.nn.Parameter(torch.randn(50, 16, device=DEV))
    opt = Muon([{"params": [w]}, {"params": [b], "algorithm": "adamw", "lr": 0.003},
                {"params": [e], "algorithm": "lion", "lr": 0.001, "cautious_wd": True}], lr=0.02)
    xb, mb, vb = b.data.cpu().clone(), torch.zeros(300), torch.zeros(300)
    xe, me = e.data.cpu().clone(), torch.zeros(50, 16)
    for step in range(1, 4):
        for p in (w, b, e):
            p.grad = torch.randn_like(p)
        opt.step()
        xb, mb, vb = oracle.adamw_update(xb, b.grad.cpu(), mb, vb, 0.003, 0.9, 0.95, 0.01, step, 1e-8)
        xe, me = oracle.lion_update(xe, e.grad.cpu(), me, 0.001, 0.9, 0.95, 0.01, True)
        assert float((b.data.double().cpu() - xb).abs().max()) <= 2e-6
        assert float((e.data.double().cpu() - xe).abs().max()) <= 2e-6
        xb, mb, vb = b.data.double().cpu(), opt.state[b]["momentum"].double().cpu(), opt.state[b]["variance"].double().cpu()
        xe, me = e.data.double().cpu(), opt.state[e]["momentum"].double().cpu()
    assert float(opt.state[b]["step_dev"]) == 3.0


@pytest.mark.parametrize("dim,k", [(70001, 17501), (32768, 100), (32769, 1), (40000, 40000)])
def test_topk_past_one_lds_chunk(dim, k):
    """Rank-counting top-k on rows longer than one LDS chunk (32 768 entries), with heavy ties and a NaN:
    the selected set is the k first entries of a stable descending sort (ties to the lower index, NaN
    first), idx ascending, map its inverse."""
    from dion_amd import _lib

    lib = _lib.load()
    torch.manual_seed(40)
    norms = torch.randint(0, 2000, (2, dim)).float()  # many equal values
    norms[1, dim // 2] = float("nan")
    nd = norms.to(DEV)
    idx = torch.empty(2, k, dtype=torch.int32, device=DEV)
    imap = torch.empty(2, dim, dtype=torch.int32, device=DEV)
    _lib.check(lib.dion_dion2_topk(nd.data_ptr(), 2, dim, k, idx.data_ptr(), imap.data_ptr(),
                                   torch.cuda.current_stream().cuda_stream), "topk")
    key = torch.nan_to_num(norms, nan=float("inf"))
    for b in range(2):
        order = torch.sort(key[b], descending=True, stable=True).indices[:k]
        ref = order.sort().values.to(torch.int32)
        assert torch.equal(idx[b].cpu(), ref)
        inv = torch.full((dim,), -1, dtype=torch.int32)
        inv[ref.long()] = torch.arange(k, dtype=torch.int32)
        assert torch.equal(imap[b].cpu(), inv)


def test_many_matrices_per_launch_are_chunked():
    """Three 3-D parameters of 30000 matrices each: more matrices than one launch addresses (65535), so
    the pointer table is cut into launches of two parameters and one; through the Dion2 select / post and
    the NorMuon statistics kernels.  More than 65535 matrices behind a single pointer are refused."""
    from dion_amd import ops

    torch.manual_seed(41)
    n, L, rows, cols = 3, 30000, 4, 8
    G = [torch.randn(L, rows, cols, device=DEV).to(torch.bfloat16) for _ in range(n)]
    M = [torch.zeros(L, rows, cols, device=DEV) for _ in range(n)]
    U, idx, imap = ops.dion2_select(G, M, 2, -2, 0.5)
    assert U.shape == (n, L, 2, cols) and idx.shape == (n * L, 2)
    g_all = torch.stack(G).view(n * L, rows, cols)
    norms = g_all.float().abs().sum(-1)
    srt = norms.sort(-1, descending=True).values
    tie_free = srt[:, 1] > srt[:, 2]
    ref = norms.topk(2, dim=-1).indices.sort(-1).values.to(torch.int32)
    assert torch.equal(idx[tie_free], ref[tie_free])
    X = [torch.randn(L, rows, cols, device=DEV) for _ in range(n)]
    x0 = torch.stack(X).view(n * L, rows, cols).clone()
    lr = torch.tensor(0.1, device=DEV)
    ops.dion2_post(X, U, imap, lr, 1.0, 0.0, -2)
    full = torch.zeros(n * L, rows, cols, device=DEV)
    full.scatter_(1, idx.long().unsqueeze(-1).expand(n * L, 2, cols), U.view(n * L, 2, cols).float())
    assert torch.allclose(torch.stack(X).view(n * L, rows, cols), x0 - 0.1 * full, rtol=1e-6, atol=1e-7)
    V = [torch.zeros(L, rows, 1, device=DEV) for _ in range(n)]
    O = torch.randn(n, L, rows, cols, device=DEV).to(torch.bfloat16)
    scale = ops.normuon_stats(O, V, 0.9)
    assert scale.shape == (n * L, rows)
    assert torch.allclose(torch.stack(V).view(n * L, rows), 0.1 * (O.view(n * L, rows, cols).float() ** 2).mean(-1),
                          rtol=1e-5)
    with pytest.raises(ValueError, match="65535"):
        ops.dion2_select([torch.zeros(70000, 2, 4, device=DEV, dtype=torch.bfloat16)],
                         [torch.zeros(70000, 2, 4, device=DEV)], 1, -2, 0.5)
