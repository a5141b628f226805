"""GPU tests of the step kernels with bfloat16 optimizer state (parameters, momentum, second moments kept
in the parameter's dtype, dion/megabatch_base.py:198-203, dion/normuon.py:122).

The kernels compute in fp32 and round a bf16 value once, when it is stored.  Two checks follow from that:
  * a bf16-state call equals the fp32-state call on the upcast state, rounded to bf16 -- bit for bit;
  * against the CPU oracle on the upcast state the stored values are within one bf16 rounding,
    |got - ref| <= 2^-8 |ref| (+ fp32 slack), far inside the reference's own bf16 arithmetic, which
    rounds after every foreach op (dion/muon.py:295-311).
Where a kernel reads back what it stored (slice norms for selection, second moments for the scale) it
reads the rounded value, as the reference does; those cases say so."""
import pytest
import torch

from oracle import dion_oracle as oracle

pytestmark = pytest.mark.gpu
DEV = "cuda"
BF = torch.bfloat16
ULP = 2.0 ** -8  # half a unit in the last place of bf16, relative


def _bf(t):
    return t.to(BF)


def _within_rounding(got, ref, slack=1e-6):
    """got (bf16) is ref (fp32/fp64) rounded once, up to fp32-level differences in ref."""
    g, r = got.double().cpu(), ref.double().cpu()
    return bool(((g - r).abs() <= ULP * r.abs() * (1 + 1e-3) + slack).all())


@pytest.mark.parametrize("shape", [(64, 128), (7, 13), (3, 40, 24)])
@pytest.mark.parametrize("nesterov", [False, True])
@pytest.mark.parametrize("gdtype", [BF, torch.float32])
def test_muon_pre_bf16_momentum(shape, nesterov, gdtype):
    from dion_amd import ops

    torch.manual_seed(0)
    n = 3
    G = [(torch.randn(shape, device=DEV) * 0.02).to(gdtype) for _ in range(n)]
    M16 = [_bf(torch.randn(shape, device=DEV) * 0.01) for _ in range(n)]
    M32 = [m.float() for m in M16]
    m0 = [m.float().cpu() for m in M16]
    U16 = ops.muon_pre(G, M16, 0.95, nesterov)
    U32 = ops.muon_pre(G, M32, 0.95, nesterov)
    assert all(m.dtype == BF for m in M16)
    for i in range(n):
        assert torch.equal(M16[i], _bf(M32[i])), "bf16 momentum = fp32 momentum rounded once"
        m_ref, u_ref = oracle.muon_pre(G[i].cpu(), m0[i], 0.95, nesterov)
        assert torch.equal(M16[i].cpu(), _bf(m_ref))
        assert torch.equal(U16[i].cpu(), u_ref)
    assert torch.equal(U16, U32), "the orthogonalization input comes from the unrounded fp32 value"


@pytest.mark.parametrize("shape", [(64, 128), (7, 13), (3, 40, 24)])
@pytest.mark.parametrize("cautious", [False, True])
@pytest.mark.parametrize("udtype", [BF, torch.float32])
def test_muon_post_bf16_parameters(shape, cautious, udtype):
    from dion_amd import ops

    torch.manual_seed(2)
    n = 2
    X16 = [_bf(torch.randn(shape, device=DEV) * 0.02) for _ in range(n)]
    X32 = [x.float() for x in X16]
    x0 = [x.float().cpu() for x in X16]
    U = (torch.randn(n, *shape, device=DEV) * 0.1).to(udtype)
    lr = torch.tensor(0.02, device=DEV)
    ops.muon_post(X16, U, lr, 0.5, 0.01, cautious)
    ops.muon_post(X32, U, lr, 0.5, 0.01, cautious)
    for i in range(n):
        assert X16[i].dtype == BF
        assert torch.equal(X16[i], _bf(X32[i]))
        ref = oracle.muon_post(x0[i], U[i].cpu(), 0.02, 0.5, 0.01, cautious)
        assert _within_rounding(X16[i], ref)


@pytest.mark.parametrize("shape", [(4, 64, 128), (2, 10, 24), (1, 2, 17, 33)])
def test_normuon_bf16_second_moments(shape):
    """V is stored rounded; the scale is computed from the stored (rounded) V, so it is compared with
    the fp32 call whose V has been replaced by the rounded one."""
    from dion_amd import ops

    torch.manual_seed(3)
    n = shape[0]
    U = (torch.randn(shape, device=DEV) * 0.05).to(BF)
    V16 = [_bf(torch.rand(*shape[1:-1], 1, device=DEV) * 1e-3) for _ in range(n)]
    V32 = [v.float() for v in V16]
    v0 = [v.float().cpu() for v in V16]
    s16 = ops.normuon_stats(U, V16, 0.95)
    s32 = ops.normuon_stats(U, V32, 0.95)
    for i in range(n):
        assert V16[i].dtype == BF
        assert torch.equal(V16[i], _bf(V32[i]))
        _, v_ref = oracle.normuon_normalize(U[i].cpu(), v0[i], 0.95)
        assert _within_rounding(V16[i], v_ref, slack=1e-12)
    # scale = f(sqrt(V)): a relative change of V by 2^-8 moves 1/sqrt(V) by 2^-9, and the Frobenius
    # renormalisation averages it out further
    assert float(((s16 - s32).abs() / s32.abs()).max()) <= 2.0 ** -8
    # zero beta2-weight: V <- mean square exactly, scale from the rounded V
    Vz = [torch.zeros(*shape[1:-1], 1, device=DEV, dtype=BF) for _ in range(n)]
    ops.normuon_stats(U, Vz, 0.0)
    ms = U.float().square().mean(dim=-1, keepdim=True)
    for i in range(n):
        assert _within_rounding(Vz[i], ms[i], slack=1e-12)


@pytest.mark.parametrize("shape,frac", [((17, 40), 0.35), ((40, 17), 0.35), ((64, 128), 0.25), ((128, 64), 0.25),
                                        ((3, 32, 48), 0.5)])
@pytest.mark.parametrize("gdtype", [BF, torch.float32])
def test_dion2_select_bf16_momentum(shape, frac, gdtype):
    """M += G is stored rounded and the slice norms are those of the stored values (dion/dion2.py:488-
    520 runs on the bf16 M), so the expected result is the fp32 sequence started from the rounded sum."""
    from dion_amd import ops

    torch.manual_seed(4)
    n = 2
    rows, cols = shape[-2:]
    sd = oracle.dion2_select_dim(rows, cols)
    dim = rows if sd == -2 else cols
    k = min(oracle.dion2_k(frac, dim), dim)
    as3 = lambda t: t.reshape(-1, rows, cols)
    G = [as3((torch.randn(shape, device=DEV) * 0.02).to(gdtype)) for _ in range(n)]
    M16 = [as3(_bf(torch.randn(shape, device=DEV) * 0.02)) for _ in range(n)]
    acc = [_bf(m.float() + g.float()) for m, g in zip(M16, G)]  # what the accumulate pass stores
    U16, idx16, map16 = ops.dion2_select(G, M16, k, sd, 0.9)
    M32 = [a.float() for a in acc]
    Z = [torch.zeros_like(g) for g in G]
    U32, idx32, map32 = ops.dion2_select(Z, M32, k, sd, 0.9)
    assert torch.equal(idx16, idx32) and torch.equal(map16, map32)
    assert torch.equal(U16, U32)
    mats = G[0].shape[0]
    for i in range(n):
        assert M16[i].dtype == BF
        assert torch.equal(M16[i], _bf(M32[i]))
        for b in range(mats):
            m_ref, u_ref, idx_ref = oracle.dion2_pre(torch.zeros(rows, cols), acc[i][b].float().cpu(), frac, 0.9, sd)
            assert torch.equal(idx16[i * mats + b].cpu().long(), idx_ref)
            assert torch.equal(U16[i, b].cpu(), u_ref)
            assert _within_rounding(M16[i][b], m_ref)


@pytest.mark.parametrize("shape,sd", [((17, 40), -2), ((40, 17), -1), ((64, 128), -2), ((128, 64), -1), ((3, 32, 48), -2)])
@pytest.mark.parametrize("udtype", [BF, torch.float32])
@pytest.mark.parametrize("with_scale", [False, True])
def test_dion2_post_bf16_parameters(shape, sd, udtype, with_scale):
    from dion_amd import ops

    if with_scale and sd != -2:
        pytest.skip("row scales go with selected rows")
    torch.manual_seed(5)
    n = 2
    rows, cols = shape[-2:]
    dim = rows if sd == -2 else cols
    k = max(1, dim // 3)
    as3 = lambda t: t.reshape(-1, rows, cols)
    X16 = [as3(_bf(torch.randn(shape, device=DEV) * 0.02)) for _ in range(n)]
    X32 = [x.float() for x in X16]
    x0 = [x.float().cpu() for x in X16]
    mats = X16[0].shape[0]
    idx = torch.stack([torch.randperm(dim, device=DEV)[:k].sort().values for _ in range(n * mats)])
    imap = ops.dion2_index_map(idx, dim)
    ush = (n, mats, k, cols) if sd == -2 else (n, mats, rows, k)
    U = (torch.randn(ush, device=DEV) * 0.1).to(udtype)
    rs = (torch.rand(n * mats, k, device=DEV) + 0.5) if with_scale else None
    lr = torch.tensor(0.02, device=DEV)
    ops.dion2_post(X16, U, imap, lr, 1.5, 0.1, sd, row_scale=rs)
    ops.dion2_post(X32, U, imap, lr, 1.5, 0.1, sd, row_scale=rs)
    for i in range(n):
        assert X16[i].dtype == BF
        assert torch.equal(X16[i], _bf(X32[i]))
        for b in range(mats):
            u = U[i, b].float().cpu()
            if with_scale:
                u = u * rs[i * mats + b].cpu()[:, None]
            ref = oracle.dion2_post(x0[i][b], u, idx[i * mats + b].cpu(), 0.02, 1.5, 0.1, sd)
            assert _within_rounding(X16[i][b], ref)


@pytest.mark.parametrize("shape,sd", [((24, 40), -2), ((40, 24), -1), ((2, 32, 48), -2), ((64, 136), -1)])
def test_dion2_post_masked_bf16_state(shape, sd):
    from dion_amd import ops

    torch.manual_seed(6)
    n = 2
    rows, cols = shape[-2:]
    dim = rows if sd == -2 else cols
    as3 = lambda t: t.reshape(-1, rows, cols)
    X16 = [as3(_bf(torch.randn(shape, device=DEV) * 0.02)) for _ in range(n)]
    M16 = [as3(_bf(torch.randn(shape, device=DEV) * 0.02)) for _ in range(n)]
    X32, M32 = [x.float() for x in X16], [m.float() for m in M16]
    x0, m0 = [x.float().cpu() for x in X16], [m.float().cpu() for m in M16]
    mats = X16[0].shape[0]
    U = (torch.randn(n, mats, rows, cols, device=DEV) * 0.1).to(BF)
    keep = torch.rand(n, mats, dim, device=DEV) < 0.4
    U = U * (keep[..., :, None] if sd == -2 else keep[..., None, :])
    norms = ops.slice_l1(U.view(n * mats, rows, cols), sd)
    lr = torch.tensor(0.02, device=DEV)
    ops.dion2_post_masked(X16, M16, U, norms, lr, 1.5, 0.1, 0.9, sd)
    ops.dion2_post_masked(X32, M32, U, norms, lr, 1.5, 0.1, 0.9, sd)
    for i in range(n):
        assert X16[i].dtype == BF and M16[i].dtype == BF
        assert torch.equal(X16[i], _bf(X32[i])) and torch.equal(M16[i], _bf(M32[i]))
        for b in range(mats):
            x_ref, m_ref = oracle.dion2_post_masked(x0[i][b], m0[i][b], U[i, b].cpu(), 0.02, 1.5, 0.1, 0.9, sd)
            assert _within_rounding(X16[i][b], x_ref) and _within_rounding(M16[i][b], m_ref)
    with pytest.raises(TypeError, match="share one dtype"):
        ops.dion2_post_masked(X16, M32, U, norms, lr, 1.5, 0.1, 0.9, sd)


@pytest.mark.parametrize("cautious", [False, True])
@pytest.mark.parametrize("gdtype", [BF, torch.float32])
def test_adamw_lion_bf16_state(cautious, gdtype):
    """Ragged lists incl. empty, odd and 2-byte-aligned views, more tensors than one launch holds."""
    from dion_amd import ops

    torch.manual_seed(31)
    sizes = [0, 1, 3, 7, 64, 129, 1000, 4096 * 9 + 5] + [17 + i for i in range(50)]
    X16 = []
    for i, sz in enumerate(sizes):
        buf = _bf(torch.randn(sz + 1, device=DEV))
        X16.append(buf[1:] if i % 3 == 0 else buf[:-1].clone())
    M16 = [_bf(torch.randn(sz, device=DEV) * 0.1) for sz in sizes]
    V16 = [_bf(torch.rand(sz, device=DEV) * 0.01) for sz in sizes]
    X32, M32, V32 = ([t.float() for t in ts] for ts in (X16, M16, V16))
    G = [torch.randn(sz, device=DEV).to(gdtype) for sz in sizes]
    lr = torch.tensor(0.01, device=DEV)
    s16 = [torch.full((), 4.0, device=DEV) for _ in sizes]
    s32 = [torch.full((), 4.0, device=DEV) for _ in sizes]
    ops.adamw_step(X16, G, M16, V16, s16, lr, 0.9, 0.95, 0.1, 1e-8, cautious)
    ops.adamw_step(X32, G, M32, V32, s32, lr, 0.9, 0.95, 0.1, 1e-8, cautious)
    for a, b in zip((X16, M16, V16), (X32, M32, V32)):
        for t16, t32 in zip(a, b):
            assert t16.dtype == BF and torch.equal(t16, _bf(t32))
    assert all(float(s) == 5.0 for s in s16)

    L16 = [x.clone() for x in X16]
    LM16 = [m.clone() for m in M16]
    L32, LM32 = [x.float() for x in L16], [m.float() for m in LM16]
    ops.lion_step(L16, G, LM16, lr, 0.9, 0.99, 0.1, cautious)
    ops.lion_step(L32, G, LM32, lr, 0.9, 0.99, 0.1, cautious)
    for t16, t32 in zip(L16 + LM16, L32 + LM32):
        assert t16.dtype == BF and torch.equal(t16, _bf(t32))
    with pytest.raises(ValueError, match="dtype of X"):
        ops.lion_step(L16, G, LM32, lr, 0.9, 0.99, 0.1, cautious)


def test_adamw_bf16_state_against_oracle():
    from dion_amd import ops

    torch.manual_seed(7)
    x = _bf(torch.randn(5000, device=DEV))
    m = _bf(torch.randn(5000, device=DEV) * 0.1)
    v = _bf(torch.rand(5000, device=DEV) * 0.01 + 1e-4)
    g = _bf(torch.randn(5000, device=DEV))
    x0, m0, v0 = x.float().cpu(), m.float().cpu(), v.float().cpu()
    ops.adamw_step([x], [g], [m], [v], [torch.full((), 2.0, device=DEV)], torch.tensor(0.01, device=DEV), 0.9, 0.95,
                   0.1, 1e-8, False)
    xr, mr, vr = oracle.adamw_update(x0, g.float().cpu(), m0, v0, 0.01, 0.9, 0.95, 0.1, 3, 1e-8, False)
    assert _within_rounding(m, mr) and _within_rounding(v, vr, slack=1e-12) and _within_rounding(x, xr)


def _params(dtype, seed):
    torch.manual_seed(seed)
    ps = [torch.nn.Parameter((torch.randn(s, device=DEV) * 0.02).to(BF).to(dtype))
          for s in [(64, 128), (64, 128), (128, 64), (2, 48, 32)]]
    bias = torch.nn.Parameter(torch.randn(300, device=DEV).to(BF).to(dtype))
    emb = torch.nn.Parameter(torch.randn(50, 16, device=DEV).to(BF).to(dtype))
    return ps, bias, emb


@pytest.mark.parametrize("name,kw", [("Muon", {}), ("Muon", {"nesterov": True, "cautious_wd": True}),
                                     ("NorMuon", {}), ("Dion2", {"fraction": 0.5}),
                                     ("Dion2", {"fraction": 0.5, "selection_scope": "global", "_assembled": True}),
                                     ("NorDion2", {"fraction": 0.5}),
                                     ("NorDion2", {"fraction": 0.5, "selection_scope": "global", "_assembled": True})])
def test_optimizer_step_with_bf16_parameters(name, kw):
    """A model kept in bf16: state is created in bf16 (dion/megabatch_base.py:198-203) and the first
    step lands on the fp32 run's result rounded once (exact for Muon / Dion2; within one more
    rounding where the update goes through the stored second moments); three further steps stay
    within a few bf16 roundings of the fp32 run."""
    import dion

    kw = dict(kw)
    assembled = kw.pop("_assembled", False)
    cls = getattr(dion, name)
    opts, models = [], []
    for dtype in (BF, torch.float32):
        ps, bias, emb = _params(dtype, 11)
        opt = cls([{"params": ps}, {"params": [bias], "algorithm": "adamw", "lr": 0.003},
                   {"params": [emb], "algorithm": "lion", "lr": 0.001}], lr=0.02, **kw)
        opt.assembled_selection = assembled
        opts.append(opt)
        models.append(ps + [bias, emb])
    exact_first = name in ("Muon", "Dion2")
    torch.manual_seed(12)
    for step in range(4):
        grads = [_bf(torch.randn_like(p, dtype=torch.float32)) for p in models[0]]
        if name in ("Dion2", "NorDion2"):
            # unambiguous top-k sets: every other slice carries 4x the gradient, on the first step only
            # (later steps start from states that differ by their rounding)
            for g in grads[:4]:
                rows, cols = g.shape[-2:]
                if name == "NorDion2" or rows <= cols:
                    g[..., ::2, :] *= 4
                else:
                    g[..., :, ::2] *= 4
        for model in models:
            for p, g in zip(model, grads):
                p.grad_dtype = None
                p.grad = g.clone()
        for opt in opts:
            opt.step()
        for p16, p32 in zip(*models):
            assert p16.dtype == BF
            st = opts[0].state[p16]
            assert st["momentum"].dtype == BF
            if "variance_neuron" in st:
                assert st["variance_neuron"].dtype == BF
            if "variance" in st:
                assert st["variance"].dtype == BF
            if step == 0 and (exact_first or p16.dim() == 1 or p16 is models[0][-1]):
                assert torch.equal(p16.data, _bf(p32.data))
            if step == 0 or name in ("Muon", "NorMuon"):
                # later Dion2 steps may select different slices once the states differ by rounding
                d = (p16.data.float() - p32.data).norm() / p32.data.norm()
                assert float(d) <= 2.0 ** -7 * (step + 1)
    sd = opts[0].state_dict()
    assert all(v.dtype in (BF, torch.float32) for s in sd["state"].values() for v in s.values()
               if isinstance(v, torch.Tensor))


def test_unsupported_parameter_dtype_is_refused():
    import dion

    p = torch.nn.Parameter(torch.randn(32, 64, device=DEV).half())
    p.grad = torch.randn_like(p)
    opt = dion.Muon([p], lr=0.01)
    with pytest.raises((NotImplementedError, TypeError)):
        opt.step()
