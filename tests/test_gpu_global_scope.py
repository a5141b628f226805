"""GPU parity of the whole-matrix ("global" selection scope) Dion2 / NorDion2 sequence, through the C
ABI: slice norms, select-inside-orthogonalization, the masked update.  Index and set results are exact;
fp32 state within 1e-5 relative (momentum bit exact); where the masked and the index-based sequence
pick the same slices they must agree bit for bit (Dion2) or to fp32 summation order (NorDion2)."""
import math

import pytest
import torch

from oracle import dion_oracle as oracle

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _rel(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / b.norm().clamp(min=1e-30))


@pytest.mark.parametrize("shape", [(3, 64, 128), (2, 7, 13), (1, 130, 36), (4, 1, 9), (2, 257, 1024)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("select_dim", [-2, -1])
def test_slice_l1(shape, dtype, select_dim):
    from dion_amd import ops

    torch.manual_seed(0)
    U = torch.randn(shape).to(dtype)
    norm_dim = -1 if select_dim == -2 else -2
    ref = U.double().abs().sum(dim=norm_dim)
    got = ops.slice_l1(U.to(DEV), select_dim).cpu()
    assert got.shape == ref.shape and got.dtype == torch.float32
    assert torch.allclose(got.double(), ref, rtol=2e-6, atol=0)
    if dtype == torch.bfloat16:
        # rounded form: what Tensor.norm(p=1) returns for a bf16 tensor, up to the fp32 summation
        # order (a sum that lands on a rounding boundary may go either way: at most one bf16 step)
        got_r = ops.slice_l1(U.to(DEV), select_dim, round_bf16=True).cpu()
        ref_r = ref.float().to(torch.bfloat16).float()
        assert torch.equal(got_r, got_r.to(torch.bfloat16).float())
        step = ref_r.abs() * 2.0 ** -7
        assert bool(((got_r - ref_r).abs() <= step).all())
        assert float((got_r == ref_r).float().mean()) > 0.98


def test_slice_l1_zero_and_empty():
    from dion_amd import ops

    U = torch.zeros(2, 5, 8, dtype=torch.bfloat16, device=DEV)
    U[1, 3, 2] = -0.5
    n = ops.slice_l1(U, -2).cpu()
    assert float(n[1, 3]) == 0.5 and float(n.sum()) == 0.5
    assert ops.slice_l1(torch.empty(2, 0, 8, dtype=torch.bfloat16, device=DEV), -1).tolist() == [[0.0] * 8] * 2
    assert ops.slice_l1(torch.empty(2, 0, 8, dtype=torch.bfloat16, device=DEV), -2).shape == (2, 0)
    with pytest.raises(ValueError):
        ops.slice_l1(U, 0)


@pytest.mark.parametrize("shape", [(3, 64, 128), (2, 7, 13), (1, 130, 36), (2, 40, 1024)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("select_dim", [-2, -1])
def test_select_then_scatter_is_a_masked_copy(shape, dtype, select_dim):
    """select_slices picks the k slices of largest norm (brute force on the host), the dense block
    holds exactly those slices in ascending order, and scattering it back reproduces the input on the
    selected slices and exact zeros elsewhere."""
    from dion_amd import ops

    torch.manual_seed(1)
    U = torch.randn(shape).to(dtype)
    dim = shape[select_dim]
    k = max(1, math.ceil(0.3 * dim))
    sub, idx, imap = ops.select_slices(U.to(DEV), k, select_dim)
    out = ops.scatter_slices(sub, imap, U.shape, select_dim).cpu()
    sub, idx, imap = sub.cpu(), idx.cpu().long(), imap.cpu()
    norm_dim = -1 if select_dim == -2 else -2
    norms = U.float().abs().sum(dim=norm_dim).to(dtype).float()
    for b in range(shape[0]):
        assert torch.equal(idx[b], idx[b].sort().values) and idx[b].unique().numel() == k
        mask = torch.zeros(dim, dtype=torch.bool)
        mask[idx[b]] = True
        # every selected slice beats (or ties) every unselected one
        assert float(norms[b][mask].min()) >= float(norms[b][~mask].max()) * (1 - 2.0 ** -7)
        assert torch.equal(imap[b][mask], torch.arange(k, dtype=torch.int32))
        assert bool((imap[b][~mask] == -1).all())
        if select_dim == -2:
            assert torch.equal(sub[b], U[b][idx[b]])
            assert torch.equal(out[b][mask], U[b][mask]) and float(out[b][~mask].abs().sum()) == 0.0
        else:
            assert torch.equal(sub[b], U[b][:, idx[b]])
            assert torch.equal(out[b][:, mask], U[b][:, mask]) and float(out[b][:, ~mask].abs().sum()) == 0.0


def test_select_and_orthogonalize_reference_padded_case():
    """tests/test_dion2_selection_scope.py:138-169 of the reference: 17 real + 3 zero rows, fraction
    0.35, true size 17 -> 6 rows (not 7), never a padded one.  Identity orthogonalization."""
    from dion_amd.global_scope import make_select_and_orthogonalize

    torch.manual_seed(0)
    X = torch.cat([torch.randn(17, 6), torch.zeros(3, 6)], dim=0).to(DEV)
    sel_ns = make_select_and_orthogonalize(lambda t, epsilon=None: t, 0.35, -2, global_select_size=17)
    out = sel_ns(X)
    assert out.shape == X.shape and out.dtype == X.dtype
    assert int((out.abs().sum(-1) > 0).sum()) == 6
    assert float(out[17:].abs().sum()) == 0.0
    ref, _ = oracle.select_and_orthogonalize(X.cpu(), 0.35, -2, lambda t: t, global_select_size=17)
    assert torch.equal(out.cpu(), ref)
    out7 = make_select_and_orthogonalize(lambda t, epsilon=None: t, 0.35, -2)(X)
    assert int((out7.abs().sum(-1) > 0).sum()) == 7
    with pytest.raises(ValueError):
        make_select_and_orthogonalize(lambda t, epsilon=None: t, 0.35, 0)


@pytest.mark.parametrize("shape,select_dim", [((4, 64, 256), -2), ((3, 256, 64), -1), ((2, 96, 96), -2)])
def test_select_and_orthogonalize_with_newton_schulz(shape, select_dim):
    """bf16 batch with the library's Newton-Schulz inside: same selected set as the CPU restatement,
    exact zeros off it, orthogonalized block within 2e-2 relative Frobenius of the restatement's."""
    from dion_amd import zeropower_via_newtonschulz5
    from dion_amd.global_scope import make_select_and_orthogonalize

    torch.manual_seed(3)
    dim = shape[select_dim]
    spread = torch.ones(dim)  # a quarter of the slices four times larger: an unambiguous top-k set
    spread[torch.randperm(dim)[:math.ceil(0.25 * dim)]] = 4.0
    X = torch.randn(shape) * (spread[:, None] if select_dim == -2 else spread[None, :])
    X = X.to(torch.bfloat16)
    sel_ns = make_select_and_orthogonalize(zeropower_via_newtonschulz5, 0.25, select_dim)
    out = sel_ns(X.to(DEV), epsilon=1e-7).cpu()
    assert out.dtype == torch.bfloat16 and out.shape == X.shape
    for b in range(shape[0]):
        ref, idx = oracle.select_and_orthogonalize(
            X[b], 0.25, select_dim, lambda u: oracle.ns_bf16_fused(u, oracle.NS5_COEFFS, 1.0, 1e-7))
        nz = out[b].float().abs().sum(dim=-1 if select_dim == -2 else -2) > 0
        assert torch.equal(nz.nonzero().flatten(), idx)
        assert _rel(out[b], ref) <= 2e-2


@pytest.mark.parametrize("shape,select_dim", [((2, 64, 128), -2), ((2, 128, 64), -1), ((3, 7, 13), -2),
                                              ((3, 13, 7), -1), ((1, 2, 40, 24), -2)])
def test_dion2_post_masked_vs_oracle_and_index_form(shape, select_dim):
    """Against the CPU restatement (X <= 1e-6 relative, M bit exact) and against the index-based kernels
    fed the same selection: X and M bit identical."""
    from dion_amd import ops
    from dion_amd.global_scope import dion2_post_orthogonalize_masked

    torch.manual_seed(4)
    n = shape[0]
    mat_shape = shape[1:]
    rows, cols = mat_shape[-2], mat_shape[-1]
    dim = mat_shape[select_dim]
    k = max(1, math.ceil(0.25 * dim))
    X = [torch.randn(mat_shape) * 0.02 for _ in range(n)]
    M = [torch.randn(mat_shape) * 0.01 for _ in range(n)]
    U = torch.zeros(n, *mat_shape)
    flat = U.view(-1, rows, cols)
    sels = []
    for b in range(flat.shape[0]):
        idx = torch.randperm(dim)[:k].sort().values
        sels.append(idx)
        if select_dim == -2:
            flat[b][idx] = torch.randn(k, cols)
        else:
            flat[b][:, idx] = torch.randn(rows, k)
    U = U.to(torch.bfloat16)
    lr = torch.tensor(0.02, device=DEV)
    Xd = [x.to(DEV) for x in X]
    Md = [m.to(DEV) for m in M]
    dion2_post_orthogonalize_masked(Xd, Md, U.to(DEV), lr, 1.5, 0.1, 0.9, select_dim)
    mats = flat.shape[0] // n
    for i in range(n):
        xr = X[i].view(mats, rows, cols)
        mr = M[i].view(mats, rows, cols)
        for j in range(mats):
            x_ref, m_ref = oracle.dion2_post_masked(xr[j], mr[j], U.view(-1, rows, cols)[i * mats + j], 0.02, 1.5,
                                                    0.1, 0.9, select_dim)
            assert torch.equal(Md[i].view(mats, rows, cols)[j].cpu(), m_ref)
            assert _rel(Xd[i].view(mats, rows, cols)[j], x_ref) <= 1e-6
    # index form on the same selection
    idx_t = torch.stack(sels).to(torch.int32).to(DEV)
    imap = torch.full((flat.shape[0], dim), -1, dtype=torch.int32)
    for b, idx in enumerate(sels):
        imap[b][idx] = torch.arange(k, dtype=torch.int32)
    imap = imap.to(DEV)
    Ud = U.to(DEV).view(-1, rows, cols)
    sub = torch.stack([Ud[b][sels[b].to(DEV)] if select_dim == -2 else Ud[b][:, sels[b].to(DEV)]
                       for b in range(flat.shape[0])]).contiguous()
    X2 = [x.to(DEV) for x in X]
    ops.dion2_post(X2, sub.view(n, *mat_shape[:-2], *sub.shape[-2:]), imap, lr, 1.5, 0.1, select_dim)
    for a, b in zip(Xd, X2):
        assert torch.equal(a, b)
    del idx_t


def test_dion2_post_masked_all_zero_update_is_decay_only():
    from dion_amd.global_scope import dion2_post_orthogonalize_masked

    torch.manual_seed(5)
    X = [torch.randn(16, 32, device=DEV)]
    M = [torch.randn(16, 32, device=DEV)]
    x0, m0 = X[0].clone(), M[0].clone()
    U = torch.zeros(1, 16, 32, dtype=torch.bfloat16, device=DEV)
    lr = torch.tensor(0.02, device=DEV)
    dion2_post_orthogonalize_masked(X, M, U, lr, 1.5, 0.1, 0.5, -2)
    a = 1 - torch.tensor(0.02) * torch.tensor(0.1)
    assert torch.equal(M[0], m0)
    assert torch.equal(X[0].cpu(), (x0.cpu() * a))


@pytest.mark.parametrize("shape", [(64, 128), (3, 40, 24), (130, 36)])
def test_nordion2_post_masked_vs_oracle(shape):
    from dion_amd.global_scope import nordion2_post_orthogonalize_masked

    torch.manual_seed(6)
    n = 2
    rows, cols = shape[-2], shape[-1]
    k = max(1, math.ceil(0.25 * rows))
    X = [torch.randn(shape) * 0.02 for _ in range(n)]
    M = [torch.randn(shape) * 0.01 for _ in range(n)]
    V = [torch.rand(*shape[:-1], 1) * 1e-2 for _ in range(n)]
    U = torch.zeros(n, *shape)
    flat = U.view(-1, rows, cols)
    for b in range(flat.shape[0]):
        idx = torch.randperm(rows)[:k]
        flat[b][idx] = torch.randn(k, cols) * 0.1
    U = U.to(torch.bfloat16)
    lr = torch.tensor(0.02, device=DEV)
    Xd, Md, Vd = ([t.to(DEV) for t in ts] for ts in (X, M, V))
    nordion2_post_orthogonalize_masked(Xd, Md, Vd, U.to(DEV), lr, 1.5, 0.1, 0.95, 0.9)
    mats = flat.shape[0] // n
    for i in range(n):
        for j in range(mats):
            u = U.view(-1, rows, cols)[i * mats + j]
            x_ref, m_ref, v_ref = oracle.nordion2_post_masked(
                X[i].view(mats, rows, cols)[j], M[i].view(mats, rows, cols)[j], V[i].view(mats, rows, 1)[j], u,
                0.02, 1.5, 0.1, 0.95, 0.9)
            assert torch.equal(Md[i].view(mats, rows, cols)[j].cpu(), m_ref)
            v_gpu = Vd[i].view(mats, rows, 1)[j].cpu()
            unsel = u.float().abs().sum(-1) == 0
            assert torch.equal(v_gpu[unsel], V[i].view(mats, rows, 1)[j][unsel])
            assert _rel(v_gpu, v_ref) <= 1e-6
            assert _rel(Xd[i].view(mats, rows, cols)[j], x_ref) <= 1e-5
    with pytest.raises(ValueError):
        nordion2_post_orthogonalize_masked(Xd, Md, Vd, U.to(DEV), lr, 1.5, 0.1, 0.95, 0.9, select_dim=-1)


def _hot_slices(dim, fraction=0.25):
    k = max(1, math.ceil(fraction * dim))
    hot = torch.ones(dim)
    hot[torch.randperm(dim)[:k]] = 4.0
    return hot


def _spread_grad(shape, select_dim, hot, gen_scale=0.02):
    """Gradient whose ``hot`` slices along select_dim are four times larger than the rest: the top-k set
    is then the same whether it is taken on fp32 norms of the fp32 momentum or on bf16-rounded norms
    of its bf16 copy."""
    g = torch.randn(shape) * gen_scale
    return g * (hot[:, None] if select_dim == -2 else hot[None, :])


@pytest.mark.parametrize("shape", [(128, 512), (512, 128), (4, 64, 96)])
def test_dion2_assembled_selection_matches_index_sequence(shape):
    """Dion2 stepping through accumulate -> select inside the orthogonalization -> masked update equals,
    bit for bit, the default index-based step when both select the same slices."""
    from dion import Dion2

    torch.manual_seed(7)
    x0 = torch.randn(shape) * 0.02
    sd = -2 if shape[-2] <= shape[-1] else -1
    hot = _hot_slices(shape[sd])
    grads = [_spread_grad(shape, sd, hot).to(torch.bfloat16) for _ in range(3)]
    outs = []
    for assembled in (False, True):
        p = torch.nn.Parameter(x0.clone().to(DEV))
        p.grad_dtype = None
        opt = Dion2([p], lr=0.02, fraction=0.25, ef_decay=0.9, weight_decay=0.01, selection_scope="global")
        opt.assembled_selection = assembled
        for g in grads:
            p.grad = g.to(DEV)
            opt.step()
        outs.append((p.data.clone(), opt.state[p]["momentum"].clone()))
    assert torch.equal(outs[0][1], outs[1][1])
    assert torch.equal(outs[0][0], outs[1][0])
    assert not torch.equal(outs[0][0].cpu(), x0)


def test_dion2_assembled_selection_needs_global_scope():
    """With the default scope the attribute changes nothing (same code path as without it)."""
    from dion import Dion2

    torch.manual_seed(8)
    x0 = torch.randn(64, 128) * 0.02
    g = (torch.randn(64, 128) * 0.02).to(torch.bfloat16)
    res = []
    for assembled in (False, True):
        p = torch.nn.Parameter(x0.clone().to(DEV))
        p.grad_dtype = None
        opt = Dion2([p], lr=0.02, fraction=0.25)
        opt.assembled_selection = assembled
        p.grad = g.to(DEV)
        opt.step()
        res.append(p.data.clone())
    assert torch.equal(res[0], res[1])


@pytest.mark.parametrize("shape", [(128, 512), (256, 64)])
def test_nordion2_assembled_selection_matches_index_sequence(shape):
    from dion import NorDion2

    torch.manual_seed(9)
    x0 = torch.randn(shape) * 0.02
    hot = _hot_slices(shape[-2])
    grads = [_spread_grad(shape, -2, hot).to(torch.bfloat16) for _ in range(3)]
    outs = []
    for assembled in (False, True):
        p = torch.nn.Parameter(x0.clone().to(DEV))
        p.grad_dtype = None
        opt = NorDion2([p], lr=0.02, fraction=0.25, mu=0.9, muon_beta2=0.95, weight_decay=0.01,
                       selection_scope="global")
        opt.assembled_selection = assembled
        for g in grads:
            p.grad = g.to(DEV)
            opt.step()
        outs.append((p.data.clone(), opt.state[p]["momentum"].clone(), opt.state[p]["variance_neuron"].clone()))
    assert torch.equal(outs[0][1], outs[1][1])
    assert _rel(outs[1][2], outs[0][2]) <= 1e-6
    assert torch.equal(outs[0][2] == 0, outs[1][2] == 0)
    assert _rel(outs[1][0], outs[0][0]) <= 1e-6


def test_dion2_assembled_step_vs_oracle():
    """Two assembled-selection Dion2 steps against the CPU restatement of the global-scope sequence
    (dion/dion2.py:301-343)."""
    from dion import Dion2

    torch.manual_seed(10)
    shape = (128, 512)
    x = torch.randn(shape) * 0.02
    p = torch.nn.Parameter(x.clone().to(DEV))
    p.grad_dtype = None
    opt = Dion2([p], lr=0.02, fraction=0.25, ef_decay=0.95, weight_decay=0.01, use_polar_express=False,
                selection_scope="global")
    opt.assembled_selection = True
    M = torch.zeros(shape)
    ratio = oracle.adjust_lr_ratio(shape, "spectral_norm")
    hot = _hot_slices(shape[-2])
    for step in range(2):
        g = _spread_grad(shape, -2, hot).to(torch.bfloat16)
        p.grad = g.to(DEV)
        opt.step()
        M, u_full = oracle.dion2_pre_accumulate(g, M)
        full, idx = oracle.select_and_orthogonalize(
            u_full, 0.25, -2, lambda u: oracle.ns_bf16_fused(u, oracle.NS5_COEFFS, 1.0, 1e-8))
        x, M = oracle.dion2_post_masked(x, M, full, 0.02, ratio, 0.01, 0.95, -2)
        assert _rel(opt.state[p]["momentum"], M) <= 1e-6
        assert _rel(p.data, x) <= 1e-3
        x = p.data.cpu().clone()
        M = opt.state[p]["momentum"].cpu().clone()


@pytest.mark.parametrize("shape,select_dim", [((24, 2048, 8192), -2), ((24, 8192, 2048), -1)])
def test_full_size_selection_and_masked_update_properties(shape, select_dim):
    """GPT-1.3B shape groups (fraction 0.25), checked through properties that do not need a CPU pass over
    400 M elements: exactly k slices survive, they carry the input, everything else is exactly zero, no
    selected slice has a smaller (bf16-rounded) norm than an unselected one; the masked update leaves
    unselected entries at exactly a*x, decays exactly the selected slices of M and moves the selected
    entries of X by -lr*adj*u to fp32 rounding."""
    from dion_amd import ops
    from dion_amd.global_scope import dion2_post_orthogonalize_masked

    torch.manual_seed(20)
    n, rows, cols = shape
    dim = shape[select_dim]
    k = math.ceil(0.25 * dim)
    U = (torch.randn(shape, device=DEV) * 0.02).to(torch.bfloat16)
    sub, idx, imap = ops.select_slices(U, k, select_dim)
    out = ops.scatter_slices(sub, imap, U.shape, select_dim)
    norm_dim = -1 if select_dim == -2 else -2
    sel = out.float().abs().sum(dim=norm_dim) > 0            # [n, dim]
    assert bool((sel.sum(dim=-1) == k).all())
    assert torch.equal(sel, imap >= 0)
    mask = sel.unsqueeze(norm_dim)                           # broadcast over the slices
    assert torch.equal(out, torch.where(mask, U, torch.zeros_like(U)))
    norms = U.float().abs().sum(dim=norm_dim).to(torch.bfloat16).float()
    lo_sel = torch.where(sel, norms, torch.full_like(norms, float("inf"))).min(dim=-1).values
    hi_uns = torch.where(sel, torch.full_like(norms, -1.0), norms).max(dim=-1).values
    assert bool((lo_sel >= hi_uns * (1 - 2.0 ** -7)).all())
    del sub, norms

    X = [torch.randn(rows, cols, device=DEV) * 0.02 for _ in range(n)]
    M = [torch.randn(rows, cols, device=DEV) * 0.01 for _ in range(n)]
    x0 = torch.stack(X)
    m0 = torch.stack(M)
    lr = torch.tensor(0.02, device=DEV)
    dion2_post_orthogonalize_masked(X, M, out, lr, 1.5, 0.1, 0.9, select_dim)
    x1 = torch.stack(X)
    m1 = torch.stack(M)
    a = 1 - lr * torch.tensor(0.1, device=DEV)
    assert torch.equal(torch.where(mask, x0 * a, x1), x0 * a)              # unselected: exactly a*x
    assert torch.equal(m1, torch.where(mask, m0 * torch.tensor(0.9, device=DEV), m0))
    ref = x0.double() * a.double() - (lr.double() * 1.5) * out.double()
    err = (x1.double() - ref).abs().max()
    assert float(err) <= 1e-8
