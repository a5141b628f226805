"""The orthogonalization whose last GEMM applies the Muon update (dion_ns_orthogonalize_update) against the
two-call sequence it replaces (dion_ns_orthogonalize, then dion_muon_post): the parameters must come out
bit-identical, whichever way the library runs it (update in the GEMM epilogue for matrices that fill whole
tiles, the two passes through the workspace tail otherwise).  The two-call sequence itself is held to the
oracle in test_gpu_newton_schulz.py / test_gpu_step_kernels.py."""
import pytest
import torch

from oracle import dion_oracle as oracle

pytestmark = pytest.mark.gpu
DEV = "cuda"
BF = torch.bfloat16


def _run_both(shape, n, xdtype, cautious, gram=False, wd=0.01, offset_view=False, coeffs=None, norm_scale=1.0,
              eps=1e-7):
    from dion_amd import newton_schulz as ns
    from dion_amd import ops

    coeffs = ns.NS5_COEFFS if coeffs is None else coeffs
    g = torch.Generator(device=DEV).manual_seed(hash((shape, n)) % 1000)
    U = (torch.randn(n, *shape, device=DEV, generator=g) * 0.02).to(BF)
    X0 = [(torch.randn(shape, device=DEV, generator=g) * 0.05).to(BF).to(xdtype) for _ in range(n)]

    def fresh():
        if not offset_view:
            return [x.clone() for x in X0]
        out = []
        for x in X0:  # element-aligned only: the start is 2 or 4 bytes past a 256-byte boundary
            buf = torch.empty(x.numel() + 1, device=DEV, dtype=xdtype)
            v = buf[1:].view(shape)
            v.copy_(x)
            out.append(v)
        return out

    lr = torch.tensor(0.02, device=DEV)
    rows, cols = shape[-2:]
    Xa, Xb = fresh(), fresh()
    O = ops.ns_orthogonalize(U.view(-1, rows, cols), coeffs, norm_scale, eps, gram=gram, gram_reset=2)
    ops.muon_post(Xa, O.view(n, -1), lr, 0.7, wd, cautious)
    ops.ns_orthogonalize_update(U.view(-1, rows, cols), Xb, coeffs, norm_scale, eps, lr, 0.7, wd, cautious,
                                gram=gram, gram_reset=2)
    return X0, O.view(n, *shape), Xa, Xb


@pytest.mark.parametrize("shape", [(256, 512), (512, 256), (128, 128), (384, 1024), (1024, 384), (2, 128, 256),
                                   (3, 256, 128)])
@pytest.mark.parametrize("xdtype", [torch.float32, BF])
@pytest.mark.parametrize("cautious", [False, True])
def test_fused_epilogue_matches_two_calls(shape, xdtype, cautious):
    X0, O, Xa, Xb = _run_both(shape, 3, xdtype, cautious)
    for x0, o, a, b in zip(X0, O, Xa, Xb):
        assert b.dtype == xdtype
        assert torch.equal(a, b)
        assert not torch.equal(b, x0)
        # and the update is the oracle's, given the orthogonalized matrices
        ref = oracle.muon_post(x0.float().cpu(), o.cpu(), 0.02, 0.7, 0.01, cautious)
        if xdtype == torch.float32:
            assert float((b.cpu() - ref).abs().max()) <= 1e-7
        else:
            assert float((b.float().cpu() - ref).abs().max()) <= 2.0 ** -8 * float(ref.abs().max())


@pytest.mark.parametrize("shape", [(100, 200), (200, 100), (64, 768), (768, 64), (3, 40, 24), (130, 130)])
@pytest.mark.parametrize("xdtype", [torch.float32, BF])
def test_padded_and_small_matrices_take_the_two_pass_route(shape, xdtype):
    _X0, _O, Xa, Xb = _run_both(shape, 2, xdtype, False)
    assert all(torch.equal(a, b) for a, b in zip(Xa, Xb))


@pytest.mark.parametrize("shape", [(256, 512), (512, 256)])
@pytest.mark.parametrize("xdtype", [torch.float32, BF])
def test_parameters_that_are_offset_views(shape, xdtype):
    """Parameter storage that is only element-aligned: the transposed epilogue falls back from 16-byte
    accesses to element accesses."""
    _X0, _O, Xa, Xb = _run_both(shape, 2, xdtype, True, offset_view=True)
    assert all(torch.equal(a, b) for a, b in zip(Xa, Xb))


@pytest.mark.parametrize("shape,xdtype", [((4096, 14336), torch.float32), ((14336, 4096), torch.float32),
                                          ((14336, 4096), BF), ((1024, 4096), BF)])
def test_llama_sized_parameters(shape, xdtype):
    """The 256x256-tile kernels at the headline shapes, both orientations."""
    _X0, _O, Xa, Xb = _run_both(shape, 2, xdtype, False)
    assert all(torch.equal(a, b) for a, b in zip(Xa, Xb))


@pytest.mark.parametrize("shape", [(128, 256), (256, 128)])
def test_more_parameters_than_one_launch_holds(shape):
    """70 parameters: the last GEMM is launched once per 64 pointers."""
    _X0, _O, Xa, Xb = _run_both(shape, 70, torch.float32, False)
    assert all(torch.equal(a, b) for a, b in zip(Xa, Xb))


@pytest.mark.parametrize("shape", [(256, 512), (512, 256), (256, 768), (768, 256)])
def test_schedules_and_options(shape):
    from dion_amd import newton_schulz as ns

    for kw in (dict(gram=True, coeffs=ns.POLAR_EXPRESS_COEFFS, norm_scale=1.02, eps=0.0),
               dict(coeffs=ns.POLAR_EXPRESS_COEFFS, norm_scale=1.02, eps=1e-6),
               dict(coeffs=[ns.KJ_COEFFS] * 3),
               dict(coeffs=[]),  # no iteration: the prepared input is the update
               dict(wd=torch.tensor(0.05, device=DEV))):
        _X0, _O, Xa, Xb = _run_both(shape, 2, torch.float32, False, **kw)
        assert all(torch.equal(a, b) for a, b in zip(Xa, Xb)), kw


def test_live_learning_rate_is_read_on_the_device():
    from dion_amd import newton_schulz as ns
    from dion_amd import ops

    torch.manual_seed(0)
    U = (torch.randn(2, 256, 256, device=DEV) * 0.02).to(BF)
    X = [torch.randn(256, 256, device=DEV) for _ in range(2)]
    x0 = [x.clone() for x in X]
    lr = torch.tensor(0.0, device=DEV)
    ops.ns_orthogonalize_update(U, X, ns.NS5_COEFFS, 1.0, 1e-7, lr, 1.0, 0.1)
    assert all(torch.equal(a, b) for a, b in zip(X, x0)), "lr = 0: nothing moves"
    lr.fill_(0.5)
    ops.ns_orthogonalize_update(U, X, ns.NS5_COEFFS, 1.0, 1e-7, lr, 1.0, 0.1)
    O = ops.ns_orthogonalize(U, ns.NS5_COEFFS, 1.0, 1e-7)
    for x, x_before, o in zip(X, x0, O):
        assert torch.allclose(x, x_before * (1 - 0.5 * 0.1) - 0.5 * o.float(), atol=1e-6, rtol=0)


def test_argument_checks():
    from dion_amd import newton_schulz as ns
    from dion_amd import ops

    U = torch.zeros(2, 128, 128, device=DEV, dtype=BF)
    lr = torch.tensor(0.1, device=DEV)
    with pytest.raises(ValueError, match="divide"):
        ops.ns_orthogonalize_update(U, [torch.zeros(128, 128, device=DEV)] * 3, ns.NS5_COEFFS, 1.0, 1e-7, lr, 1.0, 0.0)
    with pytest.raises(ValueError, match="elements"):
        ops.ns_orthogonalize_update(U, [torch.zeros(128, 64, device=DEV)] * 2, ns.NS5_COEFFS, 1.0, 1e-7, lr, 1.0, 0.0)
    with pytest.raises(TypeError):
        ops.ns_orthogonalize_update(U, [torch.zeros(128, 128, device=DEV, dtype=torch.float16)] * 2, ns.NS5_COEFFS,
                                    1.0, 1e-7, lr, 1.0, 0.0)
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.ns_orthogonalize_update(U, [torch.zeros(128, 128)] * 2, ns.NS5_COEFFS, 1.0, 1e-7, lr, 1.0, 0.0)


def _model(dtype):
    torch.manual_seed(5)
    shapes = [(256, 512), (256, 512), (512, 256), (100, 60), (2, 128, 256), (384, 128)]
    return [torch.nn.Parameter((torch.randn(s, device=DEV) * 0.02).to(BF).to(dtype)) for s in shapes]


@pytest.mark.parametrize("kw", [{}, {"nesterov": True, "cautious_wd": True}, {"use_polar_express": False},
                                {"use_gram_newton_schulz": True}, {"flatten": True}, {"adjust_lr": "rms_norm"}])
@pytest.mark.parametrize("dtype", [torch.float32, BF])
def test_muon_step_is_the_same_with_and_without_fusion(kw, dtype):
    import dion

    models, opts = [], []
    for fused in (True, False):
        ps = _model(dtype)
        heads = {} if kw.get("flatten") else {"num_heads": 3}  # the two options exclude each other
        opt = dion.Muon([{"params": ps[:5]}, {"params": ps[5:], **heads}], lr=0.02, **kw)
        opt.fused_update = fused
        models.append(ps)
        opts.append(opt)
    torch.manual_seed(6)
    for _ in range(3):
        grads = [torch.randn_like(p, dtype=torch.float32).to(BF) for p in models[0]]
        for ps in models:
            for p, g in zip(ps, grads):
                p.grad_dtype = None
                p.grad = g.clone()
        for opt in opts:
            opt.step()
        for a, b in zip(*models):
            assert torch.equal(a.data, b.data)
            assert torch.equal(opts[0].state[a]["momentum"], opts[1].state[b]["momentum"])


def test_custom_orthogonalization_keeps_the_two_call_sequence():
    import dion
    from dion_amd import zeropower_via_newtonschulz5

    calls = []

    def my_ns(X, epsilon=1e-7):
        calls.append(tuple(X.shape))
        return zeropower_via_newtonschulz5(X, epsilon)

    torch.manual_seed(7)
    pa = torch.nn.Parameter(torch.randn(256, 512, device=DEV) * 0.02)
    pb = torch.nn.Parameter(pa.data.clone())
    oa = dion.Muon([pa], lr=0.02, newton_schulz_func=my_ns)
    ob = dion.Muon([pb], lr=0.02, use_polar_express=False)
    ob.prepared_input = False  # the built-in operator on the arena in the parameters' layout, as my_ns gets it
    g = torch.randn(256, 512, device=DEV)
    pa.grad, pb.grad = g.clone(), g.clone()
    oa.step()
    ob.step()
    assert calls == [(1, 256, 512)]
    assert torch.equal(pa.data, pb.data)


def test_fused_step_under_graph_replay():
    """The fused call inside a captured step: every replay equals the eager step on the same gradients."""
    import dion
    from dion.cuda_graph import CudaGraphOptimizer

    torch.manual_seed(8)
    pe = [torch.nn.Parameter(torch.randn(256, 512, device=DEV) * 0.02) for _ in range(2)]
    pg = [torch.nn.Parameter(p.data.clone()) for p in pe]
    eager = dion.Muon(pe, lr=0.02)
    graph = CudaGraphOptimizer(dion.Muon(pg, lr=0.02), warmup_steps=1)
    for p in pe + pg:
        p.grad = torch.zeros_like(p)
    for step in range(5):
        gs = [torch.randn(256, 512, device=DEV) for _ in pe]
        for p, q, g in zip(pe, pg, gs):
            p.grad.copy_(g)
            q.grad.copy_(g)
        eager.step()
        graph.step()
        torch.cuda.synchronize()
        for p, q in zip(pe, pg):
            assert torch.equal(p.data, q.data), f"step {step}"
