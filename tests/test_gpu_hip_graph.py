"""hipGraph capture of the optimizer step (the contract of the reference's tests/test_cuda_graph.py):
a wrapped optimizer must follow the eager one bit for bit on every step -- warm-up, the capture step
and every replay -- with eager work and synchronisations of the test itself between the replays, under
a constant and a scheduled learning rate, for every optimizer of the package and mixed param groups."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"

# GPT-small-like shape groups (several small groups -> the side-stream fork/join is captured too),
# a per-head group, an AdamW and a Lion group
SHAPES = [(256, 128), (256, 128), (128, 128), (128, 128), (128, 512), (512, 128), (384, 128)]


def _build(cls_name, kwargs, seed):
    import dion

    torch.manual_seed(seed)
    mats = [torch.nn.Parameter(torch.randn(s, device=DEV) * 0.02) for s in SHAPES]
    heads = [torch.nn.Parameter(torch.randn(4 * 32, 96, device=DEV) * 0.02)]
    vec = [torch.nn.Parameter(torch.randn(300, device=DEV))]
    emb = [torch.nn.Parameter(torch.randn(64, 48, device=DEV))]
    groups = [dict(params=mats), dict(params=heads, num_heads=4),
              dict(params=vec, algorithm="adamw", lr=0.003), dict(params=emb, algorithm="lion", lr=0.001)]
    assembled = kwargs.pop("_assembled", False)
    opt = getattr(dion, cls_name)(groups, lr=0.02, **kwargs)
    if assembled:  # the whole-matrix selection sequence (accumulate, select inside, masked update)
        opt.assembled_selection = True
    return mats + heads + vec + emb, opt


CASES = [("Muon", dict(nesterov=True)), ("Muon", dict(use_polar_express=False, cautious_wd=True)),
         ("NorMuon", {}), ("Dion2", dict(fraction=0.25)), ("NorDion2", dict(fraction=0.5)),
         ("Muon", dict(weight_decay=torch.tensor(0.02))),
         ("Dion2", dict(fraction=0.25, selection_scope="global", _assembled=True)),
         ("NorDion2", dict(fraction=0.5, selection_scope="global", _assembled=True))]


@pytest.mark.parametrize("cls_name,kwargs", CASES)
def test_replay_matches_eager_bit_for_bit(cls_name, kwargs):
    from dion.cuda_graph import CudaGraphOptimizer

    p_e, o_e = _build(cls_name, dict(kwargs), 5)
    p_g, inner = _build(cls_name, dict(kwargs), 5)
    o_g = CudaGraphOptimizer(inner, warmup_steps=2)
    s_e = torch.optim.lr_scheduler.LambdaLR(o_e, lambda s: 1.0 / (1 + 0.3 * s))
    s_g = torch.optim.lr_scheduler.LambdaLR(inner, lambda s: 1.0 / (1 + 0.3 * s))
    gen = torch.Generator(device=DEV).manual_seed(9)
    for p in p_e + p_g:
        p.grad = torch.zeros_like(p)
    for step in range(8):
        for a, b in zip(p_e, p_g):
            g = torch.randn(a.shape, device=DEV, generator=gen)
            a.grad.copy_(g)
            b.grad.copy_(g)  # in place: the captured graph reads these buffers
        o_e.step()
        o_g.step()
        torch.cuda.synchronize()
        # eager work of the test between replays
        junk = torch.randn(256, 256, device=DEV) @ torch.randn(256, 256, device=DEV)
        assert torch.isfinite(junk).all()
        for i, (a, b) in enumerate(zip(p_e, p_g)):
            assert torch.equal(a.data, b.data), (cls_name, step, i)
        for a, b in zip(p_e, p_g):
            for key in o_e.state[a]:
                assert torch.equal(o_e.state[a][key], inner.state[b][key]), (cls_name, step, key)
        s_e.step()
        s_g.step()
        o_g.zero_grad(set_to_none=False)
    assert o_g.captured
    assert [g["step"] for g in inner.param_groups] == [g["step"] for g in o_e.param_groups]
    assert float(inner.state[p_g[-2]]["step_dev"]) == 8.0
    o_g.release()
    assert not o_g.captured


def test_float_lr_assignment_reaches_the_graph_and_late_live_wd_is_refused():
    from dion.cuda_graph import CudaGraphOptimizer

    p_e, o_e = _build("Muon", {}, 6)
    p_g, inner = _build("Muon", {}, 6)
    o_g = CudaGraphOptimizer(inner, warmup_steps=1)
    gen = torch.Generator(device=DEV).manual_seed(10)
    for p in p_e + p_g:
        p.grad = torch.zeros_like(p)
    for step in range(5):
        for a, b in zip(p_e, p_g):
            g = torch.randn(a.shape, device=DEV, generator=gen)
            a.grad.copy_(g)
            b.grad.copy_(g)
        lr = 0.02 / (step + 1)
        o_e.param_groups[0]["lr"] = lr      # the hand-rolled schedule idiom: a plain float
        inner.param_groups[0]["lr"] = lr
        o_e.step()
        o_g.step()
        for a, b in zip(p_e, p_g):
            assert torch.equal(a.data, b.data), step
    inner.param_groups[0]["weight_decay"] = torch.tensor(0.5, device=DEV)
    with pytest.raises(RuntimeError, match="did not exist when the step was recorded"):
        o_g.step()


def test_capture_refuses_params_without_grad():
    from dion.cuda_graph import CudaGraphOptimizer

    params, inner = _build("Muon", {}, 7)
    opt = CudaGraphOptimizer(inner, warmup_steps=1)
    for p in params[:-1]:
        p.grad = torch.randn_like(p)
    opt.step()  # warm-up step is eager and simply skips the param without a gradient
    with pytest.raises(RuntimeError, match="have no gradient yet"):
        opt.step()


def test_replay_refuses_a_gradient_buffer_that_moved():
    """The recorded kernels address .grad by raw pointer: a gradient that was re-created elsewhere would
    be ignored silently, so the wrapper refuses to replay; after release() it records again."""
    from dion.cuda_graph import CudaGraphOptimizer

    params, inner = _build("Muon", {}, 14)
    wrap = CudaGraphOptimizer(inner, warmup_steps=1)
    for p in params:
        p.grad = torch.randn_like(p)
    wrap.step()
    wrap.step()
    assert wrap.captured
    wrap.step()  # a plain replay is fine
    keep = params[0].grad
    params[0].grad = torch.randn_like(params[0])  # a new buffer, as zero_grad(set_to_none=True) + backward leaves
    assert params[0].grad.data_ptr() != keep.data_ptr()
    before = [p.data.clone() for p in params]
    with pytest.raises(RuntimeError, match="no longer the tensor it was recorded with"):
        wrap.step()
    torch.cuda.synchronize()
    assert all(torch.equal(a, p.data) for a, p in zip(before, params)), "a refused replay must not run"
    wrap.release()
    wrap.step()
    wrap.step()
    assert wrap.captured


def _zero_grads(params):
    for p in params:
        p.grad = torch.zeros_like(p)


def test_frozen_parameter_is_allowed_and_release_rewarms():
    """A parameter frozen on purpose (requires_grad=False, no gradient) does not block the capture;
    release() drops the graph and restarts the warm-up, twice in a row is a no-op, and before any
    capture it still resets the warm-up count (dion/cuda_graph.py:183-200, the contract of the reference's
    tests/test_cuda_graph.py:765-815)."""
    from dion.cuda_graph import CudaGraphOptimizer

    params, inner = _build("Dion2", dict(fraction=0.25), 8)
    wrap = CudaGraphOptimizer(inner, warmup_steps=1)
    _zero_grads(params)
    wrap.step()
    params[0].grad = None
    params[0].requires_grad_(False)
    wrap.step()
    assert wrap.captured
    wrap.release()
    assert not wrap.captured and wrap.eager_steps_done == 0
    wrap.release()
    wrap.step()
    assert not wrap.captured
    wrap.step()
    assert wrap.captured

    params, inner = _build("Dion2", dict(fraction=0.25), 8)
    wrap = CudaGraphOptimizer(inner, warmup_steps=3)
    _zero_grads(params)
    wrap.step()
    wrap.step()
    assert not wrap.captured and wrap.eager_steps_done == 2
    wrap.release()
    assert wrap.eager_steps_done == 0


def test_failed_capture_leaves_no_graph_and_lr_sync_under_capture_is_an_error():
    from dion.cuda_graph import CudaGraphOptimizer

    params, inner = _build("Muon", {}, 9)
    wrap = CudaGraphOptimizer(inner, warmup_steps=1)
    _zero_grads(params)
    wrap.step()
    real_step = inner.step

    def boom(*a, **k):
        raise RuntimeError("capture blew up")

    inner.step = boom
    with pytest.raises(RuntimeError, match="capture blew up"):
        wrap.step()
    assert not wrap.captured
    inner.step = real_step
    torch.cuda.synchronize()
    wrap.step()  # captures now
    assert wrap.captured

    # writing the lr tensor inside a capture would bake the capture-time value into every replay
    params, opt = _build("Dion2", dict(fraction=0.25), 9)
    _zero_grads(params)
    opt.step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, capture_error_mode="thread_local"):
        torch.zeros(4, device=DEV).add_(1)  # keep the capture non-empty
        for g in opt.param_groups:
            g["lr"] = 0.5
        with pytest.raises(RuntimeError, match="capture"):
            opt.bind_live_scalars()
    del graph
    torch.cuda.synchronize()


@pytest.mark.parametrize("cls_name,kwargs", [("Muon", {}), ("NorMuon", {}), ("Dion2", dict(fraction=0.25)),
                                             ("NorDion2", dict(fraction=0.5))])
def test_scheduled_lr_tracks_after_resume_and_closure(cls_name, kwargs):
    """An optimizer restored from a checkpoint (state_dict through torch.save / load with
    map_location="cpu", loaded by keyword) and then wrapped follows a scheduled learning rate under replay
    exactly like the eager one; step(closure) returns the closure's value."""
    import io

    from dion.cuda_graph import CudaGraphOptimizer

    p_src, o_src = _build(cls_name, dict(kwargs), 11)
    gen = torch.Generator(device=DEV).manual_seed(12)
    for p in p_src:
        p.grad = torch.randn(p.shape, device=DEV, generator=gen)
    o_src.step()
    o_src.step()
    buf = io.BytesIO()
    torch.save(o_src.state_dict(), buf)
    weights = [p.detach().clone() for p in p_src]

    def resumed():
        params, opt = _build(cls_name, dict(kwargs), 11)
        for p, w in zip(params, weights):
            p.data.copy_(w)
        buf.seek(0)
        sd = torch.load(buf, map_location="cpu", weights_only=True)
        return params, opt, sd

    p_e, o_e, sd = resumed()
    o_e.load_state_dict(sd)
    p_g, inner, sd = resumed()
    o_g = CudaGraphOptimizer(inner, warmup_steps=2)
    o_g.load_state_dict(state_dict=sd)
    assert inner.param_groups[0]["step"] == o_src.param_groups[0]["step"] == 2
    assert all(isinstance(g["lr"], torch.Tensor) and g["lr"].is_cuda for g in inner.param_groups)
    _zero_grads(p_e + p_g)
    for step in range(7):
        for a, b in zip(p_e, p_g):
            g = torch.randn(a.shape, device=DEV, generator=gen)
            a.grad.copy_(g)
            b.grad.copy_(g)
        for grp_e, grp_g in zip(o_e.param_groups, inner.param_groups):
            lr = 0.02 * (0.25 + 1.5 * (step + 1) / 7)
            grp_e["lr"] = lr
            grp_g["lr"] = lr
        o_e.step()
        assert o_g.step(lambda: torch.tensor(3.0)) == 3.0
        for a, b in zip(p_e, p_g):
            assert torch.equal(a.data, b.data), (cls_name, step)
    assert o_g.captured


def test_add_param_group_rewarms_before_recapturing():
    from dion.cuda_graph import CudaGraphOptimizer

    params, inner = _build("Muon", {}, 13)
    wrap = CudaGraphOptimizer(inner, warmup_steps=2)
    _zero_grads(params)
    for _ in range(3):
        wrap.step()
    assert wrap.captured
    extra = torch.nn.Parameter(torch.randn(128, 256, device=DEV) * 0.02)
    extra.grad = torch.zeros_like(extra)
    wrap.add_param_group(dict(params=[extra]))
    assert not wrap.captured and wrap.eager_steps_done == 0
    wrap.step()
    wrap.step()
    assert not wrap.captured       # two eager steps for the new group first
    wrap.step()
    assert wrap.captured
    assert isinstance(inner.param_groups[-1]["lr"], torch.Tensor)
