"""Host-side contract of the optimizers (constructor, param groups, state, validation) -- no GPU.
Mirrors what the reference pins in tests/test_state_prepopulation.py and the TestValidation class
of tests/test_optimizers.py."""
import pytest
import torch

from dion import Dion2, Dion3, Muon, NorDion2, NorMuon


def _params(shapes):
    torch.manual_seed(0)
    return [torch.nn.Parameter(torch.randn(s)) for s in shapes]


def test_state_exists_at_construction():
    p = _params([(16, 32), (32, 16)])
    for cls, keys in [(Muon, {"momentum"}), (Dion2, {"momentum"}), (NorMuon, {"momentum", "variance_neuron"}),
                      (NorDion2, {"momentum", "variance_neuron"})]:
        opt = cls(p, lr=0.01)
        for q in p:
            assert set(opt.state[q].keys()) == keys
            assert torch.equal(opt.state[q]["momentum"], torch.zeros_like(q))
        if cls in (NorMuon, NorDion2):
            assert opt.state[p[0]]["variance_neuron"].shape == (16, 1)


def test_param_group_keys_and_defaults():
    p = _params([(16, 32)])
    g = Muon(p).param_groups[0]
    assert {"lr", "mu", "beta1", "beta2", "weight_decay", "cautious_wd", "algorithm", "step", "epsilon",
            "nesterov", "flatten", "adjust_lr"} <= set(g)
    assert g["algorithm"] == "muon" and g["step"] == 0 and g["mu"] == 0.95 and g["adjust_lr"] == "spectral_norm"
    g = NorMuon(p).param_groups[0]
    assert g["algorithm"] == "normuon" and g["muon_beta2"] == 0.95
    g = Dion2(p, fraction=1).param_groups[0]
    assert g["algorithm"] == "dion2" and g["fraction"] == 1.0 and isinstance(g["fraction"], float)
    assert g["ef_decay"] == 0.95 and g["selection_scope"] == "local"
    # dion/nordion2.py:108-122
    g = NorDion2(p, fraction=1).param_groups[0]
    assert g["algorithm"] == "nordion2" and g["fraction"] == 1.0 and isinstance(g["fraction"], float)
    assert g["mu"] == 0.95 and g["muon_beta2"] == 0.95 and g["selection_scope"] == "local" and "ef_decay" not in g
    assert Dion3 is NorDion2


def test_nordion2_constructor_validation():
    p = _params([(16, 32)])
    for kw in [dict(lr=-1.0), dict(fraction=0.0), dict(fraction=1.5), dict(selection_scope="everywhere"),
               dict(mu=-0.1), dict(muon_beta2=-0.1), dict(betas=(0.9,)), dict(adjust_lr="bogus")]:
        with pytest.raises(ValueError):
            NorDion2(p, **kw)
    with pytest.raises(NotImplementedError):
        opt = NorDion2([dict(params=p, split_sizes=(8, 8))])
        p[0].grad = torch.zeros_like(p[0])
        opt.step()


def test_lr_is_a_persistent_tensor_and_state_dict_is_portable():
    p = _params([(16, 32)])
    opt = Muon(p, lr=0.02)
    lr = opt.param_groups[0]["lr"]
    assert isinstance(lr, torch.Tensor) and lr.ndim == 0 and lr.dtype == torch.float32
    sd = opt.state_dict()
    assert isinstance(sd["param_groups"][0]["lr"], float)
    assert sd["param_groups"][0]["lr"] == pytest.approx(0.02)
    # a float assigned by a hand-rolled schedule is copied into the same tensor on sync
    opt.param_groups[0]["lr"] = 0.05
    opt.bind_live_scalars()
    assert opt.param_groups[0]["lr"] is lr and float(lr) == pytest.approx(0.05)
    opt2 = Muon(_params([(16, 32)]), lr=0.5)
    opt2.load_state_dict(sd)
    assert float(opt2.param_groups[0]["lr"]) == pytest.approx(0.02)
    # LR schedulers attach like to any torch optimizer
    sched = torch.optim.lr_scheduler.LambdaLR(opt2, lambda s: 0.5)
    assert float(opt2.param_groups[0]["lr"]) == pytest.approx(0.01)
    assert sched is not None


def test_weight_decay_tensor_becomes_live():
    p = _params([(16, 32)])
    opt = Muon(p, weight_decay=torch.tensor(0.1))
    wd = opt.param_groups[0]["weight_decay"]
    assert isinstance(wd, torch.Tensor) and wd.ndim == 0
    assert isinstance(opt.state_dict()["param_groups"][0]["weight_decay"], float)


def test_constructor_validation():
    p = _params([(16, 32)])
    with pytest.raises(ValueError):
        Muon(p, lr=-0.01)
    with pytest.raises(ValueError):
        NorMuon(p, mu=-1.0)
    with pytest.raises(ValueError):
        NorMuon(p, muon_beta2=-1.0)
    with pytest.raises(ValueError):
        Dion2(p, fraction=0.0)
    with pytest.raises(ValueError):
        Dion2(p, fraction=1.5)
    with pytest.raises(ValueError):
        Dion2(p, selection_scope="shard")
    with pytest.raises(ValueError):
        Dion2(p, ef_decay=-0.1)
    with pytest.raises(ValueError):
        Muon(p, adjust_lr="invalid")
    with pytest.raises(ValueError):
        Muon(p, betas=(0.9,))
    with pytest.raises(TypeError):
        Muon(p, newton_schulz_func="not callable")
    with pytest.raises(TypeError):
        Muon(p, distributed_mesh="mesh")


def test_no_grad_step_is_a_noop_and_counts_steps():
    p = _params([(16, 32)])
    before = p[0].data.clone()
    opt = Muon(p, lr=0.01)
    opt.step()
    assert torch.equal(p[0].data, before)
    assert opt.param_groups[0]["step"] == 1


def test_step_validation_on_cpu_params():
    """Errors raised before any kernel is reached."""
    w = torch.nn.Parameter(torch.randn(64))
    w.grad = torch.randn_like(w)
    with pytest.raises(AssertionError):
        Muon([{"params": [w]}], lr=0.01).step()
    for bad in [0, -1, 2.0, "4", True]:
        w = torch.nn.Parameter(torch.randn(32, 16))
        w.grad = torch.randn_like(w)
        with pytest.raises(ValueError, match="num_heads"):
            Muon([{"params": [w], "num_heads": bad}], lr=0.01).step()
    w = torch.nn.Parameter(torch.randn(30, 16))
    w.grad = torch.randn_like(w)
    with pytest.raises(ValueError, match="num_heads"):
        Muon([{"params": [w], "num_heads": 4}], lr=0.01).step()
    w = torch.nn.Parameter(torch.randn(4, 8, 16))
    w.grad = torch.randn_like(w)
    with pytest.raises(ValueError, match="2D"):
        Muon([{"params": [w], "num_heads": 2}], lr=0.01).step()
    w = torch.nn.Parameter(torch.randn(32, 16))
    w.grad = torch.randn_like(w)
    with pytest.raises(ValueError, match="flatten"):
        Muon([{"params": [w], "num_heads": 4}], lr=0.01, flatten=True).step()
    for bad in [3, (32,), (32, 0), (32, -1), (32, 2.0), (32, "16"), (32, True)]:
        w = torch.nn.Parameter(torch.randn(64, 32))
        w.grad = torch.randn_like(w)
        with pytest.raises(ValueError, match="split_sizes"):
            Muon([{"params": [w], "split_sizes": bad}], lr=0.01).step()
    w = torch.nn.Parameter(torch.randn(60, 32))
    w.grad = torch.randn_like(w)
    with pytest.raises(ValueError, match="split_sizes"):
        Muon([{"params": [w], "split_sizes": (32, 16, 16)}], lr=0.01).step()
    w = torch.nn.Parameter(torch.randn(64, 32))
    w.grad = torch.randn_like(w)
    with pytest.raises(ValueError, match="num_heads"):
        Muon([{"params": [w], "split_sizes": (32, 16, 16), "num_heads": 4}], lr=0.01).step()
    with pytest.raises(NotImplementedError, match="split_sizes"):
        Dion2([{"params": [w], "split_sizes": (32, 16, 16)}], lr=0.01).step()
    with pytest.raises(ValueError, match="Unknown algorithm"):
        Muon([{"params": [w], "algorithm": "sgd"}], lr=0.01).step()


def test_scalar_groups_keep_their_state_contract_and_have_no_cpu_path():
    """adamw / lion groups: state keys as in dion/megabatch_base.py:198-215; the step runs on the HIP
    multi-tensor kernels only, so CPU parameters are refused, not silently updated by another path."""
    b = torch.nn.Parameter(torch.randn(8))
    c = torch.nn.Parameter(torch.randn(8))
    opt = Muon([{"params": [b], "algorithm": "adamw"}, {"params": [c], "algorithm": "lion"}], lr=0.01)
    assert set(opt.state[b].keys()) == {"momentum", "variance", "step_dev"}
    assert set(opt.state[c].keys()) == {"momentum"}
    assert float(opt.state[b]["step_dev"]) == 0.0
    b.grad = torch.randn(8)
    with pytest.raises(RuntimeError, match="no CPU path"):
        opt.step()


def test_graph_wrapper_host_contract():
    """The wrapper delegates the Optimizer API to the inner optimizer (dion/cuda_graph.py:88-181)."""
    from dion.cuda_graph import CudaGraphOptimizer
    from dion_amd import HipGraphOptimizer

    assert CudaGraphOptimizer is HipGraphOptimizer
    p = _params([(16, 32)])
    inner = Muon(p, lr=0.02)
    with pytest.raises(ValueError, match="warmup_steps"):
        CudaGraphOptimizer(inner, warmup_steps=0)
    opt = CudaGraphOptimizer(inner, warmup_steps=3)
    assert isinstance(opt, torch.optim.Optimizer)
    assert opt.param_groups is inner.param_groups and opt.state is inner.state
    assert opt.state_dict()["param_groups"][0]["lr"] == pytest.approx(0.02)
    sched = torch.optim.lr_scheduler.LambdaLR(opt, lambda s: 0.5)   # binds through the wrapper too
    assert float(inner.param_groups[0]["lr"]) == pytest.approx(0.01)
    assert sched is not None
    p[0].grad = torch.ones_like(p[0])
    with pytest.warns(RuntimeWarning, match="set_to_none"):
        opt.zero_grad(set_to_none=True)
    assert p[0].grad is not None and float(p[0].grad.abs().sum()) == 0.0
    opt.add_param_group({"params": _params([(8, 8)])})
    assert len(inner.param_groups) == 2 and opt.eager_steps_done == 0 and not opt.captured
    opt.load_state_dict(inner.state_dict())
    assert [t.data_ptr() for t in inner.live_scalar_tensors()] == [g["lr"].data_ptr() for g in inner.param_groups]
    steps = [g["step"] for g in inner.param_groups]
    inner.count_skipped_host_step()
    assert [g["step"] for g in inner.param_groups] == [s + 1 for s in steps]


def test_wrapper_subclass_tensors_are_refused():
    """A tensor wrapper subclass has no dense buffer behind data_ptr() (the case the reference routes
    around, dion/dion2_triton.py:171-190, tests/test_dion2_post_ortho_triton.py:95-159): the raw-pointer
    entry points refuse it with TypeError rather than write through a meaningless pointer."""
    import torch
    from torch.utils._pytree import tree_map

    from dion_amd import ops

    class Wrapper(torch.Tensor):
        @staticmethod
        def __new__(cls, inner):
            return torch.Tensor._make_wrapper_subclass(cls, inner.shape, dtype=inner.dtype, device=inner.device,
                                                       layout=inner.layout, strides=inner.stride(),
                                                       requires_grad=False)

        def __init__(self, inner):
            self._inner = inner

        def __tensor_flatten__(self):
            return ["_inner"], None

        @staticmethod
        def __tensor_unflatten__(inner_tensors, meta, outer_size, outer_stride):
            return Wrapper(inner_tensors["_inner"])

        @classmethod
        def __torch_dispatch__(cls, func, types, args=(), kwargs=None):
            unwrap = lambda t: t._inner if isinstance(t, Wrapper) else t
            return func(*tree_map(unwrap, args), **tree_map(unwrap, kwargs or {}))

    w = Wrapper(torch.zeros(8, 16))
    with pytest.raises(TypeError, match="wrapper subclass"):
        ops.muon_pre([w], [torch.zeros(8, 16)], 0.9, False)
    with pytest.raises(TypeError, match="wrapper subclass"):
        ops.ns_orthogonalize(w, [(1.0, 0.0, 0.0)], 1.0, 1e-7)
    # a plain dense subclass is not a wrapper
    with pytest.raises(RuntimeError, match="no CPU path"):
        ops.ns_orthogonalize(torch.nn.Parameter(torch.zeros(8, 16)), [(1.0, 0.0, 0.0)], 1.0, 1e-7)


def test_graph_wrapper_signatures_match_torch_optimizer():
    """The wrapper stands in for a torch.optim.Optimizer: every method it overrides keeps the base class's
    parameter names and kinds (callers such as distributed checkpointing pass ``state_dict=`` by keyword;
    the contract of the reference's tests/test_cuda_graph.py:818-870).  Defaults are not pinned:
    zero_grad's set_to_none defaults to False here because replay needs stable .grad buffers."""
    import inspect

    from dion.cuda_graph import CudaGraphOptimizer

    overridden = sorted(name for name, attr in vars(CudaGraphOptimizer).items()
                        if callable(attr) and not name.startswith("_") and hasattr(torch.optim.Optimizer, name))
    assert "load_state_dict" in overridden and "step" in overridden and "zero_grad" in overridden
    for name in overridden:
        base = inspect.signature(getattr(torch.optim.Optimizer, name))
        mine = inspect.signature(getattr(CudaGraphOptimizer, name))
        assert [(p.name, p.kind) for p in mine.parameters.values()] == \
               [(p.name, p.kind) for p in base.parameters.values()], name


@pytest.mark.parametrize("cls,extra", [(Muon, set()), (Dion2, set()), (NorMuon, {"variance_neuron"}),
                                       (NorDion2, {"variance_neuron"})])
def test_add_param_group_prepopulates_and_state_dict_is_complete(cls, extra):
    """State for a group added later exists at once, and a state_dict taken before any step carries
    every parameter's state and loads into a fresh optimizer (the contract of the reference's
    tests/test_state_prepopulation.py:55-86)."""
    p = _params([(16, 32)])
    opt = cls(p, lr=0.01)
    late = _params([(8, 24), (8, 24)])
    opt.add_param_group({"params": late})
    for q in late:
        assert set(opt.state[q].keys()) == {"momentum"} | extra
    assert isinstance(opt.param_groups[1]["lr"], torch.Tensor)
    sd = opt.state_dict()
    assert len(sd["state"]) == 3 and all({"momentum"} | extra <= set(s) for s in sd["state"].values())
    assert all(isinstance(g["lr"], float) for g in sd["param_groups"])
    fresh = cls([{"params": _params([(16, 32)])}, {"params": _params([(8, 24), (8, 24)])}], lr=0.5)
    fresh.load_state_dict(sd)
    assert float(fresh.param_groups[0]["lr"]) == pytest.approx(0.01)
    assert len(fresh.state) == 3


def test_empty_lists_are_accepted_by_the_list_functions():
    """The reference's foreach functions return at once on an empty list
    (tests/test_adamw_foreach.py:218-222); so do these, before any device work."""
    from dion.scalar_opts import adamw_update_foreach, lion_update_foreach

    adamw_update_foreach([], [], [], [], 0.01, 0.9, 0.95, 0.1, 1, 1e-8)
    lion_update_foreach([], [], [], 0.01, 0.9, 0.99, 0.1)


@pytest.mark.parametrize(("scalar_opt", "expected_scale"), [("adamw", 1.0), ("lion", 1 / 768 ** 0.5)])
def test_lm_head_lr_scale_by_scalar_opt(scalar_opt, expected_scale):
    """The reference's own check (tests/test_optimizers.py:42-53)."""
    from dion.opt_utils import as_scalar_tensor, lm_head_lr_scale

    assert lm_head_lr_scale(scalar_opt, model_dim=768) == pytest.approx(expected_scale)
    t = torch.tensor(0.5)
    assert as_scalar_tensor(t) is t and float(as_scalar_tensor(0.25)) == 0.25
