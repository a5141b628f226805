"""Shared host logic of the Muon / NorMuon / Dion2 / NorDion2 optimizers on one MI355X.

Mirrors the single-GPU behaviour of the reference's ``DistributedOrthoBase``
(dion/megabatch_base.py:22-632): same constructor contract, param-group keys, eager state
pre-population, live ``lr`` device tensor, float ``lr`` in ``state_dict()``, and the per-group
``num_heads`` / ``split_sizes`` options.  What differs is the execution model: the reference builds
generator tasks that interleave all-to-all communication; on one GPU every shape group is simply a
handful of kernel launches on the current stream, so ``step()`` is a plain loop.
"""
from collections import defaultdict
from typing import Callable, Dict, List, Optional, Tuple

import torch
from torch import Tensor
from torch.optim.optimizer import Optimizer

from . import newton_schulz as ns
from . import scalar_opts


class OrthoOptimizer(Optimizer):
    """Base class: orchestration, state and validation.  Subclasses implement
    ``_shape_group_phases`` (a generator: work before / during / after the orthogonalization)."""

    def __init__(self, params, distributed_mesh, algo_name: str, defaults: dict,
                 use_gram_newton_schulz: bool = False, use_triton: bool = False,
                 use_polar_express: bool = True, newton_schulz_func: Optional[Callable] = None):
        if distributed_mesh is not None:
            # One process drives one GPU here; the sharded all-to-all / all-gather paths of
            # dion/megabatch_base.py:713-857 are not part of this build.
            from torch.distributed import ProcessGroup
            from torch.distributed.device_mesh import DeviceMesh

            if not isinstance(distributed_mesh, (DeviceMesh, ProcessGroup)):
                raise TypeError(
                    f"Invalid distributed_mesh type: {type(distributed_mesh)}. "
                    f"Expected DeviceMesh or ProcessGroup."
                )
            raise NotImplementedError(
                "dion_amd runs the optimizer step on a single GPU; pass distributed_mesh=None."
            )
        super().__init__(params, defaults)
        self._algo_name = algo_name
        self._device_rank = 0
        self._world_size = 1
        self._process_group = None
        self._distributed_mesh = None

        # Which orthogonalization runs.  use_triton is accepted for signature compatibility and
        # selects nothing: there is a single implementation (dion/megabatch_base.py:70-112 picks
        # between four).
        self._custom_ns = False
        if newton_schulz_func is not None:
            if not callable(newton_schulz_func):
                raise TypeError(
                    f"newton_schulz_func must be a callable function, got {type(newton_schulz_func)}"
                )
            self._newton_schulz_func = newton_schulz_func
            self._custom_ns = True
        elif use_gram_newton_schulz:
            self._newton_schulz_func = ns.gram_newton_schulz
        elif use_polar_express:
            self._newton_schulz_func = ns.polar_express
        else:
            self._newton_schulz_func = ns.zeropower_via_newtonschulz5
        self._use_triton = bool(use_triton)

        # State for every parameter exists from construction on, so state_dict() has the same keys
        # before and after the first step (dion/megabatch_base.py:114-137).
        self._state_prepopulated = False
        self._hyper_tensors: Dict[Tuple[int, str], Tensor] = {}
        self._live_names: Dict[int, Tuple[str, ...]] = {}
        for group in self.param_groups:
            self._prepopulate(group)
        self._sync_hyperparam_tensors()
        self._state_prepopulated = True

    # ------------------------------------------------------------------ state
    def _prepopulate(self, group: dict) -> None:
        for p in group["params"]:
            self._get_or_initialize_state(p, group["algorithm"])

    def add_param_group(self, param_group: dict) -> None:
        super().add_param_group(param_group)
        if getattr(self, "_state_prepopulated", False):
            index = len(self.param_groups) - 1
            for name in self._live_hyperparams(index):
                self._ensure_hyperparam_tensor(index, name)
            self._prepopulate(self.param_groups[-1])

    def _get_or_initialize_state(self, param: Tensor, algo: str) -> dict:
        state = self.state[param]
        if not state:
            state["momentum"] = torch.zeros_like(param)
            if algo == "adamw":
                state["variance"] = torch.zeros_like(param)
        if algo == "adamw" and "step_dev" not in state:
            state["step_dev"] = torch.zeros((), dtype=torch.float32, device=param.device)
        return state

    # ------------------------------------------------- live hyper-parameters
    def _live_hyperparams(self, index: int) -> Tuple[str, ...]:
        """``lr`` always lives in a persistent 0-d device tensor; ``weight_decay`` does once the
        caller has supplied a Tensor for it (dion/megabatch_base.py:417-448)."""
        live = self._live_names.get(index)
        if live is None or "weight_decay" not in live:
            if isinstance(self.param_groups[index].get("weight_decay"), Tensor):
                live = ("lr", "weight_decay")
            elif live is None:
                live = ("lr",)
            self._live_names[index] = live
        return live

    def _ensure_hyperparam_tensor(self, index: int, name: str) -> Optional[Tensor]:
        """Keep ``param_groups[index][name]`` bound to one 0-d float32 device tensor whose identity
        never changes; floats (or foreign tensors) assigned by the caller are copied into it
        (dion/megabatch_base.py:450-501)."""
        group = self.param_groups[index]
        if not group["params"]:
            return None
        value = group[name]
        tensor = self._hyper_tensors.get((index, name))
        if value is tensor and tensor is not None:
            return tensor
        device = group["params"][0].device
        if device.type == "cuda" and torch.cuda.is_current_stream_capturing():
            raise RuntimeError(
                f"param group {index} has a {name} that is not its persistent device tensor "
                f"({type(value).__name__}) and graph capture is already underway; sync {name} "
                "before capturing."
            )
        if tensor is None or tensor.device != device:
            tensor = torch.empty((), dtype=torch.float32, device=device)
            self._hyper_tensors[(index, name)] = tensor
        if isinstance(value, Tensor):
            tensor.copy_(value)
        else:
            tensor.fill_(value)
        group[name] = tensor
        return tensor

    @property
    def _hyperparam_tensors(self) -> Dict[Tuple[int, str], Tensor]:
        """The persistent device tensors behind ``lr`` (and an opted-in ``weight_decay``); a graph
        wrapper compares their count before and after capture (dion/cuda_graph.py:212-229)."""
        return self._hyper_tensors

    def _advance_host_step_counters(self) -> None:
        """Host-side bookkeeping of one step that a graph replay does not execute
        (dion/cuda_graph.py:307-311)."""
        for group in self.param_groups:
            group["step"] += 1

    def _sync_hyperparam_tensors(self) -> None:
        for index in range(len(self.param_groups)):
            for name in self._live_hyperparams(index):
                self._ensure_hyperparam_tensor(index, name)

    def state_dict(self):
        sd = super().state_dict()
        for group in sd["param_groups"]:
            for key, value in group.items():
                if key != "params" and isinstance(value, Tensor) and value.ndim == 0:
                    group[key] = value.item()
        return sd

    def load_state_dict(self, state_dict):
        super().load_state_dict(state_dict)
        self._sync_hyperparam_tensors()
        for group in self.param_groups:
            if group["algorithm"] != "adamw":
                continue
            for p in group["params"]:
                state = self.state.get(p)
                if state is None:
                    continue
                step = state.get("step_dev")
                if step is None:
                    step = torch.full((), float(group["step"]), dtype=torch.float32, device=p.device)
                elif step.dtype != torch.float32 or step.device != p.device:
                    step = step.to(dtype=torch.float32, device=p.device)
                state["step_dev"] = step

    # ------------------------------------------------------------ validation
    def _resolve_num_heads(self, group: dict) -> Optional[int]:
        num_heads = group.get("num_heads")
        if num_heads is None:
            return None
        if isinstance(num_heads, bool) or not isinstance(num_heads, int) or num_heads < 1:
            raise ValueError(f"num_heads must be a positive integer if set, got {num_heads!r}.")
        if num_heads == 1:
            return None
        if group.get("flatten"):
            raise ValueError(
                "num_heads > 1 is incompatible with flatten=True: flattening the per-head 3D view "
                "collapses heads back into a single 2D matrix, defeating per-head Newton-Schulz."
            )
        return num_heads

    def _resolve_split_sizes(self, group: dict) -> Optional[Tuple[int, ...]]:
        split_sizes = group.get("split_sizes")
        if split_sizes is None:
            return None
        if not isinstance(split_sizes, (tuple, list)) or len(split_sizes) < 2:
            raise ValueError(
                f"split_sizes must be a tuple or list of at least 2 block sizes, got {split_sizes!r}."
            )
        if any(isinstance(s, bool) or not isinstance(s, int) or s < 1 for s in split_sizes):
            raise ValueError(f"split_sizes entries must be positive integers, got {split_sizes!r}.")
        if self._resolve_num_heads(group) is not None:
            raise ValueError(
                "split_sizes is incompatible with num_heads > 1: use num_heads for uniform per-head "
                "splits or split_sizes for uneven row blocks, not both."
            )
        if group.get("flatten"):
            raise ValueError(
                "split_sizes is incompatible with flatten=True: split_sizes applies to 2D parameters only."
            )
        return tuple(split_sizes)

    @staticmethod
    def _validate_split_shape(split_sizes: Tuple[int, ...], shape) -> None:
        if len(shape) != 2:
            raise ValueError(f"split_sizes is only supported for 2D parameters, got shape {tuple(shape)}.")
        if sum(split_sizes) != shape[0]:
            raise ValueError(
                f"split_sizes {split_sizes} must sum to dim 0 of the parameter (got shape {tuple(shape)})."
            )

    @staticmethod
    def _head_geometry(num_heads: int, shape) -> Tuple[int, int, int]:
        """(mats, rows, cols) of the per-head view of a 2D weight (dion/megabatch_base.py:304-364)."""
        if len(shape) != 2:
            raise ValueError(f"num_heads is only supported for 2D parameters, got shape {tuple(shape)}.")
        if shape[0] % num_heads != 0:
            raise ValueError(
                f"num_heads ({num_heads}) must divide dim 0 of the parameter (got shape {tuple(shape)})."
            )
        return num_heads, shape[0] // num_heads, shape[1]

    # ------------------------------------------------------------------ step
    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        self._sync_hyperparam_tensors()

        ortho, lion, adamw = [], [], []
        for group in self.param_groups:
            group["step"] += 1
            algo = group["algorithm"]
            if algo == self._algo_name:
                ortho.append(group)
            elif algo == "lion":
                lion.append(group)
            elif algo == "adamw":
                adamw.append(group)
            else:
                raise ValueError(f"Unknown algorithm: {algo}")

        work: List[Tuple[dict, List[Tensor]]] = []
        for group in ortho:
            assert all(p.ndim >= 2 for p in group["params"]), (
                f"{type(self).__name__} optimizer only supports matrix parameters."
            )
            with_grad = [p for p in group["params"] if p.grad is not None]
            if not with_grad:
                continue
            buckets: Dict[tuple, List[Tensor]] = defaultdict(list)
            for p in with_grad:
                buckets[(p.shape, p.dtype)].append(p)
            for params in buckets.values():
                work.append((group, params))
        self._run_shape_groups(work)

        for group in lion:
            scalar_opts.lion_step(self, group)
        for group in adamw:
            scalar_opts.adamw_step(self, group)
        return loss

    def _shape_group_phases(self, group: dict, params: List[Tensor]):
        """Generator over the three phases of one shape group's update: memory-bound preparation,
        ``yield``, orthogonalization (GEMM-bound), ``yield``, memory-bound update."""
        raise NotImplementedError

    def _update_shape_group(self, group: dict, params: List[Tensor]) -> None:
        for _ in self._shape_group_phases(group, params):
            pass

    # Shape groups are independent.  A group whose GEMMs cannot fill the GPU on their own (a few
    # hundred tiles) is run on one of a handful of side streams so that several such groups
    # overlap; mid-sized groups (kernels of three or four rounds of workgroups) share two streams,
    # which fills the partial last round of one group's kernels with the other's; large groups run
    # one after another on the caller's stream, where a second stream only costs L2 locality.  The reference reaches
    # the same goal by interleaving up to three generator tasks (dion/megabatch_base.py:193).
    _SMALL_GROUP_FLOP = 4e12    # below: launches of a few microseconds, four streams
    _MEDIUM_GROUP_FLOP = 3e13   # below: kernels of a few rounds of workgroups, two streams fill the tails
    _N_SIDE_STREAMS = 4

    @staticmethod
    def _group_flop(params: List[Tensor]) -> float:
        r, c = params[0].shape[-2], params[0].shape[-1]
        m, n = min(r, c), max(r, c)
        mats = len(params) * (params[0].numel() // (r * c))
        return mats * 5.0 * (4.0 * m * m * n + 2.0 * m ** 3)

    def _side_pool(self, device) -> List["torch.cuda.Stream"]:
        streams = self.__dict__.setdefault("_side_streams", {})
        pool = streams.get(device)
        if pool is None:
            pool = [torch.cuda.Stream(device=device) for _ in range(self._N_SIDE_STREAMS)]
            streams[device] = pool
        return pool

    def _run_shape_groups(self, work: List[Tuple[dict, List[Tensor]]]) -> None:
        if not work:
            return
        on_gpu = all(params[0].is_cuda for _g, params in work)
        if not on_gpu:
            for group, params in work:
                self._update_shape_group(group, params)
            return
        small = [w for w in work if self._group_flop(w[1]) < self._MEDIUM_GROUP_FLOP]
        big = [w for w in work if self._group_flop(w[1]) >= self._MEDIUM_GROUP_FLOP]
        # (Running the memory-bound phases of neighbouring large groups under these GEMMs on a
        # second stream was measured: no gain -- the chip is power-limited, not idle.)
        for group, params in big:
            self._update_shape_group(group, params)
        if len(small) < 2:
            for group, params in small:
                self._update_shape_group(group, params)
            return
        device = small[0][1][0].device
        pool = self._side_pool(device)
        if any(self._group_flop(w[1]) >= self._SMALL_GROUP_FLOP for w in small):
            pool = pool[:2]
        main = torch.cuda.current_stream(device)
        fork = main.record_event()
        used = []
        for i, (group, params) in enumerate(small):
            side = pool[i % len(pool)]
            if side not in used:
                side.wait_event(fork)
                used.append(side)
            with torch.cuda.stream(side):
                self._update_shape_group(group, params)
        for side in used:
            main.wait_stream(side)

    # ---------------------------------------------------- orthogonalization
    def _orthogonalize(self, U: Tensor, epsilon: float) -> Tensor:
        """``U`` is ``[batch, rows, cols]`` bf16; returns the same shape, bf16."""
        out = self._newton_schulz_func(U, epsilon=epsilon)
        if self._custom_ns:
            out = out.reshape(U.shape).to(torch.bfloat16).contiguous()
        return out

    def _orthogonalize_update(self, U: Tensor, epsilon: float, X: List[Tensor], lr: Tensor, adj_ratio: float,
                              weight_decay, cautious_wd: bool) -> bool:
        """Orthogonalize ``U`` and apply the Muon update to ``X`` in one library call; False (nothing done)
        when a caller-supplied orthogonalization is in use, which has to run on its own."""
        if self._custom_ns or self._newton_schulz_func not in ns.SCHEDULES:
            return False
        ns.orthogonalize_update(self._newton_schulz_func, U, epsilon, X, lr, adj_ratio, weight_decay, cautious_wd)
        return True

    def _orthogonalize_row_blocks(self, U: Tensor, split_sizes, split_scales, epsilon: float) -> Tensor:
        """Row blocks of dim -2 are orthogonalized independently, equal-height blocks batched into
        one call, each rescaled by its ``split_scales`` entry (dion/megabatch_base.py:911-949)."""
        blocks = list(U.split(list(split_sizes), dim=-2))
        by_rows: Dict[int, List[int]] = defaultdict(list)
        for i, blk in enumerate(blocks):
            by_rows[blk.size(-2)].append(i)
        out: List[Optional[Tensor]] = [None] * len(blocks)
        for idx in by_rows.values():
            stacked = torch.stack([blocks[i] for i in idx], dim=0)  # [g, N, rows_i, cols]
            ortho = self._orthogonalize(stacked.flatten(end_dim=-3), epsilon).reshape(stacked.shape)
            for j, i in enumerate(idx):
                blk = ortho[j]
                if split_scales is not None:
                    blk = blk * split_scales[i]
                out[i] = blk
        return torch.cat(out, dim=-2)


def adjust_lr_ratio(shape, adjust_lr: Optional[str], flatten: bool) -> float:
    """Shape factor of the learning rate: ``adjusted_lr = lr * ratio``
    (dion/megabatch_base.py:984-1002)."""
    if adjust_lr is None:
        return 1.0
    if flatten:
        fan_out = shape[0]
        fan_in = 1
        for s in shape[1:]:
            fan_in *= s
    else:
        fan_out, fan_in = shape[-2], shape[-1]
    if adjust_lr == "spectral_norm":
        return (fan_out / fan_in) ** 0.5
    if adjust_lr == "rms_norm":
        return 0.2 * max(fan_out, fan_in) ** 0.5
    raise ValueError(f"Unknown adjust_lr value: {adjust_lr}")


def split_lr_scales(split_sizes, shape, adjust_lr: Optional[str]):
    """Per-block correction ``ratio(block) / ratio(full)`` (dion/megabatch_base.py:952-981)."""
    if adjust_lr is None:
        return None
    full = adjust_lr_ratio(shape, adjust_lr, False)
    return tuple(adjust_lr_ratio((rows, shape[-1]), adjust_lr, False) / full for rows in split_sizes)
