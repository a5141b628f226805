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
from . import ops, scalar_opts


class LiveScalars:
    """Hyper-parameters the kernels read from device memory instead of taking by value.

    The reference keeps ``lr`` of every param group in a 0-d float32 device tensor whose identity
    never changes, and ``weight_decay`` too once the caller has passed it as a Tensor
    (dion/megabatch_base.py:417-501): LR schedulers and hand-rolled schedules keep assigning floats
    to ``group["lr"]``, a captured graph keeps reading the same address.  This class owns those
    tensors, one per (group index, name).
    """

    def __init__(self):
        self._slots: Dict[Tuple[int, str], Tensor] = {}

    def tensors(self) -> List[Tensor]:
        return list(self._slots.values())

    def _wanted(self, index: int, group: dict) -> Tuple[str, ...]:
        # weight decay stays live once it has been: a later float assignment updates the tensor
        if isinstance(group.get("weight_decay"), Tensor) or (index, "weight_decay") in self._slots:
            return ("lr", "weight_decay")
        return ("lr",)

    def bind(self, index: int, group: dict) -> None:
        if not group["params"]:
            return
        device = group["params"][0].device
        for name in self._wanted(index, group):
            slot = self._slots.get((index, name))
            current = group[name]
            if slot is not None and current is slot:
                continue  # nothing was assigned since the last bind
            if device.type == "cuda" and torch.cuda.is_current_stream_capturing():
                # a write recorded into a graph would replay the capture-time value forever
                raise RuntimeError(
                    f"group {index}: {name} was assigned ({type(current).__name__}) while a graph capture is in "
                    "progress; assign hyper-parameters before capture starts"
                )
            if slot is None or slot.device != device:
                slot = torch.zeros((), dtype=torch.float32, device=device)
                self._slots[(index, name)] = slot
            slot.copy_(current) if isinstance(current, Tensor) else slot.fill_(float(current))
            group[name] = slot


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
        self._scalars = LiveScalars()
        self._constructed = False
        for group in self.param_groups:
            self._create_state(group)
        self.bind_live_scalars()
        self._constructed = True

    # ------------------------------------------------------------------ state
    def _create_state(self, group: dict) -> None:
        for p in group["params"]:
            self._get_or_initialize_state(p, group["algorithm"])

    def add_param_group(self, param_group: dict) -> None:
        """torch calls this from ``Optimizer.__init__`` for every group and users call it later; only a
        late group needs its state and device scalars made here (construction does it for all at once)."""
        super().add_param_group(param_group)
        if not getattr(self, "_constructed", False):
            return
        self._scalars.bind(len(self.param_groups) - 1, self.param_groups[-1])
        self._create_state(self.param_groups[-1])

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
    def bind_live_scalars(self) -> None:
        """Make ``group["lr"]`` (and a ``weight_decay`` the caller gave as a Tensor) of every group the
        group's own persistent 0-d device tensor, carrying whatever value is assigned right now."""
        for index, group in enumerate(self.param_groups):
            self._scalars.bind(index, group)

    def live_scalar_tensors(self) -> List[Tensor]:
        """The persistent device tensors the step kernels read hyper-parameters from."""
        return self._scalars.tensors()

    def count_skipped_host_step(self) -> None:
        """The one piece of host state a step changes (``group["step"]``), for a caller that ran the
        step's device work without running ``step()`` -- a graph replay."""
        for group in self.param_groups:
            group["step"] += 1

    def state_dict(self):
        """Checkpoints carry plain floats where a group holds a 0-d tensor, so they load into any
        optimizer on any device (dion/megabatch_base.py:521-538)."""
        sd = super().state_dict()
        sd["param_groups"] = [
            {k: (v.item() if k != "params" and isinstance(v, Tensor) and v.ndim == 0 else v) for k, v in g.items()}
            for g in sd["param_groups"]
        ]
        return sd

    def load_state_dict(self, state_dict):
        super().load_state_dict(state_dict)
        self.bind_live_scalars()
        # AdamW's device step counter: float32 on the parameter's device whatever the checkpoint
        # held, and rebuilt from the group's host counter when the checkpoint predates it
        for group in self.param_groups:
            if group["algorithm"] != "adamw":
                continue
            for p in group["params"]:
                if p not in self.state:
                    continue
                saved = self.state[p].get("step_dev")
                value = float(group["step"]) if saved is None else float(saved)
                self.state[p]["step_dev"] = torch.full((), value, dtype=torch.float32, device=p.device)

    # ------------------------------------------------------------ validation
    # How a group's 2D weights are cut into independent matrices: ``num_heads`` equal row bands
    # (per-head orthogonalization, dion/megabatch_base.py:304-364) or ``split_sizes`` uneven row blocks
    # (fused projections, :911-981).  One or the other, never with flatten.
    @staticmethod
    def _positive_int(value) -> bool:
        return isinstance(value, int) and not isinstance(value, bool) and value >= 1

    def _resolve_num_heads(self, group: dict) -> Optional[int]:
        heads = group.get("num_heads")
        if heads is None:
            return None
        if not self._positive_int(heads):
            raise ValueError(f"num_heads: expected a positive integer or None, got {heads!r}")
        if heads == 1:
            return None  # one head is the whole matrix
        if group.get("flatten"):
            raise ValueError("num_heads > 1 cannot be combined with flatten=True (flattening would merge the heads "
                             "back into one matrix)")
        return heads

    def _resolve_split_sizes(self, group: dict) -> Optional[Tuple[int, ...]]:
        blocks = group.get("split_sizes")
        if blocks is None:
            return None
        if not isinstance(blocks, (tuple, list)) or len(blocks) < 2 or not all(self._positive_int(b) for b in blocks):
            raise ValueError(f"split_sizes: expected a tuple or list of two or more positive integers, got {blocks!r}")
        if self._resolve_num_heads(group) is not None:
            raise ValueError("split_sizes and num_heads > 1 are two ways of cutting the same rows: give one of them")
        if group.get("flatten"):
            raise ValueError("split_sizes cannot be combined with flatten=True (it applies to 2D parameters)")
        return tuple(blocks)

    @staticmethod
    def _validate_split_shape(split_sizes: Tuple[int, ...], shape) -> None:
        if len(shape) != 2:
            raise ValueError(f"split_sizes needs a 2D parameter, got shape {tuple(shape)}")
        if sum(split_sizes) != shape[0]:
            raise ValueError(f"split_sizes {split_sizes} add up to {sum(split_sizes)}, not to the {shape[0]} rows of a "
                             f"parameter of shape {tuple(shape)}")

    @staticmethod
    def _head_geometry(num_heads: int, shape) -> Tuple[int, int, int]:
        """(mats, rows, cols) of the per-head view of a 2D weight (dion/megabatch_base.py:304-364)."""
        if len(shape) != 2:
            raise ValueError(f"num_heads needs a 2D parameter, got shape {tuple(shape)}")
        if shape[0] % num_heads:
            raise ValueError(f"num_heads={num_heads} does not divide the {shape[0]} rows of a parameter of shape "
                             f"{tuple(shape)}")
        return num_heads, shape[0] // num_heads, shape[1]

    # ------------------------------------------------------------------ step
    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        self.bind_live_scalars()

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

    # Shape groups are independent.  Groups whose kernels are a few rounds of workgroups or less (GPT-small:
    # a few hundred tiles per launch; GPT-1.3B: three or four rounds) alternate between two side streams, so that
    # the partial last round of one group's kernels is filled by the other's; more streams than two measured
    # slower (the launches then share L2 and the power budget three or four ways).  Large groups run one after
    # another on the caller's stream, where a second stream only costs L2 locality.  The reference reaches
    # the same goal by interleaving up to three generator tasks (dion/megabatch_base.py:193).
    _MEDIUM_GROUP_FLOP = 3e13   # below: two streams fill the tails
    _N_SIDE_STREAMS = 2

    @staticmethod
    def _group_flop(params: List[Tensor]) -> float:
        r, c = params[0].shape[-2], params[0].shape[-1]
        m, n = min(r, c), max(r, c)
        mats = len(params) * (params[0].numel() // (r * c))
        return mats * 5.0 * (4.0 * m * m * n + 2.0 * m ** 3)

    # One pool per device for the whole process, shared by every optimizer instance: the runtime maps streams
    # onto a handful of hardware queues in creation order, and two streams created by a later instance can
    # land on one queue, where they run in sequence (measured: the step of a second optimizer in the same
    # process at the sequential figure, 2.1 instead of 1.8 ms for GPT-small).
    _side_pools: dict = {}

    def _side_pool(self, device) -> List["torch.cuda.Stream"]:
        key = torch.device(device).index if torch.device(device).index is not None else torch.cuda.current_device()
        pool = OrthoOptimizer._side_pools.get(key)
        if pool is None:
            pool = [torch.cuda.Stream(device=device) for _ in range(self._N_SIDE_STREAMS)]
            OrthoOptimizer._side_pools[key] = pool
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

    # hand the orthogonalization its input as the producing kernel writes it (False: the arena in the
    # parameters' layout, normalised and transposed by passes of the orthogonalization call)
    prepared_input = True

    def _takes_prepared(self, n_mat: int, rows: int, cols: int, select_dim: int, k: int, flat3d: bool,
                        M: List[Tensor]) -> bool:
        """Dion2 / NorDion2: whether the ``k`` slices selected along ``select_dim`` of ``n_mat`` matrices of
        ``rows x cols`` go to a built-in orthogonalization as the gather kernel writes them."""
        if not self.prepared_input or flat3d or self._custom_ns:
            return False
        if ops.dion2_prepared_blocks(rows, cols, select_dim, k) == 0:
            return False
        sr, sc = (k, cols) if select_dim == -2 else (rows, k)
        return ns.accepts_prepared(self._newton_schulz_func, n_mat, sr, sc) and \
            all(m.data_ptr() % 16 == 0 for m in M)

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
