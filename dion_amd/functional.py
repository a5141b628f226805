"""The reference's list-of-tensors operator functions, same names and call signatures, over the HIP
kernels: what its tests and callers import from ``dion.dion2``, ``dion.dion2_triton`` and
``dion.scalar_opts``.  Each is a thin host adapter; the arithmetic is in the kernels.
"""
import math
from typing import List, Optional, Tuple, Union

import torch
from torch import Tensor

from . import ops

Scalar = Union[float, Tensor]


def _host_float(v: Scalar) -> float:
    return float(v)


def _device_scalar(v: Scalar, device) -> Tensor:
    """0-d fp32 device tensor holding ``v`` (a tensor already there is passed through)."""
    if isinstance(v, Tensor) and v.is_cuda and v.dtype == torch.float32 and v.numel() == 1:
        return v
    return torch.full((), float(v), dtype=torch.float32, device=device)


def _same_shape(ts: List[Tensor], name: str) -> None:
    for t in ts:
        if t.shape != ts[0].shape or t.dtype != ts[0].dtype:
            raise ValueError(f"{name}: all tensors of one call must share shape and dtype")


def dion2_pre_orthogonalize(G: List[Tensor], M: List[Tensor], fraction: Scalar, ef_decay: Scalar, select_dim: int,
                            k_override: Optional[int] = None) -> Tuple[List[Tensor], List[Tensor]]:
    """``M += G``; top-k slices of every ``M[i]`` by L1 norm along ``select_dim``; those slices decay by
    ``ef_decay``.  Returns (list of bf16 selected blocks, list of int64 index tensors ``[*leading, k]``,
    ascending).  Same call as dion/dion2.py:439-547; ``k_override`` forces the count (clamped to what
    the matrix holds)."""
    if select_dim not in (-2, -1):
        raise ValueError(f"select_dim must be -2 or -1, got {select_dim}")
    _same_shape(M, "M")
    num_select = M[0].size(select_dim)
    k = int(k_override) if k_override is not None else max(1, int(math.ceil(_host_float(fraction) * num_select)))
    k = min(k, num_select)
    if M[0].numel() == 0 or k == 0:  # empty shard: nothing selected (dion/dion2.py:501-504)
        shape = list(M[0].shape)
        shape[select_dim] = 0
        dev = M[0].device
        return ([torch.empty(shape, dtype=torch.bfloat16, device=dev) for _ in M],
                [torch.empty((*shape[:-2], 0), dtype=torch.int64, device=dev) for _ in M])
    U, idx, _imap = ops.dion2_select([g.contiguous() for g in G], M, k, select_dim, _host_float(ef_decay))
    lead = M[0].shape[:-2]
    idx64 = idx.view(len(M), *lead, k).long()
    return list(U.unbind(0)), list(idx64.unbind(0))


def dion2_post_orthogonalize_triton(X: List[Tensor], U: List[Tensor], indices: List[Tensor], base_lr: Tensor,
                                    adjusted_lr: Tensor, weight_decay: Scalar, select_dim: int) -> None:
    """selected: ``x = (1 - base_lr*wd)*x - adjusted_lr*u``; unselected: ``x = (1 - base_lr*wd)*x``; one
    rounding.  Same call as dion/dion2_triton.py:147-155."""
    ops.dion2_post_orthogonalize_triton(X, U, indices, base_lr, adjusted_lr, weight_decay, select_dim)


# One kernel serves the three entry points of the reference (eager two-rounding form
# dion/dion2.py:666-697, single-rounding dion/dion2.py:701-740, Triton dion/dion2_triton.py:147-242);
# it has the numerics of the latter two.
dion2_post_orthogonalize = dion2_post_orthogonalize_triton
dion2_post_orthogonalize_fused = dion2_post_orthogonalize_triton


def _build_index_map(indices: Tensor, full_dim: int) -> Tensor:
    """dion/dion2_triton.py:30-47: ``[B, full_dim]`` int32, position of each listed slice, -1 elsewhere."""
    return ops.dion2_index_map(indices, full_dim)


def adamw_update_foreach(X: List[Tensor], G: List[Tensor], M: List[Tensor], V: List[Tensor], lr: Scalar,
                         beta1: Scalar, beta2: Scalar, weight_decay: Scalar, step: Optional[int] = None,
                         epsilon: float = 1e-8, cautious_wd: bool = False,
                         state_steps: Optional[List[Tensor]] = None) -> None:
    """Same call as dion/scalar_opts.py:121-134.  ``state_steps`` (per-parameter 0-d fp32 device counters,
    advanced on the device) or the legacy python-int ``step`` (the value to use for this update)."""
    if not X:
        return
    dev = X[0].device
    if state_steps is None:
        if step is None:
            raise ValueError("adamw_update_foreach needs step or state_steps")
        # the kernel advances its counter, then uses it; one counter serves a run of 48 tensors
        state_steps = []
        for i0 in range(0, len(X), 48):
            counter = torch.full((), float(int(step) - 1), dtype=torch.float32, device=dev)
            state_steps += [counter] * min(48, len(X) - i0)
    ops.adamw_step(X, [g.contiguous() for g in G], M, V, state_steps, _device_scalar(lr, dev), _host_float(beta1),
                   _host_float(beta2), weight_decay, float(epsilon), cautious_wd)


def lion_update_foreach(X: List[Tensor], G: List[Tensor], M: List[Tensor], lr: Scalar, beta1: Scalar, beta2: Scalar,
                        weight_decay: Scalar, cautious_wd: bool = False) -> None:
    """Same call as dion/scalar_opts.py:259-268."""
    if not X:
        return
    ops.lion_step(X, [g.contiguous() for g in G], M, _device_scalar(lr, X[0].device), _host_float(beta1),
                  _host_float(beta2), weight_decay, cautious_wd)
