"""The reference's list-of-tensors operator functions, same names and call signatures, over the HIP
kernels: what its tests and callers import from ``dion.muon``, ``dion.normuon``, ``dion.nordion2``,
``dion.dion2``, ``dion.dion2_triton`` and ``dion.scalar_opts``.  Each is a thin host adapter; the
arithmetic is in the kernels.
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


def muon_update_pre_orthogonalize(G: List[Tensor], M: List[Tensor], momentum: Scalar, nesterov: bool) -> List[Tensor]:
    """``M = momentum*M + G`` in place; returns the bf16 orthogonalization inputs (``M``, or
    ``momentum*M + G`` with Nesterov).  Same call as dion/muon.py:284-311; the returned tensors are views of
    one ``[N, *shape]`` arena."""
    if not G:
        return []
    _same_shape(M, "M")
    return list(ops.muon_pre([g.contiguous() for g in G], M, _host_float(momentum), bool(nesterov)).unbind(0))


def muon_update_post_orthogonalize(X: List[Tensor], U: List[Tensor], base_lr: Scalar, adjusted_lr: Scalar,
                                   weight_decay: Scalar, cautious_wd: bool = False) -> None:
    """Weight decay (plain or cautious) at ``base_lr``, then ``X -= adjusted_lr * U``.  Same call as
    dion/muon.py:315-347.  ``U`` bf16 or fp32; the list is gathered into one arena first (no copy when it
    already is the unbound arena ``muon_update_pre_orthogonalize`` / an orthogonalization returned)."""
    if not X:
        return
    dev = X[0].device
    arena = _as_arena(U)
    ops.muon_post(X, arena.view(len(X), -1), _device_scalar(base_lr, dev), 1.0, weight_decay, cautious_wd,
                  adjusted_lr=_device_scalar(adjusted_lr, dev))


def _as_arena(U: List[Tensor]) -> Tensor:
    """``[N, *shape]`` contiguous tensor holding ``U``: the tensors' own storage when they are the
    consecutive slices of one, a stacked copy otherwise."""
    u0 = U[0]
    if u0.dtype not in (torch.bfloat16, torch.float32):
        U = [u.float() for u in U]
        u0 = U[0]
    step = u0.numel() * u0.element_size()
    same = all(u.is_contiguous() and u.dtype == u0.dtype and u.shape == u0.shape
               and u.untyped_storage().data_ptr() == u0.untyped_storage().data_ptr()
               and u.data_ptr() == u0.data_ptr() + i * step for i, u in enumerate(U))
    if same:
        return u0.as_strided((len(U), *u0.shape), (u0.numel(), *u0.stride()))
    return torch.stack([u.contiguous() for u in U], dim=0)


def _normuon_block(U: Tensor, V: Tensor, beta2: float) -> Tuple[Tensor, Tensor]:
    """One ``[N, rows, cols]`` block against its ``[N, rows, 1]`` second moments (dion/normuon.py:375-399)."""
    v_new = V.contiguous().clone()
    scale = ops.normuon_stats(U.unsqueeze(0), [v_new.view(-1)], beta2)
    return ops.scale_rows(U, scale, V.dtype), v_new


def normuon_normalization_stacked(U: Tensor, V: Tensor, muon_beta2: Scalar,
                                  split_sizes: Optional[Tuple[int, ...]] = None) -> Tuple[Tensor, Tensor]:
    """NorMuon's per-row second-moment normalisation with the Frobenius-preserving rescale, out of place:
    ``U [N, rows, cols]`` (bf16, as the orthogonalization returns it), ``V [N, rows, 1]`` in the parameter
    dtype (fp32 or bf16).  Returns ``(normalized_U in the dtype of V, updated V)``.  With ``split_sizes``
    every row block is normalised on its own.  Same call as dion/normuon.py:344-373."""
    if U.dim() != 3 or V.shape != (U.shape[0], U.shape[1], 1):
        raise ValueError(f"expected U [N, rows, cols] and V [N, rows, 1], got {tuple(U.shape)} and {tuple(V.shape)}")
    if U.dtype != torch.bfloat16:
        raise TypeError(f"U must be bfloat16 (the orthogonalized update), got {U.dtype}")
    beta2 = _host_float(muon_beta2)
    if split_sizes is None:
        return _normuon_block(U.contiguous(), V, beta2)
    if sum(split_sizes) != U.shape[1]:
        raise ValueError(f"split_sizes {tuple(split_sizes)} do not add up to {U.shape[1]} rows")
    outs = [_normuon_block(u.contiguous(), v, beta2)
            for u, v in zip(U.split(list(split_sizes), dim=-2), V.split(list(split_sizes), dim=-2))]
    return torch.cat([o[0] for o in outs], dim=-2), torch.cat([o[1] for o in outs], dim=-2)


def nordion2_normalize_selected_stacked(U: Tensor, V_full: Tensor, indices: Tensor,
                                        muon_beta2: Scalar) -> Tuple[Tensor, Tensor]:
    """NorMuon normalisation of ``k`` selected rows per matrix: ``U [N, k, cols]`` bf16, ``V_full
    [N, rows, 1]`` (fp32 or bf16), ``indices [N, k]`` int64 distinct rows.  Only the selected entries of the
    second moments are read and updated.  Returns ``(normalized_U in float32, updated copy of V_full)``.
    Same call as dion/nordion2.py:430-447.  (With bf16 second moments the scale is computed from the
    stored, rounded values, as NorMuon's own bf16 path does, dion/normuon.py:376-392; the reference's
    selected-rows helper uses the unrounded fp32 values there, a difference of at most 2^-9 relative.)"""
    if U.dim() != 3 or V_full.dim() != 3 or V_full.shape[0] != U.shape[0] or V_full.shape[2] != 1:
        raise ValueError(f"expected U [N, k, cols] and V_full [N, rows, 1], got {tuple(U.shape)} and "
                         f"{tuple(V_full.shape)}")
    if U.dtype != torch.bfloat16:
        raise TypeError(f"U must be bfloat16 (the orthogonalized update), got {U.dtype}")
    if indices.shape != U.shape[:2]:
        raise ValueError(f"indices must be [N, k] = {tuple(U.shape[:2])}, got {tuple(indices.shape)}")
    v_new = V_full.contiguous().clone()
    U = U.contiguous()
    scale = ops.normuon_stats_selected(U.unsqueeze(0), [v_new.view(-1)], indices.to(torch.int32).contiguous(),
                                       _host_float(muon_beta2))
    return ops.scale_rows(U, scale, torch.float32), v_new


def lm_head_lr_scale(scalar_opt: str, model_dim: int) -> float:
    """Learning-rate scale of an lm_head trained by the scalar optimizer: ``1/sqrt(model_dim)`` for Lion,
    1 otherwise (dion/opt_utils.py:9-11)."""
    return 1 / math.sqrt(model_dim) if scalar_opt == "lion" else 1.0


def as_scalar_tensor(value: Scalar) -> Tensor:
    """A tensor passes through untouched (a live hyper-parameter must stay the same object); a number
    becomes a host scalar tensor (dion/opt_utils.py:14-23)."""
    return value if isinstance(value, Tensor) else torch.tensor(value)
