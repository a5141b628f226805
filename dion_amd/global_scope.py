"""Whole-matrix selection for Dion2 / NorDion2: the sequence the reference runs per rank under
``selection_scope="global"`` once the shards of a matrix have been assembled.

Three steps, each a thin host function over HIP kernels:

* ``dion2_pre_accumulate`` -- ``M += G`` and the whole momentum in bf16 (dion/dion2.py:546-563);
* ``make_select_and_orthogonalize`` -- wraps an orthogonalization callable so that it picks the top-k
  slices of every matrix it is handed, orthogonalizes only those and returns a full-size tensor that
  is zero elsewhere (dion/dion2.py:565-620);
* ``dion2_post_orthogonalize_masked`` / ``nordion2_post_orthogonalize_masked`` -- the update that finds
  the selected slices again as the non-zero ones (dion/dion2.py:623-659, dion/nordion2.py:448-500).

With whole matrices on one GPU the reference never takes this route (local and global selection
coincide, dion/dion2.py:249-251); ``Dion2`` / ``NorDion2`` run it when their ``assembled_selection``
attribute is set, which is how it is tested against the index-based sequence.
"""
import math
from typing import Callable, List, Optional

import torch
from torch import Tensor

from . import ops


def dion2_pre_accumulate(G: List[Tensor], M: List[Tensor]) -> Tensor:
    """``M[i] += G[i]`` in place; returns the bf16 arena ``[N, *shape]`` of the updated momenta.  No
    selection and no error-feedback decay here (dion/dion2.py:546-563)."""
    # mu = 1 makes the momentum kernel's  mu*M + G  exactly  M + G
    return ops.muon_pre(G, M, 1.0, False)


def select_count(fraction: float, select_size: int, available: int) -> int:
    """``min(max(1, ceil(fraction * select_size)), available)`` (dion/dion2.py:596-601)."""
    return min(max(1, int(math.ceil(fraction * select_size))), available)


def make_select_and_orthogonalize(newton_schulz_func: Callable, fraction: float, select_dim: int,
                                  global_select_size: Optional[int] = None) -> Callable:
    """Returns ``select_ns(X, epsilon=None)``: top-k slices of every matrix of ``X [..., rows, cols]`` by L1
    norm along ``select_dim``, ``newton_schulz_func`` on the dense block of selected slices, result
    scattered into a zero tensor shaped like ``X``.  ``k`` derives from ``global_select_size`` (the true
    size of a matrix whose assembled form carries zero padding) when given, else from ``X`` itself,
    and never exceeds what ``X`` holds (dion/dion2.py:565-620)."""
    if select_dim not in (-2, -1):
        raise ValueError(f"select_dim must be -2 or -1, got {select_dim}")

    def select_ns(X: Tensor, epsilon=None) -> Tensor:
        have = X.size(select_dim)
        k = select_count(fraction, have if global_select_size is None else global_select_size, have)
        Xc = X if X.is_contiguous() else X.contiguous()
        sub, _idx, imap = ops.select_slices(Xc, k, select_dim)
        ortho = newton_schulz_func(sub, epsilon=epsilon)
        if ortho.shape != sub.shape:
            raise ValueError(
                f"newton_schulz_func returned shape {tuple(ortho.shape)} for input {tuple(sub.shape)}")
        ortho = ortho.to(X.dtype)
        if not ortho.is_contiguous():
            ortho = ortho.contiguous()
        return ops.scatter_slices(ortho, imap, X.shape, select_dim)

    return select_ns


def _arena(U, n: int) -> Tensor:
    if isinstance(U, (list, tuple)):
        U = torch.stack(list(U))
    if U.shape[0] != n:
        raise ValueError(f"U holds {U.shape[0]} tensors, expected {n}")
    return U if U.is_contiguous() else U.contiguous()


def dion2_post_orthogonalize_masked(X: List[Tensor], M: List[Tensor], U, base_lr: Tensor, adj_ratio: float,
                                    weight_decay, ef_decay: float, select_dim: int,
                                    adjusted_lr: Optional[Tensor] = None) -> None:
    """``X[i] <- (1 - lr*wd) X[i] - lr*adj_ratio*U[i]``; the slices of ``M[i]`` at which ``U[i]`` is not all
    zero decay by ``ef_decay``.  ``U``: bf16 arena ``[N, *shape]`` (or a list of N tensors), zero off the
    selected slices.  ``base_lr`` is the 0-d device tensor of the group, the adjusted rate is
    ``base_lr * adj_ratio``, or ``adjusted_lr * adj_ratio`` when that 0-d device tensor is given
    (dion/dion2.py:623-659)."""
    U = _arena(U, len(X))
    norms = ops.slice_l1(U, select_dim)
    ops.dion2_post_masked(X, M, U, norms, base_lr, adj_ratio, weight_decay, ef_decay, select_dim,
                          adjusted_lr=adjusted_lr)


def nordion2_post_orthogonalize_masked(X: List[Tensor], M: List[Tensor], V: List[Tensor], U, base_lr: Tensor,
                                       adj_ratio: float, weight_decay, ef_decay: float, muon_beta2: float,
                                       select_dim: int = -2, adjusted_lr: Optional[Tensor] = None) -> None:
    """As ``dion2_post_orthogonalize_masked`` with NorMuon's per-row normalisation in between: the second
    moments ``V[i] [..., rows, 1]`` are updated on the selected (non-zero) rows only and the Frobenius
    norm of the update is kept (dion/nordion2.py:448-500).  Rows only."""
    if select_dim != -2:
        raise ValueError(f"NorDion2 selects rows (select_dim == -2), got {select_dim}")
    U = _arena(U, len(X))
    norms = ops.slice_l1(U, -2)
    gate = ops.mask_index(norms)
    row_scale = ops.normuon_stats_selected(U, V, gate, muon_beta2)
    ops.dion2_post_masked(X, M, U, norms, base_lr, adj_ratio, weight_decay, ef_decay, -2, row_scale=row_scale,
                          adjusted_lr=adjusted_lr)
