"""Muon, NorMuon, Dion2 and NorDion2 with the constructor / param-group / step() / state_dict()
contract of microsoft/dion (dion/muon.py:20-110, dion/normuon.py:20-133, dion/dion2.py:19-127,
dion/nordion2.py:26-136), executing on the hand-written gfx950 kernels.

Per shape group (all parameters of one shape and dtype) a step is:
  Muon     muon_pre -> orthogonalize + update (one call; the last GEMM applies the update)
  NorMuon  muon_pre -> orthogonalize -> normuon_stats -> muon_post(row_scale)
  Dion2    dion2_select -> orthogonalize(selected slices) -> dion2_post
  NorDion2 dion2_select(rows) -> orthogonalize -> normuon_stats_selected -> dion2_post(row_scale)
where the orthogonalization input/output is one dense bf16 arena ``[N, *shape]`` written and read
directly by the fused kernels (the reference stacks and unbinds lists of tensors around it,
dion/megabatch_base.py:870-881).
"""
import math
from typing import Callable, List, Optional, Tuple, Union

import torch
from torch import Tensor

from . import global_scope, ops
from . import newton_schulz as ns
from .optim_base import OrthoOptimizer, adjust_lr_ratio, split_lr_scales


def _check_common(lr, betas, adjust_lr):
    if lr < 0.0:
        raise ValueError(f"Invalid learning rate: {lr}")
    if len(betas) != 2 or betas[0] < 0.0 or betas[1] < 0.0:
        raise ValueError(f"Invalid betas: {betas}")
    if adjust_lr not in ("spectral_norm", "rms_norm", None):
        raise ValueError(
            f"Invalid adjust_lr value: {adjust_lr}. Must be 'spectral_norm', 'rms_norm', or None."
        )


def _note_stream(t: Tensor) -> None:
    """A tensor produced on one stream is about to be consumed on the current one: tell the caching
    allocator so the block is not recycled under the consumer."""
    if t.is_cuda:
        t.record_stream(torch.cuda.current_stream(t.device))


def _require_state_dtype(params: List[Tensor], who: str) -> None:
    """Parameters (and with them momentum / second moments, dion/megabatch_base.py:198-203) are kept in
    float32 or bfloat16; the kernels compute in fp32 and round a bf16 value once, on store."""
    if params[0].dtype not in (torch.float32, torch.bfloat16):
        raise NotImplementedError(
            f"{who}: the gfx950 step kernels keep parameters and optimizer state in float32 or bfloat16; "
            f"got parameter dtype {params[0].dtype}"
        )


class _MomentumOrtho(OrthoOptimizer):
    """Shared Muon / NorMuon shape-group update (dion/muon.py:194-280, dion/normuon.py:222-341)."""

    _normalize = False
    # Muon only: run orthogonalization and update as one library call (False: the two-call sequence)
    fused_update = True

    def _shape_group_phases(self, group: dict, params: List[Tensor]):
        """Generator: [momentum / cast] yield [orthogonalization GEMMs] yield [normalise / update]."""
        num_heads = self._resolve_num_heads(group)
        split_sizes = self._resolve_split_sizes(group)
        shape = params[0].shape
        flatten = group["flatten"]
        split_scales = None
        if split_sizes is not None:
            self._validate_split_shape(split_sizes, shape)
            split_scales = split_lr_scales(split_sizes, shape, group["adjust_lr"])
        if num_heads is not None:
            mats, rows, cols = self._head_geometry(num_heads, shape)
            ratio_shape = (mats, rows, cols)  # the per-head 3D view decides the lr adjustment
        else:
            rows, cols = shape[-2], shape[-1]
            mats = params[0].numel() // (rows * cols)
            ratio_shape = shape
        _require_state_dtype(params, type(self).__name__)
        n = len(params)
        X = [p.data for p in params]
        G = [p.grad.contiguous() for p in params]
        states = [self._get_or_initialize_state(p, self._algo_name) for p in params]
        M = [s["momentum"] for s in states]
        eps = float(group["epsilon"])

        ratio = adjust_lr_ratio(ratio_shape, group["adjust_lr"], flatten)
        # Matrices that fill whole GEMM tiles reach the orthogonalization as the momentum kernel writes them:
        # short side along rows, unnormalised, with the partial sums of the Frobenius norm from the same pass
        # (no separate norm / scale / transpose pass over the arena; the factor rides on the first two GEMMs).
        flat3d = flatten and len(shape) >= 3
        prepared = (self.prepared_input and split_sizes is None and not flat3d and not self._custom_ns
                    and ns.accepts_prepared(self._newton_schulz_func, n * mats, rows, cols)
                    and all(t.data_ptr() % 16 == 0 for t in G + M))
        if prepared:
            U, sumsq = ops.muon_pre_prepared(G, M, group["mu"], group["nesterov"], mats, rows, cols)
            yield
            _note_stream(U)
            _note_stream(sumsq)
            func = self._newton_schulz_func
            if not self._normalize and self.fused_update:
                ns.orthogonalize_update_prepared(func, U, sumsq, rows, cols, eps, X, group["lr"], ratio,
                                                 group["weight_decay"], group["cautious_wd"])
                return
            O = ns.orthogonalize_prepared(func, U, sumsq, rows, cols, eps)
            del U, sumsq
            yield
            _note_stream(O)
            self._normalize_and_update(group, X, states, O, n, mats, rows, cols, ratio, None)
            return

        U = ops.muon_pre(G, M, group["mu"], group["nesterov"])  # [n, *shape] bf16
        yield
        _note_stream(U)

        if not self._normalize and split_sizes is None and self.fused_update:
            # Muon proper: the update consumes the orthogonalized matrices where the last GEMM
            # produces them (same result as the two calls below, bit for bit)
            Uv = U.view(n, shape[0], -1) if flatten and len(shape) >= 3 else U.view(n * mats, rows, cols)
            if self._orthogonalize_update(Uv, eps, X, group["lr"], ratio, group["weight_decay"],
                                          group["cautious_wd"]):
                return

        # shape plumbing of muon_update_newton_schulz (dion/megabatch_base.py:884-908)
        if split_sizes is not None:
            O = self._orthogonalize_row_blocks(U, split_sizes, split_scales, eps).contiguous()
        elif flatten and len(shape) >= 3:
            O = self._orthogonalize(U.view(n, shape[0], -1), eps)
        else:
            O = self._orthogonalize(U.view(n * mats, rows, cols), eps)

        del U
        yield
        _note_stream(O)
        self._normalize_and_update(group, X, states, O, n, mats, rows, cols, ratio, split_sizes)

    def _normalize_and_update(self, group, X, states, O, n, mats, rows, cols, ratio, split_sizes) -> None:
        """NorMuon's neuron-wise normalisation (when this class normalises) and the update pass."""
        row_scale = None
        if self._normalize:
            V = [s["variance_neuron"] for s in states]
            O3 = O.view(n, mats, rows, cols)
            if split_sizes is not None:
                # per-block Frobenius-preserving rescale (dion/normuon.py:359-369)
                scales, off = [], 0
                for sz in split_sizes:
                    blk = O3[:, :, off:off + sz, :].contiguous()
                    vb = [v[off:off + sz] for v in V]
                    scales.append(ops.normuon_stats(blk, vb, group["muon_beta2"]).view(n, sz))
                    off += sz
                row_scale = torch.cat(scales, dim=1).contiguous()
            else:
                row_scale = ops.normuon_stats(O3, V, group["muon_beta2"])
        ops.muon_post(X, O.view(n, -1), group["lr"], ratio, group["weight_decay"],
                      group["cautious_wd"], row_scale=row_scale)


class Muon(_MomentumOrtho):
    """Muon on one MI355X.  Same arguments as the reference ``Muon`` (dion/muon.py:61-78);
    ``distributed_mesh`` must be None and ``use_triton`` selects nothing.

    ``flatten=True`` updates every parameter with three or more dimensions as its own
    ``[shape[0], prod(shape[1:])]`` matrix, as the reference documents it (dion/muon.py:42-44).  The
    reference's batched code path flattens the stack of same-shape parameters instead
    (dion/megabatch_base.py:903-904), which orthogonalizes one ``N x numel`` matrix across the N
    parameters of a shape group; results for such groups therefore differ from the reference's."""

    def __init__(self, params, distributed_mesh=None, lr: float = 0.01, mu: float = 0.95,
                 betas: Tuple[float, float] = (0.9, 0.95), weight_decay: Union[float, Tensor] = 0.01,
                 cautious_wd: bool = False, epsilon: float = 1e-8, nesterov: bool = False,
                 adjust_lr: Optional[str] = "spectral_norm", flatten: bool = False,
                 use_gram_newton_schulz: bool = False, use_triton: bool = False,
                 use_polar_express: bool = True, newton_schulz_func: Optional[Callable] = None):
        _check_common(lr, betas, adjust_lr)
        if mu < 0.0:
            raise ValueError(f"Invalid momentum factor (mu): {mu}")
        defaults = dict(lr=lr, mu=mu, beta1=betas[0], beta2=betas[1], weight_decay=weight_decay,
                        cautious_wd=cautious_wd, algorithm="muon", step=0, epsilon=epsilon,
                        nesterov=nesterov, flatten=flatten, adjust_lr=adjust_lr)
        super().__init__(params, distributed_mesh, "muon", defaults,
                         use_gram_newton_schulz=use_gram_newton_schulz, use_triton=use_triton,
                         use_polar_express=use_polar_express, newton_schulz_func=newton_schulz_func)


class NorMuon(_MomentumOrtho):
    """NorMuon on one MI355X.  Same arguments as the reference ``NorMuon``
    (dion/normuon.py:64-82); adds the ``variance_neuron`` state (dion/normuon.py:119-123)."""

    _normalize = True

    def __init__(self, params, distributed_mesh=None, lr: float = 0.01, mu: float = 0.95,
                 muon_beta2: float = 0.95, betas: Tuple[float, float] = (0.9, 0.95),
                 weight_decay: Union[float, Tensor] = 0.01, cautious_wd: bool = False,
                 epsilon: float = 1e-8, nesterov: bool = False,
                 adjust_lr: Optional[str] = "spectral_norm", flatten: bool = False,
                 use_gram_newton_schulz: bool = False, use_triton: bool = False,
                 use_polar_express: bool = True, newton_schulz_func: Optional[Callable] = None):
        _check_common(lr, betas, adjust_lr)
        if mu < 0.0:
            raise ValueError(f"Invalid momentum factor (mu): {mu}")
        if muon_beta2 < 0.0:
            raise ValueError(f"Invalid muon_beta2: {muon_beta2}")
        defaults = dict(lr=lr, mu=mu, muon_beta2=muon_beta2, beta1=betas[0], beta2=betas[1],
                        weight_decay=weight_decay, cautious_wd=cautious_wd, algorithm="normuon",
                        step=0, epsilon=epsilon, nesterov=nesterov, flatten=flatten,
                        adjust_lr=adjust_lr)
        super().__init__(params, distributed_mesh, "normuon", defaults,
                         use_gram_newton_schulz=use_gram_newton_schulz, use_triton=use_triton,
                         use_polar_express=use_polar_express, newton_schulz_func=newton_schulz_func)

    def _get_or_initialize_state(self, param: Tensor, algo: str) -> dict:
        state = super()._get_or_initialize_state(param, algo)
        if algo == self._algo_name and "variance_neuron" not in state:
            state["variance_neuron"] = torch.zeros_like(param[..., 0:1])
        return state


class Dion2(OrthoOptimizer):
    """Dion2 on one MI355X.  Same arguments as the reference ``Dion2`` (dion/dion2.py:60-79).
    ``triton_post_ortho`` is accepted and selects nothing (the fused single-rounding post kernel is
    the only one).  ``selection_scope="global"`` changes the sequence only for sharded parameters in
    the reference (dion/dion2.py:284); with whole matrices it is the index-based sequence unless
    ``assembled_selection`` is set, in which case the step runs what a rank runs on assembled
    matrices: accumulate, select inside the orthogonalization call, masked update."""

    _printed = set()
    assembled_selection = False

    def __init__(self, params, distributed_mesh=None, lr: float = 0.01, fraction: float = 0.25,
                 ef_decay: float = 0.95, betas: Tuple[float, float] = (0.9, 0.95),
                 weight_decay: Union[float, Tensor] = 0.01, epsilon: float = 1e-8,
                 adjust_lr: Optional[str] = "spectral_norm", flatten: bool = False,
                 use_triton: bool = False, use_polar_express: bool = True,
                 use_gram_newton_schulz: bool = False, newton_schulz_func: Optional[Callable] = None,
                 verbose: bool = False, triton_post_ortho: bool = False, selection_scope: str = "local"):
        if lr < 0.0:
            raise ValueError(f"Invalid learning rate: {lr}")
        if not (0.0 < fraction <= 1.0):
            raise ValueError(f"fraction must be in (0, 1], got {fraction}")
        if selection_scope not in ("local", "global"):
            raise ValueError(f"selection_scope must be 'local' or 'global', got {selection_scope!r}")
        if ef_decay < 0.0:
            raise ValueError(f"Invalid ef_decay: {ef_decay}")
        _check_common(lr, betas, adjust_lr)
        defaults = dict(lr=lr, ef_decay=ef_decay, fraction=float(fraction), beta1=betas[0], beta2=betas[1],
                        weight_decay=weight_decay, epsilon=epsilon, flatten=flatten, adjust_lr=adjust_lr,
                        algorithm="dion2", step=0, selection_scope=selection_scope)
        super().__init__(params, distributed_mesh, "dion2", defaults,
                         use_gram_newton_schulz=use_gram_newton_schulz, use_triton=use_triton,
                         use_polar_express=use_polar_express, newton_schulz_func=newton_schulz_func)
        self.verbose = verbose
        self._triton_post_ortho = bool(triton_post_ortho)

    def _shape_group_phases(self, group: dict, params: List[Tensor]):
        """Generator: [accumulate / select / gather] yield [orthogonalization] yield [update]."""
        num_heads = self._resolve_num_heads(group)
        if group.get("split_sizes") is not None:
            raise NotImplementedError("split_sizes is currently supported only by Muon and NorMuon.")
        shape = params[0].shape
        flatten = group["flatten"]
        if num_heads is not None:
            mats, rows, cols = self._head_geometry(num_heads, shape)
            ratio_shape = (mats, rows, cols)
        else:
            rows, cols = shape[-2], shape[-1]
            mats = params[0].numel() // (rows * cols)
            ratio_shape = shape
        _require_state_dtype(params, "Dion2")
        n = len(params)
        # unsharded: select along the shorter dimension (dion/dion2.py:270-272)
        select_dim = -2 if rows <= cols else -1
        dim = rows if select_dim == -2 else cols
        k = min(max(1, int(math.ceil(group["fraction"] * dim))), dim)
        if self.verbose:
            key = (tuple(shape), select_dim)
            if key not in Dion2._printed:
                Dion2._printed.add(key)
                what = "rows" if select_dim == -2 else "columns"
                print(f"[Dion2] Shape {tuple(shape)}: single GPU, shorter dim ({dim}) -> "
                      f"select top-{k} {what} by L1 norm")

        X = [p.data.view(mats, rows, cols) for p in params]
        G = [p.grad.contiguous().view(mats, rows, cols) for p in params]
        M = [self._get_or_initialize_state(p, self._algo_name)["momentum"].view(mats, rows, cols)
             for p in params]

        if self.assembled_selection and group["selection_scope"] == "global":
            if flatten and len(shape) >= 3:
                raise NotImplementedError("Dion2: whole-matrix selection with flatten=True is built for "
                                          "2D parameters only.")
            # accumulate -> select inside the orthogonalization call -> masked update
            # (dion/dion2.py:301-343)
            U_full = global_scope.dion2_pre_accumulate(G, M)
            yield
            _note_stream(U_full)
            select_ns = global_scope.make_select_and_orthogonalize(
                lambda t, epsilon=None: self._orthogonalize(t, float(epsilon)), group["fraction"], select_dim)
            O = select_ns(U_full.view(n * mats, rows, cols), epsilon=float(group["epsilon"]))
            del U_full
            yield
            _note_stream(O)
            ratio = adjust_lr_ratio(ratio_shape, group["adjust_lr"], flatten)
            global_scope.dion2_post_orthogonalize_masked(X, M, O.view(n, mats, rows, cols), group["lr"], ratio,
                                                         group["weight_decay"], group["ef_decay"], select_dim)
            return

        eps = float(group["epsilon"])
        sel_rows, sel_cols = (k, cols) if select_dim == -2 else (rows, k)
        if self._takes_prepared(n * mats, rows, cols, select_dim, k, flatten and len(shape) >= 3, M):
            # the gather writes the selected blocks the way the iteration carries them, with the partial sums
            # of their Frobenius norms (no norm / scale / transpose pass inside the orthogonalization call)
            U_sel, _idx, imap, sumsq = ops.dion2_select(G, M, k, select_dim, group["ef_decay"], prepared=True)
            yield
            _note_stream(U_sel)
            _note_stream(sumsq)
            O = ns.orthogonalize_prepared(self._newton_schulz_func, U_sel, sumsq, sel_rows, sel_cols, eps)
            del U_sel, sumsq
            yield
            _note_stream(O)
            ratio = adjust_lr_ratio(ratio_shape, group["adjust_lr"], flatten)
            ops.dion2_post(X, O.view(n, mats, sel_rows, sel_cols), imap, group["lr"], ratio,
                           group["weight_decay"], select_dim)
            return
        U_sel, _idx, imap = ops.dion2_select(G, M, k, select_dim, group["ef_decay"])
        yield
        _note_stream(U_sel)
        if flatten and len(shape) >= 3:
            # leading dim stays, the rest of the selected block is one long row
            # (dion/megabatch_base.py:903-904)
            lead = shape[0]
            O = self._orthogonalize(U_sel.view(n, lead, -1), eps)
        else:
            O = self._orthogonalize(U_sel.view(n * mats, sel_rows, sel_cols), eps)
        del U_sel
        yield
        _note_stream(O)
        ratio = adjust_lr_ratio(ratio_shape, group["adjust_lr"], flatten)
        ops.dion2_post(X, O.view(n, mats, sel_rows, sel_cols), imap, group["lr"], ratio,
                       group["weight_decay"], select_dim)


class NorDion2(OrthoOptimizer):
    """NorDion2 ("Dion2 update applied to NorMuon") on one MI355X.  Same arguments as the reference
    ``NorDion2`` (dion/nordion2.py:67-86).  Per shape group (dion/nordion2.py:233-428, unsharded
    branch): ``M += G``; the ``ceil(fraction * rows)`` rows of largest L1 norm are selected (always
    rows, so that a selected slice is a whole neuron); those rows of ``M`` decay by ``mu``; the
    selected block is orthogonalized; NorMuon's per-row second-moment normalisation runs on it
    against the selected entries of ``variance_neuron``; the scaled rows update ``X``.
    ``assembled_selection`` as for ``Dion2``.  ``flatten=True`` on a parameter with three or more dimensions
    orthogonalizes its selected block as one ``[shape[0], -1]`` matrix per parameter (the reference's batched
    path flattens across the stack of same-shape parameters, dion/megabatch_base.py:903-904); selection and
    the per-neuron normalisation are those of the unflattened layout."""

    assembled_selection = False

    def __init__(self, params, distributed_mesh=None, lr: float = 0.01, fraction: float = 0.25,
                 mu: float = 0.95, muon_beta2: float = 0.95, betas: Tuple[float, float] = (0.9, 0.95),
                 weight_decay: Union[float, Tensor] = 0.01, epsilon: float = 1e-8,
                 adjust_lr: Optional[str] = "spectral_norm", flatten: bool = False,
                 use_triton: bool = False, use_polar_express: bool = True,
                 use_gram_newton_schulz: bool = False, newton_schulz_func: Optional[Callable] = None,
                 triton_post_ortho: bool = False, selection_scope: str = "local"):
        if lr < 0.0:
            raise ValueError(f"Invalid learning rate: {lr}")
        if not (0.0 < fraction <= 1.0):
            raise ValueError(f"fraction must be in (0, 1], got {fraction}")
        if selection_scope not in ("local", "global"):
            raise ValueError(f"selection_scope must be 'local' or 'global', got {selection_scope!r}")
        if mu < 0.0:
            raise ValueError(f"Invalid momentum factor (mu): {mu}")
        if muon_beta2 < 0.0:
            raise ValueError(f"Invalid muon_beta2: {muon_beta2}")
        _check_common(lr, betas, adjust_lr)
        defaults = dict(lr=lr, fraction=float(fraction), mu=mu, muon_beta2=muon_beta2, beta1=betas[0],
                        beta2=betas[1], weight_decay=weight_decay, epsilon=epsilon, flatten=flatten,
                        adjust_lr=adjust_lr, algorithm="nordion2", step=0, selection_scope=selection_scope)
        super().__init__(params, distributed_mesh, "nordion2", defaults,
                         use_gram_newton_schulz=use_gram_newton_schulz, use_triton=use_triton,
                         use_polar_express=use_polar_express, newton_schulz_func=newton_schulz_func)
        self._triton_post_ortho = bool(triton_post_ortho)

    def _get_or_initialize_state(self, param: Tensor, algo: str) -> dict:
        state = super()._get_or_initialize_state(param, algo)
        if algo == self._algo_name and "variance_neuron" not in state:
            state["variance_neuron"] = torch.zeros_like(param[..., 0:1])
        return state

    def _shape_group_phases(self, group: dict, params: List[Tensor]):
        """Generator: [accumulate / select rows / gather] yield [orthogonalization] yield
        [normalise selected rows / update]."""
        num_heads = self._resolve_num_heads(group)
        if group.get("split_sizes") is not None:
            raise NotImplementedError("split_sizes is currently supported only by Muon and NorMuon.")
        shape = params[0].shape
        flatten = group["flatten"]
        if num_heads is not None:
            mats, rows, cols = self._head_geometry(num_heads, shape)
            ratio_shape = (mats, rows, cols)
        else:
            rows, cols = shape[-2], shape[-1]
            mats = params[0].numel() // (rows * cols)
            ratio_shape = shape
        _require_state_dtype(params, "NorDion2")
        n = len(params)
        select_dim = -2  # whole rows, so the per-neuron normalisation sees complete neurons
        k = min(max(1, int(math.ceil(group["fraction"] * rows))), rows)
        X = [p.data.view(mats, rows, cols) for p in params]
        G = [p.grad.contiguous().view(mats, rows, cols) for p in params]
        states = [self._get_or_initialize_state(p, self._algo_name) for p in params]
        M = [s["momentum"].view(mats, rows, cols) for s in states]
        V = [s["variance_neuron"].view(mats, rows, 1) for s in states]

        if self.assembled_selection and group["selection_scope"] == "global":
            if flatten and len(shape) >= 3:
                raise NotImplementedError("NorDion2: whole-matrix selection with flatten=True is built for "
                                          "2D parameters only.")
            # accumulate -> select inside the orthogonalization call -> masked normalisation and update
            # (dion/nordion2.py:291-335)
            U_full = global_scope.dion2_pre_accumulate(G, M)
            yield
            _note_stream(U_full)
            select_ns = global_scope.make_select_and_orthogonalize(
                lambda t, epsilon=None: self._orthogonalize(t, float(epsilon)), group["fraction"], select_dim)
            O = select_ns(U_full.view(n * mats, rows, cols), epsilon=float(group["epsilon"]))
            del U_full
            yield
            _note_stream(O)
            ratio = adjust_lr_ratio(ratio_shape, group["adjust_lr"], flatten)
            global_scope.nordion2_post_orthogonalize_masked(
                X, M, V, O.view(n, mats, rows, cols), group["lr"], ratio, group["weight_decay"], group["mu"],
                group["muon_beta2"], select_dim)
            return

        # error-feedback decay of the selected rows is the momentum factor (dion/nordion2.py:352-359)
        eps = float(group["epsilon"])
        flat3d = flatten and len(shape) >= 3
        if self._takes_prepared(n * mats, rows, cols, select_dim, k, flat3d, M):
            U_sel, idx, imap, sumsq = ops.dion2_select(G, M, k, select_dim, group["mu"], prepared=True)
            yield
            _note_stream(U_sel)
            _note_stream(sumsq)
            O = ns.orthogonalize_prepared(self._newton_schulz_func, U_sel, sumsq, k, cols, eps)
            del sumsq
        else:
            U_sel, idx, imap = ops.dion2_select(G, M, k, select_dim, group["mu"])
            yield
            _note_stream(U_sel)
            if flat3d:
                # leading dim stays, the selected rows of all the other dims form one long row (per parameter,
                # as in Muon and Dion2 here; dion/megabatch_base.py:903-904 flattens the stack instead)
                O = self._orthogonalize(U_sel.view(n, shape[0], -1), eps)
            else:
                O = self._orthogonalize(U_sel.view(n * mats, k, cols), eps)
        del U_sel
        yield
        _note_stream(O)
        O4 = O.view(n, mats, k, cols)
        row_scale = ops.normuon_stats_selected(O4, V, idx, group["muon_beta2"])
        ratio = adjust_lr_ratio(ratio_shape, group["adjust_lr"], flatten)
        ops.dion2_post(X, O4, imap, group["lr"], ratio, group["weight_decay"], select_dim,
                       row_scale=row_scale)


Dion3 = NorDion2  # the reference exports the same class under both names (dion/__init__.py:9-10)
