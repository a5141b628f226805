"""Orthogonalization operators with the reference's plug-point signature
``newton_schulz_func(input: Tensor, epsilon) -> Tensor`` (dion/muon.py:47-48).

All of them run the same hand-written gfx950 kernels; they differ only in the coefficient
table, the Frobenius safety factor and whether the Gram-matrix recurrence is used.
"""
from typing import Sequence, Tuple, Union

import torch
from torch import Tensor

from . import ops

# Quintic coefficient schedules (a, b, c), one triple per iteration.
# dion/newton_schulz_triton.py:500-506
NS5_COEFFS: Sequence[Tuple[float, float, float]] = (
    (4.0848, -6.8946, 2.9270),
    (3.9505, -6.3029, 2.6377),
    (3.7418, -5.5913, 2.3037),
    (2.8769, -3.1427, 1.2046),
    (2.8366, -3.0525, 1.2012),
)
# dion/polar_express.py:10-16 (safety factor 1.02 baked into all but the last polynomial)
POLAR_EXPRESS_COEFFS: Sequence[Tuple[float, float, float]] = (
    (8.156554524902461, -22.48329292557795, 15.878769915207462),
    (4.042929935166739, -2.808917465908714, 0.5000178451051316),
    (3.8916678022926607, -2.772484153217685, 0.5060648178503393),
    (3.285753657755655, -2.3681294933425376, 0.46449024233003106),
    (2.3465413258596377, -1.7097828382687081, 0.42323551169305323),
)
POLAR_EXPRESS_SAFETY = 1.02  # dion/polar_express.py:35
# dion/muon_reference.py:16 (Keller Jordan's fixed quintic)
KJ_COEFFS: Tuple[float, float, float] = (3.4445, -4.7750, 2.0315)


def _eps(epsilon: Union[float, Tensor, None], default: float) -> float:
    if epsilon is None:
        return default
    if isinstance(epsilon, Tensor):
        return float(epsilon)  # the optimizers pass a 0-d CPU tensor (dion/muon.py:133)
    return float(epsilon)


@torch.no_grad()
def zeropower_via_newtonschulz5(G: Tensor, epsilon: Union[float, Tensor] = 1e-7) -> Tensor:
    """NS5 schedule, ``X / (||X||_F + eps)``; same contract as
    dion/newton_schulz_triton.py:494-522 (bf16 output, shape of ``G``)."""
    return ops.ns_orthogonalize(G, NS5_COEFFS, 1.0, _eps(epsilon, 1e-7))


@torch.no_grad()
def polar_express(G: Tensor, epsilon: Union[float, Tensor] = 1e-6) -> Tensor:
    """Polar-Express schedule, ``X / (||X||_F * 1.02 + eps)``; same contract as
    dion/polar_express.py:20-50."""
    return ops.ns_orthogonalize(G, POLAR_EXPRESS_COEFFS, POLAR_EXPRESS_SAFETY, _eps(epsilon, 1e-6))


@torch.no_grad()
def gram_newton_schulz(G: Tensor, epsilon: Union[float, Tensor, None] = None) -> Tensor:
    """Gram-matrix recurrence with the Polar-Express schedule and a restart at iteration 2
    (how dion/megabatch_base.py:77-94 configures the external package; epsilon is ignored there)."""
    return ops.ns_orthogonalize(G, POLAR_EXPRESS_COEFFS, POLAR_EXPRESS_SAFETY, 0.0, gram=True, gram_reset=2)


@torch.no_grad()
def zeropower_kj(G: Tensor, steps: int = 5, eps: Union[float, Tensor] = 1e-7) -> Tensor:
    """Fixed-coefficient Newton-Schulz of the reference's un-batched Muon
    (``muon_reference.zeropower_via_newtonschulz5``, dion/muon_reference.py:11-27): ``steps``
    iterations of (3.4445, -4.7750, 2.0315) after ``X / (||X||_F + eps)``."""
    return ops.ns_orthogonalize(G, [KJ_COEFFS] * int(steps), 1.0, _eps(eps, 1e-7))


# What each built-in operator runs, as arguments of ``ops.ns_orthogonalize`` /
# ``ops.ns_orthogonalize_update``: (coeffs, norm_scale, default epsilon, gram, gram_reset).  A fixed
# epsilon of None means the caller's epsilon is ignored (the Gram form).
SCHEDULES = {
    zeropower_via_newtonschulz5: (NS5_COEFFS, 1.0, 1e-7, False, 0),
    polar_express: (POLAR_EXPRESS_COEFFS, POLAR_EXPRESS_SAFETY, 1e-6, False, 0),
    gram_newton_schulz: (POLAR_EXPRESS_COEFFS, POLAR_EXPRESS_SAFETY, None, True, 2),
}


@torch.no_grad()
def orthogonalize_update(func, G: Tensor, epsilon, X, lr: Tensor, adj_ratio: float, weight_decay,
                         cautious_wd: bool = False) -> None:
    """``ops.muon_post(X, func(G, epsilon), ...)`` for a built-in ``func`` (a key of ``SCHEDULES``), as one
    fused library call."""
    coeffs, norm_scale, default_eps, gram, reset = SCHEDULES[func]
    eps = 0.0 if default_eps is None else _eps(epsilon, default_eps)
    ops.ns_orthogonalize_update(G, X, coeffs, norm_scale, eps, lr, adj_ratio, weight_decay, cautious_wd,
                                gram=gram, gram_reset=reset)


def _schedule_args(func, epsilon):
    coeffs, norm_scale, default_eps, gram, reset = SCHEDULES[func]
    eps = 0.0 if default_eps is None else _eps(epsilon, default_eps)
    return coeffs, norm_scale, eps, gram, reset


def accepts_prepared(func, batch: int, rows: int, cols: int) -> bool:
    """True when the built-in operator ``func`` takes ``batch`` matrices of ``rows x cols`` in the prepared
    form (``ops.muon_pre_prepared``)."""
    if func not in SCHEDULES:
        return False
    coeffs, _s, _e, gram, _r = SCHEDULES[func]
    return ops.ns_accepts_prepared(batch, rows, cols, len(coeffs), gram)


@torch.no_grad()
def orthogonalize_prepared(func, U: Tensor, sumsq: Tensor, rows: int, cols: int, epsilon) -> Tensor:
    """``func(G, epsilon)`` for a built-in ``func`` on the prepared form of ``G``."""
    coeffs, norm_scale, eps, gram, reset = _schedule_args(func, epsilon)
    return ops.ns_orthogonalize_prepared(U, sumsq, rows, cols, coeffs, norm_scale, eps, gram=gram, gram_reset=reset)


@torch.no_grad()
def orthogonalize_update_prepared(func, U: Tensor, sumsq: Tensor, rows: int, cols: int, epsilon, X, lr: Tensor,
                                  adj_ratio: float, weight_decay, cautious_wd: bool = False) -> None:
    """``orthogonalize_update`` on the prepared form of ``G``."""
    coeffs, norm_scale, eps, gram, reset = _schedule_args(func, epsilon)
    ops.ns_orthogonalize_update_prepared(U, sumsq, rows, cols, X, coeffs, norm_scale, eps, lr, adj_ratio,
                                         weight_decay, cautious_wd, gram=gram, gram_reset=reset)


# The reference exposes Triton-backed twins of the two schedules; here there is one
# implementation, so the names resolve to it.
newton_schulz_triton = zeropower_via_newtonschulz5
polar_express_triton = polar_express

ns_line_1 = ops.ns_line_1
ns_line_2 = ops.ns_line_2
ns_line_3 = ops.ns_line_3
