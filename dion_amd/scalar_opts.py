"""AdamW / Lion for the non-matrix parameter groups (``algorithm="adamw"`` / ``"lion"``), as the
reference keeps them beside the orthogonalizing optimizers (dion/scalar_opts.py:7-325,
dion/megabatch_base.py:579-632): one multi-tensor HIP launch per gradient dtype covers every
parameter of the group, whatever its size.
"""
from collections import defaultdict

import torch

from . import ops


def _with_grad(group: dict):
    by_dtype = defaultdict(list)
    for p in group["params"]:
        if p.grad is not None:
            by_dtype[p.grad.dtype].append(p)
    return by_dtype


@torch.no_grad()
def lion_step(opt, group: dict) -> None:
    """U = sign(lerp(M, G, 1-beta1)); M = lerp(M, G, 1-beta2); X = X*(1-lr*wd) - lr*U
    (dion/scalar_opts.py:68-118)."""
    for params in _with_grad(group).values():
        X = [p.data for p in params]
        G = [p.grad.contiguous() for p in params]
        M = [opt._get_or_initialize_state(p, "lion")["momentum"] for p in params]
        ops.lion_step(X, G, M, group["lr"], group["beta1"], group["beta2"], group["weight_decay"],
                      group.get("cautious_wd", False))


@torch.no_grad()
def adamw_step(opt, group: dict) -> None:
    """Bias-corrected AdamW with decoupled (optionally cautious) weight decay
    (dion/scalar_opts.py:7-65); every parameter's step counter lives on the device in ``step_dev``
    and is advanced there."""
    for params in _with_grad(group).values():
        states = [opt._get_or_initialize_state(p, "adamw") for p in params]
        X = [p.data for p in params]
        G = [p.grad.contiguous() for p in params]
        ops.adamw_step(X, G, [s["momentum"] for s in states], [s["variance"] for s in states],
                       [s["step_dev"] for s in states], group["lr"], group["beta1"], group["beta2"],
                       group["weight_decay"], group["epsilon"], group.get("cautious_wd", False))
