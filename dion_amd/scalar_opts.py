"""AdamW / Lion for the non-matrix parameter groups (``algorithm="adamw"`` / ``"lion"``).

Kept so mixed param groups work as in the reference (dion/scalar_opts.py:7-118,
dion/megabatch_base.py:579-632); these element-wise rules are outside the orthogonalization hot
path and run on stock torch foreach ops.
"""
from typing import List

import torch
from torch import Tensor


def _wd_tensor(group: dict, like: Tensor) -> Tensor:
    wd = group["weight_decay"]
    return wd if isinstance(wd, Tensor) else torch.tensor(float(wd), dtype=torch.float32, device=like.device)


def _apply_weight_decay(X: List[Tensor], U: List[Tensor], lr: Tensor, wd: Tensor, cautious: bool) -> None:
    if cautious:
        coeff = lr * wd
        for x, u in zip(X, U):
            mask = (u * x >= 0).to(dtype=x.dtype)
            x.sub_((x * mask) * coeff)
    else:
        torch._foreach_mul_(X, 1 - lr * wd)


@torch.no_grad()
def lion_step(opt, group: dict) -> None:
    """U = sign(lerp(M, G, 1-beta1)); M = lerp(M, G, 1-beta2); X = X*(1-lr*wd) - lr*U
    (dion/scalar_opts.py:68-118)."""
    params = [p for p in group["params"] if p.grad is not None]
    if not params:
        return
    lr = group["lr"]
    wd = _wd_tensor(group, params[0])
    X = [p.data for p in params]
    M = [opt._get_or_initialize_state(p, "lion")["momentum"] for p in params]
    G = [p.grad.to(m.dtype) for p, m in zip(params, M)]
    U = [m.lerp(g, 1 - group["beta1"]).sign_() for m, g in zip(M, G)]
    for m, g in zip(M, G):
        m.lerp_(g, 1 - group["beta2"])
    _apply_weight_decay(X, U, lr, wd, group.get("cautious_wd", False))
    for x, u in zip(X, U):
        x.sub_(u * lr)


@torch.no_grad()
def adamw_step(opt, group: dict) -> None:
    """Bias-corrected AdamW with decoupled (optionally cautious) weight decay
    (dion/scalar_opts.py:7-65); the step counter lives on the device in ``step_dev``."""
    params = [p for p in group["params"] if p.grad is not None]
    if not params:
        return
    lr = group["lr"]
    wd = _wd_tensor(group, params[0])
    beta1, beta2, eps = group["beta1"], group["beta2"], group["epsilon"]
    for p in params:
        st = opt._get_or_initialize_state(p, "adamw")
        m, v, step = st["momentum"], st["variance"], st["step_dev"]
        g = p.grad.to(m.dtype)
        step.add_(1)
        m.lerp_(g, 1 - beta1)
        v.mul_(beta2).addcmul_(g, g, value=1 - beta2)
        bc1 = 1 - torch.pow(torch.tensor(beta1, device=p.device), step)
        bc2 = 1 - torch.pow(torch.tensor(beta2, device=p.device), step)
        denom = v.sqrt().div_(bc2.sqrt()).add_(eps)
        upd = m / denom
        _apply_weight_decay([p.data], [upd], lr, wd, group.get("cautious_wd", False))
        p.data.sub_(upd * (lr / bc1))
