"""CPU oracle for the Muon / NorMuon / Dion2 / NorDion2 optimizer-step hot path of microsoft/dion.

TEST INFRASTRUCTURE ONLY.  This module restates the reference's algorithms on the CPU (numpy
float64 for exact arithmetic, torch-CPU bfloat16/float32 for the rounding sequence of the eager
reference) so the HIP kernels can be checked against them.  Nothing under dion_amd/ imports it;
only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg do.

Each function cites the reference lines (paths relative to the reference tree) it follows.

Pinning status (what fixes each function besides re-reading the formula):
  * ns_bf16 / polar_express_bf16 / kj_ns_bf16: bit-equal to the outputs of the reference's own
    (undecorated) functions on the golden inputs of tests/golden/ns_vectors.npz; closed form on a
    constructed SVD; the orthogonality bound of the reference's own tests on their seeds and
    shapes.  ns_fp64: closed form on a constructed SVD (singular vectors preserved, singular
    values mapped by the scalar quintic composition), transpose and scale invariance, zero-row
    preservation, and both golden reference outputs (eager and torch.compile'd) within their bf16
    noise of it.  ns_bf16_fused is NOT a reference path: it is the "round after every matmul,
    fp32 inside a pointwise chain" sequence, kept as a third bf16 realisation; the compiled
    reference on the CPU keeps un-rounded fp32 values across ops and matches no such rule (its
    golden vectors are used directly instead).                   -> tests/test_oracle.py
  * muon_pre / muon_post: first-step closed forms (M == G, U == bf16((1+mu) G)), U == 0 decay
    only, brute-force cautious mask.                              -> tests/test_oracle.py
  * normuon_normalize: Frobenius norm preserved, first-step V == (1-beta2) mean(U^2),
    equal-row-energy input gives a multiple of U.                -> tests/test_oracle.py
  * dion2_pre / dion2_post: brute-force sort for the top-k set, fraction == 1 degenerate case,
    unselected entries exactly a*x.                               -> tests/test_oracle.py
  * nordion2_normalize_selected / nordion2_step: every-row selection reduces to normuon_normalize,
    unselected entries of V untouched, fraction == 1 and identity-orthogonalization closed
    forms.                                                        -> tests/test_oracle.py
  * dion2_pre_accumulate / select_and_orthogonalize / dion2_post_masked / nordion2_post_masked
    (the whole-matrix "global" selection sequence): the reference's own padded-matrix case
    (17 real + 3 zero rows, fraction 0.35 -> 6 selected, tests/test_dion2_selection_scope.py:138-169),
    brute-force top-k, and equality of the masked sequence with the index-based one (dion2_pre /
    dion2_post / nordion2_step, written separately) whenever both pick the same slices.
                                                                  -> tests/test_oracle.py
  * adamw_update / lion_update: the reference's hand-computed cautious-decay vector
    (tests/test_adamw_foreach.py:80-112), torch.optim.AdamW as an independent implementation,
    first-step and blended-sign closed forms for Lion.            -> tests/test_oracle.py
  * gram_ns_fp64: PARITY UNPINNED against the third-party gram-newton-schulz==0.1.6 package
    (not in the reference tree, not installed); pinned only by equality with ns_fp64 in exact
    arithmetic.
"""
from __future__ import annotations

import math
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch

# dion/newton_schulz_triton.py:500-506
NS5_COEFFS = [
    (4.0848, -6.8946, 2.9270),
    (3.9505, -6.3029, 2.6377),
    (3.7418, -5.5913, 2.3037),
    (2.8769, -3.1427, 1.2046),
    (2.8366, -3.0525, 1.2012),
]
# dion/polar_express.py:10-16
POLAR_EXPRESS_COEFFS = [
    (8.156554524902461, -22.48329292557795, 15.878769915207462),
    (4.042929935166739, -2.808917465908714, 0.5000178451051316),
    (3.8916678022926607, -2.772484153217685, 0.5060648178503393),
    (3.285753657755655, -2.3681294933425376, 0.46449024233003106),
    (2.3465413258596377, -1.7097828382687081, 0.42323551169305323),
]
# dion/muon_reference.py:16
KJ_COEFFS = [(3.4445, -4.7750, 2.0315)] * 5
POLAR_EXPRESS_SAFETY = 1.02  # dion/polar_express.py:35


def bf16_round(x: np.ndarray) -> np.ndarray:
    """Round float values to the nearest bfloat16 (ties to even), returned as float64."""
    t = torch.from_numpy(np.asarray(x, dtype=np.float32)).to(torch.bfloat16).to(torch.float32)
    return t.numpy().astype(np.float64)


def scalar_map(sigma: np.ndarray, coeffs: Sequence[Tuple[float, float, float]]) -> np.ndarray:
    """Composition of the quintics x -> a x + b x^3 + c x^5: what one NS run does to a singular
    value (dion/newton_schulz_triton.py:515-518 applied to a 1x1 matrix)."""
    x = np.asarray(sigma, dtype=np.float64).copy()
    for a, b, c in coeffs:
        x = a * x + b * x**3 + c * x**5
    return x


def ns_fp64(G: np.ndarray, coeffs, norm_scale: float = 1.0, eps: float = 1e-7,
            round_input: bool = True) -> np.ndarray:
    """Exact-arithmetic Newton-Schulz (dion/newton_schulz_triton.py:508-522,
    dion/polar_express.py:30-50).  Input is rounded to bf16 first as the reference does
    (``X = G.to(bfloat16)``); everything after is float64."""
    G = np.asarray(G, dtype=np.float64)
    X = bf16_round(G) if round_input else G.copy()
    tall = X.shape[-2] > X.shape[-1]
    if tall:
        X = np.swapaxes(X, -2, -1)
    nrm = np.sqrt((X * X).sum(axis=(-2, -1), keepdims=True))
    X = X / (nrm * norm_scale + eps)
    for a, b, c in coeffs:
        A = X @ np.swapaxes(X, -2, -1)
        B = b * A + c * (A @ A)
        X = a * X + B @ X
    if tall:
        X = np.swapaxes(X, -2, -1)
    return X


def gram_ns_fp64(G: np.ndarray, coeffs, norm_scale: float = POLAR_EXPRESS_SAFETY, eps: float = 0.0,
                 reset_iterations: Sequence[int] = (2,)) -> np.ndarray:
    """Gram-matrix form of the same iteration (call site dion/megabatch_base.py:77-94; the package
    itself is external).  Keeps R = X X^T and Q with X = Q X0; per iteration Z = a I + b R + c R^2,
    Q <- Z Q, R <- Z R Z; at a reset iteration X is materialised and R, Q restart."""
    G = np.asarray(G, dtype=np.float64)
    X = bf16_round(G)
    tall = X.shape[-2] > X.shape[-1]
    if tall:
        X = np.swapaxes(X, -2, -1)
    nrm = np.sqrt((X * X).sum(axis=(-2, -1), keepdims=True))
    X = X / (nrm * norm_scale + eps)
    m = X.shape[-2]
    eye = np.eye(m)
    R = X @ np.swapaxes(X, -2, -1)
    Q = np.broadcast_to(eye, R.shape).copy()
    for it, (a, b, c) in enumerate(coeffs):
        if it in reset_iterations and it > 0:
            X = Q @ X
            R = X @ np.swapaxes(X, -2, -1)
            Q = np.broadcast_to(eye, R.shape).copy()
        Z = a * eye + b * R + c * (R @ R)
        Q = Z @ Q
        R = Z @ R @ Z
    X = Q @ X
    if tall:
        X = np.swapaxes(X, -2, -1)
    return X


def ns_bf16(G: torch.Tensor, coeffs=NS5_COEFFS, norm_scale: float = 1.0, eps: float = 1e-7) -> torch.Tensor:
    """Eager torch-CPU restatement of ``zeropower_via_newtonschulz5``
    (dion/newton_schulz_triton.py:494-522): every op rounds to bf16, tall inputs are transposed."""
    X = G.to(torch.bfloat16)
    tall = G.size(-2) > G.size(-1)
    if tall:
        X = X.mT
    X = X / (X.norm(dim=(-2, -1), keepdim=True) * norm_scale + eps)
    for a, b, c in coeffs:
        A = X @ X.mT
        B = b * A + c * (A @ A)
        X = a * X + B @ X
    if tall:
        X = X.mT
    return X


def polar_express_bf16(G: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """Eager torch-CPU restatement of ``polar_express`` (dion/polar_express.py:20-50): tall inputs
    are not transposed, they use X^T X and a right multiply."""
    X = G.to(torch.bfloat16)
    tall = G.size(-2) > G.size(-1)
    X = X / (X.norm(dim=(-2, -1), keepdim=True) * POLAR_EXPRESS_SAFETY + eps)
    if tall:
        for a, b, c in POLAR_EXPRESS_COEFFS:
            A = X.mT @ X
            B = b * A + c * (A @ A)
            X = a * X + X @ B
    else:
        for a, b, c in POLAR_EXPRESS_COEFFS:
            A = X @ X.mT
            B = b * A + c * (A @ A)
            X = a * X + B @ X
    return X


def ns_bf16_fused(G: torch.Tensor, coeffs=NS5_COEFFS, norm_scale: float = 1.0, eps: float = 1e-7) -> torch.Tensor:
    """Same algorithm as ns_bf16 with fewer rounding points: every matmul result is rounded to bf16,
    each pointwise chain (normalisation, b*A + c*AA, a*X + BX) is evaluated in float32 and rounded
    once.  A third bf16 realisation of the iteration, not a reference path: the reference's
    torch.compile'd functions (dion/newton_schulz_triton.py:494, dion/polar_express.py:19) go through
    inductor, whose CPU code keeps un-rounded float32 values across ops (e.g. a*X is formed from
    the un-rounded quotient X/||X||), so the compiled output follows no fixed rounding rule and is
    represented by its golden vectors instead."""
    X = G.to(torch.bfloat16)
    tall = G.size(-2) > G.size(-1)
    if tall:
        X = X.mT
    nrm = X.float().pow(2).sum(dim=(-2, -1), keepdim=True).sqrt()
    X = (X.float() / (nrm * norm_scale + eps)).to(torch.bfloat16)
    for a, b, c in coeffs:
        A = X @ X.mT
        AA = A @ A
        B = (b * A.float() + c * AA.float()).to(torch.bfloat16)
        BX = B @ X
        X = (a * X.float() + BX.float()).to(torch.bfloat16)
    if tall:
        X = X.mT
    return X


def kj_ns_bf16(G: torch.Tensor, steps: int = 5, eps: float = 1e-7) -> torch.Tensor:
    """``muon_reference.zeropower_via_newtonschulz5`` (dion/muon_reference.py:11-27): 2-D only,
    normalised before transposing, fixed coefficients."""
    assert G.ndim == 2
    a, b, c = KJ_COEFFS[0]
    X = G.bfloat16()
    X = X / (X.norm() + eps)
    if G.size(0) > G.size(1):
        X = X.T
    for _ in range(steps):
        A = X @ X.T
        B = b * A + c * (A @ A)
        X = a * X + B @ X
    if G.size(0) > G.size(1):
        X = X.T
    return X


# ---------------------------------------------------------------------------------------------
# optimizer-step pieces (float32 torch on CPU, op order of the eager reference)
# ---------------------------------------------------------------------------------------------
def muon_pre(G: torch.Tensor, M: torch.Tensor, mu: float, nesterov: bool) -> Tuple[torch.Tensor, torch.Tensor]:
    """dion/muon.py:284-311.  Returns (M_new fp32, U bf16); does not modify its inputs."""
    g = G.to(M.dtype)
    mu_t = torch.tensor(mu, dtype=M.dtype)
    M_new = M * mu_t + g
    U = M_new * mu_t + g if nesterov else M_new
    return M_new, U.to(torch.bfloat16)


def adjust_lr_ratio(shape, adjust_lr: Optional[str], flatten: bool = False) -> float:
    """dion/megabatch_base.py:984-1002 with lr factored out."""
    if adjust_lr is None:
        return 1.0
    if flatten:
        fan_out, fan_in = shape[0], math.prod(shape[1:])
    else:
        fan_out, fan_in = shape[-2], shape[-1]
    if adjust_lr == "spectral_norm":
        return math.sqrt(fan_out / fan_in)
    if adjust_lr == "rms_norm":
        return 0.2 * math.sqrt(max(fan_out, fan_in))
    raise ValueError(f"Unknown adjust_lr value: {adjust_lr}")


def muon_post(X: torch.Tensor, U: torch.Tensor, lr: float, adj_ratio: float, wd: float,
              cautious: bool = False) -> torch.Tensor:
    """dion/muon.py:315-347 in float32 (the fused/compiled form: the product adjusted_lr*U is not
    rounded to U's dtype before the subtraction).  Returns the new X."""
    lr_t = torch.tensor(lr, dtype=torch.float32)
    wd_t = torch.tensor(wd, dtype=torch.float32)
    u = U.to(torch.float32)
    x = X.to(torch.float32)
    if cautious:
        coeff = lr_t * wd_t
        mask = torch.minimum(torch.sign(x * u) + 1, torch.tensor(1.0))
        x = x - (x * mask) * coeff
    else:
        x = x * (1 - lr_t * wd_t)
    b = lr_t * torch.tensor(adj_ratio, dtype=torch.float32)
    return x - u * b


def normuon_normalize(U: torch.Tensor, V: torch.Tensor, beta2: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """dion/normuon.py:374-399.  U [..., rows, cols], V [..., rows, 1]; returns (normalized U, new V)."""
    b2 = torch.tensor(beta2, dtype=torch.float32)
    U = U.to(V.dtype)
    norm_U = U.norm(p=2, dim=(-2, -1), keepdim=True)
    neuron = (U * U).mean(dim=-1, keepdim=True)
    V = torch.lerp(V, neuron, 1 - b2)
    denom = V.sqrt() + 1e-8
    nU = U / denom
    norm_new = nU.norm(p=2, dim=(-2, -1), keepdim=True).clamp(min=1e-8)
    return nU * (norm_U / norm_new), V


def dion2_k(fraction: float, dim: int) -> int:
    """dion/dion2.py:484."""
    return max(1, int(math.ceil(fraction * dim)))


def dion2_select_dim(rows: int, cols: int) -> int:
    """dion/dion2.py:270-272 (unsharded): the shorter dimension."""
    return -2 if rows <= cols else -1


def dion2_pre(G: torch.Tensor, M: torch.Tensor, fraction: float, ef_decay: float, select_dim: int):
    """dion/dion2.py:439-547 for one matrix.  Returns (M_new, U_sel bf16, sorted index tensor).
    Ties in the L1 norms go to the lower index (torch.topk leaves the order unspecified)."""
    M_new = M + G.to(M.dtype)
    dim = M_new.size(select_dim)
    k = min(dion2_k(fraction, dim), dim)
    norm_dim = -1 if select_dim == -2 else -2
    norms = M_new.norm(p=1, dim=norm_dim)
    order = sorted(range(dim), key=lambda i: (-float(norms[i]), i))
    idx = torch.tensor(sorted(order[:k]), dtype=torch.long)
    if select_dim == -2:
        sel = M_new[idx, :]
        M_new = M_new.clone()
        M_new[idx, :] = sel * torch.tensor(ef_decay, dtype=M.dtype)
    else:
        sel = M_new[:, idx]
        M_new = M_new.clone()
        M_new[:, idx] = sel * torch.tensor(ef_decay, dtype=M.dtype)
    return M_new, sel.to(torch.bfloat16), idx


def dion2_post(X: torch.Tensor, U: torch.Tensor, idx: torch.Tensor, lr: float, adj_ratio: float, wd: float,
               select_dim: int) -> torch.Tensor:
    """Single-rounding form (dion/dion2.py:701-740, dion/dion2_triton.py:141-142):
    selected x = a*x - b*u, unselected x = a*x."""
    lr_t = torch.tensor(lr, dtype=torch.float32)
    a = 1 - lr_t * torch.tensor(wd, dtype=torch.float32)
    b = lr_t * torch.tensor(adj_ratio, dtype=torch.float32)
    full = torch.zeros_like(X, dtype=torch.float64)
    if select_dim == -2:
        full[idx, :] = U.to(torch.float64)
    else:
        full[:, idx] = U.to(torch.float64)
    out = a.double() * X.double() - b.double() * full
    return out.to(torch.float32)


def dion2_pre_accumulate(G: torch.Tensor, M: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """dion/dion2.py:546-563 for one matrix: returns (M + G, its bf16 copy)."""
    M_new = M + G.to(M.dtype)
    return M_new, M_new.to(torch.bfloat16)


def select_and_orthogonalize(X: torch.Tensor, fraction: float, select_dim: int, ns,
                             global_select_size: Optional[int] = None):
    """dion/dion2.py:596-614 for one matrix X [rows, cols]: top-k slices by L1 norm (the norm of a
    bf16 tensor is itself bf16), ``ns`` on the dense block, scattered into zeros.  Ties go to the
    lower index.  Returns (full-size result in X.dtype, sorted index tensor)."""
    have = X.size(select_dim)
    num_select = have if global_select_size is None else global_select_size
    k = min(max(1, int(math.ceil(fraction * num_select))), have)
    norm_dim = -1 if select_dim == -2 else -2
    norms = X.float().abs().sum(dim=norm_dim).to(X.dtype)
    order = sorted(range(have), key=lambda i: (-float(norms[i]), i))
    idx = torch.tensor(sorted(order[:k]), dtype=torch.long)
    sub = X[idx, :] if select_dim == -2 else X[:, idx]
    ortho = ns(sub).to(X.dtype)
    out = torch.zeros_like(X)
    if select_dim == -2:
        out[idx, :] = ortho
    else:
        out[:, idx] = ortho
    return out, idx


def _nonzero_slices(U: torch.Tensor, select_dim: int) -> torch.Tensor:
    """dion/dion2.py:648: boolean mask, keepdim, over the slices of U that are not all zero."""
    norm_dim = -1 if select_dim == -2 else -2
    return U.to(torch.float32).abs().sum(dim=norm_dim, keepdim=True) > 0


def dion2_post_masked(X: torch.Tensor, M: torch.Tensor, U: torch.Tensor, lr: float, adj_ratio: float, wd: float,
                      ef_decay: float, select_dim: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """dion/dion2.py:623-659 for one matrix, the weight update in the single-rounding form of
    ``dion2_post``.  Returns (X_new, M_new)."""
    sel = _nonzero_slices(U, select_dim)
    M_new = M * torch.where(sel, torch.tensor(ef_decay, dtype=M.dtype), torch.ones((), dtype=M.dtype))
    lr_t = torch.tensor(lr, dtype=torch.float32)
    a = 1 - lr_t * torch.tensor(wd, dtype=torch.float32)
    b = lr_t * torch.tensor(adj_ratio, dtype=torch.float32)
    X_new = (a.double() * X.double() - b.double() * U.double()).to(torch.float32)
    return X_new, M_new


def nordion2_post_masked(X: torch.Tensor, M: torch.Tensor, V: torch.Tensor, U: torch.Tensor, lr: float,
                         adj_ratio: float, wd: float, ef_decay: float, beta2: float):
    """dion/nordion2.py:448-500 for one matrix (rows selected): NorMuon normalisation over the full,
    mostly-zero U; V written back on the non-zero rows only.  Returns (X_new, M_new, V_new)."""
    sel = _nonzero_slices(U, -2)
    M_new = M * torch.where(sel, torch.tensor(ef_decay, dtype=M.dtype), torch.ones((), dtype=M.dtype))
    nU, v_new = normuon_normalize(U, V.float(), beta2)
    V_new = torch.where(sel, v_new.to(V.dtype), V)
    lr_t = torch.tensor(lr, dtype=torch.float32)
    a = 1 - lr_t * torch.tensor(wd, dtype=torch.float32)
    b = lr_t * torch.tensor(adj_ratio, dtype=torch.float32)
    X_new = (a.double() * X.double() - b.double() * nU.double()).to(torch.float32)
    return X_new, M_new, V_new


def nordion2_normalize_selected(U: torch.Tensor, V_full: torch.Tensor, idx: torch.Tensor, beta2: float):
    """dion/nordion2.py:430-447 for one matrix: gather the selected rows of the full per-neuron
    variance buffer, run the NorMuon normalisation on them, scatter the new values back.
    U [k, cols], V_full [rows, 1], idx [k] (long).  Returns (normalized U, new V_full)."""
    V_sel = V_full[idx]
    nU, V_sel_new = normuon_normalize(U, V_sel, beta2)
    V_new = V_full.clone()
    V_new[idx] = V_sel_new.to(V_full.dtype)
    return nU, V_new


def nordion2_step(x: torch.Tensor, g: torch.Tensor, m: torch.Tensor, v: torch.Tensor, lr: float,
                  fraction: float, mu: float, beta2: float, wd: float, adjust_lr: Optional[str],
                  ns=None):
    """One NorDion2 step on one 2D parameter (dion/nordion2.py:233-428, unsharded branch): rows are
    always the selected dimension and the error-feedback decay is the momentum factor.
    ``ns`` maps the bf16 selected block to its orthogonalization (default: fused-rounding NS5)."""
    m2, u, idx = dion2_pre(g, m, fraction, mu, -2)
    o = ns(u) if ns is not None else ns_bf16_fused(u, NS5_COEFFS, 1.0, 1e-8)
    nU, v2 = nordion2_normalize_selected(o, v, idx, beta2)
    x2 = dion2_post(x, nU, idx, lr, adjust_lr_ratio(x.shape, adjust_lr), wd, -2)
    return x2, m2, v2, idx


def adamw_update(X: torch.Tensor, G: torch.Tensor, M: torch.Tensor, V: torch.Tensor, lr: float, beta1: float,
                 beta2: float, wd: float, step: int, eps: float, cautious: bool = False):
    """dion/scalar_opts.py:7-65 in float64.  Returns (X_new, M_new, V_new)."""
    X, G, M, V = (t.to(torch.float64) for t in (X, G, M, V))
    M = M + (1 - beta1) * (G - M)
    V = V * beta2 + (1 - beta2) * G * G
    bc1 = 1 - beta1 ** step
    bc2 = 1 - beta2 ** step
    denom = V.sqrt() / math.sqrt(bc2) + eps
    upd = M / denom
    if cautious:
        mask = (upd * X >= 0).to(X.dtype)
        X = X - (X * mask) * (lr * wd)
    else:
        X = X * (1 - lr * wd)
    X = X - (lr / bc1) * upd
    return X, M, V


def lion_update(X: torch.Tensor, G: torch.Tensor, M: torch.Tensor, lr: float, beta1: float, beta2: float,
                wd: float, cautious: bool = False):
    """dion/scalar_opts.py:68-118 in float64.  Returns (X_new, M_new)."""
    X, G, M = (t.to(torch.float64) for t in (X, G, M))
    U = torch.sign(M + (1 - beta1) * (G - M))
    M = M + (1 - beta2) * (G - M)
    if cautious:
        mask = (U * X >= 0).to(X.dtype)
        X = X - (X * mask) * (lr * wd)
    else:
        X = X * (1 - lr * wd)
    X = X - lr * U
    return X, M


def muon_step(X: List[torch.Tensor], G: List[torch.Tensor], M: List[torch.Tensor], lr: float, mu: float,
              wd: float, nesterov: bool, adjust_lr: Optional[str], ns: str = "polar_express",
              epsilon: float = 1e-8, cautious: bool = False, adj_ratio: Optional[float] = None):
    """One Muon step over a list of same-shape parameters (dion/muon.py:194-280 on one GPU).
    Returns (new X list, new M list, U list after orthogonalization)."""
    Xo, Mo, Uo = [], [], []
    for x, g, m in zip(X, G, M):
        m2, u = muon_pre(g, m, mu, nesterov)
        if ns == "polar_express":
            o = polar_express_bf16(u, eps=epsilon)
        elif ns == "ns5":
            o = ns_bf16(u, NS5_COEFFS, 1.0, epsilon)
        else:
            raise ValueError(ns)
        ratio = adj_ratio if adj_ratio is not None else adjust_lr_ratio(x.shape, adjust_lr)
        Xo.append(muon_post(x, o, lr, ratio, wd, cautious))
        Mo.append(m2)
        Uo.append(o)
    return Xo, Mo, Uo
