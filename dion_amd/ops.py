"""Tensor-level wrappers over the C ABI of libdion_hip.so.

Each function takes torch tensors that live on the GPU, validates shapes/dtypes on the host,
hands raw device pointers and the current stream to the library, and returns torch tensors.
torch is used for device memory and streams only; all arithmetic happens in the HIP kernels.
There is no CPU implementation behind these functions: CPU tensors raise.
"""
import math
from typing import List, Optional, Sequence, Tuple

import torch
from torch import Tensor
from torch.utils._python_dispatch import is_traceable_wrapper_subclass

from . import _lib
from ._lib import DION_BF16, DION_F32, DION_NS_GRAM, check, ptr_table


def _stream_handle(device: torch.device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


def _require_gpu(t: Tensor, name: str) -> None:
    # The kernels write through raw device pointers.  A wrapper subclass (DTensor, quantised-weight
    # wrappers) keeps its data in inner tensors and exposes no dense buffer at data_ptr()
    # (the case dion/dion2_triton.py:171-190 routes around): refuse it instead of writing somewhere.
    if is_traceable_wrapper_subclass(t):
        raise TypeError(
            f"{name}: {type(t).__name__} is a tensor wrapper subclass; pass its plain local tensor"
        )
    if not t.is_cuda:
        raise RuntimeError(
            f"{name} must be a GPU tensor (got device {t.device}); the dion_amd kernels have no CPU path"
        )


def _dtype_code(t: Tensor, name: str) -> int:
    if t.dtype == torch.bfloat16:
        return DION_BF16
    if t.dtype == torch.float32:
        return DION_F32
    raise TypeError(f"{name}: dtype {t.dtype} not supported (bfloat16 or float32)")


_workspaces = {}


def _workspace(device: torch.device, nbytes: int) -> Tensor:
    """Grow-only scratch buffer per (device, stream); NS calls on one stream reuse it in order."""
    key = (device.index, _stream_handle(device))
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = None
        _workspaces.pop(key, None)
        buf = torch.empty(nbytes, dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    return buf


def release_workspaces() -> None:
    """Drop the cached Newton-Schulz workspaces (they are re-created on demand)."""
    _workspaces.clear()


def _pad128(t: Tensor) -> Tensor:
    """Zero-pad the last two dims of a 3-D bf16 tensor to multiples of 128 (copy only if needed)."""
    r, c = t.shape[-2], t.shape[-1]
    rp, cp = -(-r // 128) * 128, -(-c // 128) * 128
    if rp == r and cp == c:
        return t.contiguous()
    out = torch.zeros(t.shape[0], rp, cp, dtype=t.dtype, device=t.device)
    out[:, :r, :c] = t
    return out


def _as_batch(t: Tensor, name: str) -> Tuple[Tensor, bool]:
    if t.ndim == 2:
        return t.unsqueeze(0), True
    if t.ndim == 3:
        return t, False
    raise ValueError(f"{name} must be a 2D or 3D tensor, got shape {tuple(t.shape)}")


def _check_bf16(t: Tensor, name: str) -> None:
    _require_gpu(t, name)
    if t.dtype != torch.bfloat16:
        raise TypeError(f"{name}: the gfx950 kernels take bfloat16 operands, got {t.dtype}")


def ns_line_1(A: Tensor, *, out: Optional[Tensor] = None) -> Tensor:
    """``A @ A.mT`` computing only the upper-triangular tiles and mirroring them.

    Mirrors ``ns_line_1`` of the reference (dion/newton_schulz_triton.py:160-203): 2D or 3D
    input, optional ``out``; ValueError for other ranks.
    """
    _check_bf16(A, "A")
    A3, squeeze = _as_batch(A, "Input tensor")
    b, m, k = A3.shape
    Ap = _pad128(A3)
    mp, kp = Ap.shape[-2:]
    res = torch.empty(b, mp, mp, dtype=torch.bfloat16, device=A.device)
    lib = _lib.load()
    check(lib.dion_ns_line_1(Ap.data_ptr(), res.data_ptr(), b, mp, kp, _stream_handle(A.device)),
          "ns_line_1")
    res = res[:, :m, :m]
    if squeeze:
        res = res[0]
    if out is not None:
        out.copy_(res)
        return out
    return res.contiguous()


def ns_line_2(A: Tensor, alpha: float, beta: float, *, out: Optional[Tensor] = None) -> Tensor:
    """``alpha * A @ A.mT + beta * A`` for symmetric ``A`` (upper tiles + mirror).

    Mirrors ``ns_line_2`` of the reference (dion/newton_schulz_triton.py:290-333).
    """
    _check_bf16(A, "A")
    A3, squeeze = _as_batch(A, "Input tensor")
    b, m, m2 = A3.shape
    if m != m2:
        raise ValueError(f"Input tensor must be square, got shape {tuple(A.shape)}")
    Ap = _pad128(A3)
    mp = Ap.shape[-1]
    res = torch.empty(b, mp, mp, dtype=torch.bfloat16, device=A.device)
    lib = _lib.load()
    check(lib.dion_ns_line_2(Ap.data_ptr(), res.data_ptr(), b, mp, float(alpha), float(beta),
                             _stream_handle(A.device)), "ns_line_2")
    res = res[:, :m, :m]
    if squeeze:
        res = res[0]
    if out is not None:
        out.copy_(res)
        return out
    return res.contiguous()


def ns_line_3(B: Tensor, X: Tensor, a: float, *, out: Optional[Tensor] = None) -> Tensor:
    """``a * X + B @ X`` for symmetric ``B``.

    Mirrors ``ns_line_3`` of the reference (dion/newton_schulz_triton.py:450-491).  X is read as it
    lies (reduction index along rows, transposing LDS reads in the kernel), as in the whole-NS
    driver.
    """
    _check_bf16(B, "B")
    _check_bf16(X, "X")
    B3, squeeze = _as_batch(B, "B")
    X3, _ = _as_batch(X, "X")
    if B3.shape[0] != X3.shape[0] or B3.shape[-1] != B3.shape[-2] or B3.shape[-1] != X3.shape[-2]:
        raise ValueError(f"shape mismatch: B {tuple(B.shape)} vs X {tuple(X.shape)}")
    b, m, n = X3.shape
    Bp = _pad128(B3)
    Xp = _pad128(X3)
    mp, np_ = Xp.shape[-2:]
    res = torch.empty(b, mp, np_, dtype=torch.bfloat16, device=X.device)
    lib = _lib.load()
    check(lib.dion_ns_line_3(Bp.data_ptr(), Xp.data_ptr(), res.data_ptr(), b, mp, np_, float(a),
                             _stream_handle(X.device)), "ns_line_3")
    res = res[:, :m, :n]
    if squeeze:
        res = res[0]
    if out is not None:
        out.copy_(res)
        return out
    return res.contiguous()


def ns_orthogonalize(G: Tensor, coeffs: Sequence[Sequence[float]], norm_scale: float, epsilon: float,
                     gram: bool = False, gram_reset: int = 0) -> Tensor:
    """Batched Newton-Schulz / Polar-Express orthogonalization of ``G[..., rows, cols]``.

    X0 = bf16(G) / (||bf16(G)||_F * norm_scale + epsilon), then ``len(coeffs)`` quintic
    iterations on the orientation with rows <= cols; result is bf16 with the shape of ``G``.
    """
    _require_gpu(G, "G")
    if G.ndim < 2:
        raise ValueError(f"expected a tensor with at least 2 dims, got shape {tuple(G.shape)}")
    if G.dtype not in (torch.bfloat16, torch.float32):
        G = G.to(torch.float32)
    shape = G.shape
    rows, cols = shape[-2], shape[-1]
    G3 = G.reshape(-1, rows, cols).contiguous()
    batch = G3.shape[0]
    out = torch.empty(batch, rows, cols, dtype=torch.bfloat16, device=G.device)
    if out.numel() == 0:
        return out.reshape(shape)
    carr, n_iters = _flat_coeffs(coeffs)
    flags = DION_NS_GRAM if gram else 0
    lib = _lib.load()
    chunk = 32768  # one library call takes at most 65535 matrices
    for b0 in range(0, batch, chunk):
        nb = min(chunk, batch - b0)
        nbytes = lib.dion_ns_workspace_bytes(nb, rows, cols, flags)
        ws = _workspace(G.device, nbytes)
        check(lib.dion_ns_orthogonalize(G3[b0:].data_ptr(), _dtype_code(G3, "G"), out[b0:].data_ptr(), nb, rows,
                                        cols, carr, n_iters, float(norm_scale), float(epsilon), flags,
                                        int(gram_reset), ws.data_ptr(), ws.numel(), _stream_handle(G.device)),
              "ns_orthogonalize")
    return out.reshape(shape)


def _flat_coeffs(coeffs):
    flat = [float(v) for abc in coeffs for v in abc]
    if len(flat) % 3:
        raise ValueError("coeffs must be (a, b, c) triples")
    return (_lib.ctypes.c_float * max(1, len(flat)))(*flat), len(flat) // 3


def ns_orthogonalize_update(G: Tensor, X: List[Tensor], coeffs: Sequence[Sequence[float]], norm_scale: float,
                            epsilon: float, lr: Tensor, adj_ratio: float, weight_decay, cautious_wd: bool = False,
                            gram: bool = False, gram_reset: int = 0) -> None:
    """``muon_post(X, ns_orthogonalize(G, ...), lr, adj_ratio, weight_decay, cautious_wd)`` in one library
    call, with the same result bit for bit (dion/muon.py:249-277).  ``G`` is ``[..., rows, cols]`` with
    ``len(X) * mats`` matrices; every ``X[i]`` is a contiguous fp32 or bf16 parameter of ``mats * rows *
    cols`` elements laid out as ``[mats, rows, cols]``.  When the matrices fill whole tiles the update runs in
    the epilogue of the last GEMM and the orthogonalized matrices never reach memory."""
    _require_gpu(G, "G")
    if G.ndim < 2:
        raise ValueError(f"expected a tensor with at least 2 dims, got shape {tuple(G.shape)}")
    n = len(X)
    if n == 0:
        raise ValueError("X is empty")
    if G.dtype not in (torch.bfloat16, torch.float32):
        G = G.to(torch.float32)
    rows, cols = G.shape[-2], G.shape[-1]
    G3 = G.reshape(-1, rows, cols).contiguous()
    batch = G3.shape[0]
    if batch == 0 or rows * cols == 0:
        return
    if batch % n:
        raise ValueError(f"{batch} matrices do not divide over {n} parameters")
    mats_per_ptr = batch // n
    xp, xcode = _state_ptrs(X, "X", mats_per_ptr * rows * cols)
    lr_p, wd_p, wd_h = _scalar_args(lr, weight_decay, G.device)
    if batch > 32768:  # past one library call: the two-pass form, which splits the batch
        O = ns_orthogonalize(G3, coeffs, norm_scale, epsilon, gram, gram_reset)
        muon_post(X, O.view(n, -1), lr, adj_ratio, weight_decay, cautious_wd)
        return
    carr, n_iters = _flat_coeffs(coeffs)
    flags = DION_NS_GRAM if gram else 0
    lib = _lib.load()
    ws = _workspace(G.device, lib.dion_ns_update_workspace_bytes(batch, rows, cols, flags, n_iters))
    check(lib.dion_ns_orthogonalize_update(G3.data_ptr(), _dtype_code(G3, "G"), xp, xcode, n, mats_per_ptr, rows,
                                           cols, carr, n_iters, float(norm_scale), float(epsilon), flags,
                                           int(gram_reset), lr_p, float(adj_ratio), wd_p, wd_h,
                                           int(bool(cautious_wd)), ws.data_ptr(), ws.numel(),
                                           _stream_handle(G.device)), "ns_orthogonalize_update")


def ns_accepts_prepared(batch: int, rows: int, cols: int, n_iters: int, gram: bool = False) -> bool:
    """True when ``batch`` matrices of ``rows x cols`` can go to the orthogonalization as ``muon_pre_prepared``
    writes them (whole GEMM tiles, not the small-matrix kernel, at least one iteration)."""
    lib = _lib.load()
    return bool(lib.dion_ns_accepts_prepared(int(batch), int(rows), int(cols), DION_NS_GRAM if gram else 0,
                                             int(n_iters)))


def _check_prepared(U: Tensor, sumsq: Tensor, rows: int, cols: int) -> Tuple[int, int]:
    _check_bf16(U, "U")
    m, n = min(rows, cols), max(rows, cols)
    if U.ndim != 3 or U.shape[1] != m or U.shape[2] != n or not U.is_contiguous():
        raise ValueError(f"a prepared input of {rows} x {cols} matrices is a contiguous [batch, {m}, {n}] tensor, "
                         f"got {tuple(U.shape)}")
    batch = U.shape[0]
    if (sumsq.dtype != torch.float32 or sumsq.ndim != 2 or sumsq.shape[0] != batch or not sumsq.is_contiguous()
            or sumsq.device != U.device):
        raise ValueError("sumsq must be a contiguous float32 [batch, blocks] tensor on the device of U")
    return batch, sumsq.shape[1]


def ns_orthogonalize_prepared(U: Tensor, sumsq: Tensor, rows: int, cols: int, coeffs, norm_scale: float,
                              epsilon: float, gram: bool = False, gram_reset: int = 0) -> Tensor:
    """``ns_orthogonalize`` of the matrices ``muon_pre_prepared`` wrote: ``U [batch, min, max]`` holds them
    with the short side along rows and unnormalised, ``sumsq [batch, blocks]`` partial sums of their squares.
    Returns ``[batch, rows, cols]`` bf16.  The Frobenius normalisation rides on the first two GEMMs."""
    batch, blocks = _check_prepared(U, sumsq, rows, cols)
    out = torch.empty(batch, rows, cols, dtype=torch.bfloat16, device=U.device)
    carr, n_iters = _flat_coeffs(coeffs)
    flags = DION_NS_GRAM if gram else 0
    lib = _lib.load()
    ws = _workspace(U.device, lib.dion_ns_workspace_bytes(batch, rows, cols, flags))
    check(lib.dion_ns_orthogonalize_prepared(U.data_ptr(), sumsq.data_ptr(), blocks, out.data_ptr(), batch, rows,
                                             cols, carr, n_iters, float(norm_scale), float(epsilon), flags,
                                             int(gram_reset), ws.data_ptr(), ws.numel(), _stream_handle(U.device)),
          "ns_orthogonalize_prepared")
    return out


def ns_orthogonalize_update_prepared(U: Tensor, sumsq: Tensor, rows: int, cols: int, X: List[Tensor], coeffs,
                                     norm_scale: float, epsilon: float, lr: Tensor, adj_ratio: float, weight_decay,
                                     cautious_wd: bool = False, gram: bool = False, gram_reset: int = 0) -> None:
    """``ns_orthogonalize_update`` on a prepared input (see ``ns_orthogonalize_prepared``): the update of
    every ``X[i]`` (``[mats, rows, cols]``) rides on the last GEMM."""
    batch, blocks = _check_prepared(U, sumsq, rows, cols)
    n = len(X)
    if n == 0 or batch % n:
        raise ValueError(f"{batch} matrices do not divide over {n} parameters")
    mats_per_ptr = batch // n
    xp, xcode = _state_ptrs(X, "X", mats_per_ptr * rows * cols)
    lr_p, wd_p, wd_h = _scalar_args(lr, weight_decay, U.device)
    carr, n_iters = _flat_coeffs(coeffs)
    flags = DION_NS_GRAM if gram else 0
    lib = _lib.load()
    ws = _workspace(U.device, lib.dion_ns_update_workspace_bytes(batch, rows, cols, flags, n_iters))
    check(lib.dion_ns_orthogonalize_update_prepared(U.data_ptr(), sumsq.data_ptr(), blocks, xp, xcode, n,
                                                    mats_per_ptr, rows, cols, carr, n_iters, float(norm_scale),
                                                    float(epsilon), flags, int(gram_reset), lr_p,
                                                    float(adj_ratio), wd_p, wd_h, int(bool(cautious_wd)),
                                                    ws.data_ptr(), ws.numel(), _stream_handle(U.device)),
          "ns_orthogonalize_update_prepared")


# ---------------------------------------------------------------------------------------------
# optimizer-step kernels on lists of same-shape parameters
# ---------------------------------------------------------------------------------------------
def _list_ptrs(ts: List[Tensor], name: str, dtype=None, numel=None):
    for t in ts:
        _require_gpu(t, name)
        if not t.is_contiguous():
            raise ValueError(f"{name}: tensors must be contiguous")
        if dtype is not None and t.dtype != dtype:
            raise TypeError(f"{name}: expected {dtype}, got {t.dtype}")
        if numel is not None and t.numel() != numel:
            raise ValueError(f"{name}: all tensors of a shape group must have {numel} elements")
    return ptr_table([t.data_ptr() for t in ts])


def _state_ptrs(ts: List[Tensor], name: str, numel=None):
    """(pointer table, dtype code) of a list of optimizer-state tensors (parameters, momentum, second
    moments): contiguous GPU tensors that share one dtype, float32 or bfloat16."""
    code = _dtype_code(ts[0], name)
    return _list_ptrs(ts, name, ts[0].dtype, numel), code


def _scalar_args(lr: Tensor, weight_decay, device):
    """lr must already be a 0-d fp32 device tensor; weight decay may be one, or a host number."""
    if not (isinstance(lr, Tensor) and lr.is_cuda and lr.dtype == torch.float32 and lr.numel() == 1):
        raise TypeError("lr must be a 0-d float32 tensor on the GPU")
    if isinstance(weight_decay, Tensor) and weight_decay.is_cuda:
        if weight_decay.dtype != torch.float32 or weight_decay.numel() != 1:
            raise TypeError("a device weight_decay must be a 0-d float32 tensor")
        return lr.data_ptr(), weight_decay.data_ptr(), 0.0
    return lr.data_ptr(), None, float(weight_decay)


def muon_pre(G: List[Tensor], M: List[Tensor], momentum: float, nesterov: bool) -> Tensor:
    """Momentum update of every ``M[i]`` in place; returns the bf16 arena ``[N, *shape]`` holding the
    orthogonalization inputs.  Mirrors ``muon_update_pre_orthogonalize`` (dion/muon.py:284-311)
    followed by the ``torch.stack`` of dion/megabatch_base.py:872."""
    n = len(G)
    assert n == len(M) and n > 0
    numel = M[0].numel()
    gp = _list_ptrs(G, "G", G[0].dtype, numel)
    mp, mcode = _state_ptrs(M, "M", numel)
    U = torch.empty((n, *M[0].shape), dtype=torch.bfloat16, device=M[0].device)
    lib = _lib.load()
    check(lib.dion_muon_pre(gp, _dtype_code(G[0], "G"), mp, mcode, U.data_ptr(), n, numel, float(momentum),
                            int(bool(nesterov)), _stream_handle(U.device)), "muon_pre")
    return U


def muon_pre_prepared(G: List[Tensor], M: List[Tensor], momentum: float, nesterov: bool, mats: int, rows: int,
                      cols: int) -> Tuple[Tensor, Tensor]:
    """``muon_pre`` for parameters made of ``mats`` matrices of ``rows x cols`` each, writing the
    orthogonalization input the way the iteration carries it: returns ``(U, sumsq)`` with ``U [N * mats,
    min(rows, cols), max(rows, cols)]`` bf16 (a tall matrix transposed) and ``sumsq [N * mats, blocks]`` fp32
    partial sums of squares of each matrix.  ``M`` is updated exactly as by ``muon_pre``."""
    n = len(G)
    assert n == len(M) and n > 0
    numel = M[0].numel()
    if numel != mats * rows * cols:
        raise ValueError(f"parameters of {numel} elements are not {mats} matrices of {rows} x {cols}")
    gp = _list_ptrs(G, "G", G[0].dtype, numel)
    mp, mcode = _state_ptrs(M, "M", numel)
    lib = _lib.load()
    blocks = lib.dion_muon_pre_sumsq_blocks(rows, cols)
    if blocks == 0:
        raise ValueError(f"muon_pre_prepared: {rows} x {cols} matrices are not whole 64 x 64 tiles")
    dev = M[0].device
    U = torch.empty((n * mats, min(rows, cols), max(rows, cols)), dtype=torch.bfloat16, device=dev)
    sumsq = torch.empty((n * mats, blocks), dtype=torch.float32, device=dev)
    check(lib.dion_muon_pre_prepared(gp, _dtype_code(G[0], "G"), mp, mcode, U.data_ptr(), sumsq.data_ptr(), n, mats,
                                     rows, cols, float(momentum), int(bool(nesterov)), _stream_handle(dev)),
          "muon_pre_prepared")
    return U, sumsq


def muon_post(X: List[Tensor], U: Tensor, lr: Tensor, adj_ratio: float, weight_decay, cautious_wd: bool = False,
              row_scale: Optional[Tensor] = None, adjusted_lr: Optional[Tensor] = None) -> None:
    """In-place weight decay + update of every ``X[i]`` from the arena ``U[i]``.  Mirrors
    ``muon_update_post_orthogonalize`` (dion/muon.py:315-347); ``row_scale`` folds NorMuon's
    per-row normalisation into the same pass; ``adjusted_lr`` (0-d fp32 device tensor) replaces
    ``lr * adj_ratio`` in the update term."""
    n = len(X)
    assert n > 0 and U.shape[0] == n
    numel = X[0].numel()
    cols = X[0].shape[-1]
    xp, xcode = _state_ptrs(X, "X", numel)
    if not U.is_contiguous() or U.numel() != n * numel:
        raise ValueError("U must be a contiguous [N, *shape] arena")
    lr_p, wd_p, wd_h = _scalar_args(lr, weight_decay, U.device)
    rs_p = None
    if row_scale is not None:
        if row_scale.dtype != torch.float32 or row_scale.numel() != n * (numel // cols):
            raise ValueError("row_scale must be float32 [N, rows]")
        rs_p = row_scale.data_ptr()
    alr = None
    if adjusted_lr is not None:
        if not (adjusted_lr.is_cuda and adjusted_lr.dtype == torch.float32 and adjusted_lr.numel() == 1):
            raise TypeError("adjusted_lr must be a 0-d float32 GPU tensor")
        alr = adjusted_lr.data_ptr()
    lib = _lib.load()
    check(lib.dion_muon_post(xp, xcode, U.data_ptr(), _dtype_code(U, "U"), n, numel, cols, rs_p, lr_p, alr,
                             float(adj_ratio), wd_p, wd_h, int(bool(cautious_wd)),
                             _stream_handle(U.device)), "muon_post")


def scale_rows(U: Tensor, scale: Tensor, dtype: torch.dtype) -> Tensor:
    """``U[..., r, :] * scale[r]`` for a contiguous bf16 ``U [..., rows, cols]`` and fp32 ``scale`` with one
    entry per row of ``U``; result in ``dtype`` (float32 or bfloat16)."""
    _check_bf16(U, "U")
    if not U.is_contiguous():
        raise ValueError("U must be contiguous")
    cols = U.shape[-1]
    n_rows = U.numel() // cols if cols else 0
    if scale.dtype != torch.float32 or not scale.is_contiguous() or scale.numel() != n_rows or not scale.is_cuda:
        raise ValueError("scale must be a contiguous float32 GPU tensor with one entry per row of U")
    out = torch.empty(U.shape, dtype=dtype, device=U.device)
    lib = _lib.load()
    check(lib.dion_scale_rows(U.data_ptr(), scale.data_ptr(), out.data_ptr(), _dtype_code(out, "out"), n_rows,
                              cols, _stream_handle(U.device)), "scale_rows")
    return out


def normuon_stats(U: Tensor, V: List[Tensor], beta2: float) -> Tensor:
    """Updates every ``V[i]`` (``[..., rows, 1]``, fp32 or bf16) in place from the orthogonalized arena
    ``U [N, ..., rows, cols]`` and returns the per-row scales ``[n_mat, rows]`` that turn ``U`` into the
    NorMuon-normalised update.  Mirrors ``normuon_normalization_stacked`` (dion/normuon.py:345-399)."""
    n = len(V)
    assert n > 0 and U.shape[0] == n
    _check_bf16(U, "U")
    rows, cols = U.shape[-2], U.shape[-1]
    n_mat = U.numel() // (rows * cols)
    mats_per_ptr = n_mat // n
    vp, vcode = _state_ptrs(V, "V", mats_per_ptr * rows)
    scale = torch.empty(n_mat, rows, dtype=torch.float32, device=U.device)
    lib = _lib.load()
    check(lib.dion_normuon_stats(U.data_ptr(), vp, vcode, n, mats_per_ptr, rows, cols, float(beta2),
                                 scale.data_ptr(), _stream_handle(U.device)), "normuon_stats")
    return scale


def normuon_stats_selected(U: Tensor, V: List[Tensor], idx: Tensor, beta2: float) -> Tensor:
    """NorMuon statistics for an update made of ``k`` selected rows per matrix: ``U [N, ..., k, cols]``
    bf16, ``idx [n_mat, k]`` int32 (rows of the parameter), ``V[i]`` the full ``[..., rows, 1]`` fp32 or bf16
    buffers, of which only the selected entries are read and updated.  Returns the per-row scales
    ``[n_mat, k]``.  Mirrors ``nordion2_normalize_selected_stacked`` (dion/nordion2.py:430-447)."""
    n = len(V)
    assert n > 0 and U.shape[0] == n
    _check_bf16(U, "U")
    k, cols = U.shape[-2], U.shape[-1]
    n_mat = U.numel() // (k * cols)
    mats_per_ptr = n_mat // n
    v_rows = V[0].numel() // mats_per_ptr
    vp, vcode = _state_ptrs(V, "V", mats_per_ptr * v_rows)
    if idx.dtype != torch.int32 or not idx.is_contiguous() or idx.numel() != n_mat * k:
        raise ValueError("idx must be a contiguous int32 tensor of n_mat * k entries")
    scale = torch.empty(n_mat, k, dtype=torch.float32, device=U.device)
    lib = _lib.load()
    check(lib.dion_normuon_stats_selected(U.data_ptr(), vp, vcode, n, mats_per_ptr, k, cols, idx.data_ptr(), v_rows,
                                          float(beta2), scale.data_ptr(), _stream_handle(U.device)),
          "normuon_stats_selected")
    return scale


def dion2_prepared_blocks(rows: int, cols: int, select_dim: int, k: int) -> int:
    """Partial sums per matrix that ``dion2_select(..., prepared=True)`` writes for ``k`` slices of a
    ``rows x cols`` matrix along ``select_dim``; 0 when the selected block has no prepared form."""
    return int(_lib.load().dion_dion2_gather_sumsq_blocks(int(rows), int(cols), int(select_dim), int(k)))


def dion2_select(G: List[Tensor], M: List[Tensor], k: int, select_dim: int, ef_decay: float, prepared: bool = False):
    """``M += G``; pick the ``k`` slices of largest L1 norm along ``select_dim`` of every matrix; return
    (U_sel bf16 arena, idx int32 [n_mat, k] ascending, map int32 [n_mat, dim]) and decay the selected
    slices of ``M`` by ``ef_decay``.  Mirrors ``dion2_pre_orthogonalize`` (dion/dion2.py:439-547).

    ``prepared=True`` (only where ``dion2_prepared_blocks`` is not 0): the selected blocks are written as a
    prepared orthogonalization input -- ``U_sel [n_mat, min, max]`` with the short side of the block along rows
    (a tall block transposed) -- and a fourth result ``sumsq [n_mat, blocks]`` holds partial sums of their
    squares."""
    if select_dim not in (-2, -1):
        raise ValueError(f"select_dim must be -2 or -1, got {select_dim}")
    n = len(G)
    assert n == len(M) and n > 0
    shape = M[0].shape
    rows, cols = shape[-2], shape[-1]
    numel = M[0].numel()
    mats_per_ptr = numel // (rows * cols)
    n_mat = n * mats_per_ptr
    gp = _list_ptrs(G, "G", G[0].dtype, numel)
    mp, mcode = _state_ptrs(M, "M", numel)
    dev = M[0].device
    dim = rows if select_dim == -2 else cols
    norms = torch.empty(n_mat, dim, dtype=torch.float32, device=dev)
    idx = torch.empty(n_mat, k, dtype=torch.int32, device=dev)
    imap = torch.empty(n_mat, dim, dtype=torch.int32, device=dev)
    sel_shape = (n, *shape[:-2], k, cols) if select_dim == -2 else (n, *shape[:-2], rows, k)
    U = torch.empty(sel_shape, dtype=torch.bfloat16, device=dev)
    lib = _lib.load()
    st = _stream_handle(dev)
    sbytes = lib.dion_dion2_accumulate_scratch_bytes(n_mat, rows, cols, select_dim)
    scratch = torch.empty(sbytes, dtype=torch.uint8, device=dev) if sbytes else None
    check(lib.dion_dion2_accumulate(gp, _dtype_code(G[0], "G"), mp, mcode, n, mats_per_ptr, rows, cols, select_dim,
                                    norms.data_ptr(), scratch.data_ptr() if sbytes else None, sbytes, st),
          "dion2_accumulate")
    check(lib.dion_dion2_topk(norms.data_ptr(), n_mat, dim, k, idx.data_ptr(), imap.data_ptr(), st),
          "dion2_topk")
    if prepared:
        blocks = dion2_prepared_blocks(rows, cols, select_dim, k)
        if blocks == 0:
            raise ValueError(f"dion2_select: {k} slices of {rows} x {cols} along dim {select_dim} have no prepared form")
        sr, sc = (k, cols) if select_dim == -2 else (rows, k)
        U = U.view(n_mat, min(sr, sc), max(sr, sc))
        sumsq = torch.empty(n_mat, blocks, dtype=torch.float32, device=dev)
        check(lib.dion_dion2_gather_prepared(mp, mcode, n, mats_per_ptr, rows, cols, select_dim, idx.data_ptr(), k,
                                             float(ef_decay), U.data_ptr(), sumsq.data_ptr(), st),
              "dion2_gather_prepared")
        return U, idx, imap, sumsq
    check(lib.dion_dion2_gather(mp, mcode, n, mats_per_ptr, rows, cols, select_dim, idx.data_ptr(), k,
                                float(ef_decay), U.data_ptr(), st), "dion2_gather")
    return U, idx, imap


def dion2_post(X: List[Tensor], U: Tensor, imap: Tensor, lr: Tensor, adj_ratio: float, weight_decay,
               select_dim: int, row_scale: Optional[Tensor] = None, adjusted_lr: Optional[Tensor] = None) -> None:
    """Fused ``x = (1 - lr*wd)*x - lr*adj_ratio*u[map]`` over every ``X[i]``.  Mirrors
    ``dion2_post_orthogonalize_triton`` (dion/dion2_triton.py:147-242).  ``U`` bf16 or fp32 arena.
    ``row_scale [n_mat, k]`` (rows selected only) multiplies each selected row of ``U`` first;
    ``adjusted_lr`` (0-d fp32 device tensor) replaces ``lr`` in the update term."""
    if select_dim not in (-2, -1):
        raise ValueError(f"select_dim must be -2 or -1, got {select_dim}")
    n = len(X)
    assert n > 0
    shape = X[0].shape
    rows, cols = shape[-2], shape[-1]
    numel = X[0].numel()
    mats_per_ptr = numel // (rows * cols)
    xp, xcode = _state_ptrs(X, "X", numel)
    _require_gpu(U, "U")
    if not U.is_contiguous():
        raise ValueError("U must be contiguous")
    k = U.shape[-2] if select_dim == -2 else U.shape[-1]
    lr_p, wd_p, wd_h = _scalar_args(lr, weight_decay, U.device)
    lib = _lib.load()
    rs = None
    if row_scale is not None:
        if row_scale.dtype != torch.float32 or not row_scale.is_contiguous() or \
                row_scale.numel() != n * mats_per_ptr * k:
            raise ValueError("row_scale must be a contiguous float32 tensor of n_mat * k entries")
        rs = row_scale.data_ptr()
    alr = None
    if adjusted_lr is not None:
        if not (adjusted_lr.is_cuda and adjusted_lr.dtype == torch.float32 and adjusted_lr.numel() == 1):
            raise TypeError("adjusted_lr must be a 0-d float32 GPU tensor")
        alr = adjusted_lr.data_ptr()
    check(lib.dion_dion2_post(xp, xcode, n, mats_per_ptr, rows, cols, select_dim, U.data_ptr(), _dtype_code(U, "U"), k,
                              imap.data_ptr(), rs, lr_p, alr, float(adj_ratio), wd_p, wd_h,
                              _stream_handle(U.device)), "dion2_post")


def dion2_index_map(indices: Tensor, dim: int) -> Tensor:
    """int32 ``[n_mat, dim]`` inverse map of ``indices [..., k]`` (int64, distinct, any order): position of
    each slice in the list, -1 where not listed.  Mirrors ``_build_index_map``
    (dion/dion2_triton.py:30-47)."""
    _require_gpu(indices, "indices")
    if indices.dtype != torch.int64:
        raise TypeError(f"indices must be int64, got {indices.dtype}")
    k = indices.shape[-1]
    idx = indices.reshape(-1, k).contiguous()
    imap = torch.empty(idx.shape[0], dim, dtype=torch.int32, device=indices.device)
    lib = _lib.load()
    check(lib.dion_dion2_index_map(idx.data_ptr(), idx.shape[0], k, dim, imap.data_ptr(),
                                   _stream_handle(indices.device)), "dion2_index_map")
    return imap


def dion2_post_orthogonalize_triton(X: List[Tensor], U: List[Tensor], indices: List[Tensor], base_lr: Tensor,
                                    adjusted_lr: Tensor, weight_decay, select_dim: int) -> None:
    """Same call as the reference's ``dion2_post_orthogonalize_triton`` (dion/dion2_triton.py:147-155):
    per tensor ``x`` ``[*leading, M, N]`` fp32 or bf16, contiguous, ``u`` the selected slices (bf16 or fp32),
    ``indices [*leading, k]`` int64; ``selected: x = (1 - base_lr*wd)*x - adjusted_lr*u``, unselected:
    ``x = (1 - base_lr*wd)*x``.  ``base_lr`` / ``adjusted_lr`` are 0-d fp32 device tensors read in the
    kernel.  Empty tensors are skipped; non-contiguous ``x`` raises ``ValueError``."""
    if select_dim not in (-2, -1):
        raise ValueError(f"select_dim must be -2 or -1, got {select_dim}")
    for x, u, idx in zip(X, U, indices):
        if x.numel() == 0:
            continue
        if not x.is_contiguous():
            raise ValueError("dion2_post_orthogonalize_triton requires contiguous X tensors")
        if u.dtype not in (torch.bfloat16, torch.float32):
            u = u.float()
        dim = x.shape[select_dim]
        imap = dion2_index_map(idx, dim)
        dion2_post([x], u.contiguous().unsqueeze(0), imap, base_lr, 1.0, weight_decay, select_dim,
                   adjusted_lr=adjusted_lr)


# ---------------------------------------------------------------------------------------------
# whole-matrix selection (selection_scope="global"): select inside the orthogonalization call,
# update keyed off the non-zero slices
# ---------------------------------------------------------------------------------------------
def _stacked(U: Tensor, name: str) -> Tuple[int, int, int, int]:
    """(dtype code, n_mat, rows, cols) of a contiguous stacked ``[..., rows, cols]`` GPU tensor."""
    _require_gpu(U, name)
    if U.dim() < 2:
        raise ValueError(f"{name} must have at least 2 dimensions, got shape {tuple(U.shape)}")
    if not U.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    rows, cols = U.shape[-2], U.shape[-1]
    n_mat = U.numel() // (rows * cols) if rows * cols else math.prod(U.shape[:-2])
    return _dtype_code(U, name), n_mat, rows, cols


def slice_l1(U: Tensor, select_dim: int, round_bf16: bool = False) -> Tensor:
    """L1 norm of every slice of ``U [..., rows, cols]`` (bf16 or fp32) along ``select_dim``: fp32
    ``[n_mat, dim]``.  ``round_bf16`` rounds the result to bf16 precision, which is what
    ``X.norm(p=1, dim=...)`` returns for a bf16 ``X`` (dion/dion2.py:602)."""
    if select_dim not in (-2, -1):
        raise ValueError(f"select_dim must be -2 or -1, got {select_dim}")
    code, n_mat, rows, cols = _stacked(U, "U")
    dim = rows if select_dim == -2 else cols
    norms = torch.empty(n_mat, dim, dtype=torch.float32, device=U.device)
    lib = _lib.load()
    check(lib.dion_slice_l1(U.data_ptr(), code, n_mat, rows, cols, select_dim, int(bool(round_bf16)),
                            norms.data_ptr(), _stream_handle(U.device)), "slice_l1")
    return norms


def select_slices(U: Tensor, k: int, select_dim: int):
    """Top-``k`` slices of every matrix of ``U [..., rows, cols]`` by L1 norm along ``select_dim``
    (dion/dion2.py:600-610).  Returns (sub, idx int32 [n_mat, k] ascending, map int32 [n_mat, dim]);
    ``sub`` is ``[..., k, cols]`` or ``[..., rows, k]`` in the dtype of ``U``."""
    code, n_mat, rows, cols = _stacked(U, "U")
    dim = rows if select_dim == -2 else cols
    if not (0 <= k <= dim):
        raise ValueError(f"k={k} outside [0, {dim}]")
    norms = slice_l1(U, select_dim, round_bf16=U.dtype == torch.bfloat16)
    dev = U.device
    idx = torch.empty(n_mat, k, dtype=torch.int32, device=dev)
    imap = torch.empty(n_mat, dim, dtype=torch.int32, device=dev)
    sub_shape = (*U.shape[:-2], k, cols) if select_dim == -2 else (*U.shape[:-2], rows, k)
    sub = torch.empty(sub_shape, dtype=U.dtype, device=dev)
    lib = _lib.load()
    st = _stream_handle(dev)
    check(lib.dion_dion2_topk(norms.data_ptr(), n_mat, dim, k, idx.data_ptr(), imap.data_ptr(), st),
          "dion2_topk")
    check(lib.dion_gather_slices(U.data_ptr(), code, n_mat, rows, cols, select_dim, idx.data_ptr(), k,
                                 sub.data_ptr(), st), "gather_slices")
    return sub, idx, imap


def scatter_slices(sub: Tensor, imap: Tensor, shape, select_dim: int) -> Tensor:
    """Full-size tensor of ``shape [..., rows, cols]`` that holds ``sub`` at the slices ``imap`` marks and
    zero elsewhere (dion/dion2.py:612-613)."""
    if select_dim not in (-2, -1):
        raise ValueError(f"select_dim must be -2 or -1, got {select_dim}")
    code, n_mat, srows, scols = _stacked(sub, "sub")
    rows, cols = shape[-2], shape[-1]
    k = srows if select_dim == -2 else scols
    if (select_dim == -2 and scols != cols) or (select_dim == -1 and srows != rows):
        raise ValueError(f"sub {tuple(sub.shape)} does not fit into {tuple(shape)} along dim {select_dim}")
    dim = rows if select_dim == -2 else cols
    if imap.dtype != torch.int32 or not imap.is_contiguous() or imap.numel() != n_mat * dim:
        raise ValueError("map must be a contiguous int32 tensor of n_mat * dim entries")
    out = torch.empty(tuple(shape), dtype=sub.dtype, device=sub.device)
    if out.numel() != n_mat * rows * cols:
        raise ValueError(f"shape {tuple(shape)} does not hold {n_mat} matrices")
    lib = _lib.load()
    check(lib.dion_scatter_slices(sub.data_ptr(), code, n_mat, rows, cols, select_dim, imap.data_ptr(), k,
                                  out.data_ptr(), _stream_handle(sub.device)), "scatter_slices")
    return out


def mask_index(norms: Tensor) -> Tensor:
    """int32 ``[n_mat, dim]``: the slice's own index where its norm is > 0, -1 elsewhere."""
    _require_gpu(norms, "norms")
    if norms.dtype != torch.float32 or norms.dim() != 2 or not norms.is_contiguous():
        raise ValueError("norms must be a contiguous float32 [n_mat, dim] tensor")
    gate = torch.empty(norms.shape, dtype=torch.int32, device=norms.device)
    lib = _lib.load()
    check(lib.dion_mask_index(norms.data_ptr(), norms.shape[0], norms.shape[1], gate.data_ptr(),
                              _stream_handle(norms.device)), "mask_index")
    return gate


def dion2_post_masked(X: List[Tensor], M: List[Tensor], U: Tensor, norms: Tensor, lr: Tensor,
                      adj_ratio: float, weight_decay, ef_decay: float, select_dim: int,
                      row_scale: Optional[Tensor] = None, adjusted_lr: Optional[Tensor] = None) -> None:
    """``x = (1 - lr*wd)*x - lr*adj_ratio*u`` over every ``X[i]`` and ``m *= ef_decay`` on the slices of
    ``M[i]`` whose entry of ``norms`` (``slice_l1(U)``) is > 0.  ``U [N, ..., rows, cols]`` bf16 is zero
    off the selected slices.  Mirrors ``dion2_post_orthogonalize_masked`` (dion/dion2.py:623-659);
    ``row_scale [n_mat, rows]`` (rows selected only) multiplies each row of ``U`` first; ``adjusted_lr``
    (0-d fp32 device tensor) replaces ``lr`` in the update term."""
    if select_dim not in (-2, -1):
        raise ValueError(f"select_dim must be -2 or -1, got {select_dim}")
    n = len(X)
    assert n > 0 and len(M) == n
    shape = X[0].shape
    rows, cols = shape[-2], shape[-1]
    numel = X[0].numel()
    mats_per_ptr = numel // (rows * cols)
    n_mat = n * mats_per_ptr
    xp, xcode = _state_ptrs(X, "X", numel)
    mp, mcode = _state_ptrs(M, "M", numel)
    if xcode != mcode:
        raise TypeError(f"X ({X[0].dtype}) and M ({M[0].dtype}) must share one dtype")
    _check_bf16(U, "U")
    if not U.is_contiguous() or U.numel() != n * numel:
        raise ValueError("U must be a contiguous [N, *shape] arena")
    dim = rows if select_dim == -2 else cols
    if norms.dtype != torch.float32 or not norms.is_contiguous() or norms.numel() != n_mat * dim:
        raise ValueError("norms must be a contiguous float32 tensor of n_mat * dim entries")
    rs = None
    if row_scale is not None:
        if row_scale.dtype != torch.float32 or not row_scale.is_contiguous() or \
                row_scale.numel() != n_mat * rows:
            raise ValueError("row_scale must be a contiguous float32 tensor of n_mat * rows entries")
        rs = row_scale.data_ptr()
    lr_p, wd_p, wd_h = _scalar_args(lr, weight_decay, U.device)
    alr = None
    if adjusted_lr is not None:
        if not (adjusted_lr.is_cuda and adjusted_lr.dtype == torch.float32 and adjusted_lr.numel() == 1):
            raise TypeError("adjusted_lr must be a 0-d float32 GPU tensor")
        alr = adjusted_lr.data_ptr()
    lib = _lib.load()
    check(lib.dion_dion2_post_masked(xp, mp, xcode, n, mats_per_ptr, rows, cols, select_dim, U.data_ptr(),
                                     norms.data_ptr(), rs, lr_p, alr, float(adj_ratio), wd_p, wd_h,
                                     float(ef_decay), _stream_handle(U.device)), "dion2_post_masked")


# ---------------------------------------------------------------------------------------------
# multi-tensor AdamW / Lion for the non-matrix parameter groups
# ---------------------------------------------------------------------------------------------
def _mta_tables(X: List[Tensor], G: List[Tensor], states: List[List[Tensor]]):
    n = len(X)
    assert n > 0 and len(G) == n and all(len(s) == n for s in states)
    gdt = G[0].dtype
    sdt = X[0].dtype
    for x, g in zip(X, G):
        _require_gpu(x, "X")
        _require_gpu(g, "G")
        if x.dtype != sdt:
            raise TypeError("X: one parameter dtype per call")
        if g.dtype != gdt:
            raise TypeError("G: one gradient dtype per call")
        if not x.is_contiguous() or not g.is_contiguous() or g.numel() != x.numel():
            raise ValueError("X / G must be contiguous and of equal size")
    for name, st in zip("MV", states):
        for x, s in zip(X, st):
            if s.dtype != sdt or not s.is_contiguous() or s.numel() != x.numel() or not s.is_cuda:
                raise ValueError(f"{name}: optimizer state must be contiguous GPU tensors shaped like X, in the "
                                 f"dtype of X ({sdt})")
    numels = (_lib.ctypes.c_int64 * n)(*[x.numel() for x in X])
    tabs = [ptr_table([t.data_ptr() for t in ts]) for ts in (X, G, *states)]
    return tabs, numels, _dtype_code(G[0], "G"), _dtype_code(X[0], "X")


def adamw_step(X: List[Tensor], G: List[Tensor], M: List[Tensor], V: List[Tensor], steps: List[Tensor],
               lr: Tensor, beta1: float, beta2: float, weight_decay, epsilon: float,
               cautious_wd: bool = False) -> None:
    """One fused AdamW step over tensors of any sizes (dion/scalar_opts.py:7-65, :121-268).  ``steps``
    are 0-d float32 device counters (one per tensor; tensors may share one), advanced on the device."""
    (xp, gp, mp, vp), numels, gcode, scode = _mta_tables(X, G, [M, V])
    for s in steps:
        if not (s.is_cuda and s.dtype == torch.float32 and s.numel() == 1):
            raise TypeError("steps must be 0-d float32 GPU tensors")
    sp = ptr_table([s.data_ptr() for s in steps])
    lr_p, wd_p, wd_h = _scalar_args(lr, weight_decay, X[0].device)
    lib = _lib.load()
    check(lib.dion_adamw_step(xp, gp, gcode, mp, vp, scode, sp, numels, len(X), lr_p, float(beta1), float(beta2),
                              float(epsilon), wd_p, wd_h, int(bool(cautious_wd)), _stream_handle(X[0].device)),
          "adamw_step")


def lion_step(X: List[Tensor], G: List[Tensor], M: List[Tensor], lr: Tensor, beta1: float, beta2: float,
              weight_decay, cautious_wd: bool = False) -> None:
    """One fused Lion step over tensors of any sizes (dion/scalar_opts.py:68-118, :271-325)."""
    (xp, gp, mp), numels, gcode, scode = _mta_tables(X, G, [M])
    lr_p, wd_p, wd_h = _scalar_args(lr, weight_decay, X[0].device)
    lib = _lib.load()
    check(lib.dion_lion_step(xp, gp, gcode, mp, scode, numels, len(X), lr_p, float(beta1), float(beta2), wd_p, wd_h,
                             int(bool(cautious_wd)), _stream_handle(X[0].device)), "lion_step")
