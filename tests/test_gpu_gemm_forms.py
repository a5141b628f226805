"""The GEMM kernel through the C ABI (dion_ns_line_1/2/3) over the shapes that exercise every launch
path: 128- and 256-wide tiles, ragged tile counts, triangular enumeration past one super-block, batch
counts that do not divide the XCD count, X' = a X + B X with and without the addend.  Each result is
compared with the float64 product of the same bf16 inputs (error no worse than a bf16 torch matmul's);
repeated launches must reproduce the first bit for bit."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _lib():
    from dion_amd import _lib as L

    return L.load(), L.check


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _err(res, ref64):
    d = np.abs(res.float().cpu().numpy().astype(np.float64) - ref64)
    return d.mean(), d.max()


# (batch, m, n): m, n multiples of 128
SHAPES = [(1, 128, 128), (3, 128, 384), (5, 384, 128), (2, 640, 1152), (9, 256, 512), (1, 2304, 256),
          (7, 1280, 2560), (33, 512, 768), (2, 2560, 2304)]


@pytest.mark.parametrize("batch,m,n", SHAPES)
def test_line_1_and_2_all_tile_paths(batch, m, n):
    lib, check = _lib()
    torch.manual_seed(batch * 1000 + m + n)
    X = torch.randn(batch, m, n, device=DEV).to(torch.bfloat16)
    A = torch.empty(batch, m, m, device=DEV, dtype=torch.bfloat16)
    check(lib.dion_ns_line_1(X.data_ptr(), A.data_ptr(), batch, m, n, _stream()), "line_1")
    x64 = X.float().cpu().numpy().astype(np.float64)
    ref = x64 @ np.swapaxes(x64, -2, -1)
    mean, mx = _err(A, ref)
    bmean, bmx = _err(X @ X.mT, ref)
    assert mean <= bmean * 1.05 + 1e-6 and mx <= bmx * 1.5 + 1e-6
    assert torch.equal(A, A.mT)

    S = (A.float() / n ** 0.5).to(torch.bfloat16)  # symmetric, O(1) entries
    S = torch.maximum(S, S.mT)                     # exactly symmetric after the rescale
    B = torch.empty_like(S)
    check(lib.dion_ns_line_2(S.data_ptr(), B.data_ptr(), batch, m, ctypes.c_float(0.73), ctypes.c_float(-1.31),
                             _stream()), "line_2")
    s64 = S.float().cpu().numpy().astype(np.float64)
    ref2 = 0.73 * (s64 @ s64) - 1.31 * s64
    mean, mx = _err(B, ref2)
    bmean, bmx = _err(0.73 * (S @ S) - 1.31 * S, ref2)
    assert mean <= bmean * 1.05 + 1e-6 and mx <= bmx * 1.5 + 1e-6
    assert torch.equal(B, B.mT)


@pytest.mark.parametrize("a", [0.0, 3.4445])
@pytest.mark.parametrize("batch,m,n", SHAPES)
def test_line_3_all_tile_paths(batch, m, n, a):
    lib, check = _lib()
    torch.manual_seed(batch * 77 + m + n)
    X = torch.randn(batch, m, n, device=DEV).to(torch.bfloat16)
    Bm = torch.randn(batch, m, m, device=DEV)
    Bm = ((Bm + Bm.mT) / 2).to(torch.bfloat16)
    C = torch.empty_like(X)
    check(lib.dion_ns_line_3(Bm.data_ptr(), X.data_ptr(), C.data_ptr(), batch, m, n, ctypes.c_float(a), _stream()),
          "line_3")
    x64 = X.float().cpu().numpy().astype(np.float64)
    b64 = Bm.float().cpu().numpy().astype(np.float64)
    ref = a * x64 + b64 @ x64
    mean, mx = _err(C, ref)
    bmean, bmx = _err(a * X + Bm @ X, ref)
    assert mean <= bmean * 1.05 + 1e-6 and mx <= bmx * 1.5 + 1e-6


@pytest.mark.parametrize("batch,m,n", [(24, 512, 8192), (24, 512, 2048), (8, 256, 1024), (3, 128, 384)])
def test_line_3_short_reduction_many_launches(batch, m, n):
    """X' = B X with only a few k-slabs per tile, launched back to back: the epilogue starts right behind the
    last fragment reads of the main loop.  (Those reads are issued from assembly; their destination registers
    have to stay allocated until the LDS queue has drained, or the epilogue's addresses get overwritten.)
    Every launch must reproduce the first one bit for bit, and that one must be the product."""
    lib, check = _lib()
    torch.manual_seed(batch + m + n)
    X = torch.randn(batch, m, n, device=DEV).to(torch.bfloat16)
    Bm = torch.randn(batch, m, m, device=DEV)
    Bm = ((Bm + Bm.mT) / 2).to(torch.bfloat16)
    st = _stream()
    first = torch.empty_like(X)
    check(lib.dion_ns_line_3(Bm.data_ptr(), X.data_ptr(), first.data_ptr(), batch, m, n, ctypes.c_float(0.0), st),
          "line_3")
    ref = torch.bmm(Bm.float(), X.float())
    assert float((first.float() - ref).norm() / ref.norm()) <= 4e-3
    outs = [torch.empty_like(X) for _ in range(4)]
    for rep in range(40):
        out = outs[rep % 4]
        check(lib.dion_ns_line_3(Bm.data_ptr(), X.data_ptr(), out.data_ptr(), batch, m, n, ctypes.c_float(0.0), st),
              "line_3")
    torch.cuda.synchronize()
    assert all(torch.equal(o, first) for o in outs)
    # the transposed-output form of the same kernel is the last product of a tall orthogonalization
    from dion_amd import zeropower_via_newtonschulz5

    wide = zeropower_via_newtonschulz5(X)
    tall_in = X.mT.contiguous()
    for _ in range(6):
        assert torch.equal(zeropower_via_newtonschulz5(tall_in), wide.mT)


@pytest.mark.parametrize("batch,m,n", [(24, 512, 8192), (5, 1024, 14336), (3, 2304, 10240), (2, 4096, 8192),
                                       (33, 768, 4096), (4, 768, 8192), (3, 1280, 7168), (7, 2048, 3584)])
def test_line_3_thousand_tile_launches(batch, m, n):
    """X' = B X over hundreds to thousands of 256-wide tiles (tile counts that are and are not multiples of the
    CU count, so that workgroups of the tile-walking kernel -- reductions up to 2048 -- take unequal numbers
    of tiles; both tile orders; longer reductions on the one-tile-per-workgroup kernel): the product, and
    the same bits on every launch."""
    lib, check = _lib()
    torch.manual_seed(batch + m + n)
    X = torch.randn(batch, m, n, device=DEV).to(torch.bfloat16)
    Bm = torch.randn(batch, m, m, device=DEV)
    Bm = ((Bm + Bm.mT) / 2).to(torch.bfloat16)
    st = _stream()
    first = torch.empty_like(X)
    check(lib.dion_ns_line_3(Bm.data_ptr(), X.data_ptr(), first.data_ptr(), batch, m, n, ctypes.c_float(0.0), st),
          "line_3")
    ref = torch.bmm(Bm.float(), X.float())
    assert float((first.float() - ref).norm() / ref.norm()) <= 4e-3
    del ref
    for rep in range(3):
        C = torch.full_like(X, float("nan"))
        check(lib.dion_ns_line_3(Bm.data_ptr(), X.data_ptr(), C.data_ptr(), batch, m, n, ctypes.c_float(0.0), st),
              "line_3")
        assert torch.equal(C, first), rep
    if m <= 2048:
        # the transposed-output form (last product of a tall orthogonalization) of the same launches
        from dion_amd import zeropower_via_newtonschulz5

        del first, C
        wide = zeropower_via_newtonschulz5(X)
        tall_in = X.mT.contiguous()
        for _ in range(2):
            assert torch.equal(zeropower_via_newtonschulz5(tall_in), wide.mT)


def test_line_3_seeded_sweep_of_walked_tile_lists():
    """Twenty seeded (batch, m, n) with 256-wide tiles, reductions of 256..2048 and 384..1500 tiles: lists whose
    length is anything modulo the CU count, matrices that end in the middle of a workgroup's share."""
    lib, check = _lib()
    rng = np.random.default_rng(20240607)
    st = _stream()
    done = 0
    while done < 20:
        m = 256 * int(rng.integers(1, 9))
        n = 256 * int(rng.integers(1, 33))
        batch = int(rng.integers(1, 41))
        tiles = (m // 256) * (n // 256) * batch
        if not 384 <= tiles <= 1500:
            continue
        done += 1
        torch.manual_seed(done)
        X = torch.randn(batch, m, n, device=DEV).to(torch.bfloat16)
        Bm = torch.randn(batch, m, m, device=DEV)
        Bm = ((Bm + Bm.mT) / 2).to(torch.bfloat16)
        C = torch.full_like(X, float("nan"))
        check(lib.dion_ns_line_3(Bm.data_ptr(), X.data_ptr(), C.data_ptr(), batch, m, n, ctypes.c_float(0.0), st),
              "line_3")
        ref = torch.bmm(Bm.float(), X.float())
        err = float((C.float() - ref).norm() / ref.norm())
        assert err <= 4e-3, (batch, m, n, tiles, err)


def test_line_3_argument_errors():
    lib, check = _lib()
    from dion_amd._lib import DionHipError

    X = torch.zeros(1, 128, 128, device=DEV, dtype=torch.bfloat16)
    Y = torch.zeros(1, 128, 128, device=DEV, dtype=torch.bfloat16)
    with pytest.raises((DionHipError, ValueError)):
        check(lib.dion_ns_line_3(X.data_ptr(), X.data_ptr(), None, 1, 128, 128, ctypes.c_float(0.0), _stream()),
              "no output")
    with pytest.raises((DionHipError, ValueError)):
        check(lib.dion_ns_line_3(X.data_ptr(), X.data_ptr(), X.data_ptr(), 1, 128, 128, ctypes.c_float(0.0),
                                 _stream()), "in place")
    with pytest.raises((DionHipError, ValueError)):
        check(lib.dion_ns_line_3(X.data_ptr(), X.data_ptr(), Y.data_ptr(), 1, 100, 128, ctypes.c_float(0.0),
                                 _stream()), "extent not a multiple of 128")
