"""dion_ns_orthogonalize_static -- the entry point that allocates nothing and brings its own fixed
device scratch array -- against dion_ns_orthogonalize (caller workspace), through the C ABI.

Both run the same driver and kernels, so the bar is bit equality of the bf16 outputs.  The array is
shared by every call on a GPU and keeps the previous call's contents: each case runs two calls in a
row, the second on a smaller input, and both must match."""
import ctypes

import pytest
import torch

from dion_amd import _lib
from dion_amd.newton_schulz import NS5_COEFFS, POLAR_EXPRESS_COEFFS

DEV = "cuda"


def _coeffs(table):
    flat = [float(v) for abc in table for v in abc]
    return (ctypes.c_float * len(flat))(*flat), len(flat) // 3


def _with_workspace(lib, G, table, norm_scale, eps, flags, reset):
    b, r, c = G.shape
    out = torch.empty(b, r, c, dtype=torch.bfloat16, device=G.device)
    carr, n = _coeffs(table)
    nbytes = lib.dion_ns_workspace_bytes(b, r, c, flags)
    ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=G.device)
    st = torch.cuda.current_stream(G.device).cuda_stream
    code = _lib.DION_BF16 if G.dtype == torch.bfloat16 else _lib.DION_F32
    _lib.check(lib.dion_ns_orthogonalize(G.data_ptr(), code, out.data_ptr(), b, r, c, carr, n, norm_scale, eps,
                                         flags, reset, ws.data_ptr(), ws.numel(), st), "dion_ns_orthogonalize")
    return out


def _static(lib, G, table, norm_scale, eps, flags, reset):
    b, r, c = G.shape
    out = torch.empty(b, r, c, dtype=torch.bfloat16, device=G.device)
    carr, n = _coeffs(table)
    st = torch.cuda.current_stream(G.device).cuda_stream
    code = _lib.DION_BF16 if G.dtype == torch.bfloat16 else _lib.DION_F32
    _lib.check(lib.dion_ns_orthogonalize_static(G.data_ptr(), code, out.data_ptr(), b, r, c, carr, n, norm_scale,
                                                eps, flags, reset, st), "dion_ns_orthogonalize_static")
    return out


CASES = [
    # (first shape, smaller second shape, coefficient table, norm_scale, flags, gram_reset, dtype)
    ((1, 768, 3072), (2, 256, 512), NS5_COEFFS, 1.0, 0, 0, torch.bfloat16),
    ((2, 1024, 512), (1, 200, 136), POLAR_EXPRESS_COEFFS, 1.02, 0, 0, torch.bfloat16),     # tall, then padded
    ((4, 640, 1280), (3, 128, 128), POLAR_EXPRESS_COEFFS, 1.02, _lib.DION_NS_GRAM, 2, torch.float32),
    ((2, 512, 2048), (5, 64, 768), NS5_COEFFS, 1.0, 0, 0, torch.bfloat16),                 # second: LDS-resident kernel
]


@pytest.mark.gpu
@pytest.mark.parametrize("case", range(len(CASES)))
def test_static_scratch_matches_caller_workspace(case):
    first, second, table, scale, flags, reset, dtype = CASES[case]
    lib = _lib.load()
    torch.manual_seed(100 + case)
    for shape in (first, second):
        print("dion_ns_orthogonalize_static case", case, "shape", shape, flush=True)
        G = torch.randn(shape, device=DEV).to(dtype)
        assert lib.dion_ns_workspace_bytes(*shape, flags) <= _lib.DION_NS_STATIC_SCRATCH_BYTES
        want = _with_workspace(lib, G, table, scale, 1e-7, flags, reset)
        got = _static(lib, G, table, scale, 1e-7, flags, reset)
        torch.cuda.synchronize()
        assert torch.equal(got, want), f"{shape}: static-scratch result differs from the caller-workspace result"
        assert torch.isfinite(got.float()).all()


@pytest.mark.gpu
def test_static_scratch_refuses_what_does_not_fit():
    lib = _lib.load()
    shape = (8, 2048, 4096)
    assert lib.dion_ns_workspace_bytes(*shape, 0) > _lib.DION_NS_STATIC_SCRATCH_BYTES
    G = torch.randn(shape, device=DEV).to(torch.bfloat16)
    out = torch.full(shape, 7.0, dtype=torch.bfloat16, device=DEV)
    carr, n = _coeffs(NS5_COEFFS)
    st = torch.cuda.current_stream().cuda_stream
    rc = lib.dion_ns_orthogonalize_static(G.data_ptr(), _lib.DION_BF16, out.data_ptr(), *shape, carr, n, 1.0, 1e-7,
                                          0, 0, st)
    assert rc == -2
    msg = lib.dion_last_error().decode()
    assert "fixed" in msg and str(_lib.DION_NS_STATIC_SCRATCH_BYTES) in msg
    torch.cuda.synchronize()
    assert bool((out == 7.0).all()), "a refused call must not touch the output"


@pytest.mark.gpu
def test_static_entry_point_allocates_no_device_memory():
    """Free device memory as the driver reports it (hipMemGetInfo) is the same before and after warm calls of
    the entry point: nothing is allocated or freed, on any of the three kernel routes (tiled, padded,
    LDS-resident).  Outputs are allocated before the reading is taken."""
    lib = _lib.load()
    torch.manual_seed(5)
    cases = [(2, 256, 512), (1, 200, 136), (5, 64, 768)]
    Gs = [torch.randn(shape, device=DEV).to(torch.bfloat16) for shape in cases]
    outs = [torch.empty_like(G) for G in Gs]
    carr, n = _coeffs(NS5_COEFFS)
    st = torch.cuda.current_stream().cuda_stream

    def call(G, out):
        b, r, c = G.shape
        _lib.check(lib.dion_ns_orthogonalize_static(G.data_ptr(), _lib.DION_BF16, out.data_ptr(), b, r, c, carr, n,
                                                    1.0, 1e-7, 0, 0, st), "dion_ns_orthogonalize_static")

    for G, out in zip(Gs, outs):  # warm: code objects loaded, the array's address resolved
        call(G, out)
    torch.cuda.synchronize()
    free_before, _total = torch.cuda.mem_get_info()
    for _ in range(3):
        for G, out in zip(Gs, outs):
            call(G, out)
    torch.cuda.synchronize()
    free_after, _total = torch.cuda.mem_get_info()
    assert free_after == free_before, (free_before, free_after)
