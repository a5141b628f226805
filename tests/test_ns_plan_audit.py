"""Host-only walk over the launch lists of the orthogonalization driver (no GPU, no device work).

dion_ns_orthogonalize plans a call first -- workspace layout and every kernel launch with its operands
-- and checks the list against the buffers the call owns before the first launch.  This test runs
that planner and checker through dion_ns_plan_audit for every shape of the benchmark configurations
(wide, tall, padded, per-head, Dion2 sub-matrices), every schedule length, Gram on and off and the
fused-update form: each launch must read inside {input, workspace} and write inside {workspace,
output, parameter}, with tile shapes that divide the padded extents.  It also shows the check has
teeth: the same plans audited against a workspace that is too short must be refused, naming the
launch and the operand."""
import os

import pytest

from dion_amd import _lib

pytestmark = pytest.mark.skipif(not os.path.exists(_lib.LIB_PATH), reason="libdion_hip.so not built in this checkout")

BF16, F32, GRAM = _lib.DION_BF16, _lib.DION_F32, _lib.DION_NS_GRAM

# (batch, rows, cols) of every shape group of the benchmark configurations, plus ragged ones
CONFIG_SHAPES = [
    (1, 768, 3072),                                                            # one matrix
    (12, 2304, 768), (12, 768, 768), (12, 3072, 768), (12, 768, 3072),         # GPT-small
    (432, 64, 768),                                                            # per-head (LDS-resident kernel)
    (24, 6144, 2048), (24, 2048, 2048), (24, 8192, 2048), (24, 2048, 8192),    # GPT-1.3B
    (24, 6144, 512), (24, 512, 2048), (24, 8192, 512), (24, 512, 8192),        # Dion2 sub-matrices, fraction 0.25
    (64, 4096, 4096), (64, 1024, 4096), (64, 14336, 4096), (32, 4096, 14336),  # Llama-3-8B
    (8, 4096, 4096), (8, 1024, 4096), (8, 14336, 4096), (4, 4096, 14336),      # one GPU's share of eight
]
RAGGED_SHAPES = [(3, 256, 512), (3, 512, 256), (3, 128, 128), (3, 100, 36), (1, 17, 33), (2, 48, 1000), (2, 1000, 130),
                 (5, 768, 64), (2, 100, 200), (3, 100, 300), (1, 200, 136), (7, 65, 65), (2, 129, 257), (1, 1, 1),
                 (300, 72, 80)]


def _audit(lib, shape, n_iters=5, flags=0, in_dtype=BF16, with_update=0, x_dtype=F32, mats_per_ptr=1, ws=0, reset=2):
    b, r, c = shape
    return lib.dion_ns_plan_audit(b, r, c, in_dtype, n_iters, flags, reset, with_update, x_dtype, mats_per_ptr, ws)


@pytest.mark.parametrize("shape", CONFIG_SHAPES + RAGGED_SHAPES)
def test_every_launch_stays_inside_the_calls_buffers(shape):
    lib = _lib.load()
    b, r, c = shape
    small = min(r, c) <= 64
    for flags in (0, GRAM):
        for n_iters in (0, 1, 5):
            for in_dtype in (BF16, F32):
                n = _audit(lib, shape, n_iters, flags, in_dtype)
                assert n > 0, (shape, flags, n_iters, lib.dion_last_error().decode())
                if small:
                    assert n == 1  # one LDS-resident launch
                elif not flags or max(r, c) < 3 * min(r, c):
                    # norm + prepare + three GEMMs per iteration (+ unpad when padding is in the way); a wide
                    # bf16 input that fills whole tiles is read where it lies: no prepare pass
                    in_place = (in_dtype == BF16 and r <= c and n_iters > 0
                                and bool(lib.dion_ns_accepts_prepared(b, r, c, flags, n_iters)))
                    want = (1 + 3 * n_iters,) if in_place else (2 + 3 * n_iters, 3 + 3 * n_iters)
                    assert n in want, (shape, n_iters, in_dtype, n)
                else:
                    assert n >= 2 + n_iters


@pytest.mark.parametrize("shape", [s for s in CONFIG_SHAPES if min(s[1:]) > 64 and s[1] % 128 == 0 and s[2] % 128 == 0])
def test_fused_update_launches_stay_inside_the_parameters(shape):
    lib = _lib.load()
    b = shape[0]
    for x_dtype in (F32, BF16):
        for flags in (0, GRAM):
            for mpp in sorted({1, 2 if b % 2 == 0 else 1, b}):
                n = _audit(lib, shape, 5, flags, BF16, with_update=1, x_dtype=x_dtype, mats_per_ptr=mpp)
                assert n > 0, (shape, flags, mpp, lib.dion_last_error().decode())
    # more than 64 parameters: the last GEMM is split into launches of 64 pointers each
    n1 = _audit(lib, (shape[0], shape[1], shape[2]), 5, 0, BF16, with_update=1)
    in_place = shape[1] <= shape[2] and bool(lib.dion_ns_accepts_prepared(b, shape[1], shape[2], 0, 5))
    assert n1 == (1 if in_place else 2) + 3 * 4 + 2 + (b + 63) // 64  # norm (+ prepare), 4 iterations, A, B, last X' 


def test_padded_shapes_do_not_take_the_fused_update():
    lib = _lib.load()
    for shape in [(3, 100, 300), (5, 768, 64), (432, 64, 768)]:
        assert _audit(lib, shape, 5, 0, BF16, with_update=1) == -1
        assert "does not take the fused update" in lib.dion_last_error().decode()


@pytest.mark.parametrize("shape", [(1, 768, 3072), (12, 2304, 768), (3, 512, 256), (3, 100, 300), (2, 1000, 130),
                                   (32, 4096, 14336)])
def test_a_short_workspace_is_caught_launch_by_launch(shape):
    lib = _lib.load()
    for flags in (0, GRAM):
        total = lib.dion_ns_workspace_bytes(*shape, flags)
        assert _audit(lib, shape, 5, flags, ws=total) > 0
        # short by the last buffer of the layout (the reciprocal norms, one 256-byte slot)
        assert _audit(lib, shape, 5, flags, ws=total - 256) == -1
        msg = lib.dion_last_error().decode()
        # (the norm is launch 0, or launch 1 behind the transposing copy of a tall input)
        assert "(frobenius norm)" in msg and "reciprocal norms" in msg, msg
        # cut in the middle of the layout: whatever launch first touches a buffer past the cut is named
        x_bytes = 2 * shape[0] * max(shape[1], shape[2]) * min(shape[1], shape[2])
        assert _audit(lib, shape, 5, flags, ws=x_bytes // 2) == -1
        msg = lib.dion_last_error().decode()
        assert "outside the call's buffers" in msg, msg


def test_static_scratch_limit_is_checked_before_any_device_work():
    import ctypes

    lib = _lib.load()
    c = (ctypes.c_float * 15)(*[1.0] * 15)
    rc = lib.dion_ns_orthogonalize_static(0x1000, BF16, 0x2000, 8, 2048, 4096, c, 5, ctypes.c_float(1.0),
                                          ctypes.c_float(0.0), 0, 0, None)
    assert rc == -2
    msg = lib.dion_last_error().decode()
    assert str(_lib.DION_NS_STATIC_SCRATCH_BYTES) in msg and "caller workspace" in msg


def _audit_prepared(lib, shape, n_iters=5, flags=0, with_update=0, x_dtype=F32, mats_per_ptr=1, ws=0, reset=2):
    b, r, c = shape
    return lib.dion_ns_plan_audit_prepared(b, r, c, n_iters, flags, reset, with_update, x_dtype, mats_per_ptr, ws)


@pytest.mark.parametrize("shape", CONFIG_SHAPES + RAGGED_SHAPES)
def test_prepared_input_plans(shape):
    """The prepared form (input in the iteration's layout, norm partials from the caller): taken exactly by
    the shapes that fill whole tiles; no norm pass over the input (one small launch turns the partial sums
    into the per-matrix factor) and no transposing copy of a tall one, every launch
    inside the call's buffers, the fused update included."""
    lib = _lib.load()
    b, r, c = shape
    for flags in (0, GRAM):
        takes = bool(lib.dion_ns_accepts_prepared(b, r, c, flags, 5))
        whole = min(r, c) > 64 and r % 128 == 0 and c % 128 == 0
        if takes:
            assert whole, shape
        if not whole:
            assert not takes, shape
        n = _audit_prepared(lib, shape, 5, flags)
        if not takes:
            assert n == -1 and "does not take a prepared input" in lib.dion_last_error().decode(), shape
            continue
        # the plain form of the same call: a norm launch where this one finalizes the caller's partial sums,
        # plus the transposing copy of a tall input (a wide one is read where it lies in both forms)
        plain = _audit(lib, shape, 5, flags)
        assert n == plain - (1 if r > c else 0), (shape, flags, n, plain)
        assert _audit_prepared(lib, shape, 0, flags) == -1  # no iteration to carry the normalisation
        for x_dtype in (F32, BF16):
            assert _audit_prepared(lib, shape, 5, flags, with_update=1, x_dtype=x_dtype) > 0, \
                (shape, lib.dion_last_error().decode())
        # a workspace cut short is caught for this form too
        assert _audit_prepared(lib, shape, 5, flags, ws=4096) == -1
