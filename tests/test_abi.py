"""The C-ABI library loads and exports every symbol include/dion_hip.h declares (no compute)."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "dion_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dion_[a-z0-9_]+)\s*\(", text)))


def _declared_prototypes():
    """name -> list of C parameter declarations, from the header text."""
    text = open(os.path.join(ROOT, "include", "dion_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    out = {}
    for name, args in re.findall(r"\b(dion_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text):
        args = " ".join(args.split())
        out[name] = [] if args in ("", "void") else [a.strip() for a in args.split(",")]
    return out


def test_ctypes_prototypes_follow_the_header():
    """Argument count and kind (pointer / float / integer) of every ctypes prototype match the header."""
    import ctypes

    from dion_amd import _lib

    protos = _declared_prototypes()
    assert set(protos) == set(_declared_symbols())
    for name, cargs in protos.items():
        _res, argtypes = _lib.SIGNATURES[name]
        assert len(argtypes) == len(cargs), f"{name}: header has {len(cargs)} parameters, ctypes {len(argtypes)}"
        for decl, ct in zip(cargs, argtypes):
            if "*" in decl:
                kind = "ptr"
            elif decl.startswith("float"):
                kind = "float"
            else:
                kind = "int"
            if ct is ctypes.c_float:
                got = "float"
            elif ct in (ctypes.c_int, ctypes.c_int64, ctypes.c_size_t):
                got = "int"
            else:
                got = "ptr"
            assert kind == got, f"{name}: `{decl}` bound as {ct}"
            if kind == "int":
                want = ctypes.c_int64 if decl.startswith("int64_t") else \
                    ctypes.c_size_t if decl.startswith("size_t") else ctypes.c_int
                assert ct is want, f"{name}: `{decl}` bound as {ct}"


def test_header_declares_the_expected_surface():
    syms = _declared_symbols()
    for name in ["dion_ns_line_1", "dion_ns_line_2", "dion_ns_line_3", "dion_ns_orthogonalize",
                 "dion_ns_workspace_bytes", "dion_muon_pre", "dion_muon_post", "dion_normuon_stats",
                 "dion_dion2_accumulate", "dion_dion2_topk", "dion_dion2_gather", "dion_dion2_post",
                 "dion_last_error", "dion_abi_version"]:
        assert name in syms


def test_library_exports_every_declared_symbol():
    from dion_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("libdion_hip.so not built in this checkout")
    lib = _lib.load()
    for name in _declared_symbols():
        assert hasattr(lib, name), f"{name} declared in dion_hip.h but not exported"
        assert name in _lib.SIGNATURES, f"{name} has no ctypes prototype"
    assert lib.dion_abi_version() == _lib.ABI_VERSION
    # pure host entry points
    assert lib.dion_ns_workspace_bytes(0, 128, 128, 0) == 0
    n = lib.dion_ns_workspace_bytes(2, 768, 3072, 0)
    assert n >= 2 * 768 * 3072 * 2 * 3  # X ping-pong pair + one X^T
    assert lib.dion_ns_workspace_bytes(2, 3072, 768, 0) == n
    # Gram recurrence: four more m x m buffers, but only where it is used (long matrices)
    assert lib.dion_ns_workspace_bytes(2, 768, 3072, _lib.DION_NS_GRAM) >= n + 4 * 2 * 768 * 768 * 2
    assert lib.dion_ns_workspace_bytes(2, 768, 1024, _lib.DION_NS_GRAM) == lib.dion_ns_workspace_bytes(2, 768, 1024, 0)


def test_missing_library_is_a_hard_error(monkeypatch, tmp_path):
    from dion_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(ImportError):
        _lib.load()


def test_cpu_tensors_are_rejected():
    import torch

    from dion_amd import polar_express

    with pytest.raises(RuntimeError, match="no CPU path"):
        polar_express(torch.randn(8, 8))


def test_argument_validation_happens_before_any_device_work():
    """Bad arguments are refused on the host with DION_E_INVALID (-1) and a message, without a GPU."""
    import ctypes

    from dion_amd import _lib

    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("libdion_hip.so not built in this checkout")
    lib = _lib.load()
    f = ctypes.c_float

    def refused(rc, needle):
        assert rc == -1
        assert needle in lib.dion_last_error().decode()

    refused(lib.dion_slice_l1(None, 0, 1, 8, 8, 0, 0, None, None), "select_dim")
    refused(lib.dion_slice_l1(None, 7, 1, 8, 8, -2, 0, None, None), "dtype")
    refused(lib.dion_slice_l1(None, 0, 70000, 8, 8, -2, 0, None, None), "65535")
    refused(lib.dion_gather_slices(None, 0, 1, 8, 8, -2, None, 9, None, None), "k outside")
    refused(lib.dion_scatter_slices(None, 0, 1, 8, 8, -1, None, -1, None, None), "k outside")
    refused(lib.dion_mask_index(None, -1, 4, None, None), "bad size")
    refused(lib.dion_dion2_index_map(None, 1, 9, 8, None, None), "bad size")
    refused(lib.dion_dion2_post(None, 1, 1, 1, 8, 8, -2, None, 5, 2, None, None, None, None, f(1.0), None, f(0.0),
                                None), "u_dtype")
    refused(lib.dion_dion2_post(None, 1, 1, 1, 8, 8, 1, None, 0, 2, None, None, None, None, f(1.0), None, f(0.0),
                                None), "select_dim")
    refused(lib.dion_dion2_post(None, 3, 1, 1, 8, 8, -2, None, 0, 2, None, None, None, None, f(1.0), None, f(0.0),
                                None), "x_dtype")
    refused(lib.dion_dion2_post_masked(None, None, 1, 1, 0, 8, 8, -2, None, None, None, None, None, f(1.0), None,
                                       f(0.0), f(0.9), None), "bad size")
    refused(lib.dion_muon_pre(None, 0, None, 2, None, 1, 8, f(0.9), 0, None), "m_dtype")
    refused(lib.dion_adamw_step(None, None, 0, None, None, -1, None, None, 1, None, f(0.9), f(0.9), f(1e-8), None,
                                f(0.0), 0, None), "s_dtype")
    refused(lib.dion_ns_orthogonalize(None, 9, None, 1, 8, 8, None, 0, f(1.0), f(0.0), 0, 0, None, 0, None),
            "in_dtype")
    refused(lib.dion_ns_line_1(None, None, 1, 128, 128, None), "null argument")
    refused(lib.dion_ns_line_2(None, None, 1, 128, f(1.0), f(1.0), None), "null argument")
    refused(lib.dion_ns_line_3(None, None, None, 1, 128, 128, f(0.0), None), "null argument")
    refused(lib.dion_ns_line_1(None, None, 1, 100, 128, None), "multiples of 128")
    refused(lib.dion_ns_line_1(0x1002, 0x2000, 1, 128, 128, None), "X is not 16-byte aligned")
    refused(lib.dion_ns_line_2(0x1000, 0x2008, 1, 128, f(1.0), f(1.0), None), "B is not 16-byte aligned")
    refused(lib.dion_ns_line_3(0x1000, 0x2000, 0x3004, 1, 128, 128, f(0.0), None), "C is not 16-byte aligned")
    refused(lib.dion_ns_orthogonalize(0x1000, 0, 0x2002, 1, 128, 128, (ctypes.c_float * 3)(1.0, 1.0, 1.0), 1, f(1.0),
                                      f(0.0), 0, 0, 0x4000, 1 << 30, None), "out is not 16-byte aligned")
    # empty problems are accepted and do nothing
    assert lib.dion_slice_l1(None, 0, 0, 8, 8, -2, 0, None, None) == 0
    assert lib.dion_gather_slices(None, 0, 1, 8, 8, -2, None, 0, None, None) == 0
    assert lib.dion_dion2_index_map(None, 0, 0, 8, None, None) == 0
