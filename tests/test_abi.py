"""The C-ABI library loads and exports every symbol include/dion_hip.h declares (no compute)."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "dion_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dion_[a-z0-9_]+)\s*\(", text)))


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
    assert lib.dion_abi_version() >= 1
    # pure host entry points
    assert lib.dion_ns_workspace_bytes(0, 128, 128, 0) == 0
    n = lib.dion_ns_workspace_bytes(2, 768, 3072, 0)
    assert n >= 2 * 768 * 3072 * 2 * 3  # X ping-pong pair + one X^T
    assert lib.dion_ns_workspace_bytes(2, 3072, 768, 0) == n
    assert lib.dion_ns_workspace_bytes(2, 768, 3072, _lib.DION_NS_CARRY_XT) >= n + 2 * 768 * 3072 * 2


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
