"""The library called from a C program (tests/c_caller/ns_caller.c, built with the host C compiler by
`python -m dion_amd._build --c-caller`): dion_ns_orthogonalize and dion_ns_orthogonalize_static through nothing
but the C header, the result checked in the program itself (rows orthonormal to the accuracy of five bf16
Polar-Express iterations, the two entry points bit-identical).  The program runs as a child process."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "c_caller", "ns_caller")


@pytest.mark.gpu
def test_c_program_orthogonalizes_through_the_c_abi():
    if not os.path.exists(BIN):
        import shutil

        if shutil.which("gcc") is None:
            pytest.skip("tests/c_caller/ns_caller is not built and gcc is not installed")
        from dion_amd import _build

        _build.build_c_caller(verbose=False)
    run = subprocess.run([BIN], capture_output=True, text=True, timeout=120)
    print(run.stdout, run.stderr)
    assert run.returncode == 0, (run.returncode, run.stdout, run.stderr)


def test_header_is_valid_c11(tmp_path):
    """include/dion_hip.h compiles as strict C11 on its own (no C++ in the boundary), and the caller compiles
    against it and the HIP runtime's C API with the host C compiler."""
    import shutil

    if shutil.which("gcc") is None:
        pytest.skip("gcc is not installed")
    inc = os.path.join(os.path.dirname(HERE), "include")
    tu = tmp_path / "only_header.c"
    tu.write_text('#include "dion_hip.h"\nint main(void) { return dion_abi_version() < 0; }\n')
    run = subprocess.run(["gcc", "-std=c11", "-Wall", "-Wextra", "-Werror", "-pedantic", "-fsyntax-only", "-I" + inc,
                          str(tu)], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, run.stderr
    if not os.path.exists("/opt/rocm/include/hip/hip_runtime_api.h"):
        pytest.skip("the HIP headers are not installed")
    run = subprocess.run(["gcc", "-std=c11", "-Wall", "-Werror", "-fsyntax-only", "-D__HIP_PLATFORM_AMD__",
                          "-I/opt/rocm/include", "-I" + inc, os.path.join(HERE, "c_caller", "ns_caller.c")],
                         capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, run.stderr
