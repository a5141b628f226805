"""Compile the HIP sources under dion_amd/csrc into dion_amd/libdion_hip.so (gfx950 only)."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_PATH = os.path.join(HERE, "libdion_hip.so")
SOURCES = ["gemm_nt.hip", "elementwise.hip", "select_scope.hip", "ns_small.hip", "scalar_opts.hip", "capi.hip"]

# -packed-fp32-ops off: keep hipcc from forming v_pk_*_f32 out of scalar float code.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


# The step kernels keep the reference's separate multiply / add roundings (mul_ then add_), so no
# FMA contraction there; the GEMM epilogues may contract.
EXTRA_FLAGS = {"elementwise.hip": ["-ffp-contract=off"], "select_scope.hip": ["-ffp-contract=off"], "scalar_opts.hip": ["-ffp-contract=off"]}


def hipcc_path() -> str:
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cand = os.path.join(rocm, "bin", "hipcc")
    return cand if os.path.exists(cand) else "hipcc"


def build(verbose: bool = True) -> str:
    """Compile every source and link the shared library. Always recompiles."""
    objs = []
    procs = []
    for src in SOURCES:
        obj = os.path.join(CSRC, src.replace(".hip", ".o"))
        cmd = [hipcc_path(), *HIPCC_FLAGS, *EXTRA_FLAGS.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(obj)
    for src, proc in procs:
        out, _ = proc.communicate()
        lines = [l for l in out.splitlines() if "packed-fp32-ops" not in l]
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n" + "\n".join(lines))
        if verbose and lines:
            print("\n".join(lines))
    cmd = [hipcc_path(), "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB_PATH


C_CALLER_SRC = os.path.join(os.path.dirname(HERE), "tests", "c_caller", "ns_caller.c")
C_CALLER_BIN = os.path.join(os.path.dirname(HERE), "tests", "c_caller", "ns_caller")


def build_c_caller(verbose: bool = True) -> str:
    """The C program under tests/c_caller (a caller of the library with no Python or C++ in it), compiled
    with the host C compiler against include/dion_hip.h and linked to the library just built."""
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = ["gcc", "-std=c11", "-Wall", "-D__HIP_PLATFORM_AMD__", f"-I{rocm}/include",
           "-I" + os.path.join(os.path.dirname(HERE), "include"), C_CALLER_SRC, "-o", C_CALLER_BIN,
           "-L" + HERE, "-ldion_hip", f"-L{rocm}/lib", "-lamdhip64", "-lm",
           "-Wl,-rpath,$ORIGIN/../../dion_amd", f"-Wl,-rpath,{rocm}/lib"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return C_CALLER_BIN


if __name__ == "__main__":
    # `--c-caller` builds only the C test program (needs gcc and a built library); the default builds the
    # library (needs hipcc only) and, when gcc is there, the C test program as well.
    import shutil

    if "--c-caller" in sys.argv[1:]:
        print(build_c_caller())
        sys.exit(0)
    build()
    print(LIB_PATH)
    if shutil.which("gcc") is not None:
        print(build_c_caller())
    sys.exit(0)
