"""The GEMM kernels issue the LDS reads of their MFMA fragments (ds_read_b128, ds_read_b64_tr_b16) from assembly and
wait for them with hand-counted s_waitcnt lgkmcnt(N), so the compiler does not know that a result is still on its
way when the statement has executed: it may hand a destination register it considers dead to something else, and a
read that lands late then overwrites that value (once: the lane index ahead of the epilogue's address arithmetic, a
GPU memory fault); and a wait counted one too high lets an MFMA read a fragment that has not arrived.  This test
compiles gemm_nt.hip to gfx950 assembly and walks every kernel (gemm_nt_kernel, gemm_qk_walk_kernel) in program
order (each loop back-edge taken once), modelling the LDS return queue (in-order; s_waitcnt lgkmcnt(N) retires all
but the newest N entries): no instruction may read or write a register while an LDS read into it is in flight.
Needs hipcc, no GPU."""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "dion_amd", "csrc", "gemm_nt.hip")


def _regs(tok):
    tok = tok.rstrip(",")
    m = re.match(r"v\[(\d+):(\d+)\]$", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"v(\d+)$", tok)
    return {int(m.group(1))} if m else set()


def walk(body):
    """Returns (number of LDS reads seen, list of hazards) for one kernel's assembly lines.

    The instruction stream is followed along both outcomes of every conditional branch, each branch
    outcome once, carrying the queues of outstanding reads as they stand on first arrival (so a loop
    body is walked a second time with what its first pass left in flight)."""
    labels = {l.split(":")[0].strip(): i for i, l in enumerate(body) if re.match(r"\.L\w+:", l.strip())}
    in_asm_at, inside = [], False
    for l in body:
        if "#ASMSTART" in l:
            inside = True
        elif "#ASMEND" in l:
            inside = False
        in_asm_at.append(inside)
    explored, hazards, reads = set(), {}, set()
    stack = [(0, [], [])]
    steps = 0
    while stack and steps < 4000000:
        pc, queue, vmq = stack.pop()
        while pc < len(body) and steps < 4000000:
            steps += 1
            cur, s = pc, body[pc].split(";")[0].strip()
            in_asm = in_asm_at[pc]
            pc += 1
            if not s or s.startswith(".") or s.endswith(":"):
                continue
            op, *args = s.split()
            if op == "s_endpgm":
                break
            if op.startswith("s_cbranch") or op == "s_branch":
                tgt = labels.get(args[0])
                if op == "s_branch":
                    if tgt is None or (cur, True) in explored:
                        break
                    explored.add((cur, True))
                    pc = tgt
                    continue
                if tgt is not None and (cur, True) not in explored:
                    explored.add((cur, True))
                    stack.append((tgt, list(queue), list(vmq)))
                if (cur, False) in explored:
                    break
                explored.add((cur, False))
                continue
            if op == "s_waitcnt":
                m = re.search(r"lgkmcnt\((\d+)\)", s)
                if m:
                    del queue[: max(0, len(queue) - int(m.group(1)))]
                m = re.search(r"vmcnt\((\d+)\)", s)
                if m:
                    del vmq[: max(0, len(vmq) - int(m.group(1)))]
                continue
            inflight = set().union(*[q for q in queue + vmq if q]) if queue or vmq else set()
            if re.match(r"(buffer|global|flat|scratch)_", op):
                # vector memory: returns in order, counted by vmcnt.  The destination of a load issued from an
                # assembly statement is in flight until a wait retires it (the compiler guards its own loads)
                is_load = in_asm and "_load" in op and "_lds_" not in op and not op.endswith("_lds")
                dest = _regs(args[0]) if is_load else set()
                touched = set().union(*[_regs(a) for a in args]) if args else set()
                if touched & inflight:
                    hazards[cur] = s
                vmq.append(dest)
                continue
            if op.startswith("ds_read"):
                dest = _regs(args[0])
                reads.add(cur)
                if dest & inflight:
                    hazards[cur] = s
                queue.append(dest)
                continue
            touched = set().union(*[_regs(a) for a in args]) if args else set()
            if touched & inflight:
                hazards[cur] = s
            if op.startswith("ds_") or op.startswith("s_load") or op.startswith("s_buffer_load"):
                queue.append(set())
    return len(reads), sorted(hazards.items())


def test_the_walk_flags_a_register_reused_before_the_wait():
    bad = ["ds_read_b64_tr_b16 v[10:11], v3", "v_and_b32_e32 v10, 63, v0", "s_waitcnt lgkmcnt(0)", "s_endpgm"]
    good = ["ds_read_b64_tr_b16 v[10:11], v3", "ds_read_b128 v[20:23], v4", "ds_read_b128 v[30:33], v4", "s_waitcnt lgkmcnt(1)",
            "v_mfma_f32_32x32x16_bf16 v[0:15], v[20:23], v[10:13], v[0:15]", "v_and_b32_e32 v10, 63, v0", "s_endpgm"]
    early = ["ds_read_b64_tr_b16 v[10:11], v3", "ds_read_b128 v[20:23], v4", "ds_read_b128 v[30:33], v4", "s_waitcnt lgkmcnt(2)",
             "v_mfma_f32_32x32x16_bf16 v[0:15], v[20:23], v[10:13], v[0:15]", "s_endpgm"]
    plain = ["ds_read_b128 v[20:23], v4", "ds_read_b128 v[24:27], v4 offset:4096", "s_waitcnt lgkmcnt(1)",
             "v_mfma_f32_32x32x16_bf16 v[0:15], v[20:23], v[24:27], v[0:15]", "s_endpgm"]
    two_loads = [";;#ASMSTART", "buffer_load_dwordx4 v[40:43], v1, s[4:7], s8 offen", ";;#ASMEND",
                 ";;#ASMSTART", "buffer_load_dwordx4 v[44:47], v1, s[4:7], s9 offen", ";;#ASMEND", "s_waitcnt vmcnt(1)"]
    staged_bad = two_loads + ["ds_write_b128 v2, v[44:47]", "s_endpgm"]
    staged_ok = two_loads + ["ds_write_b128 v2, v[40:43]", "s_endpgm"]
    assert walk(bad)[1] and not walk(good)[1] and walk(early)[1] and walk(plain)[1]
    assert walk(staged_bad)[1] and not walk(staged_ok)[1]


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="hipcc not on PATH")
def test_no_kernel_touches_a_register_a_transposing_read_is_in_flight_to(tmp_path):
    out = tmp_path / "gemm_nt.s"
    cmd = ["hipcc", "--offload-arch=gfx950", "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang",
           "-packed-fp32-ops", "-Wno-unused-command-line-argument", "-S", "--cuda-device-only", SRC, "-o", str(out)]
    subprocess.run(cmd, check=True, capture_output=True, timeout=900)
    kernels, name, body = {}, None, []
    for line in out.read_text().split("\n"):
        if name is None:
            if re.match(r"_ZN4dion\d+gemm_(nt|qk_walk)_kernel\S*:", line):
                name, body = line.split(":")[0], []
        else:
            body.append(line)
            if "s_endpgm" in line:
                kernels[name], name = body, None
    assert len(kernels) >= 22, "expected every gemm_nt_kernel / gemm_qk_walk_kernel instantiation in the assembly"
    assert sum("gemm_qk_walk_kernel" in k for k in kernels) == 2
    with_tr = 0
    for kname, kbody in kernels.items():
        n_reads, hazards = walk(kbody)
        assert n_reads > 0, kname
        with_tr += any("ds_read_b64_tr" in l for l in kbody)
        assert not hazards, (kname, hazards[:5])
    assert with_tr >= 8, "the K-major instantiations should contain transposing reads"
    # and nothing is spilled between the first and the last MFMA of a kernel (the software-pipelined loop)
    for kname, kbody in kernels.items():
        mfma = [i for i, l in enumerate(kbody) if "v_mfma" in l]
        assert not [l for l in kbody[mfma[0]:mfma[-1] + 1] if "scratch_" in l], kname
