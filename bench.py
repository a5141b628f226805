#!/usr/bin/env python3
"""Benchmark of the Muon optimizer-step hot path on one MI355X.

A "step" is one full ``Muon.step()`` over synthetic parameters of the named model shape list
(momentum + Nesterov, batched Newton-Schulz orthogonalization, weight decay + update), inputs
resident in HBM.  ``value`` is the algorithmic Newton-Schulz TFLOP/s of the whole step,
``5*(4 m^2 n + 2 m^3)`` FLOP per matrix (the reference's benchmark/benchmark_newton_shultz.py:40-49
convention, not reduced for symmetry) summed over all matrices, divided by the full step time.

Prints ONE JSON line; see --help for the workloads.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA
PEAK_HBM_GBS = 8000.0

# (name, rows, cols, count) per workload; counts are whole-model totals.
WORKLOADS = {
    # Llama-3-8B: 32 layers, d 4096, GQA 32q/8kv, MLP 14336
    "llama3_8b": [("q_o", 4096, 4096, 64), ("k_v", 1024, 4096, 64), ("gate_up", 14336, 4096, 64),
                  ("down", 4096, 14336, 32)],
    # GPT-small 160M: 12 layers, d 768
    "gpt_small": [("qkv", 2304, 768, 12), ("attn_out", 768, 768, 12), ("fc", 3072, 768, 12),
                  ("proj", 768, 3072, 12)],
    # 1.3B: 24 layers, d 2048, MLP 8192
    "gpt_1p3b": [("qkv", 6144, 2048, 24), ("out", 2048, 2048, 24), ("fc", 8192, 2048, 24),
                 ("proj", 2048, 8192, 24)],
    # what one GPU of an 8-GPU node would run for llama3_8b: ceil(N/8) whole matrices of every shape
    # group through orthogonalization, and the same element count through momentum / update
    "llama3_8b_share8": [("q_o", 4096, 4096, 8), ("k_v", 1024, 4096, 8), ("gate_up", 14336, 4096, 8),
                         ("down", 4096, 14336, 4)],
    # the headline shape group on its own
    "ns_4096x14336": [("down", 4096, 14336, 32)],
    # a single 768x3072 matrix (the reference's CPU-runnable case): pure launch latency on a GPU
    "one_768x3072": [("proj", 768, 3072, 1)],
    # GPT-small with per-head Newton-Schulz on the fused qkv weight (36 heads of 64x768 per layer)
    "gpt_small_heads": [("qkv", 2304, 768, 12), ("attn_out", 768, 768, 12), ("fc", 3072, 768, 12),
                        ("proj", 768, 3072, 12)],
}
NUM_HEADS = {"gpt_small_heads": {"qkv": 36}}


def ns_flops(rows: int, cols: int, iters: int = 5) -> float:
    m, n = min(rows, cols), max(rows, cols)
    return iters * (4.0 * m * m * n + 2.0 * m ** 3)


def cpu_baseline(ns: str):
    """Oracle (torch-CPU restatement of the reference's bf16 path) timed on the host cores on a
    bounded sample: one 4096x14336 matrix, Frobenius normalisation + 5 iterations."""
    import torch

    from oracle import dion_oracle as oracle

    cores = os.cpu_count() or 1
    cores = min(cores, int(os.environ.get("OMP_NUM_THREADS", cores)))
    torch.set_num_threads(cores)
    g = torch.Generator().manual_seed(1234)
    G = (torch.randn(4096, 14336, generator=g) * 0.02).to(torch.bfloat16)
    oracle.ns_bf16(G[:256, :1024].contiguous())  # warm the thread pool
    done, t0 = 0, time.perf_counter()
    while done < 32:
        if ns == "polar_express":
            oracle.polar_express_bf16(G, eps=1e-8)
        else:
            oracle.ns_bf16(G, oracle.NS5_COEFFS, 1.0, 1e-8)
        done += 1
        if time.perf_counter() - t0 > 12.0:
            break
    dt = time.perf_counter() - t0
    return {
        "value": round(done * ns_flops(4096, 14336) / dt * 1e-12, 4),
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "sample": f"{done} of the 32 4096x14336 matrices of the headline group, Frobenius normalisation + "
                  f"5 {ns} iterations each, torch-CPU bf16 matmul, {dt:.1f} s",
    }


def measured_traffic():
    """HBM bytes per launch of the dominant kernel, from the committed rocprofv3 --pmc summary
    (profiles/gemm_xprime_traffic.json: FETCH_SIZE + WRITE_SIZE, each scaled by the same counter's
    reading for a streaming kernel of known traffic in the same run).  None when
    the file is absent."""
    path = os.path.join(ROOT, "profiles", "gemm_xprime_traffic.json")
    try:
        with open(path) as f:
            return json.load(f).get("hbm_bytes_per_launch")
    except (OSError, ValueError):
        return None


def main() -> int:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload", default="llama3_8b", choices=sorted(WORKLOADS))
    ap.add_argument("--ns", default="ns5", choices=["ns5", "polar_express", "gram"])
    ap.add_argument("--optimizer", default="muon", choices=["muon", "normuon", "dion2", "nordion2"])
    ap.add_argument("--selection-scope", default="local", choices=["local", "global"],
                    help="dion2 / nordion2: 'global' runs the whole-matrix sequence (accumulate, select inside the "
                         "orthogonalization call, masked update) that a rank runs on assembled matrices")
    ap.add_argument("--state-dtype", default="fp32", choices=["fp32", "bf16"],
                    help="dtype of parameters and optimizer state (the headline configuration is fp32)")
    ap.add_argument("--two-call-update", action="store_true",
                    help="Muon: orthogonalize and update as two library calls instead of the fused one")
    ap.add_argument("--graph", action="store_true",
                    help="capture the step into a hipGraph during warm-up and time replays (needs --warmup >= 2)")
    ap.add_argument("--breakdown", action="store_true",
                    help="also time momentum / orthogonalization / update of every shape group on its own "
                         "(adds a 'groups' list to the JSON line)")
    ap.add_argument("--stream-compare", action="store_true",
                    help="time muon_pre / muon_post on the headline group next to a plain device copy that moves the "
                         "same number of bytes (adds a 'streaming' object to the JSON line)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-variants", action="store_true",
                    help="skip timing the step with the Polar-Express and Gram schedules (default Muon run only)")
    ap.add_argument("--no-kernel-timing", action="store_true")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="skip timing the Muon step of the smaller workloads (default llama3_8b Muon run only)")
    args = ap.parse_args()

    if args.gpus != 1:
        print("bench.py: this build drives one GPU per process and has no multi-GPU path; "
              "run with --gpus 1 (the step of an N-GPU job is this step on 1/N of each shape group).",
              file=sys.stderr)
        return 2

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    from dion import Dion2, Muon, NorDion2, NorMuon
    from dion_amd import _lib, ops

    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    spec = WORKLOADS[args.workload]

    others = None
    # ---- the Muon step of the smaller workloads (default run only): the regimes below the headline size,
    # timed by whoever runs this file rather than quoted.  Same optimizer settings, same FLOP convention.
    # They run first: after the headline step the chip is at its power limit, which these short launches
    # pay for in clock (GPT-small 2.1 instead of 1.8 ms).
    if args.workload == "llama3_8b" and args.optimizer == "muon" and args.ns == "ns5" and not args.graph \
            and not args.two_call_update and args.state_dtype == "fp32" and not args.no_other_workloads:
        others = {}
        gen = torch.Generator(device=dev).manual_seed(4321)
        for wname, wsteps in (("gpt_1p3b", 10), ("gpt_small", 30), ("gpt_small_heads", 30), ("one_768x3072", 30)):
            wgroups, wflops = [], 0.0
            for name, rows, cols, count in WORKLOADS[wname]:
                these = []
                for _ in range(count):
                    p = torch.nn.Parameter(torch.empty(rows, cols, device=dev).normal_(0.0, 0.02, generator=gen))
                    p.grad_dtype = None
                    p.grad = torch.empty(rows, cols, device=dev).normal_(0.0, 0.02, generator=gen).to(torch.bfloat16)
                    these.append(p)
                heads = NUM_HEADS.get(wname, {}).get(name)
                wgroups.append({"params": these, "num_heads": heads} if heads else {"params": these})
                r, c = (rows // heads, cols) if heads else (rows, cols)
                wflops += count * (heads or 1) * ns_flops(r, c)
            wopt = Muon(wgroups, lr=0.02, mu=0.95, nesterov=True, weight_decay=0.01, adjust_lr="spectral_norm")
            for _ in range(3):
                wopt.step()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(wsteps):
                wopt.step()
            torch.cuda.synchronize()
            wms = (time.perf_counter() - t0) * 1e3 / wsteps
            others[wname] = {"ms_per_step": round(wms, 3), "tflops": round(wflops / (wms * 1e-3) * 1e-12, 2),
                             "pct_of_bf16_peak": round(100.0 * wflops / (wms * 1e-3) * 1e-12 / PEAK_BF16_TFLOPS, 2),
                             "matrices": ", ".join(f"{c}x({r}x{k})" for _n, r, k, c in WORKLOADS[wname])}
            del wopt, wgroups
            ops.release_workspaces()
            torch.cuda.empty_cache()


    # ---- synthetic model: X ~ N(0, 0.02), G ~ N(0, 0.02) bf16, momentum zeros in the dtype of X (fp32 unless
    # --state-dtype bf16)
    sdt = torch.float32 if args.state_dtype == "fp32" else torch.bfloat16
    params = []
    groups = []
    gen = torch.Generator(device=dev).manual_seed(1234)
    total_flops = 0.0
    total_elems = 0
    fraction = 0.25
    for name, rows, cols, count in spec:
        these = []
        for _ in range(count):
            p = torch.nn.Parameter(torch.empty(rows, cols, device=dev).normal_(0.0, 0.02, generator=gen).to(sdt))
            p.grad_dtype = None
            p.grad = torch.empty(rows, cols, device=dev).normal_(0.0, 0.02, generator=gen).to(torch.bfloat16)
            these.append(p)
        params += these
        heads = NUM_HEADS.get(args.workload, {}).get(name)
        groups.append({"params": these, "num_heads": heads} if heads else {"params": these})
        r, c = (rows // heads, cols) if heads else (rows, cols)
        mult = heads or 1
        if args.optimizer == "dion2":  # NS runs on the selected quarter of the shorter dimension
            k = -(-min(r, c) * 25 // 100)
            r, c = (k, c) if r <= c else (r, k)
        elif args.optimizer == "nordion2":  # always the selected quarter of the rows
            r = -(-r * 25 // 100)
        total_flops += count * mult * ns_flops(r, c)
        total_elems += count * rows * cols
    ns_kw = dict(use_polar_express=(args.ns == "polar_express"), use_gram_newton_schulz=(args.ns == "gram"))
    if args.optimizer == "muon":
        opt = Muon(groups, lr=0.02, mu=0.95, nesterov=True, weight_decay=0.01, adjust_lr="spectral_norm", **ns_kw)
    elif args.optimizer == "normuon":
        opt = NorMuon(groups, lr=0.02, mu=0.95, muon_beta2=0.95, nesterov=True, weight_decay=0.01,
                      adjust_lr="spectral_norm", **ns_kw)
    elif args.optimizer == "nordion2":
        opt = NorDion2(groups, lr=0.02, fraction=fraction, mu=0.95, muon_beta2=0.95, weight_decay=0.01,
                       adjust_lr="spectral_norm", selection_scope=args.selection_scope, **ns_kw)
    else:
        opt = Dion2(groups, lr=0.02, fraction=fraction, ef_decay=0.95, weight_decay=0.01,
                    adjust_lr="spectral_norm", selection_scope=args.selection_scope, **ns_kw)
    if args.two_call_update:
        opt.fused_update = False
    if args.selection_scope == "global":
        if args.optimizer not in ("dion2", "nordion2"):
            print("bench.py: --selection-scope applies to dion2 / nordion2", file=sys.stderr)
            return 2
        opt.assembled_selection = True

    if args.graph:
        if args.warmup < 2:
            print("bench.py: --graph needs --warmup >= 2 (one eager step, one capture step)", file=sys.stderr)
            return 2
        from dion.cuda_graph import CudaGraphOptimizer

        opt = CudaGraphOptimizer(opt, warmup_steps=args.warmup - 1)
    for _ in range(args.warmup):
        opt.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        opt.step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps
    value = total_flops / (ms_per_step * 1e-3) * 1e-12

    # ---- the other orthogonalization schedules of the same step (default Muon run only): one warm
    # step and three timed ones each, on the same parameters
    variants = None
    if args.optimizer == "muon" and args.ns == "ns5" and not args.graph and not args.two_call_update \
            and not args.no_variants:
        variants = {}
        for vname, vkw in (("polar_express", dict(use_polar_express=True)),
                           ("gram", dict(use_polar_express=True, use_gram_newton_schulz=True))):
            fresh = [{k: g[k] for k in ("params", "num_heads") if k in g} for g in groups]
            vopt = Muon(fresh, lr=0.02, mu=0.95, nesterov=True, weight_decay=0.01, adjust_lr="spectral_norm", **vkw)
            vopt.step()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(3):
                vopt.step()
            torch.cuda.synchronize()
            vms = (time.perf_counter() - t0) * 1e3 / 3
            variants[vname] = {"ms_per_step": round(vms, 3),
                               "tflops": round(total_flops / (vms * 1e-3) * 1e-12, 2),
                               "pct_of_bf16_peak": round(100.0 * total_flops / (vms * 1e-3) * 1e-12 / PEAK_BF16_TFLOPS, 2)}
            del vopt

    result = {
        "metric": "Newton-Schulz TFLOP/s (% bf16 MFMA peak) + full optimizer-step ms, 1 GPU",
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 3),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": f"{args.workload}: full {type(getattr(opt, 'optimizer', opt)).__name__}.step() ("
                        + ("hipGraph replay, " if args.graph else "") + f"{args.ns}, wd 0.01, lr 0.02"
                        + ({"dion2": ", fraction 0.25, ef_decay 0.95", "nordion2": ", fraction 0.25, mu 0.95"}
                           .get(args.optimizer, ", nesterov mu=0.95"))
                        + (", whole-matrix selection" if args.selection_scope == "global" else "")
                        + (", bf16 parameters and state" if args.state_dtype == "bf16" else "")
                        + (", two-call update" if args.two_call_update else "")
                        + (", muon_beta2 0.95" if args.optimizer in ("normuon", "nordion2") else "") + ") over "
                        + ", ".join(f"{c}x({r}x{k})" for _n, r, k, c in spec),
            "matrices": sum(c for *_x, c in spec),
            "elements": total_elems,
            "ns_flop_per_step": total_flops,
        },
        "pct_of_bf16_peak": round(100.0 * value / PEAK_BF16_TFLOPS, 2),
    }
    if variants is not None:
        # same step, same FLOP convention (the standard iteration's count), other schedules
        result["variants"] = variants
    if others is not None:
        result["other_workloads"] = others

    # ---- free the model, then time kernels of the headline shape group on their own
    del opt
    for p in params:
        p.grad = None
    del params
    ops.release_workspaces()
    torch.cuda.empty_cache()

    if not args.no_kernel_timing:
        lib = _lib.load()
        B, m, n = 32, 4096, 14336
        if args.workload in ("gpt_small", "gpt_small_heads"):
            B, m, n = 12, 768, 3072
        elif args.workload == "one_768x3072":
            B, m, n = 1, 768, 3072
        elif args.workload == "gpt_1p3b":
            B, m, n = 24, 2048, 8192
        st = torch.cuda.current_stream().cuda_stream
        X = (torch.randn(B, m, n, device=dev) * 0.01).to(torch.bfloat16)
        Bm = (torch.randn(B, m, m, device=dev) * 0.01)
        Bm = ((Bm + Bm.mT) * 0.5).to(torch.bfloat16)
        C = torch.empty_like(X)

        def time_kernel(fn, iters=10):
            # warm-up: at least 30 ms of the same launches, so that short kernels are not timed while the
            # clocks are still coming up from idle (24 x (2048 x 8192) X X^T: 0.93 ms cold, 0.80 ms warm)
            fn()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            fn()
            torch.cuda.synchronize()
            once = max(time.perf_counter() - t0, 1e-6)
            for _ in range(min(2000, int(0.03 / once))):
                fn()
            torch.cuda.synchronize()
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(iters):
                fn()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / iters

        # The three GEMMs of one iteration on the headline group, each timed on its own with events on
        # the launch stream.  "executed" counts the MFMA work actually issued (upper-triangle tiles only
        # for the two symmetric products), "algorithmic" the full product.
        A = torch.empty(B, m, m, device=dev, dtype=torch.bfloat16)
        # executed share of a symmetric product: upper tiles only, with the tile edge the library picks
        T = m // lib.dion_gemm_tile_edge(B, m, m, 1)
        tri = (T + 1) / (2.0 * T)
        ms1 = time_kernel(lambda: lib.dion_ns_line_1(X.data_ptr(), A.data_ptr(), B, m, n, st))
        ms2 = time_kernel(lambda: lib.dion_ns_line_2(Bm.data_ptr(), A.data_ptr(), B, m, 1.0, 1.0, st))
        # dominant kernel: X' = B X with a*I folded into B, reading X as it lies; one launch per NS
        # iteration
        ms3 = time_kernel(lambda: lib.dion_ns_line_3(Bm.data_ptr(), X.data_ptr(), C.data_ptr(), B, m, n, 0.0, st))
        # the vendor library's bf16 GEMM (hipBLASLt behind torch.bmm) on the same operands, same box, same
        # run: the full product X X^T ("NT": both operands contiguous along the reduction index) and
        # B X ("NN": X read as it lies, the form of the dominant launch)
        ms_v_nt = time_kernel(lambda: torch.bmm(X, X.mT, out=A))
        ms_v_nn = time_kernel(lambda: torch.bmm(Bm, X, out=C))
        result["vendor_bf16_gemm"] = {
            "X X^T, full product": {"ms": round(ms_v_nt, 4),
                                    "tflops": round(2.0 * B * m * m * n / (ms_v_nt * 1e-3) * 1e-12, 1)},
            "B X": {"ms": round(ms_v_nn, 4), "tflops": round(2.0 * B * m * m * n / (ms_v_nn * 1e-3) * 1e-12, 1)},
        }
        del A

        def gemm_row(ms, flop_full, executed_share):
            ex = flop_full * executed_share / (ms * 1e-3) * 1e-12
            return {"ms": round(ms, 4), "tflops_executed": round(ex, 1),
                    "frac_executed": round(ex / PEAK_BF16_TFLOPS, 4),
                    "tflops_algorithmic": round(flop_full / (ms * 1e-3) * 1e-12, 1)}

        result["gemms"] = {
            "A = X X^T": gemm_row(ms1, 2.0 * B * m * m * n, tri),
            "B = c A A + b A + a I": gemm_row(ms2, 2.0 * B * m * m * m, tri),
            "X' = B X": gemm_row(ms3, 2.0 * B * m * m * n, 1.0),
        }
        flop3 = 2.0 * B * m * m * n
        achieved = flop3 / (ms3 * 1e-3) * 1e-12
        result["roofline"] = {
            "bound": "mfma",
            "kernel": "gemm_nt_kernel<256x256x64, 8 waves, 16x16x32 MFMAs, direct-to-LDS loads, K-major second operand> (X' = B X)",
            "achieved": round(achieved, 2),
            "peak": PEAK_BF16_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
            "traffic": measured_traffic() if (B, m, n) == (32, 4096, 14336) else None,
            "algorithmic_bytes": B * (m * m + 2 * m * n) * 2,
            "launch_ms": round(ms3, 4),
            "launch_shape": f"{B}x({m}x{m})·({m}x{n})",
        }
        # whole NS on the headline group
        from dion_amd import polar_express, zeropower_via_newtonschulz5

        from dion_amd import gram_newton_schulz

        fn = {"polar_express": polar_express, "gram": gram_newton_schulz}.get(args.ns, zeropower_via_newtonschulz5)
        del C, Bm
        ms_ns = time_kernel(lambda: fn(X, 1e-8), iters=3)
        ns_tf = B * ns_flops(m, n) / (ms_ns * 1e-3) * 1e-12
        result["ns_headline"] = {
            "shape": f"{B}x({m}x{n})",
            "ms": round(ms_ns, 3),
            "tflops": round(ns_tf, 2),
            "pct_of_bf16_peak": round(100.0 * ns_tf / PEAK_BF16_TFLOPS, 2),
        }
        del X
        if args.workload == "gpt_small_heads":
            # the per-head group on its own: 36 heads x 12 layers of 64 x 768, one LDS-resident launch
            Xh = (torch.randn(432, 64, 768, device=dev) * 0.01).to(torch.bfloat16)
            ms_h = time_kernel(lambda: fn(Xh, 1e-8), iters=20)
            h_tf = 432 * ns_flops(64, 768) / (ms_h * 1e-3) * 1e-12
            result["ns_per_head"] = {"shape": "432x(64x768)", "us": round(ms_h * 1e3, 1), "tflops": round(h_tf, 1),
                                     "pct_of_bf16_peak": round(100.0 * h_tf / PEAK_BF16_TFLOPS, 2)}
            del Xh
        torch.cuda.empty_cache()

    if args.stream_compare:
        # memory-bound kernels of the step against a plain copy with the same read and write volume, same
        # run: muon_pre reads 6 B and writes 6 B per element (G bf16 + M fp32 -> M fp32 + U bf16), muon_post
        # reads 6 B and writes 4 B (U bf16 + X fp32 -> X fp32)
        name, rows, cols, count = max(spec, key=lambda g: g[1] * g[2] * g[3])
        count = min(count, 16)
        Gs = [torch.empty(rows, cols, device=dev).normal_(0.0, 0.02, generator=gen).to(torch.bfloat16)
              for _ in range(count)]
        Ms = [torch.zeros(rows, cols, device=dev) for _ in range(count)]
        Xs = [torch.empty(rows, cols, device=dev).normal_(0.0, 0.02, generator=gen) for _ in range(count)]
        n_el = count * rows * cols
        lr_t = torch.tensor(0.02, device=dev)

        def ev(f, iters=10):
            f()
            torch.cuda.synchronize()
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(iters):
                f()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / iters

        ms_pre = ev(lambda: ops.muon_pre(Gs, Ms, 0.95, True))
        U = ops.muon_pre(Gs, Ms, 0.95, True)
        ms_post = ev(lambda: ops.muon_post(Xs, U.view(count, -1), lr_t, 0.5, 0.01))
        src = torch.empty(n_el * 6, dtype=torch.uint8, device=dev).view(torch.float32)
        dst = torch.empty_like(src)
        ms_copy = ev(lambda: dst.copy_(src))                 # device-to-device memcpy (no kernel in a trace)
        ms_mul = ev(lambda: torch.mul(src, 1.0, out=dst))    # the plainest streaming kernel: one read, one write
        src2 = torch.empty_like(src)
        ms_add = ev(lambda: torch.add(src, src2, out=dst))   # two read streams, one write stream

        def row(ms, nbytes):
            return {"ms": round(ms, 4), "GBps": round(nbytes / (ms * 1e-3) * 1e-9, 1),
                    "frac_of_hbm_peak": round(nbytes / (ms * 1e-3) / (PEAK_HBM_GBS * 1e9), 4)}

        result["streaming"] = {
            "group": f"{count}x({rows}x{cols}) {name}",
            "muon_pre (12 B/element)": row(ms_pre, n_el * 12),
            "muon_post (10 B/element)": row(ms_post, n_el * 10),
            "device memcpy, 6 B read + 6 B written per element": row(ms_copy, n_el * 12),
            "torch.mul(src, 1, out=dst) fp32, 6 B read + 6 B written per element": row(ms_mul, n_el * 12),
            "torch.add(src, src2, out=dst) fp32, 12 B read + 6 B written per element": row(ms_add, n_el * 18),
        }
        del Gs, Ms, Xs, U, src, src2, dst
        torch.cuda.empty_cache()

    if args.breakdown:
        # every shape group on its own: Muon's three phases, timed with events on the launch stream
        from dion_amd import gram_newton_schulz, polar_express, zeropower_via_newtonschulz5

        fn = {"polar_express": polar_express, "gram": gram_newton_schulz}.get(args.ns, zeropower_via_newtonschulz5)

        def timed(f, iters):
            f()
            torch.cuda.synchronize()
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(iters):
                f()
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) / iters

        lr_t = torch.tensor(0.02, device=dev)
        rows_out = []
        for name, rows, cols, count in spec:
            Xs = [torch.empty(rows, cols, device=dev).normal_(0.0, 0.02, generator=gen) for _ in range(count)]
            Gs = [torch.empty(rows, cols, device=dev).normal_(0.0, 0.02, generator=gen).to(torch.bfloat16)
                  for _ in range(count)]
            Ms = [torch.zeros(rows, cols, device=dev) for _ in range(count)]
            n_el = count * rows * cols
            it = 20 if n_el < 5e8 else 5
            ms_pre = timed(lambda: ops.muon_pre(Gs, Ms, 0.95, True), it)
            U = ops.muon_pre(Gs, Ms, 0.95, True)
            ms_ns = timed(lambda: fn(U, 1e-8), max(3, it // 2))
            O = fn(U, 1e-8)
            ms_post = timed(lambda: ops.muon_post(Xs, O.view(count, -1), lr_t, 0.5, 0.01), it)
            tf = count * ns_flops(rows, cols) / (ms_ns * 1e-3) * 1e-12
            rows_out.append({
                "group": f"{count}x({rows}x{cols}) {name}",
                "ns_ms": round(ms_ns, 4), "ns_tflops": round(tf, 1),
                "ns_pct_of_bf16_peak": round(100.0 * tf / PEAK_BF16_TFLOPS, 2),
                "pre_ms": round(ms_pre, 4), "pre_GBps": round(n_el * 12 / (ms_pre * 1e-3) * 1e-9, 1),
                "pre_pct_of_hbm_peak": round(100.0 * n_el * 12 / (ms_pre * 1e-3) / 8e12, 2),
                "post_ms": round(ms_post, 4), "post_GBps": round(n_el * 10 / (ms_post * 1e-3) * 1e-9, 1),
                "post_pct_of_hbm_peak": round(100.0 * n_el * 10 / (ms_post * 1e-3) / 8e12, 2),
            })
            del Xs, Gs, Ms, U, O
            ops.release_workspaces()
            torch.cuda.empty_cache()
        result["groups"] = rows_out

    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline("polar_express" if args.ns == "gram" else args.ns)

    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
