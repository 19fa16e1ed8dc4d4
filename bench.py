#!/usr/bin/env python3
"""bench.py — GEMM throughput of the engine on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

A step is one pass of the hot path over one batch of synthetic input: one launch of the tuned
kernel for fp32 C[4096,4096] = A[4096,4096] · B[4096,4096] (row-major A[M,K], B[K,N]; seeded
uniform[-1,1) inputs already resident in HBM).  The JSON line printed at the end carries

  value / ms_per_step : whole-job throughput over exactly K steps between two device synchronisations
  roofline            : 2MNK / (average launch duration measured with HIP events on the launch
                        stream over the same K launches) against the fp32 MFMA peak of MI355X
  roofline_steady     : the same kernel after 100 untimed launches, HIP-event average over 200 launches (the
                        part's clocks need several milliseconds under load to settle; with a short warm-up that
                        ramp lies inside the K timed steps)
  fp16, bf16          : the same figures for the 16-bit-input / fp32-accumulate kernels at 4096^3, each checked
                        against the oracle on a row panel
  cpu_baseline        : the CPU oracle (a port of the reference's hostMatmul arithmetic) timed on this
                        box's host cores on a bounded row panel of the same product

Only one GPU is ever used; --gpus above 1 exits with a message.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_TFLOPS = {"f32": 157.3, "f16": 2516.6, "bf16": 2516.6}   # MI355X dense matrix peaks
HBM_PEAK_GBS = 8000.0

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (two passes), each scaled by what
# the same counter read for a copy kernel of known size: kept in profiles/traffic.json (full kernel name ->
# KiB per dispatch, scale factors, the command that produced them).  A kernel that was not profiled reports
# null with the reason.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")


def measured_traffic(kernel_name):
    """-> (bytes per launch or None, note)."""
    try:
        with open(TRAFFIC_FILE) as f:
            doc = json.load(f)
    except (OSError, ValueError) as e:
        return None, f"profiles/traffic.json unreadable: {e}"
    entry = doc.get("kernels", {}).get(kernel_name)
    if entry is None:
        return None, "this kernel has no entry in profiles/traffic.json (not profiled since it was last re-tuned)"
    sc = doc["scale"]
    nbytes = int(round((entry["FETCH_SIZE_KiB"] * sc["FETCH_SIZE"] + entry["WRITE_SIZE_KiB"] * sc["WRITE_SIZE"]) * 1024))
    return nbytes, "profiles/traffic.json"


def load_tuned(name):
    path = name if os.path.isabs(name) or os.path.exists(name) else os.path.join(ROOT, "codegendemo_amd", "TunedConfigs", name)
    with open(path) as f:
        return json.load(f)["cfgs"][0]


def build_kernel(config):
    from codegendemo_amd.kcg.CompiledKernelFactory import CompiledKernelFactory, EnumOperator, UserInputs
    from codegendemo_amd.kcg.KCGCompiler import KCGCompiler
    from codegendemo_amd.kcg.Operators.matmul import kernelArgFromConfig
    kpm = kernelArgFromConfig(config)
    comp = KCGCompiler()
    path, name, gx, gy, gz, bx, by, bz = comp.compileKernel(kpm)[0]
    ui = UserInputs(path, name, kpm)
    ui.m_gridDims, ui.m_blockDims = [gx, gy, gz], [bx, by, bz]
    ui.m_ldsBytes = comp.lastInfo["lds_bytes"]
    ui.operatorKind = EnumOperator.Matmul
    kernel = CompiledKernelFactory.getKernel(ui, 0)
    kernel.n_regs           # loads the code object now (otherwise the first launch would)
    return kpm, kernel, comp.lastInfo


def make_inputs(kpm, dist):
    import torch
    from codegendemo_amd.kcg import SeededInputs as SI
    if dist == "uniform":
        a = SI.uniform((kpm.M, kpm.K), SI.STREAM_A)
        b = SI.uniform((kpm.K, kpm.N), SI.STREAM_B)
    else:
        a = SI.normal((kpm.M, kpm.K), SI.STREAM_A, std=0.5)
        b = SI.normal((kpm.K, kpm.N), SI.STREAM_B, std=0.5)
    ta = kpm.dtypeTorch('A')
    A = torch.from_numpy(SI.a_operand(a, kpm.isATranspose)).to("cuda:0").to(ta)
    B = torch.from_numpy(b).to("cuda:0").to(ta)
    C = torch.zeros((kpm.M, kpm.N), dtype=kpm.dtypeTorch('C'), device="cuda:0")
    return a, b, A, B, C


def make_inputs_host(kpm16):
    """The 16-bit workload's operands as the kernel sees them: normal(0, 0.5) rounded to fp16 (or bf16), upcast
    to fp32."""
    import torch
    from codegendemo_amd.kcg import SeededInputs as SI
    tt = kpm16.dtypeTorch('A')
    a = torch.from_numpy(SI.normal((kpm16.M, kpm16.K), SI.STREAM_A, std=0.5)).to(tt).to(torch.float32).numpy()
    b = torch.from_numpy(SI.normal((kpm16.K, kpm16.N), SI.STREAM_B, std=0.5)).to(tt).to(torch.float32).numpy()
    return a, b


def time_steps(kernel, A, B, C, steps, warmup):
    """-> (wall ms per step over K steps, HIP-event average launch duration in ms)."""
    import torch
    for _ in range(warmup):
        kernel.run(A, B, C)
    torch.cuda.synchronize()
    stream = torch.cuda.current_stream()
    ev0 = torch.cuda.Event(enable_timing=True)
    ev1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record(stream)               # the kernel is launched on this same (torch current) stream
    for _ in range(steps):
        kernel.run(A, B, C)
    ev1.record(stream)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    return (t1 - t0) * 1e3 / steps, ev0.elapsed_time(ev1) / steps


def reference_style_ms(kernel, A, B, C, samples=20):
    """The reference's own measurement (KCGTask.py:124-130,164-171): one launch between a pair of events, host
    synchronisation after every sample, median over the samples; includes what the launch costs from Python."""
    import torch
    ev0 = torch.cuda.Event(enable_timing=True)
    ev1 = torch.cuda.Event(enable_timing=True)
    ms = []
    for _ in range(samples):
        ev0.record()
        kernel.run(A, B, C)
        ev1.record()
        torch.cuda.synchronize()
        ms.append(ev0.elapsed_time(ev1))
    ms.sort()
    return 0.5 * (ms[(len(ms) - 1) // 2] + ms[len(ms) // 2])


RAMP_LAUNCHES, STEADY_LAUNCHES = 100, 200


def steady_roofline(kernel, A, B, C, flops, peak):
    """The same kernel after the part's clocks have settled: RAMP_LAUNCHES untimed launches, then the HIP-event
    average over STEADY_LAUNCHES.  (`steps`/`warmup` of the command line are honoured as given for the headline
    figures; clocks on this part take several milliseconds to reach their level under load, which a short
    warm-up leaves inside the timed region.)"""
    _, ms = time_steps(kernel, A, B, C, STEADY_LAUNCHES, RAMP_LAUNCHES)
    ach = flops / (ms * 1e-3) / 1e12
    return {"achieved": ach, "peak": peak, "unit": "TFLOP/s", "frac": ach / peak, "launch_ms": ms,
            "ramp_launches": RAMP_LAUNCHES, "timed_launches": STEADY_LAUNCHES}


def half_parity(C_dev, a_host, b_host, rows=(2048, 2112)):
    """A row panel of a 16-bit-input result against the oracle run on the upcast inputs; bar: 2e-2 relative to
    the RMS magnitude of C."""
    import numpy as np
    from tests import oracle_binding
    r0, r1 = rows
    want = oracle_binding.load().matmul(a_host, b_host, 0, rows=(r0, r1))
    got = C_dev[r0:r1].cpu().numpy()
    scale = float(np.sqrt(np.mean(want.astype(np.float64) ** 2)))
    rel = float(np.abs(got - want).max()) / scale
    return {"rows_checked": r1 - r0, "max_rel_err": rel, "tolerance": 2e-2, "ok": bool(rel <= 2e-2)}


def time_library_gemm(A, B, a_trans, steps, warmup):
    """The vendor library's GEMM (torch.matmul -> rocBLAS/hipBLASLt) on the same device buffers, timed like
    time_steps: for orientation only, it is neither the oracle nor part of the product."""
    import torch
    a = A.t() if a_trans else A
    for _ in range(warmup):
        torch.matmul(a, B)
    torch.cuda.synchronize()
    ev0 = torch.cuda.Event(enable_timing=True)
    ev1 = torch.cuda.Event(enable_timing=True)
    ev0.record()
    for _ in range(steps):
        torch.matmul(a, B)
    ev1.record()
    torch.cuda.synchronize()
    return ev0.elapsed_time(ev1) / steps


def cpu_baseline(a, b, ijk_seconds=5.0):
    """Times the CPU oracle on this box's host cores: the threaded loop over the WHOLE 4096^3 product
    (best of 3; it is also the parity reference for the GPU result) and, for the record, the
    reference's own loop order (i-j-k, one thread) on a row panel sized to a few seconds."""
    from tests import oracle_binding
    orc = oracle_binding.load()
    M, K = a.shape
    N = b.shape[1]
    threads = orc.max_threads()
    best = None
    full = None
    spent = 0.0
    for _ in range(3):
        t0 = time.perf_counter()
        full = orc.matmul(a, b, 0)
        dt = time.perf_counter() - t0
        spent += dt
        best = dt if best is None else min(best, dt)
        if spent > 20.0:
            break
    t0 = time.perf_counter()
    orc.ijk(a, b, 0, rows=(0, 1))
    probe = time.perf_counter() - t0
    rows_ijk = int(max(1, min(64, ijk_seconds / max(probe, 1e-4))))
    t0 = time.perf_counter()
    panel_ijk = orc.ijk(a, b, 0, rows=(0, rows_ijk))
    dt_ijk = time.perf_counter() - t0
    out = {
        "value": 2.0 * M * N * K / best / 1e12, "unit": "TFLOPS", "cores": threads, "kind": "port",
        "sample": f"whole fp32 4096^3 product on the same inputs, best of 3 runs ({best:.2f} s each), "
                  f"i-k-j loop order, OpenMP over rows",
        "reference_loop_order": {"value": 2.0 * rows_ijk * N * K / dt_ijk / 1e12, "unit": "TFLOPS", "cores": 1,
                                 "sample": f"i-j-k order (hostMatmul), first {rows_ijk} rows of C, {dt_ijk:.1f} s"},
    }
    # the reference's own hostMatmul (matmul.cpp:2349-2360, built by oracle/Makefile where the reference tree was
    # present) on the same row panel: it wants A stored [K, M], so the panel's rows go in as a [K, rows] operand
    ref = oracle_binding.load_reference_build()
    if ref is not None:
        import numpy as np
        a_km = np.ascontiguousarray(a[:rows_ijk].T)
        t0 = time.perf_counter()
        got = ref(a_km, b)
        dt_ref = time.perf_counter() - t0
        out["reference_build"] = {"value": 2.0 * rows_ijk * N * K / dt_ref / 1e12, "unit": "TFLOPS", "cores": 1, "kind": "reference",
                                  "sample": f"the reference's hostMatmul compiled from its own source, first {rows_ijk} rows of C, {dt_ref:.1f} s",
                                  "bit_equal_to_port": bool(np.array_equal(got, panel_ijk))}
    return out, full, M


def power_and_clocks(kernel, A, B, C, seconds=2.0):
    """Socket power and the clock of each XCD while `kernel` runs back to back, read once with amd-smi about a
    second into the run.  Returns None when the tool is missing or says nothing useful (the figures are
    evidence for the roofline discussion, not part of the measurement)."""
    import subprocess
    import threading
    import torch
    stop = threading.Event()

    def spin():
        while not stop.is_set():
            for _ in range(100):
                kernel.run(A, B, C)
            torch.cuda.synchronize()

    t = threading.Thread(target=spin)
    t.start()
    out = None
    try:
        time.sleep(seconds / 2)
        p = subprocess.run(["amd-smi", "metric", "--power", "--clock", "--json"], capture_output=True, text=True, timeout=30)
        doc = json.loads(p.stdout)
        gpu = (doc.get("gpu_data") if isinstance(doc, dict) else doc)[0]
        clocks = [gpu["clock"][f"gfx_{i}"]["clk"]["value"] for i in range(8) if f"gfx_{i}" in gpu["clock"]]
        out = {"socket_power_w": gpu["power"]["socket_power"]["value"], "gfx_clk_mhz_by_xcd": clocks,
               "max_clk_mhz": gpu["clock"]["gfx_0"]["max_clk"]["value"], "source": "amd-smi metric --power --clock"}
        time.sleep(seconds / 2)
    except Exception:   # noqa: BLE001 - an absent or differently shaped tool output must not fail the benchmark
        out = None
    finally:
        stop.set()
        t.join()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-fp16", action="store_true", help="skip the fp16 side measurement")
    ap.add_argument("--fp32-config", default="", help="JSON file ({'cfgs': [...]}) to use instead of the tuned fp32 config")
    ap.add_argument("--fp16-config", default="", help="same for the fp16 side measurement")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="profiling aid: first run a plain 256 MiB device copy three times, so that HBM counters "
                         "(FETCH_SIZE / WRITE_SIZE) of the same profiler run can be scaled by a kernel of known traffic")
    ap.add_argument("--hiprtc", default="", help="path of the hiprtc library that builds the kernels (default: the one this "
                    "process carries, i.e. the ROCm that PyTorch bundles); 'system' = /opt/rocm/lib/libhiprtc.so.7")
    ap.add_argument("--only-fp16", action="store_true",
                    help="profiling aid: run only the fp16 kernel (prints a reduced JSON line)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one MI355X; this engine has no multi-GPU path (--gpus must be 1)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    from codegendemo_amd import _native
    _native.lib()   # raises if the native library is missing: there is no fallback
    if args.hiprtc:
        os.environ["KCG_HIPRTC_LIB"] = _native.SYSTEM_HIPRTC if args.hiprtc == "system" else args.hiprtc
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)

    if args.calibrate_copy:
        src = torch.ones(64 * 1024 * 1024, dtype=torch.float32, device="cuda:0")     # 256 MiB
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        for _ in range(3):
            dst.copy_(src)          # one elementwise copy kernel: reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
        del src, dst

    if args.only_fp16:
        cfg16 = load_tuned(args.fp16_config or "gemm_4096_fp16.json")
        kpm16, kernel16, info16 = build_kernel(cfg16)
        _, _, A16, B16, C16 = make_inputs(kpm16, "normal")
        ms_step16, ms_launch16 = time_steps(kernel16, A16, B16, C16, args.steps, args.warmup)
        fl = 2.0 * kpm16.M * kpm16.N * kpm16.K
        print(json.dumps({"only": "fp16", "kernel": info16["kernel_name"], "launch_ms": ms_launch16,
                          "tflops": fl / (ms_launch16 * 1e-3) / 1e12, "compiler": _native.compiler_identity()}))
        return

    # ---- preparation: every kernel built and loaded, every operand resident in HBM, before anything is timed.
    # The timed legs below then follow each other without host work in between (input generation takes
    # seconds, during which an idle GPU drops its clocks again).
    cfg32 = load_tuned(args.fp32_config or "gemm_4096_fp32.json")
    kpm, kernel, info = build_kernel(cfg32)
    a, b, A, B, C = make_inputs(kpm, "uniform")
    flops = 2.0 * kpm.M * kpm.N * kpm.K
    legs16 = []           # (key, label, kpm, kernel, info, A, B, C)
    if not args.no_fp16:
        cfg16 = load_tuned(args.fp16_config or "gemm_4096_fp16.json")
        cfgb = dict(cfg16)
        cfgb["DATATYPE_A"] = cfgb["DATATYPE_B"] = 3      # the same config with bfloat16 inputs
        cfgh = dict(cfg16)
        cfgh["DATATYPE_C"] = 2                           # ... and with fp16 output (what the library's fp16 GEMM returns)
        for key, label, cfg in (("fp16", "f16", cfg16), ("bf16", "bf16", cfgb), ("fp16_out16", "f16", cfgh)):
            k_, kern_, info_ = build_kernel(cfg)
            if key == "fp16_out16":                      # the fp16 leg's operands, a result buffer of its own
                A_, B_ = legs16[0][5], legs16[0][6]
                C_ = torch.zeros((k_.M, k_.N), dtype=k_.dtypeTorch('C'), device="cuda:0")
            else:
                _, _, A_, B_, C_ = make_inputs(k_, "normal")
            legs16.append((key, label, k_, kern_, info_, A_, B_, C_))
    torch.cuda.synchronize()

    # ---- timed legs
    ms_step, ms_launch = time_steps(kernel, A, B, C, args.steps, args.warmup)
    value = flops / (ms_step * 1e-3) / 1e12
    achieved = flops / (ms_launch * 1e-3) / 1e12
    steady32 = steady_roofline(kernel, A, B, C, flops, PEAK_TFLOPS["f32"])
    ref_ms = reference_style_ms(kernel, A, B, C)
    traffic32, traffic32_note = measured_traffic(info["kernel_name"])

    out = {
        "metric": "GEMM TFLOPS and % of dtype MFMA roofline at M=N=K=4096, 1 MI355X",
        "value": value, "unit": "TFLOPS", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": ("fp32 GEMM M=N=K=4096" if (kpm.M, kpm.N, kpm.K) == (4096, 4096, 4096)
                                else f"fp32 GEMM M={kpm.M} N={kpm.N} K={kpm.K} (--fp32-config)")
                               + (", A stored [K,M]" if kpm.isATranspose else ", row-major A[M,K]")
                               + " B[K,N], uniform[-1,1) seeded, tuned config",
                   "kernel": info["kernel_name"], "kind": {1: "simt", 2: "mfma"}[info["kind"]],
                   "lds_bytes": info["lds_bytes"], "grid": info["grid"][0], "block": info["block"][0],
                   "compiler": _native.compiler_identity(), "vgprs": info["vgprs"], "scratch_bytes": info["scratch_bytes"],
                   "build_flags": info["build_flags"]},
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": PEAK_TFLOPS["f32"], "unit": "TFLOP/s",
                     "frac": achieved / PEAK_TFLOPS["f32"], "traffic": traffic32, "traffic_source": traffic32_note,
                     "launch_ms": ms_launch,
                     "hbm_gbs_algorithmic": (4.0 * (kpm.M * kpm.K + kpm.K * kpm.N + kpm.M * kpm.N)) / (ms_launch * 1e-3) / 1e9},
        "roofline_steady": steady32,
        "reference_style_timing": {"ms": ref_ms, "tflops": flops / (ref_ms * 1e-3) / 1e12, "samples": 20,
                                   "what": "one launch per event pair with a host synchronisation per sample, median (the reference's PerfTester)"},
    }
    for key, label, k_, kern_, info_, A_, B_, C_ in legs16:
        ms_step_, ms_launch_ = time_steps(kern_, A_, B_, C_, args.steps, args.warmup)
        ach_ = flops / (ms_launch_ * 1e-3) / 1e12
        traffic_, traffic_note_ = measured_traffic(info_["kernel_name"])
        out[key] = {"value": flops / (ms_step_ * 1e-3) / 1e12, "unit": "TFLOPS", "ms_per_step": ms_step_,
                    "dtype": f"{label} in, f32 accumulate/out" if k_.dtypeTorch('C') == torch.float32 else f"{label} in, f32 accumulate, {label} out",
                    "kernel": info_["kernel_name"],
                    "roofline": {"bound": "mfma", "achieved": ach_, "peak": PEAK_TFLOPS[label], "unit": "TFLOP/s",
                                 "frac": ach_ / PEAK_TFLOPS[label], "traffic": traffic_, "traffic_source": traffic_note_,
                                 "launch_ms": ms_launch_},
                    "roofline_steady": steady_roofline(kern_, A_, B_, C_, flops, PEAK_TFLOPS[label])}
    # the vendor library's GEMM on the same buffers, after the engine's own legs (orientation only)
    c_host = C.cpu().numpy()
    lib_ms = time_library_gemm(A, B, kpm.isATranspose, args.steps, args.warmup)
    out["library_gemm"] = {"source": "torch.matmul (rocBLAS/hipBLASLt) on the same buffers, same timing loop",
                           "f32_tflops": flops / (lib_ms * 1e-3) / 1e12}
    if legs16:
        _, _, k_, _, _, A_, B_, _ = legs16[0]
        lib16_ms = time_library_gemm(A_, B_, k_.isATranspose, args.steps, args.warmup)
        out["library_gemm"]["f16_tflops"] = flops / (lib16_ms * 1e-3) / 1e12
        out["library_gemm"]["f16_note"] = ("torch.matmul on fp16 operands returns fp16: the library writes 32 MiB of C, this engine's fp16 leg 64 MiB "
                                           "of fp32 (BASELINE config 5); its fp16_out16 leg is the like-for-like figure")

    # ---- checks and side information (nothing below is timed)
    if not args.no_cpu:     # (skipped in profiling runs, like the CPU leg)
        for key, label, k_, kern_, info_, A_, B_, C_ in legs16:
            # a 64-row panel of the result against the oracle run on the upcast 16-bit values
            ah, bh = make_inputs_host(k_)
            out[key]["parity"] = half_parity(C_, ah, bh)
            del ah, bh
            if not out[key]["parity"]["ok"]:
                print(json.dumps(out))
                print(f"bench.py: {key} GPU result differs from the oracle beyond tolerance", file=sys.stderr)
                sys.exit(1)
        if legs16:
            _, _, _, kern_, _, A_, B_, C_ = legs16[0]
            pc = power_and_clocks(kern_, A_, B_, C_)
            if pc:
                out["fp16"]["power_and_clocks"] = pc
            pc = power_and_clocks(kernel, A, B, C)
            if pc:
                out["roofline"]["power_and_clocks"] = pc
    if legs16:
        # What the matrix pipeline alone sustains on this box (register operands, no memory traffic), on
        # zeros and on data like the workload's: the stand-alone runner measures it in a child process.
        # fp16 GEMMs on this part run at its power limit, so the second figure bounds any fp16 kernel.
        runner = os.path.join(ROOT, "codegendemo_amd", "kcg_runner")
        if os.path.exists(runner):
            import subprocess
            p = subprocess.run([runner, "--mfma-peak", "f16"], capture_output=True, text=True, timeout=120)
            if p.returncode == 0:
                out["fp16"]["mfma_only_sustained"] = json.loads(p.stdout.strip().splitlines()[-1])["mfma_peak"]
    del legs16

    if not args.no_cpu:
        base, panel, rows = cpu_baseline(a, b)
        out["cpu_baseline"] = base
        err = float(np.abs(c_host[:rows] - panel).max())
        tol = 1e-4 * kpm.K * float(np.abs(a).max()) * float(np.abs(b).max())
        out["parity"] = {"rows_checked": rows, "max_abs_err": err, "tolerance": tol, "ok": bool(err <= tol)}
        if err > tol:
            print(json.dumps(out))
            print("bench.py: GPU result differs from the oracle beyond tolerance", file=sys.stderr)
            sys.exit(1)

    print(json.dumps(out))


if __name__ == "__main__":
    main()
