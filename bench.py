#!/usr/bin/env python3
"""Benchmark of the batched joint log-likelihood path on one MI355X.

A step is one pass of the compiled SPN kernel over one batch of synthetic inputs that already sit in HBM
(``spnc_hip_execute_device``). The headline workload is configuration C1, the README's product of six
Categorical leaves at 64M int32 rows: the configuration the path's throughput target is quoted on. The other
configurations are measured with the same number of steps and reported under "others" in the same JSON line.

Prints ONE JSON line: samples/s, the roofline of the kernel (HIP-event timed launches on the launch stream), the
rate of the host path (numpy in, numpy out, through ``spnc_hip_execute``) and a CPU baseline per configuration (the
restated CPUCompiler-equivalent kernel of oracle/cgen.py, or the oracle's interpreting evaluator for the
region graph, on the host cores).
"""
import argparse
import contextlib
import hashlib
import io
import json
import os
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "spn-compiler_amd"))

HBM_PEAK_GBS = 8000.0            # MI355X HBM3E, published
FP32_VECTOR_PEAK_TFLOPS = 157.3  # MI355X FP32 vector, published
FP64_VECTOR_PEAK_TFLOPS = 78.6   # MI355X FP64 vector, published
ALL = ["c1", "c2", "c3", "c4", "c5", "c5_f64", "c4_f64"]
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")


def kernel_key(kernel, n):
    """Identifies what a counter run measured: the generated device code (or interpreter program) and the launch size."""
    return hashlib.sha1(kernel.source().encode() + b"|%d" % n).hexdigest()[:16]


_INPUTS = {}


def make_inputs(name, cfg, n):
    """The configuration's seeded inputs, the same arrays the parity tests use (NumPy generators; spnc/synthetic.py).
    Configuration 5 is configuration 2's batch with NaNs put in, so the normals are drawn once for both."""
    import numpy as np
    if name in ("c2", "c5"):
        if ("c2", n) not in _INPUTS:
            _INPUTS.clear()
            from spnc import synthetic as syn
            _INPUTS[("c2", n)] = syn.c2_inputs(n)
        x = _INPUTS[("c2", n)]
        if name == "c2":
            return x
        if ("c5", n) not in _INPUTS:
            x5 = x.copy()
            x5[np.random.default_rng(105).random(x5.shape) < 0.2] = np.nan      # spnc.synthetic.c5_inputs
            _INPUTS[("c5", n)] = x5
        return _INPUTS[("c5", n)]
    _INPUTS.clear()
    return cfg["inputs"](n)


def make_device_inputs(name, cfg, n, torch, device):
    """Inputs of the same shape and distribution drawn on the device (seconds instead of a minute for all configurations);
    used by the counter runs of profile_counters.py, where only the launch matters."""
    from spnc import synthetic as syn
    g = torch.Generator(device=device)
    g.manual_seed(7)
    F = cfg["features"]
    if name == "c1":
        return torch.randint(0, 3, (n, F), generator=g, device=device, dtype=torch.int32)
    if name in ("c3", "c3_deep"):
        doms = torch.tensor([d for _, d in syn.c3_domains()], device=device, dtype=torch.float32)
        u = torch.rand((n, F), generator=g, device=device)
        return torch.minimum((u * doms).floor(), doms - 1).to(torch.int32)
    x = torch.randn((n, F), generator=g, device=device, dtype=torch.float32)
    if name == "c5":
        x[torch.rand((n, F), generator=g, device=device) < 0.2] = float("nan")
    return x


_SUSTAINED = {}


def sustained_issue_rate(f64):
    """Lane-operations per second of independent v_add_f32 (v_fma_f64) chains on every SIMD, measured now, in this process,
    for about half a second: what the vector units of this box sustain at the clock it holds under load. The published
    peak is quoted at the nominal clock. None when the calibration library is not built."""
    if f64 not in _SUSTAINED:
        import ctypes
        path = os.path.join(ROOT, "spn-compiler_amd", "libspnc_issue_rate.so")
        rate = ctypes.c_double(0.0)
        try:
            lib = ctypes.CDLL(path)
            lib.spnc_issue_rate.argtypes = [ctypes.c_int, ctypes.c_double, ctypes.POINTER(ctypes.c_double)]
            ok = lib.spnc_issue_rate(1 if f64 else 0, 0.5, ctypes.byref(rate)) == 0
        except OSError:
            ok = False
        _SUSTAINED[f64] = rate.value if ok else None
    return _SUSTAINED[f64]


def measure(name, n, steps, warmup, torch, device, extra_options=None, fast_inputs=False):
    from spnc import synthetic as syn
    from spnc.hip import HIPCompiler
    workload_key, extra_given = name, bool(extra_options)
    if name.endswith("_f64"):   # the same configuration computed in float64 log-space (c5: straight-line kernel, c4: interpreter)
        name, extra_options = name[:-4], dict(extra_options or {}, **{"hip-compute-type": "float64"})
    cfg = syn.CONFIGS[name]
    n = n or cfg["n"]
    spn = cfg["spn"]()
    t0 = time.time()
    kernel = HIPCompiler(**(extra_options or {})).compile_ll(spn, cfg["dtype"], supportMarginal=cfg["marginal"])
    compile_s = time.time() - t0
    info = kernel.info()
    if fast_inputs:
        x_host, x = None, make_device_inputs(name, cfg, n, torch, device)
    else:
        x_host = make_inputs(name, cfg, n)
        x = torch.from_numpy(x_host).to(device)
    out = torch.empty(n, device=device, dtype=torch.float32 if info["dtype"] == "float32" else torch.float64)
    stream = torch.cuda.current_stream().cuda_stream   # the launches and the timing events share this stream

    def step():
        kernel.execute_device(n, x.data_ptr(), out.data_ptr(), stream)

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    t0 = time.perf_counter()
    for i in range(steps):
        starts[i].record()
        step()
        ends[i].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    launch_ms = sum(s.elapsed_time(e) for s, e in zip(starts, ends)) / steps
    finite = bool(torch.isfinite(out[: min(n, 1 << 20)]).all().item())
    head = out[: min(n, 1 << 12)].cpu().numpy()   # what the CPU baseline leg compares its own results with

    bytes_per_sample = cfg["features"] * info["bytes_per_feature"] + info["bytes_per_result"]
    flops, trans = info["flops_min"], info["trans_min"]
    # Issue slots: one per flop, four per transcendental, and one instead of two for every multiply-add pair that a
    # fused instruction computes (Gaussian leaves and the product adds they feed), so that the fraction cannot pass 1.
    slots = flops - info["fused_min"] + 3 * trans
    props = torch.cuda.get_device_properties(device)
    clock_hz = props.clock_rate * 1e3 if hasattr(props, "clock_rate") else 2.4e9
    # FP32 VALU issue rate: 128 lane-operations per CU per clock (a wave64 instruction issues in
    # two cycles on each of the four SIMDs). This is what the published 157.3 TFLOP/s is made of
    # (256 CUs x 128 lanes x 2 flops per FMA x 2.4 GHz); a transcendental takes four such slots.
    f64 = info["dtype"] == "float64"
    valu_peak = props.multi_processor_count * (64 if f64 else 128) * clock_hz  # lane-operations per second
    t_launch = launch_ms * 1e-3
    hbm_gbs = bytes_per_sample * n / t_launch / 1e9
    tflops = flops * n / t_launch / 1e12
    t_min_hbm = bytes_per_sample * n / (HBM_PEAK_GBS * 1e9)
    t_min_valu = slots * n / valu_peak
    hbm_bound = t_min_hbm >= t_min_valu
    # Compute-bound kernels are priced in issue slots (simple op 1, transcendental 4) against the
    # FP32 vector peak for single-flop instructions, i.e. half the published FMA figure.
    slot_tflops = slots * n / t_launch / 1e12
    slot_peak = (FP64_VECTOR_PEAK_TFLOPS if f64 else FP32_VECTOR_PEAK_TFLOPS) / 2
    roof = {
        "bound": "hbm" if hbm_bound else ("valu-fp64" if f64 else "valu-fp32"),
        "achieved": round(hbm_gbs if hbm_bound else slot_tflops, 3),
        "peak": HBM_PEAK_GBS if hbm_bound else slot_peak,
        "unit": "GB/s" if hbm_bound else "TFLOP/s",
        "frac": round((hbm_gbs / HBM_PEAK_GBS) if hbm_bound else (slot_tflops / slot_peak), 4),
        "traffic": None,
        "peak_note": ("published HBM3E bandwidth" if hbm_bound else
                      "published vector peak (FP32 157.3, FP64 78.6 TFLOP/s) counts an FMA as 2 flops; this path issues mostly single-flop "
                      "instructions, so the ceiling is half of it in issue slots/s; achieved = (flops - fused multiply-add pairs + "
                      "3*transcendentals) per sample"),
        "fma_flops_tflops": round(tflops, 3),
        "kernel": "spn_kernel (hipRTC straight-line)" if info["kernel_kind"] == 1 else "spn_interp_kernel",
        "launch_ms": round(launch_ms, 4),
        "bytes_per_sample": bytes_per_sample,
        "flops_per_sample": flops,
        "transcendentals_per_sample": trans,
        "transcendental_wave_instructions_per_launch": trans * (n // 64),   # derived: no transcendental counter on gfx950
        "fused_multiply_adds_per_sample": info["fused_min"],
        "issue_slots_per_sample": slots,
        "valu_issue_peak_per_s": valu_peak,
        "valu_issue_frac": round(t_min_valu / t_launch, 4),
        "hbm_frac": round(t_min_hbm / t_launch, 4),
    }
    if not hbm_bound:
        sustained = sustained_issue_rate(f64)
        if sustained:
            roof["sustained_issue_per_s"] = sustained                      # measured in this process, see sustained_issue_rate()
            roof["sustained_over_published"] = round(sustained / valu_peak, 4)
            roof["frac_of_sustained"] = round(slots * n / sustained / t_launch, 4)
    if f64:
        # A float64 exp or log is not one quarter-rate instruction as in float32 but a routine of its own: nine
        # double-rate instructions, three to six integer ones and one LDS read here. Priced at the nine the same launch reads:
        slots_real = flops - info["fused_min"] + 8 * trans
        roof["issue_slots_per_sample_exp_log_at_9"] = slots_real
        roof["frac_exp_log_at_9"] = round(slots_real * n / valu_peak / t_launch, 4)
    # HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (scaled by what a plain copy of known
    # size reads on the same counters): written to profiles/traffic.json by profile_counters.py together with a hash of
    # the kernel's code and launch size, so that an entry measured on another kernel is not passed on.
    try:
        entry = json.load(open(TRAFFIC_FILE)).get(workload_key)
    except (OSError, ValueError):
        entry = None
    if entry and not extra_given:
        if entry.get("kernel_key") == kernel_key(kernel, n):
            roof["traffic"] = entry["bytes"]
            roof["traffic_over_algorithmic"] = round(entry["bytes"] / (bytes_per_sample * n), 3)
        else:
            roof["traffic_note"] = "profiles/traffic.json was measured on another kernel or launch size; run profile_counters.py"
    res = {
        "workload": name, "desc": cfg["desc"], "n": n, "samples_per_s": n * steps / wall, "ms_per_step": wall / steps * 1e3,
        "roofline": roof, "compile_s": round(compile_s, 2), "nodes": info["num_nodes"], "finite": finite,
        "kernel_key": kernel_key(kernel, n),
    }
    return res, kernel, x_host, cfg, spn, head


def host_path(kernel, x_host, torch):
    """samples/s of one spnc_hip_execute call: host array in, host array out, copies over PCIe included."""
    n = x_host.shape[0]
    kernel.execute(min(n, 1 << 20), x_host)       # staging buffers and streams exist after the first call
    best = 0.0
    for _ in range(2):
        t0 = time.perf_counter()
        kernel.execute(n, x_host)
        best = max(best, n / (time.perf_counter() - t0))
    res = {"pageable_samples_per_s": round(best, 1), "n": n,
           "note": "numpy -> numpy through spnc_hip_execute: threaded copy into pinned staging, H2D, kernel, D2H, chunks of 32 MiB "
                   "double-buffered on two streams"}
    try:   # the same call on buffers the caller has pinned: no staging copy
        xp = torch.from_numpy(x_host).pin_memory()
        op = torch.empty(n, dtype=torch.float32 if kernel.dataType() == "float32" else torch.float64).pin_memory()
        import ctypes
        from spnc import spncpy
        lib = spncpy._load()
        t0 = time.perf_counter()
        rc = lib.spnc_hip_execute(kernel._handle, n, ctypes.c_void_p(xp.data_ptr()), ctypes.c_void_p(op.data_ptr()))
        dt = time.perf_counter() - t0
        if rc == 0:
            res["pinned_samples_per_s"] = round(n / dt, 1)
    except RuntimeError:
        pass
    return res


def cpu_baseline(name, cfg, spn, x_host, gpu_head=None):
    """The restated CPUCompiler-equivalent kernel, timed on this host on a bounded sample of the same inputs, on all
    OpenMP threads and on one. Its results for the first rows are also held against what the GPU kernel wrote for them
    (`max_abs_diff_vs_gpu`; rows where both are minus infinity agree)."""
    sys.path.insert(0, ROOT)
    from oracle import c_oracle, cgen, spn_model as sm
    from xspn.serialization.binary.BinarySerialization import BinarySerializer
    from xspn.structure.Model import SPNModel
    from xspn.structure.Query import JointProbability
    with tempfile.TemporaryDirectory() as td:
        path = os.path.join(td, "q.bin")
        with contextlib.redirect_stdout(io.StringIO()):
            BinarySerializer(path).serialize_to_file(JointProbability(SPNModel(spn, cfg["dtype"], "cpu"), batchSize=4096,
                                                                      supportMarginal=cfg["marginal"]))
        model = sm.load_model(path)
        if name == "c4":
            # 46k sum terms as straight-line C take gcc minutes to compile; the region graph is timed on the oracle's
            # interpreting evaluator (oracle/spn_oracle.c, same operation order, OpenMP over samples).
            how = "oracle/spn_oracle.c (interpreting evaluator, gcc -O2 + OpenMP over samples)"
            threads = c_oracle.threads()
            run = lambda X: c_oracle.ll_f32(model, X, marginal=cfg["marginal"])   # noqa: E731
            set_threads = lambda t: c_oracle.threads(set_to=t)                    # noqa: E731
        else:
            how = "oracle/cgen.py (generated straight-line C, gcc -O3 -march=native, OpenMP chunks of 4096)"
            so, _ = cgen.build(model, cfg["marginal"], workdir=td)
            run = cgen.load(so, cfg["dtype"])
            threads = run.threads()
            set_threads = run.set_threads

        def rate(budget_s):
            probe_n = min(x_host.shape[0], 1 << 12)
            t0 = time.perf_counter()
            run(x_host[:probe_n])
            r = probe_n / (time.perf_counter() - t0)
            sample_n = int(min(x_host.shape[0], max(probe_n, r * budget_s)))
            t0 = time.perf_counter()
            run(x_host[:sample_n])
            return sample_n / (time.perf_counter() - t0), sample_n

        all_rate, all_n = rate(2.0)
        set_threads(1)
        one_rate, one_n = rate(1.5)
        set_threads(threads)
        diff = None
        if gpu_head is not None and len(gpu_head):
            import numpy as np
            ref = np.asarray(run(x_host[:len(gpu_head)]), dtype=np.float64)
            got = np.asarray(gpu_head, dtype=np.float64)
            both = np.isfinite(ref) & np.isfinite(got)
            same_inf = (np.isneginf(ref) == np.isneginf(got)).all() and not np.isnan(got).any()
            diff = float(np.abs(ref[both] - got[both]).max(initial=0.0)) if same_inf else float("inf")
    return {"value": all_rate, "unit": "samples/s", "cores": threads, "kind": "port", "one_thread_value": one_rate,
            "max_abs_diff_vs_gpu": diff,
            "sample": f"first {all_n} rows of the same batch ({one_n} for the one-thread figure), one pass each; {how}"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # Defaults: the chip takes 25-40 ms of load to settle (power management: launch 2 of the 100-feature discrete
    # configuration runs 0.60 ms, launches 5-8 0.75 ms, from about launch 40 on 0.58 ms; the 16-feature Gaussian one
    # falls from 1.9 to 1.57 ms over its first 12 launches). A job of many batches runs in the settled state.
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--config", default="c1", choices=["c1", "c2", "c3", "c3_deep", "c4", "c5", "c5_f64", "c4_f64"])
    ap.add_argument("--n", type=int, default=0, help="override the number of samples")
    ap.add_argument("--no-others", action="store_true", help="measure only the selected configuration")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baselines")
    ap.add_argument("--no-host", action="store_true", help="skip the host-path (numpy to numpy) rates")
    ap.add_argument("--fast-inputs", action="store_true",
                    help="draw the inputs on the device (same shapes and distributions) instead of the seeded NumPy arrays; implies "
                         "--no-cpu --no-host")
    ap.add_argument("--opt", action="append", default=[], help="extra compiler option key=value")
    ap.add_argument("--copy-gib", type=float, default=0.0,
                    help="instead of the benchmark, run a plain copy kernel (torch.mul by 1.0 into a second buffer) over this many GiB per step "
                         "(reference point for rocprofv3's FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: samples are independent, a multi-GPU run would only split the batch; use --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    device = torch.device("cuda:0")
    if args.copy_gib > 0:
        nbytes = int(args.copy_gib * 2 ** 30)
        a = torch.ones(nbytes // 4, dtype=torch.float32, device=device)
        b = torch.empty_like(a)
        # an elementwise kernel (a device-to-device copy_ would go to the runtime's copy engine path instead of a kernel)
        for _ in range(args.warmup):
            torch.mul(a, 1.0, out=b)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            torch.mul(a, 1.0, out=b)
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / args.steps
        print(json.dumps({"mode": "copy", "bytes_read_per_step": nbytes, "bytes_written_per_step": nbytes, "steps": args.steps,
                          "ms_per_step": dt * 1e3, "GB/s": 2 * nbytes / dt / 1e9}))
        return
    extra = dict(kv.split("=", 1) for kv in args.opt)
    log = io.StringIO()
    if args.fast_inputs:
        args.no_cpu = args.no_host = True

    def one(name):
        with contextlib.redirect_stdout(log):
            res, kernel, x_host, cfg, spn, head = measure(name, args.n if name == args.config else 0, args.steps, args.warmup, torch, device, extra,
                                                          args.fast_inputs)
        torch.cuda.empty_cache()
        if not args.no_host and name in ("c1", "c2"):
            with contextlib.redirect_stdout(log):
                res["host_path"] = host_path(kernel, x_host, torch)
        if not args.no_cpu:
            res["cpu_baseline"] = cpu_baseline(res["workload"], cfg, spn, x_host, head)
            if res.get("host_path") and res["cpu_baseline"]["value"] > 0:
                # below 1: for data that starts in host memory, the host's own cores finish sooner than the trip over PCIe
                res["host_path_vs_cpu_baseline"] = round(res["host_path"]["pageable_samples_per_s"] / res["cpu_baseline"]["value"], 3)
        os.remove(kernel.fileName())
        del kernel, x_host
        torch.cuda.empty_cache()
        return res

    res = one(args.config)
    others = {}
    if not args.no_others:
        for name in ALL:
            if name == args.config:
                continue
            r = one(name)
            others[name] = {k: (round(v, 4) if isinstance(v, float) else v) for k, v in r.items()
                            if k in ("samples_per_s", "n", "ms_per_step", "roofline", "nodes", "cpu_baseline", "host_path", "kernel_key",
                                     "compile_s", "host_path_vs_cpu_baseline")}
    line = {
        "metric": "samples/sec log-likelihood on 1 MI355X + % of HBM/FP32 roofline",
        "value": round(res["samples_per_s"], 1),
        "unit": "samples/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(res["ms_per_step"], 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f64" if args.config.endswith("_f64") else "f32",
        "data": ("synthetic (seeded NumPy generators for SPN parameters; inputs drawn on the device)" if args.fast_inputs else
                 "synthetic (seeded NumPy generators for SPN parameters and inputs, the arrays of the parity tests; inputs resident in HBM "
                 "before the timed region)"),
        "config": {"workload": f"{args.config}: {res['desc']}", "samples": res["n"], "nodes": res["nodes"], "kernel_key": res["kernel_key"]},
        "compile_s": res["compile_s"],      # compile_ll: serialise, build the graph, generate and hipRTC-compile the kernel (log_likelihood = this + execute)
        "roofline": res["roofline"],
        "cpu_baseline": res.get("cpu_baseline"),
        "host_path": res.get("host_path"),
        "host_path_vs_cpu_baseline": res.get("host_path_vs_cpu_baseline"),
        "target": {"samples_per_s": 1e9, "on": "c1 at 64M rows", "device_resident_met": None, "host_path_met": None},
        "others": others,
    }
    c1 = res if args.config == "c1" else others.get("c1")
    if c1:
        line["target"]["device_resident_met"] = bool(c1["samples_per_s"] >= 1e9)
        if c1.get("host_path"):
            line["target"]["host_path_met"] = bool(c1["host_path"]["pageable_samples_per_s"] >= 1e9)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
