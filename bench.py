#!/usr/bin/env python3
"""Benchmark of the batched joint log-likelihood path on one MI355X.

A step is one pass of the compiled SPN kernel over one batch of synthetic inputs that already
sit in HBM. The headline workload is configuration C2 (random sum/product tree over 16 Gaussian
features, 16M float32 rows); ``--config`` selects another one, and the remaining configurations
are measured with a few steps each and reported under "others" in the same JSON line.

Prints ONE JSON line: samples/s, the roofline of the kernel (HIP-event timed launches) and a CPU
baseline (the restated CPUCompiler-equivalent kernel of oracle/cgen.py on the host cores).
"""
import argparse
import json
import os
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "spn-compiler_amd"))

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
FP32_VECTOR_PEAK_TFLOPS = 157.3  # MI355X FP32 vector, published
FP64_VECTOR_PEAK_TFLOPS = 78.6   # MI355X FP64 vector, published

# HBM bytes per launch from the counter runs summarised in profiles/<kernel>_<workload>.txt:
# workload -> (samples per launch, bytes). Only valid for that launch size and the default options.
MEASURED_HBM_TRAFFIC = {
    "c1": (67108864, 1879038771),
    "c2": (16777216, 1142069219),
    "c3": (8388608, 3394635282),
    "c4": (4194304, 5884685364),
    "c5": (16777216, 1141489239),
    "c5_f64": (16777216, 1210340500),
}


def make_inputs(name, cfg, n, torch, device):
    """Synthetic inputs of the configuration's shape and distribution, generated on the device."""
    from spnc import synthetic as syn
    g = torch.Generator(device=device)
    g.manual_seed({"c1": 1, "c2": 102, "c3": 103, "c3_deep": 103, "c4": 104, "c5": 102}[name])
    F = cfg["features"]
    if name == "c1":
        return torch.randint(0, 3, (n, F), generator=g, device=device, dtype=torch.int32)
    if name in ("c3", "c3_deep"):
        doms = torch.tensor([d for _, d in syn.c3_domains()], device=device, dtype=torch.float32)
        u = torch.rand((n, F), generator=g, device=device)
        return torch.minimum((u * doms).floor(), doms - 1).to(torch.int32)
    x = torch.randn((n, F), generator=g, device=device, dtype=torch.float32)
    if name == "c5":
        g2 = torch.Generator(device=device)
        g2.manual_seed(105)
        mask = torch.rand((n, F), generator=g2, device=device) < 0.2
        x[mask] = float("nan")
    return x


def measure(name, n, steps, warmup, torch, device, extra_options=None):
    from spnc import synthetic as syn
    from spnc.hip import HIPCompiler
    workload_key, extra_given = name, bool(extra_options)
    if name == "c5_f64":   # configuration 5 computed in float64 log-space
        name, extra_options = "c5", dict(extra_options or {}, **{"hip-compute-type": "float64"})
    cfg = syn.CONFIGS[name]
    n = n or cfg["n"]
    spn = cfg["spn"]()
    t0 = time.time()
    kernel = HIPCompiler(**(extra_options or {})).compile_ll(spn, cfg["dtype"], supportMarginal=cfg["marginal"])
    compile_s = time.time() - t0
    info = kernel.info()
    x = make_inputs(name, cfg, n, torch, device)
    out = torch.empty(n, device=device, dtype=torch.float32 if info["dtype"] == "float32" else torch.float64)
    stream = torch.cuda.current_stream().cuda_stream

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
                      "published vector peak (FP32 157.3, FP64 78.6 TFLOP/s) counts an FMA as 2 flops; this path issues "
                      "mostly single-flop instructions, so the ceiling is half of it in issue slots/s; achieved = (flops - fused "
                      "multiply-add pairs + 3*transcendentals) per sample; a float64 exp/log is in fact about 11 double-rate instructions and an LDS read, not 4 slots"),
        "fma_flops_tflops": round(tflops, 3),
        "kernel": "spn_kernel (hipRTC straight-line)" if info["kernel_kind"] == 1 else "spn_interp_kernel",
        "launch_ms": round(launch_ms, 4),
        "bytes_per_sample": bytes_per_sample,
        "flops_per_sample": flops,
        "transcendentals_per_sample": trans,
        "fused_multiply_adds_per_sample": info["fused_min"],
        "issue_slots_per_sample": slots,
        "valu_issue_peak_per_s": valu_peak,
        "valu_issue_frac": round(t_min_valu / t_launch, 4),
        "hbm_frac": round(t_min_hbm / t_launch, 4),
    }
    # HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (scaled by what a
    # plain copy of known size reads on the same counters); recorded per workload under profiles/.
    entry = MEASURED_HBM_TRAFFIC.get(workload_key)
    if entry and entry[0] == n and not extra_given:
        roof["traffic"] = entry[1]
        roof["traffic_over_algorithmic"] = round(entry[1] / (bytes_per_sample * n), 3)
    res = {
        "workload": name, "desc": cfg["desc"], "n": n, "samples_per_s": n * steps / wall, "ms_per_step": wall / steps * 1e3,
        "roofline": roof, "compile_s": round(compile_s, 2), "nodes": info["num_nodes"], "finite": finite,
    }
    os.remove(kernel.fileName())
    return res, x, cfg, spn


def cpu_baseline(name, cfg, spn, x_dev, torch):
    """The restated CPUCompiler-equivalent kernel (oracle/cgen.py), timed on this host on a bounded
    sample of the same inputs."""
    sys.path.insert(0, ROOT)
    from oracle import cgen, spn_model as sm
    from xspn.serialization.binary.BinarySerialization import BinarySerializer
    from xspn.structure.Model import SPNModel
    from xspn.structure.Query import JointProbability
    import contextlib
    import io
    with tempfile.TemporaryDirectory() as td:
        path = os.path.join(td, "q.bin")
        with contextlib.redirect_stdout(io.StringIO()):
            BinarySerializer(path).serialize_to_file(JointProbability(SPNModel(spn, cfg["dtype"], "cpu"), batchSize=4096,
                                                                      supportMarginal=cfg["marginal"]))
        model = sm.load_model(path)
        so, _ = cgen.build(model, cfg["marginal"], workdir=td)
        run = cgen.load(so, cfg["dtype"])
        cores = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(16, os.cpu_count() or 1)
        probe_n = min(x_dev.shape[0], 1 << 16)
        xp = x_dev[:probe_n].cpu().numpy()
        run(xp[:4096])
        t0 = time.perf_counter()
        run(xp)
        rate = probe_n / (time.perf_counter() - t0)
        sample_n = int(min(x_dev.shape[0], max(probe_n, rate * 5.0)))  # about 5 s per pass
        xs = x_dev[:sample_n].cpu().numpy()
        best = 0.0
        t_all = time.perf_counter()
        for _ in range(3):
            t0 = time.perf_counter()
            run(xs)
            best = max(best, sample_n / (time.perf_counter() - t0))
            if time.perf_counter() - t_all > 20:
                break
    return {"value": best, "unit": "samples/s", "cores": cores, "kind": "port",
            "sample": f"first {sample_n} rows of the same batch, best of up to 3 passes, gcc -O3 -march=native + OpenMP chunks of 4096"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", default="c2", choices=["c1", "c2", "c3", "c3_deep", "c4", "c5", "c5_f64"])
    ap.add_argument("--n", type=int, default=0, help="override the number of samples")
    ap.add_argument("--no-others", action="store_true", help="measure only the selected configuration")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--opt", action="append", default=[], help="extra compiler option key=value")
    ap.add_argument("--copy-gib", type=float, default=0.0,
                    help="instead of the benchmark, run a plain device-to-device copy of this many GiB per step "
                         "(reference point for rocprofv3's FETCH_SIZE / WRITE_SIZE counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: samples are independent, a multi-GPU run would only split the batch; use --gpus 1",
              file=sys.stderr)
        sys.exit(2)
    import contextlib
    import io
    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    device = torch.device("cuda:0")
    if args.copy_gib > 0:
        nbytes = int(args.copy_gib * 2 ** 30)
        a = torch.ones(nbytes // 4, dtype=torch.float32, device=device)
        b = torch.empty_like(a)
        for _ in range(args.warmup):
            b.copy_(a)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            b.copy_(a)
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / args.steps
        print(json.dumps({"mode": "copy", "bytes_read_per_step": nbytes, "bytes_written_per_step": nbytes, "steps": args.steps,
                          "ms_per_step": dt * 1e3, "GB/s": 2 * nbytes / dt / 1e9}))
        return
    extra = dict(kv.split("=", 1) for kv in args.opt)
    log = io.StringIO()
    with contextlib.redirect_stdout(log):
        res, x, cfg, spn = measure(args.config, args.n, args.steps, args.warmup, torch, device, extra)
    cpu = None
    if not args.no_cpu:
        cpu = cpu_baseline(args.config, cfg, spn, x, torch)
    del x
    torch.cuda.empty_cache()
    others = {}
    if not args.no_others:
        for name in ["c1", "c2", "c3", "c4", "c5", "c5_f64"]:
            if name == args.config:
                continue
            with contextlib.redirect_stdout(log):
                r, xo, _, _ = measure(name, 0, max(3, args.steps // 4), 2, torch, device, extra)
            del xo
            torch.cuda.empty_cache()
            others[name] = {"samples_per_s": round(r["samples_per_s"], 1), "n": r["n"], "ms_per_step": round(r["ms_per_step"], 4),
                            "roofline": r["roofline"], "nodes": r["nodes"]}
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
        "dtype": "f32",
        "data": "synthetic (seeded, generated on the device; random SPN parameters from seeded NumPy generators)",
        "config": {"workload": f"{args.config}: {res['desc']}", "samples": res["n"], "nodes": res["nodes"]},
        "roofline": res["roofline"],
        "cpu_baseline": cpu,
        "others": others,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
