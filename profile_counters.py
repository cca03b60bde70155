#!/usr/bin/env python3
"""Collects the rocprofv3 evidence behind bench.py's roofline figures, on a machine with an MI355X.

For every benchmark configuration it runs bench.py under rocprofv3 (kernel trace, then the HBM traffic counters
FETCH_SIZE and WRITE_SIZE, then two sets of SQ counters), each in a pass of its own, and writes

  profiles/<kernel>_<config>.txt   the figures, with the command of every pass
  profiles/copy_kernel_counters.txt  what the traffic counters read for a plain 4 GiB device copy (their calibration)
  profiles/traffic.json            HBM bytes per launch per configuration, with bench.py's key of the kernel measured

usage: python3 profile_counters.py [config ...]       (default: all seven; raw profiler output goes to a temporary directory)
"""
import glob
import json
import os
import re
import shutil
import sqlite3
import subprocess
import sys
import tempfile

ROOT = os.path.dirname(os.path.abspath(__file__))
BENCH = os.path.join(ROOT, "bench.py")
STEPS, WARMUP = 50, 50   # bench.py's own defaults: the timed launches start once the chip has settled under the load
KERNELS = {"c1": "spn_kernel", "c2": "spn_kernel", "c3": "spn_kernel", "c4": "spn_interp_kernel", "c5": "spn_kernel", "c5_f64": "spn_kernel", "c4_f64": "spn_interp_kernel"}
SQ_SETS = [
    "SQ_INSTS_VALU SQ_INSTS_SALU SQ_INSTS_SMEM SQ_INSTS_LDS SQ_WAVE_CYCLES SQ_BUSY_CYCLES SQ_ACTIVE_INST_VALU SQ_WAIT_INST_ANY",
    "SQ_WAVES SQ_INSTS_VALU_TRANS SQ_ACTIVE_INST_LDS SQ_LDS_BANK_CONFLICT SQ_INSTS_VMEM_RD SQ_INSTS_VMEM_WR SQ_INSTS_MFMA SQ_ACTIVE_INST_ANY",
    "SQ_LDS_IDX_ACTIVE SQ_LDS_ADDR_CONFLICT SQ_WAIT_INST_LDS SQ_WAIT_ANY SQ_INST_CYCLES_VMEM",
]


def rocprof(work, tag, profiler_args, program_args, timeout=400):
    """One rocprofv3 pass; returns (sqlite connection, stdout of the program). The program follows `--` directly."""
    out = os.path.join(work, tag)
    cmd = ["rocprofv3"] + profiler_args + ["-d", out, "-o", tag, "--", "python3", BENCH] + program_args
    env = dict(os.environ, TMPDIR="/tmp")
    print("  pass " + tag, flush=True)
    r = subprocess.run(cmd, cwd="/tmp", env=env, capture_output=True, text=True, timeout=timeout)
    if r.returncode != 0:
        raise RuntimeError("rocprofv3 failed: %s\n%s" % (" ".join(cmd), r.stderr[-2000:]))
    dbs = glob.glob(os.path.join(out, "**", "*.db"), recursive=True)
    shown = "rocprofv3 " + " ".join(profiler_args) + " -- python3 bench.py " + " ".join(program_args)
    return sqlite3.connect(dbs[0]), r.stdout, shown


def kernel_stats(con):
    rows = con.execute("select name, count(*), avg(end-start), min(end-start), max(end-start), sum(end-start) from kernels "
                       "group by name order by sum(end-start) desc").fetchall()
    total = sum(r[5] for r in rows)
    lines = ["%-46s %6s %12s %12s %12s %7s" % ("kernel", "calls", "avg_ns", "min_ns", "max_ns", "%time")]
    for r in rows[:4]:
        lines.append("%-46s %6d %12.0f %12d %12d %6.1f%%" % (r[0][:46], r[1], r[2], r[3], r[4], 100.0 * r[5] / total))
    return lines, rows


def timed_launches(con, like, steps):
    """Average duration (ns) of the kernel's last `steps` dispatches: the ones bench.py times, after its warm-up launches."""
    rows = con.execute("select end-start from kernels where name like ? order by start desc limit ?", (like, steps)).fetchall()
    return sum(r[0] for r in rows) / len(rows), len(rows)


def counters(con, like):
    return con.execute("select counter_name, sum(counter_value)/count(distinct dispatch_id), count(distinct dispatch_id) from pmc_events "
                       "where name like ? group by counter_name order by counter_name", (like,)).fetchall()


def main():
    configs = sys.argv[1:] or list(KERNELS)
    work = tempfile.mkdtemp(prefix="spn_prof_", dir="/tmp")
    prof = os.path.join(ROOT, "profiles")
    os.makedirs(prof, exist_ok=True)
    # ---- calibration: what the traffic counters read for a copy of known size ----
    units, copy_lines = {}, []
    for counter in ("FETCH_SIZE", "WRITE_SIZE"):
        con, _, shown = rocprof(work, "copy_" + counter, ["--pmc", counter], ["--copy-gib", "4", "--steps", "5", "--warmup", "1"])
        # all dispatches of the copy kernel (the library may split one copy over several), not the fill that makes its input
        total = con.execute("select sum(counter_value) from pmc_events where counter_name = ? and (name like '%Mul%' or name like '%mul%')",
                            (counter,)).fetchone()[0]
        value = total / 6.0   # per copy: five timed and one warm-up
        units[counter] = 4 * 1048576.0 / value      # KiB per counter unit
        copy_lines += ["$ " + shown, "%-46s %-12s per 4 GiB copy=%.1f" % ("copy kernel", counter, value)]
    with open(os.path.join(prof, "copy_kernel_counters.txt"), "w") as f:
        f.write("Plain copy kernel over 4 GiB (torch.mul(a, 1.0, out=b) on float32), the reference point for the FETCH_SIZE and WRITE_SIZE\n"
                "counters of rocprofv3 on MI355X: the copy reads 4 GiB and writes 4 GiB (4194304 KiB each; far more than the 256 MiB\n"
                "of last-level cache could hold back from HBM).\n"
                "Made by: python3 profile_counters.py\n\n" + "\n".join(copy_lines) +
                "\n\nOne FETCH_SIZE unit is %.3f KiB, one WRITE_SIZE unit %.3f KiB.\n" % (units["FETCH_SIZE"], units["WRITE_SIZE"]))
    try:
        traffic = json.load(open(os.path.join(prof, "traffic.json")))
    except (OSError, ValueError):
        traffic = {}
    for cfg in configs:
        name = KERNELS[cfg]
        like = "%" + name + "%"
        common = ["--config", cfg, "--no-others", "--fast-inputs"]
        con, stdout, shown = rocprof(work, "stats_" + cfg, ["--kernel-trace", "--stats"], common + ["--steps", str(STEPS), "--warmup", str(WARMUP)])
        line = json.loads(stdout.strip().splitlines()[-1])
        roof, n = line["roofline"], line["config"]["samples"]
        stats, rows = kernel_stats(con)
        avg_ns, timed = timed_launches(con, like, STEPS)
        stats.append("%-46s %6d %12.0f   (the last %d calls: the launches bench.py times, after %d warm-up launches)" % (name[:46], timed, avg_ns, timed, WARMUP))
        text = ["Kernel %s, workload %s" % (name, line["config"]["workload"]),
                "MI355X (gfx950), %d samples per launch. Made by: python3 profile_counters.py %s" % (n, cfg),
                "Every pass is one rocprofv3 run of bench.py (inputs drawn on the device: --fast-inputs); figures are read from the sqlite",
                "database rocprofv3 writes (kernels: name, count, avg/min/max of end-start; pmc_events: counter sums per dispatch).", "",
                "$ " + shown] + stats
        per_launch = {}
        for counter in ("FETCH_SIZE", "WRITE_SIZE"):
            con, _, shown = rocprof(work, counter + "_" + cfg, ["--pmc", counter], common + ["--steps", "5"])
            value = next(r[1] for r in counters(con, like) if r[0] == counter)
            per_launch[counter] = value
            text += ["$ " + shown, "%-46s %-12s per-dispatch=%.1f units" % (name, counter, value)]
        hbm_bytes = (per_launch["FETCH_SIZE"] * units["FETCH_SIZE"] + per_launch["WRITE_SIZE"] * units["WRITE_SIZE"]) * 1024
        algorithmic = roof["bytes_per_sample"] * n
        text += ["", "bench.py, same run as the kernel trace: %.4g samples/s, launch %.4f ms (HIP events); rocprofv3 average of the same launches %.4f ms."
                 % (line["value"], roof["launch_ms"], avg_ns / 1e6),
                 "roofline bound %s, achieved %s of %s %s = %s." % (roof["bound"], roof["achieved"], roof["peak"], roof["unit"], roof["frac"]),
                 "Counter calibration (profiles/copy_kernel_counters.txt): FETCH_SIZE x %.3f, WRITE_SIZE x %.3f give KiB of HBM traffic."
                 % (units["FETCH_SIZE"], units["WRITE_SIZE"]),
                 "HBM traffic per launch: %.3f GiB; algorithmic bytes (inputs + results) %.3f GiB; ratio %.3f."
                 % (hbm_bytes / 2 ** 30, algorithmic / 2 ** 30, hbm_bytes / algorithmic), "",
                 "Instruction and cycle counters, summed over the chip, per launch (one wave-level instruction covers 64 samples,",
                 "%d wavefronts' worth of samples per launch):" % (n // 64)]
        seen = set()
        for k, counters_list in enumerate(SQ_SETS):
            con, _, shown = rocprof(work, "sq%d_%s" % (k, cfg), ["--pmc"] + counters_list.split(), common + ["--steps", "3"])
            text.append("$ " + shown)
            for cname, value, dispatches in counters(con, like):
                seen.add(cname)
                text.append("%-26s %.5g per dispatch (%d dispatches)" % (cname, value, dispatches))
        if "SQ_INSTS_VALU_TRANS" not in seen:
            text += ["SQ_INSTS_VALU_TRANS is requested above and comes back without rows: rocprofv3 exposes no transcendental counter on gfx950.",
                     "Derived instead: %d transcendentals per sample (algorithmic count of the graph) x %d wavefronts = %.4g wave-level"
                     % (roof["transcendentals_per_sample"], n // 64, roof["transcendental_wave_instructions_per_launch"]),
                     "transcendental instructions per launch (each a quarter-rate instruction, i.e. four issue slots)."]
        with open(os.path.join(prof, "%s_%s.txt" % (name, cfg)), "w") as f:
            f.write("\n".join(text) + "\n")
        traffic[cfg] = {"n": n, "bytes": int(round(hbm_bytes)), "kernel_key": line["config"]["kernel_key"],
                        "fetch_units": per_launch["FETCH_SIZE"], "write_units": per_launch["WRITE_SIZE"]}
        with open(os.path.join(prof, "traffic.json"), "w") as f:
            json.dump(traffic, f, indent=1, sort_keys=True)
            f.write("\n")
        print("%-7s %.4g samples/s launch %.4f ms (rocprofv3 avg %.4f ms) %s frac %.4f traffic x%.3f"
              % (cfg, line["value"], roof["launch_ms"], avg_ns / 1e6, roof["bound"], roof["frac"], hbm_bytes / algorithmic), flush=True)
    shutil.rmtree(work, ignore_errors=True)


if __name__ == "__main__":
    main()
