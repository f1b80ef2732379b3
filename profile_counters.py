"""Summarises rocprofv3 runs of bench.py into profiles/: one short text file a pass and profiles/counters.json, the
per-kernel hardware counters bench.py quotes in its `roofline` object.  counters.json is stamped with the cache keys of
the kernel files the counters were measured on (shadow_engine_amd.program_keys()); bench.py prints the counters only while
those keys are the keys of the sources it runs, so a kernel edit turns the quoted figures into null until the passes below
have been run again.

The passes, each a run of its own from the repository root after `cd /tmp && export TMPDIR=/tmp && cd <repo>`; W is a
workload of bench.py, ARGS its flags (`--workload W`, nothing for the default one), D = PROF/W for a scratch directory PROF:

    python3 bench.py ARGS --no-cpu-baseline --no-other-configs > D/plain.json                      (no profiler: the timings)
    rocprofv3 --kernel-trace --stats -d D/trace -o run -- python3 bench.py ARGS --steps 20 --warmup 3 --no-cpu-baseline --no-other-configs
    rocprofv3 --pmc FETCH_SIZE -d D/fetch -o run -- python3 bench.py ARGS --steps 2 --warmup 1 --no-cpu-baseline --no-other-configs --copy-calibration 1073741824
    rocprofv3 --pmc WRITE_SIZE -d D/write -o run -- python3 bench.py ARGS --steps 2 --warmup 1 --no-cpu-baseline --no-other-configs --copy-calibration 1073741824
    rocprofv3 --pmc SQ_INSTS_VALU SQ_ACTIVE_INST_VALU SQ_BUSY_CYCLES SQ_WAVES SQ_WAVE_CYCLES SQ_WAIT_INST_ANY SQ_INSTS_SALU SQ_INSTS_LDS -d D/sq -o run -- python3 bench.py ARGS --steps 2 --warmup 1 --no-cpu-baseline --no-other-configs
    rocprofv3 --pmc SQ_INSTS_MFMA SQ_VALU_MFMA_BUSY_CYCLES SQ_LDS_BANK_CONFLICT SQ_ACTIVE_INST_LDS SQ_INSTS_VMEM_RD SQ_WAIT_ANY SQ_ACTIVE_INST_ANY SQ_INSTS_VMEM_WR -d D/sq2 -o run -- python3 bench.py ARGS --steps 2 --warmup 1 --no-cpu-baseline --no-other-configs
    rocprofv3 --pmc TCC_HIT_sum TCC_MISS_sum TCC_REQ_sum TCC_EA0_RDREQ_sum -d D/l2 -o run -- python3 bench.py ARGS --steps 2 --warmup 1 --no-cpu-baseline --no-other-configs

then, in the same session (the databases are large and are not kept):

    python3 profile_counters.py PROF

A workload may have any subset of the passes.  Memory counters are scaled by what the same counter reads for the plain
copy of known size that `--copy-calibration` appends to the run (copy_words16: 1 GiB read, 1 GiB written).
"""
import json
import os
import sqlite3
import sys

ROOT = os.path.dirname(os.path.abspath(__file__))
OURS = ("verify_", "decode_", "head_", "argmax_merge", "copy_", "matvec_", "route_", "swiglu", "moe_", "prefill_", "quant_act", "scatter_", "exl3_", "topk_", "proxy_")
NAMES = {"config5": ("verify_round_config5", "the default benchmark workload (config 5: 48-layer verify round on a 4-row batch, mixed EXL3 K in {2,3,4}, Q8_0 lm_head)", ""),
         "config5_mode2": ("verify_round_config5_matrix_cores", "bench.py --expert-mode 2 (the config-5 round with the experts on the matrix cores: plan of distinct experts, f16 products, the linearised codebook)",
                           " --expert-mode 2"),
         "config5_mode3": ("verify_round_config5_f16_inputs", "bench.py --expert-mode 3 (the config-5 round with the exact launches' inputs rounded to f16, two products an instruction)",
                           " --expert-mode 3"),
         "exl3prefill": ("prefill_chunk_exl3_k3", "bench.py --workload exl3prefill (prefill chunk: 512 tokens through 512 EXL3 K=3 experts + the shared one, f16 matrix cores)", " --workload exl3prefill"),
         "config3": ("verify_layer_and_head_config3", "bench.py --workload config3 (one EXL3 K=3 MoE layer for 4 tokens + Q8_0 head + acceptance)", " --workload config3"),
         "config1": ("matvec_q8_0_config1", "bench.py --workload config1 (one Q8_0 1024 x 2048 matrix-vector product)", " --workload config1"),
         "config2": ("iq3s_decode_layer_config2", "bench.py --workload config2 (IQ3_S MoE layer for one token, 8 different layers a step)", " --workload config2"),
         "config4": ("prefill_chunk_config4", "bench.py --workload config4 (prefill chunk: 512 tokens through 512 IQ3_S experts, int8 matrix cores)", " --workload config4"),
         "exl3head": ("head_exl3_k4_lm_head", "bench.py --workload exl3head (EXL3 K=4 lm_head 151936 x 2048, 4-row batch, arg-max fused in)", " --workload exl3head"),
         "exl3top": ("head_exl3_k4_top64", "bench.py --workload exl3top (top-64 hand-off of the EXL3 K=4 lm_head 151936 x 2048 for 4 rows, exact)", " --workload exl3top"),
         "exl3top_screen": ("head_exl3_k4_top64_screened", "bench.py --workload exl3top --screen 128 (the same hand-off through the inexact 2-bit screen, 128 blocks a row)",
                            " --workload exl3top --screen 128"),
         "stage": ("stage_exl3_layer", "bench.py --workload stage (one EXL3 layer of a safetensors checkpoint staged into HBM)", " --workload stage"),
         "snapshot": ("copy_ranges_snapshot", "bench.py --workload snapshot (73 device ranges saved and put back)", " --workload snapshot")}
SQ1 = "SQ_INSTS_VALU SQ_ACTIVE_INST_VALU SQ_BUSY_CYCLES SQ_WAVES SQ_WAVE_CYCLES SQ_WAIT_INST_ANY SQ_INSTS_SALU SQ_INSTS_LDS"
SQ2 = "SQ_INSTS_MFMA SQ_VALU_MFMA_BUSY_CYCLES SQ_LDS_BANK_CONFLICT SQ_ACTIVE_INST_LDS SQ_INSTS_VMEM_RD SQ_WAIT_ANY SQ_ACTIVE_INST_ANY SQ_INSTS_VMEM_WR"
L2 = "TCC_HIT_sum TCC_MISS_sum TCC_REQ_sum TCC_EA0_RDREQ_sum"
TAIL = " --no-cpu-baseline --no-other-configs"
SHADER_ENGINES = 32          # SQ_BUSY_CYCLES is summed over the 32 shader engines (8 XCDs x 4)
SIMDS = 1024
PROF = "PROF"              # the directory the passes wrote to, as the summaries quote it in their commands


def rows(db, sql):
    con = sqlite3.connect(db)
    try:
        return list(con.cursor().execute(sql))
    finally:
        con.close()


def ours(name):
    return any(name.startswith(o) for o in OURS)


def clean(name):
    return name[:-3] if name.endswith(".kd") else name


def trace_summary(d, plain, title, args):
    r = rows(os.path.join(d, "trace", "run_results.db"),
             "select name, count(*), sum(duration), avg(duration), min(duration), max(duration) from kernels group by name order by 3 desc")
    r = [(clean(n), c, t, a, mn, mx) for n, c, t, a, mn, mx in r if ours(clean(n))]
    tot = sum(x[2] for x in r) or 1
    out = ["Kernel trace of %s on one MI355X." % title,
           "Command (from the repository root after cd /tmp && export TMPDIR=/tmp && cd <repo>; the rocpd database it writes is summarised by",
           "python3 profile_counters.py with: select name, count(*), sum(duration), avg, min, max from kernels group by name):",
           "  rocprofv3 --kernel-trace --stats -d %s/W/trace -o run -- python3 bench.py%s --steps 20 --warmup 3%s" % (PROF, args, TAIL), "",
           "%-28s %7s %12s %10s %10s %10s %7s" % ("kernel (this library's only)", "calls", "total_us", "avg_us", "min_us", "max_us", "pct")]
    for n, c, t, a, mn, mx in r:
        out.append("%-28s %7d %12.1f %10.2f %10.2f %10.2f %7.2f" % (n, c, t / 1e3, a / 1e3, mn / 1e3, mx / 1e3, 100 * t / tot))
    durations = {n: a / 1e3 for n, c, t, a, mn, mx in r}
    if plain:
        out += ["", "The calls include the timed steps (graph replays where the workload has a graph), the warm-up and the eager steps that bench.py",
                "times launch by launch.  bench.py's own per-kernel averages (start/stop events that carry the dispatch's time stamps, eager steps)",
                "from a run of the same command without the profiler (python3 bench.py%s%s):" % (args, TAIL)]
        for k, v in plain["kernels"].items():
            out.append("  %-28s avg_us %8.2f  launches/step %d%s" % (k, v["avg_us"], v["launches_per_step"],
                                                                    ("   trace/bench %.3f" % (durations[k] / v["avg_us"])) if k in durations and v["avg_us"] else ""))
        out.append("  step: ms_per_step %.4f, value %.1f GB/s algorithmic (%s%% of 8 TB/s)" % (plain["ms_per_step"], plain["value"], plain["pct_of_8TBps"]))
    return "\n".join(out) + "\n", durations


def pmc(db):
    """{kernel: {counter: (launches, mean value, mean duration ns)}}"""
    out = {}
    for k, c, n, v, dur in rows(db, "select kernel_name, counter_name, count(*), avg(value), avg(duration) from counters_collection group by 1, 2"):
        out.setdefault(clean(k), {})[c] = (n, v, dur)
    return out


def traffic_summary(d, plain, title, args):
    f, w = pmc(os.path.join(d, "fetch", "run_results.db")), pmc(os.path.join(d, "write", "run_results.db"))
    copy_kib = (1 << 30) / 1024.0
    # the calibration launch is the largest copy of the run (a workload's cold-cache measurement launches smaller ones)
    biggest = lambda p, c: rows(os.path.join(d, p, "run_results.db"),
                                "select max(value) from counters_collection where counter_name = '%s' and kernel_name like 'copy_words16%%'" % c)[0][0]
    fcal, wcal = biggest("fetch", "FETCH_SIZE"), biggest("write", "WRITE_SIZE")
    fs, ws = copy_kib / fcal, copy_kib / wcal
    out = ["HBM traffic per launch of the kernels of %s, from the memory counters, one counter a run, on one MI355X." % title,
           "Commands (each from the repository root, after cd /tmp && export TMPDIR=/tmp && cd <repo>):",
           "  rocprofv3 --pmc FETCH_SIZE -d %s/W/fetch -o run -- python3 bench.py%s --steps 2 --warmup 1%s --copy-calibration 1073741824" % (PROF, args, TAIL),
           "  rocprofv3 --pmc WRITE_SIZE -d %s/W/write -o run -- python3 bench.py%s --steps 2 --warmup 1%s --copy-calibration 1073741824" % (PROF, args, TAIL), "",
           "Calibration: the run ends with one launch of copy_words16 that reads 1 GiB and writes 1 GiB (1048576 KiB each).",
           "  FETCH_SIZE reads %.1f for it -> scale %.5f      WRITE_SIZE reads %.1f for it -> scale %.5f" % (fcal, fs, wcal, ws), "",
           "%-26s %6s %14s %14s %14s %16s %8s" % ("kernel", "calls", "fetched KiB", "written KiB", "traffic bytes", "algorithmic bytes", "ratio")]
    traffic = {}
    for k in sorted(f):
        if k == "copy_words16" or not ours(k) or "FETCH_SIZE" not in f[k]:
            continue
        fk = f[k]["FETCH_SIZE"][1] * fs
        wk = w.get(k, {}).get("WRITE_SIZE", (0, 0.0, 0))[1] * ws
        tb = (fk + wk) * 1024
        traffic[k] = int(tb)
        alg = plain["kernels"].get(k, {}).get("bytes_per_launch") if plain else None
        out.append("%-26s %6d %14.1f %14.1f %14d %16s %8s" % (k, f[k]["FETCH_SIZE"][0], fk, wk, tb, alg if alg else "-", ("%.3f" % (tb / alg)) if alg else "-"))
    out += ["", "Algorithmic bytes are bench.py's: every distinct weight byte a launch touches once, plus the activations and partial sums it reads",
            "and writes.  A kernel that works on (token, expert) pairs fetches an expert chosen by two tokens of the batch, and the shared expert",
            "of every token, once a pair; not every repeat hits in L2, which is what a ratio above 1 shows."]
    return "\n".join(out) + "\n", traffic, {"FETCH_SIZE": fs, "WRITE_SIZE": ws}


def sq_summary(d, title, args):
    c = pmc(os.path.join(d, "sq", "run_results.db"))
    second = os.path.join(d, "sq2", "run_results.db")
    c2 = pmc(second) if os.path.exists(second) else {}
    out = ["Shader counters per launch of the kernels of %s on one MI355X." % title,
           "Commands (each from the repository root, after cd /tmp && export TMPDIR=/tmp && cd <repo>; averaged over a kernel's launches with",
           "select kernel_name, counter_name, count(*), avg(value), avg(duration) from counters_collection group by 1, 2):",
           "  rocprofv3 --pmc %s -d %s/W/sq -o run -- python3 bench.py%s --steps 2 --warmup 1%s" % (SQ1, PROF, args, TAIL)]
    if c2:
        out.append("  rocprofv3 --pmc %s -d %s/W/sq2 -o run -- python3 bench.py%s --steps 2 --warmup 1%s" % (SQ2, PROF, args, TAIL))
    out += ["", "%-26s %6s %9s %12s %12s %10s %9s %7s %9s %10s" % ("kernel", "calls", "waves", "INSTS_VALU", "ACTIVE_VALU", "cycles", "us (pmc)", "GHz", "VALU busy", "wait-issue")]
    kernels = {}
    for k in sorted(c, key=lambda k: -c[k].get("SQ_INSTS_VALU", (0, 0, 0))[1] * c[k].get("SQ_INSTS_VALU", (0, 0, 0))[0]):
        v = c[k]
        if not ours(k) or "SQ_BUSY_CYCLES" not in v:
            continue
        n, busy, dur = v["SQ_BUSY_CYCLES"]
        cycles = busy / SHADER_ENGINES
        ghz = cycles / dur if dur else 0.0
        valu, act = v["SQ_INSTS_VALU"][1], v["SQ_ACTIVE_INST_VALU"][1]
        busy_frac = act * 4.0 / SIMDS / cycles if cycles else 0.0
        wait = v["SQ_WAIT_INST_ANY"][1] / v["SQ_WAVE_CYCLES"][1] if v.get("SQ_WAVE_CYCLES", (0, 0, 0))[1] else 0.0
        out.append("%-26s %6d %9d %12d %12d %10d %9.2f %7.3f %8.1f%% %9.1f%%" % (k, n, v["SQ_WAVES"][1], valu, act, cycles, dur / 1e3, ghz, 100 * busy_frac, 100 * wait))
        e = {"launches": n, "SQ_WAVES": round(v["SQ_WAVES"][1]), "SQ_INSTS_VALU": round(valu), "SQ_ACTIVE_INST_VALU": round(act), "busy_cycles": round(cycles),
             "duration_us_in_counter_run": round(dur / 1e3, 2), "clock_ghz": round(ghz, 3), "valu_busy_frac": round(busy_frac, 4),
             "SQ_INSTS_SALU": round(v["SQ_INSTS_SALU"][1]), "SQ_INSTS_LDS": round(v["SQ_INSTS_LDS"][1]), "wait_to_issue_frac": round(wait, 4)}
        for name, val in c2.get(k, {}).items():
            e[name] = round(val[1])
        kernels[k] = e
    out += ["", "cycles = SQ_BUSY_CYCLES / 32 (the counter is summed over the 32 shader engines); GHz = cycles / the launch's duration in the same run;",
            "VALU busy = SQ_ACTIVE_INST_VALU (quad-cycles) x 4 / 1024 SIMDs / cycles; wait-issue = SQ_WAIT_INST_ANY / SQ_WAVE_CYCLES (the share of",
            "its life a wave spends with an instruction ready that the SIMD does not take)."]
    if c2:
        names = SQ2.split()
        out += ["", "%-26s " % "kernel" + " ".join("%14s" % n.replace("SQ_", "")[:14] for n in names)]
        for k in kernels:
            if k in c2:
                out.append("%-26s " % k + " ".join("%14d" % c2[k].get(n, (0, 0, 0))[1] for n in names))
    third = os.path.join(d, "l2", "run_results.db")
    if os.path.exists(third):
        c3 = pmc(third)
        out += ["", "The L2 caches (summed over the 8 XCDs' channels), averages a launch:",
                "  rocprofv3 --pmc %s -d %s/W/l2 -o run -- python3 bench.py%s --steps 2 --warmup 1%s" % (L2, PROF, args, TAIL),
                "%-26s %14s %14s %14s %14s %9s" % ("kernel", "TCC_REQ", "TCC_HIT", "TCC_MISS", "EA0_RDREQ", "hit rate")]
        for k in kernels:
            v = c3.get(k)
            if not v or "TCC_HIT_sum" not in v:
                continue
            hit, miss = v["TCC_HIT_sum"][1], v["TCC_MISS_sum"][1]
            rate = hit / (hit + miss) if hit + miss else 0.0
            out.append("%-26s %14d %14d %14d %14d %8.1f%%" % (k, v.get("TCC_REQ_sum", (0, 0, 0))[1], hit, miss, v.get("TCC_EA0_RDREQ_sum", (0, 0, 0))[1], 100 * rate))
            kernels[k]["l2_hit_rate"] = round(rate, 4)
    return "\n".join(out) + "\n", kernels


def main(prof, out_dir):
    global PROF
    import shadow_engine_amd as sz
    PROF = prof.rstrip("/")
    os.makedirs(out_dir, exist_ok=True)
    counters = {"kernel_keys": sz.program_keys(), "made_by": "python3 profile_counters.py (commands in its docstring and in profiles/*.txt)",
                "peaks": {"simds": SIMDS, "cycles_per_wave64_vector_instruction": 4}, "workloads": {}}
    try:
        # workloads summarised earlier on the same kernel sources stay; a file of other sources is started afresh
        before = json.load(open(os.path.join(out_dir, "counters.json")))
        if before.get("kernel_keys") == counters["kernel_keys"]:
            counters["workloads"] = before.get("workloads", {})
    except (OSError, ValueError):
        pass
    for wl in sorted(os.listdir(prof)):
        d = os.path.join(prof, wl)
        if wl not in NAMES or not os.path.isdir(d):
            continue
        stem, title, args = NAMES[wl]
        plain = None
        try:
            plain = json.loads(open(os.path.join(d, "plain.json")).read().strip().splitlines()[-1])
        except (OSError, ValueError, IndexError):
            pass
        entry = {"kernels": {}}
        if os.path.exists(os.path.join(d, "trace", "run_results.db")):
            text, durations = trace_summary(d, plain, title, args)
            open(os.path.join(out_dir, stem + "_kernel_trace.txt"), "w").write(text.replace("/W/", "/%s/" % wl))
            for k, us in durations.items():
                entry["kernels"].setdefault(k, {})["trace_avg_us"] = round(us, 2)
        if os.path.exists(os.path.join(d, "sq", "run_results.db")):
            text, ks = sq_summary(d, title, args)
            open(os.path.join(out_dir, stem + "_shader_counters.txt"), "w").write(text.replace("/W/", "/%s/" % wl))
            for k, e in ks.items():
                entry["kernels"].setdefault(k, {}).update(e)
        if os.path.exists(os.path.join(d, "fetch", "run_results.db")) and os.path.exists(os.path.join(d, "write", "run_results.db")):
            text, traffic, scale = traffic_summary(d, plain, title, args)
            open(os.path.join(out_dir, stem + "_hbm_traffic.txt"), "w").write(text.replace("/W/", "/%s/" % wl))
            entry["copy_scale"] = {k: round(v, 5) for k, v in scale.items()}
            for k, tb in traffic.items():
                entry["kernels"].setdefault(k, {})["traffic_bytes"] = tb
        if plain:
            entry["bench_line_without_profiler"] = {"ms_per_step": plain["ms_per_step"], "value": plain["value"],
                                                    "kernels": {k: v["avg_us"] for k, v in plain["kernels"].items()}}
        counters["workloads"][wl] = entry
        print("summarised", wl, sorted(p for p in os.listdir(d)))
    json.dump(counters, open(os.path.join(out_dir, "counters.json"), "w"), indent=1, sort_keys=True)
    print("wrote", os.path.join(out_dir, "counters.json"))


if __name__ == "__main__":
    if len(sys.argv) < 2:
        print(__doc__)
        sys.exit(2)
    main(sys.argv[1], sys.argv[2] if len(sys.argv) > 2 else os.path.join(ROOT, "profiles"))
