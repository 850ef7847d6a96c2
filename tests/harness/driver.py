#!/usr/bin/env python3
"""Drives the single-translation-unit harness mains the way the reference's Python scripts do.

    python tests/harness/driver.py bench -p skinny_gemm -a "8 4096 4096" -t 3 [-sb] [-m msg]
    python tests/harness/driver.py grid  -p skinny_gemm -a "8 4096 4096" [-s N] [-r I] [--timeout S]

`bench` reproduces the reference's bench.py (arguments :12-18, test loop :26-42, time parsing
:45-56, statistics :58-66): compile and run test.cu `-t` times and keep the maximum of the
deltas (repeated runs are the race probe), compile and run bench.cu, parse
"w0, w1, ..., End of warmup, t0, ...", report mean / std / median.  `grid` reproduces grid.py:
it rewrites the lines of projects/<p>/core.cu that start with "#define <NAME>" for the
tunables B_LANES_, OPS_, A_PRODUCERS_, B_PRODUCERS_, CONSUMERS_, QSIZE_, SK_ (:33-37,
:106-116), skips combinations that cannot fit (:13-31, with gfx950's 160 KB of LDS), turns a
time-out or a failed run into the sentinel mean 1e17 (:128-133) and restores core.cu at the end
(:101-104).  The reference's own bench.py / grid.py can drive the same tree unchanged when run
from tests/harness with HIPCC_COMPILE_FLAGS_APPEND carrying the flags in HIPCC_FLAGS below.
"""
import argparse
import itertools
import json
import os
import statistics
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
BUILD = os.path.join(HERE, "build")
HIPCC_FLAGS = ["-O3", "--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
               "-Wno-inline-asm", "-Wno-unused-command-line-argument"]
SENTINEL = 100000000000000000
TUNABLES = ("B_LANES_", "OPS_", "A_PRODUCERS_", "B_PRODUCERS_", "CONSUMERS_", "QSIZE_", "SK_", "OP_M_")


def project_dir(name):
    d = os.path.join(HERE, "projects", name)
    assert os.path.isdir(d), "Directory %s does not exist" % d
    return d


def _sources(project):
    """Everything a main of `project` is compiled from: its own directory, the shared harness header, the library's
    kernel sources and the oracle's C file."""
    root = os.path.dirname(os.path.dirname(HERE))
    dirs = [project_dir(project), os.path.join(root, "rocm_dev_amd", "csrc"), os.path.join(root, "oracle")]
    files = [os.path.join(HERE, "projects", "common.cuh")]
    for d in dirs:
        files += [os.path.join(d, f) for f in os.listdir(d) if f.endswith((".cu", ".cuh", ".h", ".hip", ".c"))]
    return files


def compile_main(project, c_file, force=False):
    """hipcc <project>/<c_file> -> build/<project>.<stem>.out; an executable newer than all of its sources is kept
    (the mains are compiled ahead of a GPU run, which then only executes them)."""
    os.makedirs(BUILD, exist_ok=True)
    out = os.path.join(BUILD, "%s.%s.out" % (project, c_file.split(".")[0]))
    if not force and os.path.exists(out) and os.path.getmtime(out) >= max(os.path.getmtime(f) for f in _sources(project)):
        return out
    res = subprocess.run(["hipcc"] + HIPCC_FLAGS + [os.path.join(project_dir(project), c_file), "-o", out],
                         capture_output=True, text=True)
    if res.returncode != 0:
        raise subprocess.CalledProcessError(res.returncode, "hipcc", stderr=res.stderr[-2000:])
    return out


PROJECTS = ("skinny_gemm", "async_gemm_sparse", "async_gemm_blanes", "async_gemm_16x16x64", "tiled_sum_reduce",
            "tiled_sum_reduce_async")


def compile_all(jobs=6):
    """Compiles test.cu and bench.cu of every project (what a build step runs ahead of the GPU tests)."""
    from concurrent.futures import ThreadPoolExecutor
    with ThreadPoolExecutor(jobs) as pool:
        return list(pool.map(lambda pf: compile_main(*pf), [(p, f) for p in PROJECTS for f in ("test.cu", "bench.cu")]))


def run_main(exe, arguments, timeout=None):
    return subprocess.check_output([exe] + arguments.split(), timeout=timeout).decode()


def parse_test_output(text):
    """One JSON object with max_delta and total_delta; a bare nan is tolerated (bench.py:34-39)."""
    parsed = json.loads(text.replace("nan", '"nan"'))
    return float(parsed["max_delta"]), float(parsed["total_delta"])


def parse_bench_output(stdout_text):
    """The reference's slicing, applied to what its Project.run would have returned: it drops the
    first two and the last three characters, then the first three fields, then pops from the end
    until 'End of warmup' (bench.py:49-56)."""
    times = stdout_text[2:-3].split(", ")[3:]
    bench_ts, t = [], times.pop()
    while t != "End of warmup":
        bench_ts.append(float(t))
        t = times.pop()
    warmup_ts = [float(x) for x in times]
    return bench_ts, warmup_ts


def stats(ts):
    return {"mean": statistics.fmean(ts), "std": statistics.pstdev(ts), "median": statistics.median(ts)}


def cmd_bench(args):
    max_deltas, sum_deltas = ([], []) if args.test_runs > 0 else ([-1], [-1])
    exe = None
    for i in range(args.test_runs):
        if i == 0:
            exe = compile_main(args.project, "test.cu")
        mx, tot = parse_test_output(run_main(exe, args.arguments))
        max_deltas.append(mx)
        sum_deltas.append(tot)
    if args.skip_bench:
        data = {"mean": 0.0, "std": 0.0, "median": 0.0}
    else:
        bench_ts, _ = parse_bench_output(run_main(compile_main(args.project, "bench.cu"), args.arguments))
        data = stats(bench_ts)
    data.update({"message": args.message,
                 "max_deltas": "%.4f <- [%s]" % (max(max_deltas), ", ".join("%.4f" % x for x in max_deltas)),
                 "sum_deltas": "%.4f <- [%s]" % (max(sum_deltas), ", ".join("%.4f" % x for x in sum_deltas))})
    print(json.dumps(data, indent=4))
    return data


def skip(p, max_lds=159 * 1024):
    """Combinations that cannot run: too many waves, ring deeper than the hardware counter,
    LDS over budget (the reference's constraints.py:6-36 with 65,536 replaced by gfx950's LDS)."""
    waves = p["A_PRODUCERS_"] + p["B_PRODUCERS_"] + p["CONSUMERS_"]
    if waves > 16:
        return True
    mt = 2 if p["OP_M_"] == 32 else 1
    stage_k = (512 // p["OP_M_"]) * p["OPS_"]
    ring = p["A_PRODUCERS_"] + p["B_PRODUCERS_"] > 0
    xu = 4 * mt
    if ring:
        if stage_k != 256 or p["A_PRODUCERS_"] < 1 or p["B_PRODUCERS_"] < 1 or p["SK_"] != 1:
            return True
        if p["QSIZE_"] < max(p["A_PRODUCERS_"], p["B_PRODUCERS_"] // p["B_LANES_"], p["CONSUMERS_"]):
            return True
        lds = p["QSIZE_"] * (p["B_LANES_"] * 4 + xu) * 1024 + 2 * p["B_LANES_"] * mt * p["CONSUMERS_"] * 1024 + 5120
        return lds > max_lds
    if stage_k == 256 and p["QSIZE_"] >= 2 and p["B_LANES_"] in (1, 2, 4):
        per_stage = p["B_LANES_"] * 4 + xu
        return (p["QSIZE_"] - 1) * per_stage > 63 or p["CONSUMERS_"] * p["QSIZE_"] * per_stage * 1024 + 4096 > max_lds
    if stage_k % 64:
        return True
    regs = p["QSIZE_"] * (stage_k // 64) * (p["B_LANES_"] + mt) * 4 + p["B_LANES_"] * mt * 4 + 28
    return regs > 500 or p["CONSUMERS_"] * p["B_LANES_"] * mt * 1024 > 64 * 1024


def rewrite_core(core_path, original_lines, params):
    lines = list(original_lines)
    for k, v in params.items():
        for i, line in enumerate(lines):
            if line.startswith("#define %s" % k):
                lines[i] = "#define %s %d\n" % (k, v)
    with open(core_path, "w") as f:
        f.writelines(lines)


def cmd_grid(args):
    core_path = os.path.join(project_dir(args.project), "core.cu")
    original = open(core_path).readlines()
    space = {"B_LANES_": [1, 2, 4], "OPS_": [4], "A_PRODUCERS_": [0, 1], "B_PRODUCERS_": [0, 4],
             "CONSUMERS_": [1, 2, 3, 4], "QSIZE_": [2, 4, 6, 8], "SK_": [1, 2], "OP_M_": [8]}
    keys = list(space)
    combos = [dict(zip(keys, v)) for v in itertools.product(*(space[k] for k in keys))]
    combos = [c for c in combos if (c["A_PRODUCERS_"] > 0) == (c["B_PRODUCERS_"] > 0)]
    best = (SENTINEL, -1, None)
    try:
        for i, params in enumerate(combos):
            if i < args.restart or (args.stop is not None and i >= args.stop) or skip(params):
                continue
            rewrite_core(core_path, original, params)
            try:
                bench_ts, _ = parse_bench_output(run_main(compile_main(args.project, "bench.cu"), args.arguments,
                                                          timeout=args.timeout))
                data = stats(bench_ts)
            except subprocess.TimeoutExpired:
                print("ERROR: End of timeout.")
                data = {"mean": SENTINEL}
            except subprocess.CalledProcessError as e:
                print("ERROR: %s." % (e.stderr,))
                data = {"mean": SENTINEL}
            print("%d/%d %s -> %s" % (i, len(combos), params, data), flush=True)
            if data["mean"] < best[0]:
                best = (data["mean"], i, params)
    finally:
        with open(core_path, "w") as f:   # write back the original core
            f.writelines(original)
    print("\n\nBEST OVERALL: %s at %s with %s" % best)
    return best


def main(argv=None):
    ap = argparse.ArgumentParser()
    sub = ap.add_subparsers(dest="cmd", required=True)
    b = sub.add_parser("bench")
    b.add_argument("--project", "-p", required=True)
    b.add_argument("--message", "-m", default="")
    b.add_argument("--arguments", "-a", default="")
    b.add_argument("--test-runs", "-t", type=int, default=1)
    b.add_argument("--skip-bench", "-sb", action="store_true")
    g = sub.add_parser("grid")
    g.add_argument("--project", "-p", required=True)
    g.add_argument("--arguments", "-a", default="")
    g.add_argument("--stop", "-s", type=int, default=None)
    g.add_argument("--restart", "-r", type=int, default=0)
    g.add_argument("--timeout", type=float, default=100.0)
    args = ap.parse_args(argv)
    return cmd_bench(args) if args.cmd == "bench" else cmd_grid(args)


if __name__ == "__main__":
    main()
