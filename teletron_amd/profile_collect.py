"""Runs, on a GPU box, the commands whose output teletron_amd.profile_summary turns into the text under
profiles/: bench.py without a profiler, under `rocprofv3 --kernel-trace --stats`, and under one
`rocprofv3 --pmc` pass per counter group (rocprofv3 does not split counters over passes, and a pass that asks
one block for more counters than it has hangs).  Tuning variants are built here too, with
`python -m teletron_amd.build --variant <dir>/variants/lib_<name>.so`, so every command a summary prints
is the command that ran, on committed files only.

    python -m teletron_amd.profile_collect cfg4      --dir rocprof_out
    python -m teletron_amd.profile_collect workloads --dir rocprof_out [--only cfg1 cfg3 ...]
    python -m teletron_amd.profile_collect stream    --dir rocprof_out
    python -m teletron_amd.profile_collect variants  --dir rocprof_out [--only base unpacked ...]
    python -m teletron_amd.profile_collect runs      --dir rocprof_out
    python -m teletron_amd.profile_collect cached    --dir rocprof_out
    python -m teletron_amd.profile_collect wide      --dir rocprof_out [--only base onewave ...]
    python -m teletron_amd.profile_collect timeline  --dir rocprof_out

This process never touches the GPU itself (it starts children and nothing else), every child runs under a
time limit, a failed step ends the collection, and each step prints one line when it starts.
"""
from __future__ import annotations

import argparse
import os
import subprocess
import sys
import time

from teletron_amd.build import ROOT
from teletron_amd.profile_summary import (CACHED_VARIANTS, CFG4_PASSES, PASS_COUNTERS, RUN_LENGTHS, VARIANTS, WIDE_VARIANTS,
                                          WIDE_WORKLOADS, WORKLOAD_INFO)

BENCH = ["python3", "bench.py"]
QUICK = ["--steps", "3", "--warmup", "1", "--no-cpu-baseline"]


def run(cmd, out=None, env=None, limit=300):
    """One child under a time limit; stdout to `out` (a path) when given.  Returns nothing; raises on failure."""
    print(f"[collect] {' '.join(cmd)}" + (f"  > {out}" if out else ""), flush=True)
    t0 = time.time()
    full_env = dict(os.environ, TMPDIR="/tmp", **(env or {}))
    with (open(out, "w") if out else open(os.devnull, "w")) as f:
        try:
            p = subprocess.run(cmd, cwd=ROOT, env=full_env, stdout=f, stderr=subprocess.PIPE, text=True, timeout=limit)
        except subprocess.TimeoutExpired:
            raise SystemExit(f"[collect] time limit of {limit} s reached; stopping (nothing else is started)")
    if p.returncode != 0:
        sys.stderr.write(p.stderr[-3000:])
        raise SystemExit(f"[collect] exit status {p.returncode}; stopping (nothing else is started)")
    print(f"[collect]   done in {time.time() - t0:.1f} s", flush=True)


def trace(directory, name, bench_args, env=None):
    run(["rocprofv3", "--kernel-trace", "--stats", "-d", os.path.join(directory, name), "-o", "bench", "--", *BENCH,
         *bench_args], out=os.path.join(directory, name + ".log"), env=env)


def pmc(directory, name, counters, bench_args, env=None):
    run(["rocprofv3", "--pmc", *counters.split(), "-d", os.path.join(directory, name), "-o", "r", "--", *BENCH,
         *bench_args], out=os.path.join(directory, name + ".log"), env=env, limit=240)


def cfg4(directory, only):
    run([*BENCH, "--steps", "100", "--warmup", "20", "--no-cpu-baseline"], out=os.path.join(directory, "bench.json"))
    trace(directory, "trace", ["--steps", "30", "--warmup", "5", "--no-cpu-baseline"])
    pmc(directory, "fetch", "FETCH_SIZE", QUICK)
    pmc(directory, "write", "WRITE_SIZE", QUICK)
    for p in CFG4_PASSES:
        pmc(directory, p, PASS_COUNTERS[p], QUICK)


def workloads(directory, only):
    for w in (only or WORKLOAD_INFO):
        args = ["--steps", "30", "--warmup", "5", "--no-cpu-baseline", "--workload", w]
        run([*BENCH, *args], out=os.path.join(directory, f"bench_{w}.json"))
        trace(directory, f"trace_{w}", args)


def stream(directory, only):
    run([*BENCH, "--workload", "stream-ceiling", "--steps", "20", "--warmup", "8"], out=os.path.join(directory, "stream.json"),
        limit=600)
    quick = ["--workload", "stream-ceiling", "--steps", "3", "--warmup", "4"]
    pmc(directory, "stream_stall", PASS_COUNTERS["stall"], quick)
    pmc(directory, "stream_fetch", "FETCH_SIZE", quick)
    pmc(directory, "stream_write", "WRITE_SIZE", quick)


def _build_variants(directory, table, only):
    """All variant libraries of `table` ([(name, flags, what)]), a few compilers at a time."""
    vdir = os.path.join(directory, "variants")
    os.makedirs(vdir, exist_ok=True)
    todo = [(n, f) for n, f, _ in table if f and (not only or n in only)]
    for i in range(0, len(todo), 3):
        procs = []
        for name, flags in todo[i:i + 3]:
            cmd = [sys.executable, "-m", "teletron_amd.build", "--variant", os.path.join(vdir, f"lib_{name}.so"),
                   *[f"--flag={f}" for f in flags]]
            print(f"[collect] {' '.join(cmd)}", flush=True)
            procs.append((name, subprocess.Popen(cmd, cwd=ROOT, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        for name, p in procs:
            out, _ = p.communicate(timeout=900)
            if p.returncode != 0:
                sys.stderr.write(out[-3000:])
                raise SystemExit(f"[collect] building variant {name} failed; stopping")
    return vdir


def variants(directory, only):
    vdir = _build_variants(directory, VARIANTS, only)
    for name, flags, _ in VARIANTS:
        if only and name not in only:
            continue
        env = {"TELETRON_AMD_LIB": os.path.join(vdir, f"lib_{name}.so")} if flags else None
        run([*BENCH, "--steps", "50", "--warmup", "10", "--no-cpu-baseline"], out=os.path.join(directory, f"variant_{name}.json"),
            env=env)
        pmc(directory, f"variant_{name}_sq", PASS_COUNTERS["variant_sq"], QUICK, env=env)
        pmc(directory, f"variant_{name}_stall", PASS_COUNTERS["variant_stall"], QUICK, env=env)


def runs(directory, only):
    table = [(f"run{n}", [f"-DTTN_STRIDED_RUN={n}"], "") for n in RUN_LENGTHS]
    vdir = _build_variants(directory, table, only)
    for name, _, _ in table:
        if only and name not in only:
            continue
        env = {"TELETRON_AMD_LIB": os.path.join(vdir, f"lib_{name}.so")}
        for w in ("cfg2-strided-rope", "cfg2-strided"):
            run([*BENCH, "--steps", "50", "--warmup", "10", "--no-cpu-baseline", "--workload", w],
                out=os.path.join(directory, f"run_{name}_{w}.json"), env=env)
        trace(directory, f"run_{name}_trace", ["--steps", "30", "--warmup", "5", "--no-cpu-baseline", "--workload",
                                               "cfg2-strided-rope"], env=env)


def cached(directory, only):
    # (a) small working sets through the shipped library; (b) the full-size step with the backward kernels'
    # rows wrapped to 1024 (timing only: every wavefront re-reads and re-writes one row, which stays in L2)
    run([*BENCH, "--workload", "cached-set", "--steps", "200", "--warmup", "20"], out=os.path.join(directory, "cached_rows.json"))
    vdir = _build_variants(directory, CACHED_VARIANTS, only)
    for name, _, _ in CACHED_VARIANTS:
        run([*BENCH, "--steps", "50", "--warmup", "10", "--no-cpu-baseline"], out=os.path.join(directory, f"cached_{name}.json"),
            env={"TELETRON_AMD_LIB": os.path.join(vdir, f"lib_{name}.so")})


def wide(directory, only):
    table = [("wide_" + n, f, w) for n, f, w in WIDE_VARIANTS]
    vdir = _build_variants(directory, table, ["wide_" + o for o in only] if only else None)
    for name, flags, _ in WIDE_VARIANTS:
        if only and name not in only:
            continue
        env = {"TELETRON_AMD_LIB": os.path.join(vdir, f"lib_wide_{name}.so")} if flags else None
        for w in WIDE_WORKLOADS + (["w4096-bf16-gated"] if not flags else []):
            run([*BENCH, "--steps", "30", "--warmup", "5", "--no-cpu-baseline", "--workload", w],
                out=os.path.join(directory, f"wide_{name}_{w}.json"), env=env)


def timeline(directory, only):
    vdir = _build_variants(directory, [("waveclock", ["-DTTN_WAVE_CLOCK=1"], "")], None)
    env = {"TELETRON_AMD_LIB": os.path.join(vdir, "lib_waveclock.so")}
    run([*BENCH, "--workload", "timeline-cfg3", "--steps", "25", "--warmup", "6"], out=os.path.join(directory, "timeline_cfg3.json"), env=env)
    run([*BENCH, "--workload", "timeline-cfg4", "--steps", "15", "--warmup", "4"], out=os.path.join(directory, "timeline_cfg4.json"), env=env)


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("what", choices=("cfg4", "workloads", "stream", "variants", "runs", "cached", "wide", "timeline"))
    ap.add_argument("--dir", required=True, help="where the rocprofv3 databases and bench.py lines go")
    ap.add_argument("--only", nargs="*", default=None, help="workloads / variant names to restrict the collection to")
    a = ap.parse_args()
    os.makedirs(a.dir, exist_ok=True)
    {"cfg4": cfg4, "workloads": workloads, "stream": stream, "variants": variants, "runs": runs, "cached": cached,
     "wide": wide, "timeline": timeline}[a.what](a.dir, a.only)
    print(f"[collect] {a.what}: complete; summarise with `python -m teletron_amd.profile_summary {a.what} --dir {a.dir}`",
          flush=True)


if __name__ == "__main__":
    main()
