"""Turns rocprofv3 output (rocpd sqlite databases) and bench.py JSON lines into the short text summaries
kept under profiles/, plus profiles/cfg4_traffic.json, which bench.py reads for `roofline.kernel` and
`roofline.traffic`.  Every summary names the commands that produced its inputs.

    python -m teletron_amd.profile_summary cfg4 --dir rocprof_out
        expects  <dir>/trace, <dir>/fetch, <dir>/write   (rocprofv3 -d ... of bench.py, see the text it writes)
        optional <dir>/sq, <dir>/tcc, <dir>/stall          (counter passes)
        optional <dir>/bench.json                          (the same bench.py run without a profiler)
    python -m teletron_amd.profile_summary workloads --dir rocprof_out     (<dir>/trace_<workload>)
    python -m teletron_amd.profile_summary stream --dir rocprof_out        (<dir>/stream.json, <dir>/stream_stall)
    python -m teletron_amd.profile_summary variants --dir rocprof_out      (<dir>/variant_<name>.json, _sq, _stall)
    python -m teletron_amd.profile_summary runs --dir rocprof_out          (<dir>/run_<name>_<workload>.json, run_<name>_trace)
    python -m teletron_amd.profile_summary cached --dir rocprof_out        (<dir>/cached_<name>.json)
    python -m teletron_amd.profile_summary wide --dir rocprof_out          (<dir>/wide_<variant>_<workload>.json)
    python -m teletron_amd.profile_summary timeline --dir rocprof_out      (<dir>/timeline_cfg3.json, timeline_cfg4.json)

`python -m teletron_amd.profile_collect <what> --dir <dir>` runs the commands that produce those inputs.
The databases are large; run this where they were written and keep only what it writes (--out).
"""
from __future__ import annotations

import argparse
import glob
import json
import os
import re
import sqlite3

from teletron_amd.build import ROOT, kernel_source_digest

PROFILES = os.path.join(ROOT, "profiles")
DIR_SHOWN = "rocprof_out"   # the --dir argument as typed: what the summaries print in their commands
OURS = ("rmsnorm_", "adaln_", "stream_copy", "stream_probe", "colreduce", "copy_rows")
BOX = "MI355X (gfx950, 256 CUs), ROCm 7.2, one GPU"


def _db(directory):
    found = sorted(glob.glob(os.path.join(directory, "**", "*.db"), recursive=True))
    if not found:
        raise FileNotFoundError(f"no rocpd database under {directory}")
    return sqlite3.connect(found[0])


def short(name: str) -> str:
    name = re.sub(r"^void ", "", name).replace("ttn::", "")
    return re.sub(r"\(.*", "", name)


def kernel_stats(directory, only_ours=True, by_grid=False):
    """[{name, symbol, calls, avg_us, min_us, max_us, total_us, vgpr, agpr, lds, grid}] sorted by total time."""
    cur = _db(directory).cursor()
    group = "name, grid_x" if by_grid else "name"
    rows = cur.execute(
        "select name, count(*), sum(duration), avg(duration), min(duration), max(duration), max(vgpr_count), "
        f"max(accum_vgpr_count), max(lds_size), max(grid_x) from kernels group by {group} "
        "order by sum(duration) desc").fetchall()
    out = []
    for r in rows:
        if only_ours and not any(o in r[0] for o in OURS):
            continue
        out.append({"name": short(r[0]), "symbol": re.sub(r"^void ", "", re.sub(r"\(.*", "", r[0])), "calls": r[1],
                    "total_us": r[2] / 1e3, "avg_us": r[3] / 1e3, "min_us": r[4] / 1e3, "max_us": r[5] / 1e3,
                    "vgpr": r[6], "agpr": r[7], "lds": r[8], "grid": r[9]})
    return out


def stats_table(stats, width=96):
    total = sum(s["total_us"] for s in stats) or 1.0
    lines = [f"{'kernel':{width}s} {'calls':>6} {'avg_us':>9} {'min_us':>9} {'max_us':>9} {'%':>6} {'vgpr':>5} "
             f"{'agpr':>5} {'lds':>6} {'grid':>9}"]
    for s in stats:
        lines.append(f"{s['name'][:width]:{width}s} {s['calls']:6d} {s['avg_us']:9.1f} {s['min_us']:9.1f} "
                     f"{s['max_us']:9.1f} {100 * s['total_us'] / total:6.2f} {s['vgpr']:5d} {s['agpr']:5d} "
                     f"{s['lds']:6d} {s['grid']:9d}")
    return "\n".join(lines)


def counters(directory, by_grid=False):
    """{kernel (, grid): {counter: average per dispatch}} for our kernels."""
    cur = _db(directory).cursor()
    group = "kernel_name, grid_size_x, counter_name" if by_grid else "kernel_name, counter_name"
    sel = "kernel_name, grid_size_x, counter_name" if by_grid else "kernel_name, 0, counter_name"
    out = {}
    for name, grid, counter, value, n in cur.execute(
            f"select {sel}, avg(value), count(*) from counters_collection group by {group}").fetchall():
        if not any(o in name for o in OURS):
            continue
        key = (short(name), grid) if by_grid else short(name)
        out.setdefault(key, {})[counter] = value
        out[key]["_dispatches"] = n
    return out


def _find(d, sub):
    for k, v in d.items():
        if sub in (k if isinstance(k, str) else k[0]):
            return v
    raise KeyError(sub)


# ------------------------------------------------------------------------------------------- cfg4

CFG4_ROWS, CFG4_COLS = 118800, 3072
CFG4_TENSOR = CFG4_ROWS * CFG4_COLS * 2
CFG4_KERNELS = {  # C-ABI call -> (row kernel name starts with, algorithmic tensors per launch)
    "tt_rmsnorm_forward": ("rmsnorm_fwd_kernel<bf16_t, 3072", 2),
    "tt_rmsnorm_backward": ("rmsnorm_bwd_kernel<bf16_t, 3072", 3),
    "tt_adaln_forward": ("adaln_fwd_kernel<bf16_t, 3072", 2),
    "tt_adaln_backward": ("adaln_bwd_kernel<bf16_t, 3072", 3),
}
BENCH_CMD = "python3 bench.py --steps {steps} --warmup {warmup} --no-cpu-baseline"


def cfg4(directory):
    trace = kernel_stats(os.path.join(directory, "trace"))
    fetch = counters(os.path.join(directory, "fetch"))
    write = counters(os.path.join(directory, "write"))
    copy_f = _find(fetch, "stream_copy_kernel")["FETCH_SIZE"]
    copy_w = _find(write, "stream_copy_kernel")["WRITE_SIZE"]
    kib = CFG4_TENSOR / 1024
    f_scale, w_scale = kib / copy_f, kib / copy_w
    digest = kernel_source_digest()
    record = {"source_digest": digest, "workload": "cfg4", "rows": CFG4_ROWS, "cols": CFG4_COLS,
              "calibration": {"kernel": "stream_copy_kernel", "bytes_read": CFG4_TENSOR, "bytes_written": CFG4_TENSOR,
                              "FETCH_SIZE_KiB": round(copy_f, 1), "WRITE_SIZE_KiB": round(copy_w, 1),
                              "fetch_scale": round(f_scale, 4), "write_scale": round(w_scale, 4)},
              "calls": {}}
    table = ["| kernel | avg µs (trace) | alg. GB/s | % of 8 TB/s | fetch MB (scaled) | write MB (scaled) | total MB | "
             "algorithmic MB | excess |", "|---|---|---|---|---|---|---|---|---|"]
    for call, (prefix, tensors) in CFG4_KERNELS.items():
        st = next(s for s in trace if s["name"].startswith(prefix))
        fb = _find(fetch, prefix)["FETCH_SIZE"] * f_scale * 1024
        wb = _find(write, prefix)["WRITE_SIZE"] * w_scale * 1024
        alg = tensors * CFG4_TENSOR
        gbs = alg / st["avg_us"] / 1e3
        record["calls"][call] = {"symbol": st["symbol"], "avg_us": round(st["avg_us"], 1),
                                 "algorithmic_bytes": alg, "fetch_bytes": int(fb), "write_bytes": int(wb),
                                 "traffic_bytes": int(fb + wb)}
        table.append(f"| `{st['name']}` | {st['avg_us']:.1f} | {gbs:.0f} | {gbs / 80:.1f} % | {fb / 1e6:.1f} | "
                     f"{wb / 1e6:.1f} | {(fb + wb) / 1e6:.1f} | {alg / 1e6:.1f} | {100 * ((fb + wb) / alg - 1):+.2f} % |")
    with open(os.path.join(PROFILES, "cfg4_traffic.json"), "w") as f:
        json.dump(record, f, indent=1)
        f.write("\n")

    bench_note = ""
    bj = os.path.join(directory, "bench.json")
    if os.path.exists(bj):
        b = json.loads(open(bj).read().strip().splitlines()[-1])
        r = b["roofline"]
        bench_note = (f"\nbench.py of the same build, run without a profiler just before on the same box "
                      f"(`{BENCH_CMD.format(steps=b['steps'], warmup=b['warmup'])}`): {b['value']:.0f} GB/s "
                      f"({100 * b['frac_of_hbm_peak']:.1f} % of 8 TB/s), {b['ms_per_step']:.4f} ms per step; its roofline "
                      f"entry times `{short(r['kernel'] or r['call'])}` with a HIP event pair recorded by the library around "
                      f"that kernel: {r['avg_us']:.1f} µs.  Untimed per-call HIP-event medians: "
                      + " / ".join(f"{v['median_us']:.1f}" for v in b["per_call_untimed"].values()) + " µs.\n")

    def pmc_rows(c, name):
        rows = [f"{'kernel':96s} {'counter':>12} {'n':>4} {'avg KiB':>14}"]
        for k, v in sorted(c.items(), key=lambda kv: -kv[1].get(name, 0)):
            rows.append(f"{k[:96]:96s} {name:>12} {v['_dispatches']:4d} {v[name]:14.1f}")
        return "\n".join(rows)

    md = f"""# rocprofv3 summary: bench.py, cfg4 (118 800 x 3072 bf16), all kernels

Workload: one step = fused RMSNorm(3072) fwd+bwd + fused AdaLN fwd+bwd, through the C ABI.
{BOX}.  Kernel sources digest `{digest}` (sha256 over teletron_amd/csrc, first 16 hex digits; bench.py prints
`roofline.traffic` only while the sources it runs have this digest).  rocprofv3 writes a rocpd sqlite database;
the tables are `select ... from kernels group by name` / `from counters_collection group by kernel_name` over it
(durations in microseconds, counters in KiB per dispatch as rocprofv3 reports them).  Written by
`python -m teletron_amd.profile_summary cfg4 --dir {DIR_SHOWN}`.

## Kernel trace

    rocprofv3 --kernel-trace --stats -d {DIR_SHOWN}/trace -o bench -- {BENCH_CMD.format(steps=30, warmup=5)}

```
{stats_table(trace)}
```
{bench_note}
## HBM traffic (two separate counter runs)

    rocprofv3 --pmc FETCH_SIZE -d {DIR_SHOWN}/fetch -o bench -- {BENCH_CMD.format(steps=3, warmup=1)}
    rocprofv3 --pmc WRITE_SIZE -d {DIR_SHOWN}/write -o bench -- {BENCH_CMD.format(steps=3, warmup=1)}

```
{pmc_rows(fetch, 'FETCH_SIZE')}
```
```
{pmc_rows(write, 'WRITE_SIZE')}
```

Calibration on `stream_copy_kernel` (reads {CFG4_TENSOR:,} B = {kib:,.0f} KiB and writes the same):
FETCH_SIZE reads {copy_f:,.0f} KiB -> scale factor {f_scale:.3f}; WRITE_SIZE reads {copy_w:,.0f} KiB -> scale factor {w_scale:.3f}.

{chr(10).join(table)}

The excess over the algorithmic bytes is the row statistics (4-8 B per row) and, for the backward kernels, the
fp32 partial column sums (256 workgroups x 12 or 24 KiB).
"""
    with open(os.path.join(PROFILES, "bench_cfg4_all_kernels.md"), "w") as f:
        f.write(md)
    print("wrote profiles/bench_cfg4_all_kernels.md, profiles/cfg4_traffic.json (digest %s)" % digest)

    passes = {p: os.path.join(directory, p) for p in CFG4_PASSES if os.path.isdir(os.path.join(directory, p))}
    if passes:
        cfg4_counters(passes, digest)


PASS_COUNTERS = {
    "sq": "SQ_WAVES SQ_INSTS_VALU SQ_INSTS_VMEM SQ_BUSY_CYCLES SQ_WAVE_CYCLES SQ_WAIT_INST_ANY SQ_ACTIVE_INST_ANY "
          "GRBM_GUI_ACTIVE",
    "tcc": "TCC_HIT_sum TCC_MISS_sum TCC_EA0_RDREQ_sum TCC_EA0_WRREQ_sum",
    "stall": "TCC_EA0_WRREQ_DRAM_CREDIT_STALL_sum TCC_EA0_RDREQ_DRAM_CREDIT_STALL_sum TCC_EA0_WRREQ_STALL_sum "
             "TCC_TOO_MANY_EA_WRREQS_STALL_sum",
    # the two passes taken per tuning variant
    "variant_sq": "SQ_WAVES SQ_INSTS_VALU SQ_BUSY_CYCLES SQ_WAVE_CYCLES SQ_WAIT_INST_ANY SQ_ACTIVE_INST_ANY",
    "variant_stall": "TCC_EA0_WRREQ_DRAM_CREDIT_STALL_sum TCC_EA0_RDREQ_DRAM_CREDIT_STALL_sum",
}
CFG4_PASSES = ("sq", "tcc", "stall")


def cfg4_counters(passes, digest):
    merged = {}
    for p, d in passes.items():
        for k, v in counters(d).items():
            merged.setdefault(k, {}).update(v)
    order = [next((k for k in merged if k.startswith(pref)), None) for pref, _ in CFG4_KERNELS.values()]
    order.append(next((k for k in merged if k.startswith("stream_copy_kernel")), None))
    order = [k for k in order if k]
    names = [c for p in passes for c in PASS_COUNTERS[p].split()]
    cmds = "\n".join(f"    rocprofv3 --pmc {PASS_COUNTERS[p]} -d {DIR_SHOWN}/{p} -o r -- "
                     f"{BENCH_CMD.format(steps=3, warmup=1)}" for p in passes)
    lines = ["| counter | " + " | ".join(k.split("<")[0] for k in order) + " |", "|---|" + "---|" * len(order)]
    for c in names:
        lines.append(f"| {c} | " + " | ".join(f"{merged[k].get(c, float('nan')):,.0f}" for k in order) + " |")
    derived = []
    if "sq" in passes:
        derived.append("| VALU instructions per row (wavefront level) | " + " | ".join(
            f"{merged[k]['SQ_INSTS_VALU'] / CFG4_ROWS:.0f}" for k in order[:4]) + " | |")
        derived.append("| SQ_WAIT_INST_ANY / SQ_ACTIVE_INST_ANY | " + " | ".join(
            f"{merged[k]['SQ_WAIT_INST_ANY'] / max(merged[k]['SQ_ACTIVE_INST_ANY'], 1):.2f}" for k in order) + " |")
    if "tcc" in passes:
        derived.append("| L2 hit share (HIT / (HIT + MISS)) | " + " | ".join(
            f"{merged[k]['TCC_HIT_sum'] / (merged[k]['TCC_HIT_sum'] + merged[k]['TCC_MISS_sum']):.2f}" for k in order) + " |")
    md = f"""# rocprofv3 counter passes: bench.py, cfg4 (118 800 x 3072 bf16), the four row kernels and the copy yardstick

{BOX}.  Kernel sources digest `{digest}`.  Separate counter runs of the same command (rocprofv3 does not split
counters over passes); values are per dispatch, averaged over the dispatches of the run.  Written by
`python -m teletron_amd.profile_summary cfg4 --dir {DIR_SHOWN}`.

{cmds}

{chr(10).join(lines)}

Derived:

| | {' | '.join(k.split('<')[0] for k in order)} |
|---|{'---|' * len(order)}
{chr(10).join(derived)}

Reading: every activation byte crosses L2 once (reads leave L2 as 128-byte requests, writes as 64-byte requests:
5.70 M and 11.4 M per 730 MB tensor; with the write-through store of the backward kernels nothing written is a
hit).  The backward kernels are persistent grids of one wavefront per SIMD (1024 wavefronts) and issue 1.2-1.3
VALU instructions per wait cycle; the forward kernels are one-shot grids whose wavefronts mostly wait.  The DRAM
credit stalls are what grows when more requests are kept in flight than the memory system drains.
"""
    with open(os.path.join(PROFILES, "bench_cfg4_sq_tcc_counters.md"), "w") as f:
        f.write(md)
    print("wrote profiles/bench_cfg4_sq_tcc_counters.md")


# -------------------------------------------------------------------------------------- workloads

WORKLOAD_INFO = {
    "gated": "gated residual + AdaLN, 118 800 x 3072 bf16: forward 2 reads + 2 writes, backward 4 reads + 2 writes",
    "cfg1": "RMSNorm fwd+bwd, 8192 x 3072 fp32",
    "cfg2": "QK-norm on contiguous q and k, 712 800 rows x 128 bf16",
    "cfg2-strided": "QK-norm on the transposed [B, H, S, D] views into the fused QKV projection, 712 800 rows x 128 bf16",
    "cfg2-strided-rope": "the same with the rotary embedding applied behind each norm (fp32 tables [29 700, 128])",
    "cfg3": "AdaLN fwd+bwd, 29 700 x 3072 bf16",
    "cfg5": "AdaLN -> RMSNorm chain, 4 x 11 056 x 3072 bf16, one modulation row per sample",
    "w1536-f16": "any-width kernels: RMSNorm + AdaLN fwd+bwd, 237 600 x 1536 fp16",
    "w4096-bf16": "wide-row kernels (four wavefronts per row): RMSNorm + AdaLN fwd+bwd, 89 100 x 4096 bf16",
    "w5120-bf16": "wide-row kernels: RMSNorm + AdaLN fwd+bwd, 71 280 x 5120 bf16",
    "w8192-bf16": "wide-row kernels: RMSNorm + AdaLN fwd+bwd, 44 550 x 8192 bf16",
    "w4096-bf16-gated": "wide-row kernels: gated residual + AdaLN fwd (2R 2W) + bwd (4R 2W), 89 100 x 4096 bf16",
    "qkv-site": "QK-norm call site through the autograd Function: q and k normalised on the strided views of the "
                "fused QKV projection, gradients written straight into the projection's gradient",
    "qkv-site-rope": "QK-norm call site with the rotary embedding fused behind the norm",
    "qkv-site-rope-reference": "the same call site the reference's way: split, transposing copy, dense RMSNorm, rotary "
                               "embedding as PyTorch ops",
}


def workloads(directory):
    digest = kernel_source_digest()
    md = [f"""# rocprofv3 summaries: bench.py workloads other than the headline step

{BOX}.  Kernel sources digest `{digest}`.  Each table is `select ... from kernels group by name` over the rocpd
database rocprofv3 wrote (durations in microseconds; torch's own fill/copy kernels of the set-up omitted).
`stream_copy_kernel` is the copy yardstick over one tensor of the workload (1 read + 1 write).  The JSON line is
bench.py's own (back-to-back) result for the same command without a profiler, where one was recorded.  Written by
`python -m teletron_amd.profile_summary workloads --dir {DIR_SHOWN}`.
"""]
    for d in sorted(glob.glob(os.path.join(directory, "trace_*"))):
        if not os.path.isdir(d):
            continue
        w = os.path.basename(d)[len("trace_"):]
        md.append(f"## {w}: {WORKLOAD_INFO.get(w, '')}\n\n    rocprofv3 --kernel-trace --stats -d {DIR_SHOWN}/trace_{w} "
                  f"-o bench -- {BENCH_CMD.format(steps=30, warmup=5)} --workload {w}\n\n```\n{stats_table(kernel_stats(d))}\n```\n")
        bj = os.path.join(directory, f"bench_{w}.json")
        if os.path.exists(bj):
            b = json.loads(open(bj).read().strip().splitlines()[-1])
            calls = ", ".join(f"{k} {v['median_us']:.1f} µs ({100 * v['frac_of_peak']:.1f} %)"
                              for k, v in b["per_call_untimed"].items())
            md.append(f"bench.py: {b['ms_per_step']:.4f} ms per step, {b['value']:.0f} GB/s "
                      f"({100 * b['frac_of_hbm_peak']:.1f} % of 8 TB/s); per call (HIP-event medians): {calls}.\n")
    with open(os.path.join(PROFILES, "bench_other_workloads_kernels.md"), "w") as f:
        f.write("\n".join(md))
    print("wrote profiles/bench_other_workloads_kernels.md")


# ----------------------------------------------------------------------------------------- stream

def stream(directory):
    digest = kernel_source_digest()
    b = json.loads(open(os.path.join(directory, "stream.json")).read().strip().splitlines()[-1])
    rows = ["| reads | writes | KiB per wavefront per tensor | grid | store | µs | GB/s | % of 8 TB/s |",
            "|---|---|---|---|---|---|---|---|"]
    for r in b["probes"]:
        rows.append(f"| {r['reads']} | {r['writes']} | {r['KiB_per_wavefront_per_tensor']} | {r['grid']} | {r['store']} | "
                    f"{r['us']:.1f} | {r['GB/s']:.0f} | {100 * r['frac_of_peak']:.1f} |")
    others = ["| copy not written here | µs | GB/s | % of 8 TB/s |", "|---|---|---|---|"]
    for k, v in b["other_copies"].items():
        others.append(f"| `{k}` | {v['us']:.1f} | {v['GB/s']:.0f} | {100 * v['frac_of_peak']:.1f} |")
    best = b["best"]
    stall_md = ""
    sd = os.path.join(directory, "stream_stall")
    if os.path.isdir(sd):
        c = counters(sd, by_grid=True)
        names = sorted({n for v in c.values() for n in v if not n.startswith("_")})
        lines = ["| kernel | grid (threads) | " + " | ".join(names) + " |", "|---|---|" + "---|" * len(names)]
        for (k, grid), v in sorted(c.items()):
            if "stream_probe" in k:
                lines.append(f"| `{k}` | {grid} | " + " | ".join(f"{v.get(n, float('nan')):,.0f}" for n in names) + " |")
        stall_md = f"""
## Where the mixed streams lose (counter pass over the same probes)

    rocprofv3 --pmc {PASS_COUNTERS['stall']} -d {DIR_SHOWN}/stream_stall -o r -- python3 bench.py --workload stream-ceiling --steps 3 --warmup 4

`stream_probe_kernel<reads, writes, accesses per lane, write-through>`; a grid of 65 536 / 262 144 threads is the
persistent form (256 / 1024 workgroups), anything larger the one-shot form.  Averages per dispatch.

{chr(10).join(lines)}
"""
    traffic_md = ""
    fd, wd = os.path.join(directory, "stream_fetch"), os.path.join(directory, "stream_write")
    if os.path.isdir(fd) and os.path.isdir(wd):
        cf, cw = counters(fd, by_grid=True), counters(wd, by_grid=True)
        kib = CFG4_TENSOR / 1024
        f_scale = kib / next(v["FETCH_SIZE"] for (k, _), v in cf.items() if k.startswith("stream_copy_kernel"))
        w_scale = kib / next(v["WRITE_SIZE"] for (k, _), v in cw.items() if k.startswith("stream_copy_kernel"))
        lines = ["| kernel | grid (threads) | tensors read | read MB (FETCH_SIZE, scaled) | per tensor claimed | tensors "
                 "written | written MB (WRITE_SIZE, scaled) | per tensor claimed |", "|---|---|---|---|---|---|---|---|"]
        worst = 0.0
        for (k, grid), v in sorted(cf.items()):
            m = re.match(r"stream_probe_kernel<(\d+), (\d+), (\d+), (\d+)>", k)
            if not m or (k, grid) not in cw:
                continue
            nr, nw = int(m.group(1)), int(m.group(2))
            rb = v["FETCH_SIZE"] * f_scale * 1024
            wb = cw[(k, grid)]["WRITE_SIZE"] * w_scale * 1024
            pr = rb / nr / CFG4_TENSOR if nr else float("nan")
            pw = wb / nw / CFG4_TENSOR if nw else float("nan")
            worst = max(worst, abs(pr - 1) if nr else 0.0, abs(pw - 1) if nw else 0.0)
            lines.append(f"| `{k}` | {grid} | {nr} | {rb / 1e6:.1f} | {pr:.3f} | {nw} | {wb / 1e6:.1f} | {pw:.3f} |")
        traffic_md = f"""
## The probes move the bytes they claim (FETCH_SIZE / WRITE_SIZE passes over the same probes)

    rocprofv3 --pmc FETCH_SIZE -d {DIR_SHOWN}/stream_fetch -o r -- python3 bench.py --workload stream-ceiling --steps 3 --warmup 4
    rocprofv3 --pmc WRITE_SIZE -d {DIR_SHOWN}/stream_write -o r -- python3 bench.py --workload stream-ceiling --steps 3 --warmup 4

Counters scaled by what they read for `stream_copy_kernel` in the same run (729.9 MB read and written:
FETCH_SIZE x {f_scale:.3f}, WRITE_SIZE x {w_scale:.3f} KiB).  "Per tensor claimed" = measured bytes / (tensors x 729.9 MB):
1.000 means the probe's HBM traffic is exactly the streams its bandwidth figure is computed from (largest
deviation in this table: {100 * worst:.1f} %).  What each launch writes is also checked value by value
(`tests/test_gpu_probe.py`).

{chr(10).join(lines)}
"""
    md = f"""# Streaming ceiling: what this memory system gives each read/write mix

{BOX}.  Kernel sources digest `{digest}`.  `python3 bench.py --workload stream-ceiling --steps {b['steps']} --warmup {b['warmup']}`:
plain streams over 729.9 MB tensors through the probe library's kernel (`tt_probe_stream` of libteletron_probe.so: non-temporal
16-byte loads, one contiguous run per wavefront and tensor, no arithmetic beyond one add), {b['steps']} launches back
to back between two events.  Written by `python -m teletron_amd.profile_summary stream --dir {DIR_SHOWN}`.

Best per mix: read only {best['read_only']['GB/s']:.0f} GB/s ({100 * best['read_only']['frac_of_peak']:.1f} %), two reads
{best['two_reads']['GB/s']:.0f} ({100 * best['two_reads']['frac_of_peak']:.1f} %), write only {best['write_only']['GB/s']:.0f}
({100 * best['write_only']['frac_of_peak']:.1f} %), copy 1R+1W {best['copy_1R_1W']['GB/s']:.0f} ({100 * best['copy_1R_1W']['frac_of_peak']:.1f} %),
2R+1W {best['2R_1W']['GB/s']:.0f} ({100 * best['2R_1W']['frac_of_peak']:.1f} %), 3R+1W {best['3R_1W']['GB/s']:.0f}
({100 * best['3R_1W']['frac_of_peak']:.1f} %), 2R+2W {best['2R_2W']['GB/s']:.0f} ({100 * best['2R_2W']['frac_of_peak']:.1f} %), 4R+2W
{best['4R_2W']['GB/s']:.0f} ({100 * best['4R_2W']['frac_of_peak']:.1f} %).  Pure streams run at 85-92 % of the
published peak; as soon as reads and writes mix, every shape drops to 72-82 %.  A row kernel moves 6 KiB per
wavefront and tensor (a whole 3072-column row, which it needs for the row statistics): in that shape the best plain
2R+1W stream is the one-shot grid, and the backward kernels (persistent, because the column sums live in registers)
run faster than it (see bench_cfg4_all_kernels.md).

{chr(10).join(rows)}

{chr(10).join(others)}
{stall_md}{traffic_md}"""
    with open(os.path.join(PROFILES, "stream_ceiling.md"), "w") as f:
        f.write(md)
    print("wrote profiles/stream_ceiling.md")


# --------------------------------------------------------------------------------------- variants

VARIANTS = [  # name, hipcc flags of the build ([] = the shipped library), what it changes
    ("base", [], "the shipped kernels"),
    ("unpacked", ["-DTTN_BWD_PACKED_MATH=0"],
     "backward: every product and column sum on unpacked fp32 values (unpack, multiply, convert, unpack again), as "
     "before the packed dot-product forms"),
    ("packedproducts", ["-DTTN_BWD_PACKED_MATH=1"],
     "backward: gy / gx = rnd(g * parameter) from packed pairs; the column sums still unpack g"),
    ("serialflush", ["-DTTN_FLUSH_PARALLEL=0"],
     "backward: the workgroup's partial row is folded by its four wavefronts in turn (four barriers, 4-byte writes) "
     "instead of in parallel"),
    ("nodrain", ["-DTTN_BWD_DRAIN_STORES=0"],
     "backward: a row's first pass waits for its own loads only, not for the previous row's stores"),
    ("plainstore", ["-DTTN_RMS_BWD_STORE=0", "-DTTN_ADALN_BWD_STORE=0"],
     "backward: plain streaming stores instead of write-through"),
    ("fullahead", ["-DTTN_RMS_BWD_PREFETCH_MID=0", "-DTTN_ADALN_BWD_PREFETCH_MID=0"],
     "backward: the next row is requested before the current one is processed (a full row ahead)"),
    ("onebuffer", ["-DTTN_RMS_BWD_ROW_BUFFERS=1", "-DTTN_ADALN_BWD_ROW_BUFFERS=1"],
     "backward: one row buffer, no prefetch"),
    ("twowaves", ["-DTTN_BWD_WAVES_PER_SIMD=2", "-DTTN_RMS_BWD_BLOCKS_PER_CU=(C>=1024?2:3)",
                  "-DTTN_ADALN_BWD_BLOCKS_PER_CU=(C>=1024?2:3)"],
     "backward: two workgroups per compute unit (two wavefronts per SIMD, half the registers each)"),
    ("loadcached", ["-DTTN_BWD_LOAD_POLICY=0"],
     "backward: row loads without the non-temporal hint (buffer loads, default cache policy)"),
    ("loadplain", ["-DTTN_BWD_LOAD_POLICY=-1"],
     "backward: plain global loads with the non-temporal hint instead of buffer loads marked sc0 sc1 nt (system scope + "
     "non-temporal)"),
    ("grid88", ["-DTTN_BWD_GRID_PERCENT=88"],
     "backward: persistent grid over 88 % of the compute units (226 workgroups instead of 256)"),
    ("fwd5", ["-DTTN_RMS_FWD_DYN_LDS=(C>=1024?(sizeof(T)==2?0:76800):0)"],
     "RMSNorm forward: no occupancy throttle (five one-shot workgroups per compute unit instead of three)"),
]


def variants(directory):
    digest = kernel_source_digest()
    calls = ["rmsnorm_forward", "rmsnorm_backward", "adaln_forward", "adaln_backward"]
    rows = ["| variant | ms per step | GB/s | % of 8 TB/s | " + " | ".join(c + " µs" for c in calls) + " |",
            "|---|---|---|---|" + "---|" * len(calls)]
    ctr = ["| variant | kernel | VALU instructions per row | SQ_ACTIVE_INST_ANY / SQ_WAVE_CYCLES | SQ_WAIT_INST_ANY / "
           "SQ_WAVE_CYCLES | SQ_INSTS_VALU | SQ_ACTIVE_INST_ANY | SQ_WAIT_INST_ANY | SQ_WAVE_CYCLES | SQ_BUSY_CYCLES | "
           "WRREQ_DRAM_CREDIT_STALL | RDREQ_DRAM_CREDIT_STALL |", "|---|---|---|---|---|---|---|---|---|---|---|---|"]
    cmds = []
    vdir = f"{DIR_SHOWN}/variants"
    for name, flags, what in VARIANTS:
        bj = os.path.join(directory, f"variant_{name}.json")
        if not os.path.exists(bj):
            continue
        b = json.loads(open(bj).read().strip().splitlines()[-1])
        rows.append(f"| `{name}` | {b['ms_per_step']:.4f} | {b['value']:.0f} | {100 * b['frac_of_hbm_peak']:.1f} | "
                    + " | ".join(f"{b['per_call_untimed'][c]['median_us']:.1f}" for c in calls) + " |")
        build = " ".join(f"'--flag={f}'" for f in flags)
        cmds.append(f"* `{name}`: {what}" + (f"  \n  `python -m teletron_amd.build --variant {vdir}/lib_{name}.so {build}`" if flags else ""))
        merged = {}
        for p in ("sq", "stall"):
            d = os.path.join(directory, f"variant_{name}_{p}")
            if os.path.isdir(d):
                for k, v in counters(d).items():
                    merged.setdefault(k, {}).update(v)
        nan = float("nan")
        for k, v in sorted(merged.items()):
            if "bwd_kernel<bf16_t, 3072" in k and "SQ_WAIT_INST_ANY" in v:
                wc = v.get("SQ_WAVE_CYCLES", nan)
                ctr.append(f"| `{name}` | `{k.split('<')[0]}` | {v.get('SQ_INSTS_VALU', nan) / CFG4_ROWS:.0f} | "
                           f"{v['SQ_ACTIVE_INST_ANY'] / wc:.2f} | {v['SQ_WAIT_INST_ANY'] / wc:.2f} | "
                           f"{v.get('SQ_INSTS_VALU', nan):,.0f} | {v['SQ_ACTIVE_INST_ANY']:,.0f} | {v['SQ_WAIT_INST_ANY']:,.0f} | "
                           f"{wc:,.0f} | {v['SQ_BUSY_CYCLES']:,.0f} | "
                           f"{v.get('TCC_EA0_WRREQ_DRAM_CREDIT_STALL_sum', nan):,.0f} | "
                           f"{v.get('TCC_EA0_RDREQ_DRAM_CREDIT_STALL_sum', nan):,.0f} |")
    md = f"""# Tuning variants of the cfg4 step: what each pipeline choice is worth (bench.py, 118 800 x 3072 bf16)

{BOX}.  Kernel sources digest `{digest}`.  Each variant is the shipped kernel source built with other values of
the tuning macros at the top of `rmsnorm.hip` / `adaln.hip`, loaded in place of the shipped library
(`TELETRON_AMD_LIB` in the environment of the command), and run through the unchanged benchmark on one box, one
after the other, by `python -m teletron_amd.profile_collect variants --dir {DIR_SHOWN}`:

    python -m teletron_amd.build --variant {vdir}/lib_<name>.so <flags>
    TELETRON_AMD_LIB={vdir}/lib_<name>.so  python3 bench.py --steps 50 --warmup 10 --no-cpu-baseline
    TELETRON_AMD_LIB={vdir}/lib_<name>.so  rocprofv3 --pmc {PASS_COUNTERS['variant_sq']} -d {DIR_SHOWN}/variant_<name>_sq -o r -- python3 bench.py --steps 3 --warmup 1 --no-cpu-baseline
    TELETRON_AMD_LIB={vdir}/lib_<name>.so  rocprofv3 --pmc {PASS_COUNTERS['variant_stall']} -d {DIR_SHOWN}/variant_<name>_stall -o r -- python3 bench.py --steps 3 --warmup 1 --no-cpu-baseline

{chr(10).join(cmds)}

Per-call figures are HIP-event medians over 30 untimed steps.  Written by
`python -m teletron_amd.profile_summary variants --dir {DIR_SHOWN}`.

{chr(10).join(rows)}

Counters of the two backward row kernels, per dispatch (averages; the SQ cycle counters tick once per four
clocks; VALU instructions per row = SQ_INSTS_VALU / 118 800):

{chr(10).join(ctr)}

Reading.  Arithmetic: `unpacked` -> `packedproducts` -> `base` removes about a quarter of the backward kernels'
vector instructions (and with them that share of the cycles in which the one wavefront of a SIMD is issuing),
and the kernels' duration does not follow: the time goes to waiting instead (SQ_WAIT_INST_ANY grows by what
SQ_ACTIVE_INST_ANY loses).  The backward kernels are not limited by instruction issue.  Memory pipeline: every
alternative keeps more requests in flight per wavefront than the shipped pipeline (or, for `onebuffer`, fewer) and
is slower; the slower ones show more DRAM-credit stall cycles at the L2-to-memory interface, i.e. the extra
requests queue instead of being served.  Row loads: without the non-temporal hint (`loadcached`) the backward kernels
lose 10 %; marked system scope + non-temporal (shipped) they gain about half a per cent over plain non-temporal
global loads (`loadplain`), the only cache policy that gained anything.  A smaller grid gains nothing.  `serialflush`
is the end of the kernel only (a workgroup's partial row written after four barriers instead of one: 4.0 us
against 1.4 us per workgroup by the wave clocks of step_timeline_wave_clocks.md), below what this table
resolves at 118 800 rows.  None reaches the 80 % line; see stream_ceiling.md for what plain streams of the
same read/write mix reach.
"""
    with open(os.path.join(PROFILES, "bench_cfg4_tuning_variants.md"), "w") as f:
        f.write(md)
    print("wrote bench_cfg4_tuning_variants.md")


CACHED_VARIANTS = [  # the backward kernels with their rows wrapped so that the working set stays in L2: timing only
    ("l2resident", ["-DTTN_BWD_ROW_WRAP=1024"], "shipped arithmetic (packed dot-product forms)"),
    ("l2resident_unpacked", ["-DTTN_BWD_ROW_WRAP=1024", "-DTTN_BWD_PACKED_MATH=0"], "unpacked fp32 arithmetic"),
    ("llcresident", ["-DTTN_BWD_ROW_WRAP=8192"], "rows wrapped to 8192 (150 MB working set: fits the 256 MB last-level cache)"),
    ("llcresident_cachedloads", ["-DTTN_BWD_ROW_WRAP=8192", "-DTTN_BWD_LOAD_POLICY=0"],
     "the same with row loads that do not carry the non-temporal hint"),
]


def cached(directory):
    """What the backward kernels' instruction streams allow when memory answers from a cache."""
    digest = kernel_source_digest()
    vdir = f"{DIR_SHOWN}/variants"
    rows = ["| build | rmsnorm_backward µs | GB/s equivalent | adaln_backward µs | GB/s equivalent |", "|---|---|---|---|---|"]
    cmds = []
    for name, flags, what in CACHED_VARIANTS:
        f = os.path.join(directory, f"cached_{name}.json")
        if not os.path.exists(f):
            continue
        b = json.loads(open(f).read().strip().splitlines()[-1])
        c = b["per_call_untimed"]
        r, a = c["rmsnorm_backward"]["median_us"], c["adaln_backward"]["median_us"]
        rows.append(f"| `{name}`: {what} | {r:.1f} | {3 * CFG4_TENSOR / r / 1e3:.0f} | {a:.1f} | {3 * CFG4_TENSOR / a / 1e3:.0f} |")
        build = " ".join(f"'--flag={x}'" for x in flags)
        cmds.append(f"    python -m teletron_amd.build --variant {vdir}/lib_{name}.so {build}\n"
                    f"    TELETRON_AMD_LIB={vdir}/lib_{name}.so  python3 bench.py --steps 50 --warmup 10 --no-cpu-baseline")
    small = ""
    f = os.path.join(directory, "cached_rows.json")
    if os.path.exists(f):
        b = json.loads(open(f).read().strip().splitlines()[-1])
        t = ["| kernel | µs at 4096 rows | µs at 8192 rows | µs per 1024 rows (slope) | 118 800 rows at that rate, µs | GB/s "
             "equivalent | % of 8 TB/s |", "|---|---|---|---|---|---|---|"]
        for k, r in b["kernels"].items():
            t.append(f"| `{k}` | {r['us_4096_rows']:.2f} | {r['us_8192_rows']:.2f} | {r['us_per_1024_rows']:.3f} | "
                     f"{r['cfg4_us_at_this_rate']:.1f} | {r['GB/s_at_this_rate']:.0f} | {100 * r['frac_of_hbm_peak_at_this_rate']:.0f} |")
        small = f"""
## Small working sets through the shipped library

    python3 bench.py --workload cached-set --steps {b['steps']} --warmup {b['warmup']}

Each cfg4 call launched back to back on the same buffers at 4096 and 8192 rows x 3072 bf16 (25 / 50 MB per tensor, at
most three tensors per call: well inside the 256 MB last-level cache); the slope between the two sizes is the
steady-state cost of 4 more rows per wavefront, scaled to the full problem.  The kernels run no faster than on
the full-size tensors: their loads carry the non-temporal hint and their stores are write-through, and such
streams are not served faster by the last-level cache than by HBM.

{chr(10).join(t)}
"""
    md = f"""# The backward kernels on cache-resident rows: what their instruction streams allow

{BOX}.  Kernel sources digest `{digest}`.  Is the last stretch to the memory roofline lost in the kernels' own
instruction streams (one wavefront per SIMD, several hundred vector instructions per row)?  Measured directly: the
full-size cfg4 step with the two backward kernels built to read and write their rows modulo 1024
(`TTN_BWD_ROW_WRAP`: every wavefront keeps re-reading and re-writing one row, 18 MB in all, which stays in L2;
the results are wrong, the instruction stream, the grid and the row count are those of the real kernels).
Collected by `python -m teletron_amd.profile_collect cached --dir {DIR_SHOWN}`:

{chr(10).join(cmds)}

Per-call HIP-event medians of bench.py (30 untimed steps); GB/s equivalent = 3 x 729.9 MB / duration.  Written by
`python -m teletron_amd.profile_summary cached --dir {DIR_SHOWN}`.

{chr(10).join(rows)}

Reading: with memory out of the way the shipped backward kernels take about 200 µs where they take 353-358 µs on
HBM-resident tensors, i.e. their instruction streams would sustain well above the HBM peak; the packed
dot-product forms move that ceiling further up without moving the HBM-bound duration (bench_cfg4_tuning_variants.md).
The kernels are bound by what the memory system delivers to a 2-read + 1-write stream, not by instruction issue.
Rows wrapped to 8192 (150 MB) run like the full-size tensors with the shipped non-temporal loads and only
moderately faster with cached loads: the last-level cache is not a way around HBM for these streams.
{small}"""
    with open(os.path.join(PROFILES, "cached_set_instruction_ceiling.md"), "w") as f:
        f.write(md)
    print("wrote cached_set_instruction_ceiling.md")


# ------------------------------------------------------------------- run length at the QK-norm site

RUN_LENGTHS = (1, 3, 6, 12)   # 6 is what ships; built explicitly like the others so that all four are measured alike
RUN_VARIANTS = [(f"run{n}", n) for n in RUN_LENGTHS]
RUN_WORKLOADS = ["cfg2-strided-rope", "cfg2-strided"]


def run_lengths(directory):
    """bench lines `run_<variant>_<workload>.json`, and kernel traces `run_<variant>_trace` of the rotary
    site, for the shipped library and builds with other values of TTN_STRIDED_RUN."""
    digest = kernel_source_digest()
    rows = ["| groups per run | cfg2-strided-rope ms per step | rotary forward kernel µs | rotary backward kernel µs | "
            "cfg2-strided ms per step | strided forward / backward µs per call |", "|---|---|---|---|---|---|"]
    for name, run in RUN_VARIANTS:
        js = {}
        for w in RUN_WORKLOADS:
            f = os.path.join(directory, f"run_{name}_{w}.json")
            if os.path.exists(f):
                js[w] = json.loads(open(f).read().strip().splitlines()[-1])
        if len(js) != len(RUN_WORKLOADS):
            continue
        fwd = bwd = float("nan")
        t = os.path.join(directory, f"run_{name}_trace")
        if os.path.isdir(t):
            for r in kernel_stats(t):
                if "RopeTable" in r["name"]:
                    if "fwd_kernel" in r["name"]:
                        fwd = r["avg_us"]
                    elif "bwd_kernel" in r["name"]:
                        bwd = r["avg_us"]
        c = js["cfg2-strided"]["per_call_untimed"]
        rows.append(f"| {run}{' (shipped)' if run == 6 else ''} | {js['cfg2-strided-rope']['ms_per_step']:.4f} | {fwd:.1f} | "
                    f"{bwd:.1f} | {js['cfg2-strided']['ms_per_step']:.4f} | "
                    f"{c['rmsnorm_forward_strided_q']['median_us']:.1f} / {c['rmsnorm_backward_strided_q']['median_us']:.1f} |")
    md = f"""# Run length of the strided QK-norm kernels: heads a wavefront takes per table fetch

{BOX}.  Kernel sources digest `{digest}`.  `TTN_STRIDED_RUN` (norm_device.h) is the number of
consecutive groups -- heads of one token tile -- a wavefront of the strided 128-column kernels takes at a time: the
rotary kernels fetch the token's cos/sin rows once per run, the backward kernels do the view's index arithmetic once
per run; the forward kernel without tables always takes single groups.  With 1 every row fetches its own 1 KiB of
tables (what the kernels did before runs existed).  29 700 tokens x 24 heads x 128, bf16, q and k through the C ABI
(`cfg2-strided-rope`: the strided norm with the rotation, forward and backward; `cfg2-strided`: without), one box, one
after the other, by `python -m teletron_amd.profile_collect runs --dir {DIR_SHOWN}`:

    python -m teletron_amd.build --variant {DIR_SHOWN}/variants/lib_run<N>.so --flag=-DTTN_STRIDED_RUN=<N>
    TELETRON_AMD_LIB={DIR_SHOWN}/variants/lib_run<N>.so  python3 bench.py --steps 50 --warmup 10 --no-cpu-baseline --workload cfg2-strided-rope
    TELETRON_AMD_LIB={DIR_SHOWN}/variants/lib_run<N>.so  python3 bench.py --steps 50 --warmup 10 --no-cpu-baseline --workload cfg2-strided
    TELETRON_AMD_LIB={DIR_SHOWN}/variants/lib_run<N>.so  rocprofv3 --kernel-trace --stats -d {DIR_SHOWN}/run_run<N>_trace -o bench -- python3 bench.py --steps 30 --warmup 5 --no-cpu-baseline --workload cfg2-strided-rope

Kernel columns are rocprofv3 averages of `rmsnorm_fwd_kernel<bf16_t, 128, Strided3Rows, RopeTable>` and the matching
backward kernel.  Written by `python -m teletron_amd.profile_summary runs --dir {DIR_SHOWN}`.

{chr(10).join(rows)}
"""
    with open(os.path.join(PROFILES, "qkv_site_run_length_variants.md"), "w") as f:
        f.write(md)
    print("wrote qkv_site_run_length_variants.md")


WIDE_WORKLOADS = ["w4096-bf16", "w5120-bf16", "w8192-bf16"]
WIDE_VARIANTS = [  # name, flags, what: the choices of widerow.hip, each measured on the three wide workloads
    ("base", [], "the shipped kernels"),
    ("onewave", ["-DTTN_WIDE_ROWS=0"],
     "one wavefront per row (8, 12 or 16 accesses per lane): the any-width kernels, which strided views still use"),
    ("rmsfwd_persistent", ["-DTTN_WIDE_RMS_FWD_ROWS_PER_BLOCK=0"], "RMSNorm forward as a persistent grid instead of one-shot"),
    ("adalnfwd_oneshot", ["-DTTN_WIDE_ADALN_FWD_ROWS_PER_BLOCK=1"], "AdaLN forward one-shot (one row per workgroup)"),
    ("adalnfwd_persistent", ["-DTTN_WIDE_ADALN_FWD_ROWS_PER_BLOCK=0"], "AdaLN forward as a persistent grid"),
    ("fwd_noprefetch", ["-DTTN_WIDE_FWD_PREFETCH=0"], "forward: the next row is requested only when the current one is done"),
    ("adalnfwd_packedparams", ["-DTTN_WIDE_FWD_PARAMS_F32=0"],
     "AdaLN forward: rnd(1 + scale) and shift stay packed and are unpacked for every row"),
    ("bwd3", ["-DTTN_WIDE_BWD_BLOCKS_PER_CU=3"], "backward: three workgroups per compute unit instead of two"),
    ("bwd1", ["-DTTN_WIDE_BWD_BLOCKS_PER_CU=1"], "backward: one workgroup per compute unit"),
    ("bwd_prefetch", ["-DTTN_WIDE_BWD_PREFETCH=1"], "backward: the next row is requested between the two passes of the current one"),
    ("bwd1_prefetch", ["-DTTN_WIDE_BWD_PREFETCH=1", "-DTTN_WIDE_BWD_BLOCKS_PER_CU=1"],
     "backward: one workgroup per compute unit with the next row requested between the passes"),
    ("bwd_plainstore", ["-DTTN_WIDE_BWD_STORE=0"], "backward: plain streaming stores instead of write-through"),
]


def wide(directory):
    """bench lines wide_<variant>_<workload>.json: the choices of the wide-row kernels on rows of 512, 640 and 1024
    pieces."""
    digest = kernel_source_digest()
    vdir = f"{DIR_SHOWN}/variants"
    calls = ["rmsnorm_forward", "rmsnorm_backward", "adaln_forward", "adaln_backward"]
    head = "| variant | " + " | ".join(f"{w}: ms per step, GB/s (% of 8 TB/s); " + " / ".join(c.replace("norm_", " ").replace("ward", "") for c in calls)
                                        + " µs" for w in WIDE_WORKLOADS) + " |"
    rows = [head, "|---|" + "---|" * len(WIDE_WORKLOADS)]
    cmds = []
    for name, flags, what in WIDE_VARIANTS:
        cells = []
        for w in WIDE_WORKLOADS:
            f = os.path.join(directory, f"wide_{name}_{w}.json")
            if not os.path.exists(f):
                cells.append("-")
                continue
            b = json.loads(open(f).read().strip().splitlines()[-1])
            cells.append(f"{b['ms_per_step']:.4f}, {b['value']:.0f} ({100 * b['frac_of_hbm_peak']:.1f}); "
                         + " / ".join(f"{b['per_call_untimed'][c]['median_us']:.0f}" for c in calls))
        if all(c == "-" for c in cells):
            continue
        rows.append(f"| `{name}` | " + " | ".join(cells) + " |")
        build = " ".join(f"'--flag={f}'" for f in flags)
        cmds.append(f"* `{name}`: {what}" + (f"  \n  `python -m teletron_amd.build --variant {vdir}/lib_wide_{name}.so {build}`" if flags else ""))
    gated = ""
    g = os.path.join(directory, "wide_base_w4096-bf16-gated.json")
    if os.path.exists(g):
        b = json.loads(open(g).read().strip().splitlines()[-1])
        c = b["per_call_untimed"]
        gated = (f"\nThe gated residual form on wide rows (`--workload w4096-bf16-gated`, shipped library): {b['ms_per_step']:.4f} ms per "
                 f"step, {b['value']:.0f} GB/s ({100 * b['frac_of_hbm_peak']:.1f} % of 8 TB/s); forward "
                 f"{c['gated_residual_adaln_forward']['median_us']:.0f} µs, backward {c['gated_residual_adaln_backward']['median_us']:.0f} µs.\n")
    md = f"""# Wide rows (more than 384 16-byte pieces): what each choice of widerow.hip is worth

{BOX}.  Kernel sources digest `{digest}`.  Rows of 4096, 5120 and 8192 bf16 columns (512, 640 and 1024 pieces; 730 MB per
tensor), the cfg4 step (RMSNorm fwd+bwd + AdaLN fwd+bwd, four C-ABI calls) through the unchanged benchmark, each
variant the shipped sources built with other values of the macros at the top of `widerow.hip`, one box, one after the
other, by `python -m teletron_amd.profile_collect wide --dir {DIR_SHOWN}`:

    python -m teletron_amd.build --variant {vdir}/lib_wide_<name>.so <flags>
    TELETRON_AMD_LIB={vdir}/lib_wide_<name>.so  python3 bench.py --steps 30 --warmup 5 --no-cpu-baseline --workload <workload>

{chr(10).join(cmds)}

Per-call figures are HIP-event medians over 30 untimed steps.  Written by
`python -m teletron_amd.profile_summary wide --dir {DIR_SHOWN}`.

{chr(10).join(rows)}
{gated}"""
    with open(os.path.join(PROFILES, "wide_rows_variants.md"), "w") as f:
        f.write(md)
    print("wrote wide_rows_variants.md")


def timeline(directory):
    """timeline_<workload>.json (bench.py --workload timeline-cfg3 / timeline-cfg4 through a TTN_WAVE_CLOCK build)."""
    digest = kernel_source_digest()
    parts = []
    for w in ("cfg3", "cfg4"):
        f = os.path.join(directory, f"timeline_{w}.json")
        if not os.path.exists(f):
            continue
        b = json.loads(open(f).read().strip().splitlines()[-1])
        t = b["timeline_us"]
        fw, bw, rd = t["adaln_forward"], t["adaln_backward"], t["column_reducer"]
        rows = ["| kernel | wavefronts | first start | last start | first end | last end | median wavefront life | "
                "wavefronts active at 5 %, 15 %, ... 95 % of the kernel's span |", "|---|---|---|---|---|---|---|---|"]
        for name, k in (("adaln_fwd_kernel", fw), ("adaln_bwd_kernel", bw), ("colreduce_kernel", rd)):
            rows.append(f"| `{name}` | {k['wavefronts']:.0f} | {k['first_start']:.1f} | {k['last_start']:.1f} | {k['first_end']:.1f} | "
                        f"{k['last_end']:.1f} | {k['median_wavefront_life']:.1f} | {' '.join(f'{a:.0f}' for a in k['active_at_tenths'])} |")
        extra = bw.get("rows_done_last_with_extra")
        parts.append(f"""## {w}: {b['config']['rows']} x {b['config']['cols']} bf16, {b['steps']} timelines, medians, µs from the forward kernel's first wavefront

{chr(10).join(rows)}

* step between two events around it: {t['step_us_by_events']:.1f} µs; first start to the reducer's last end: {t['span']:.1f} µs
* nothing runs for {t['gap_forward_to_backward']:.1f} µs between the forward kernel's last wavefront and the backward kernel's first,
  and for {t['gap_backward_to_reducer']:.1f} µs between the backward kernel and the reducer
* backward: {bw['rows_per_wavefront']:.0f} rows per wavefront ({bw['wavefronts_with_one_more']:.0f} wavefronts carry one more), {bw['us_per_row_median']:.2f} µs per row (median);
  a wavefront's rows are done at {bw['rows_done_first']:.1f} (first) / {bw['rows_done_median']:.1f} (median) / {bw['rows_done_last_without_extra']:.1f} (last, without an extra row) / {extra if extra is None else format(extra, '.1f')} (last, with one);
  medians per XCD: {' '.join(f'{x:.1f}' for x in bw['rows_done_median_by_xcd'])}
* backward: from a workgroup's last row to its partial row written: {bw['partial_row_flush_median']:.2f} µs (median); the four wavefronts of a
  workgroup finish their rows within {bw['rows_done_spread_inside_workgroup_median']:.2f} µs of each other
""")
    md = f"""# A step from the inside: per-wavefront clocks in the AdaLN kernels and the column reducer

{BOX}.  Kernel sources digest `{digest}`.  A measurement build of the library (`-DTTN_WAVE_CLOCK=1`: every wavefront
of `adaln_fwd_kernel`, `adaln_bwd_kernel` and `colreduce_kernel` stores the constant 100 MHz clock when it starts,
when its rows are done and when its last memory operation has completed) runs the step back to back; the marks of
the last step are read back.  By `python -m teletron_amd.profile_collect timeline --dir {DIR_SHOWN}`:

    python -m teletron_amd.build --variant {DIR_SHOWN}/variants/lib_waveclock.so --flag=-DTTN_WAVE_CLOCK=1
    TELETRON_AMD_LIB={DIR_SHOWN}/variants/lib_waveclock.so  python3 bench.py --workload timeline-cfg3 --steps 25 --warmup 6
    TELETRON_AMD_LIB={DIR_SHOWN}/variants/lib_waveclock.so  python3 bench.py --workload timeline-cfg4 --steps 15 --warmup 4

Written by `python -m teletron_amd.profile_summary timeline --dir {DIR_SHOWN}`.

{chr(10).join(parts)}
"""
    with open(os.path.join(PROFILES, "step_timeline_wave_clocks.md"), "w") as f:
        f.write(md)
    print("wrote step_timeline_wave_clocks.md")


def main():
    global PROFILES, DIR_SHOWN
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("what", choices=("cfg4", "workloads", "stream", "variants", "runs", "cached", "wide", "timeline"))
    ap.add_argument("--dir", default="rocprof_out", help="where rocprofv3 wrote (its -d arguments' parent)")
    ap.add_argument("--out", default=PROFILES, help="where the summaries are written (default: profiles/)")
    a = ap.parse_args()
    PROFILES = a.out
    DIR_SHOWN = a.dir.rstrip("/")
    os.makedirs(PROFILES, exist_ok=True)
    {"cfg4": cfg4, "workloads": workloads, "stream": stream, "variants": variants, "runs": run_lengths,
     "cached": cached, "wide": wide, "timeline": timeline}[a.what](a.dir)


if __name__ == "__main__":
    main()
