#!/usr/bin/env python3
"""rocprofv3 counter harness for the TTT-MLP kernels: one JSON per workload under profiles/.

    python ttt-tk_amd/profile_counters.py --workload c4 [--workload c5 ...] [--raw DIR] [--out DIR]

For each workload it runs `python3 bench.py --workload W ...` under rocprofv3 five times, each pass a run of its own
(counters are never combined with tracing options other than the kernel trace):
  1. --kernel-trace --stats                      -> calls and average duration per kernel
  2. --pmc FETCH_SIZE    (+ a 1 GiB copy kernel) -> KiB read from HBM per dispatch, scaled by what the same
  3. --pmc WRITE_SIZE    (+ a 1 GiB copy kernel)    counter reads for the copy of known size
  4. --pmc SQ_INSTS_VALU SQ_INSTS_MFMA SQ_VALU_MFMA_BUSY_CYCLES SQ_BUSY_CYCLES SQ_WAVE_CYCLES
           SQ_LDS_BANK_CONFLICT SQ_ACTIVE_INST_LDS SQ_WAIT_ANY
  5. --pmc SQ_INSTS_LDS SQ_INSTS_VMEM_RD SQ_INSTS_VMEM_WR SQ_INSTS_SALU SQ_ACTIVE_INST_VALU SQ_WAIT_INST_ANY
           SQ_INSTS_VALU_TRANS_F32 SQ_WAIT_INST_LDS
and writes profiles/ttt_mlp_<W>_counters.json with, per TTT-MLP kernel: average duration, HBM bytes read / written
per launch and the GB/s they amount to, MFMA-pipe busy %, vector-ALU busy %, the share of LDS-pipeline cycles lost
to bank conflicts, the share of wave cycles spent waiting, instruction counts, waves per SIMD and LDS bytes per
workgroup; and per launch (`launches`: forward / backward, summed over the kernels it is made of) the algorithmic
FLOPs and bytes, the fraction of the bf16 MFMA peak, measured HBM bytes per (batch, head, mini-batch) unit and their
ratio to the algorithmic bytes, and vector-ALU / MFMA / LDS instructions per unit.  The file carries the sha256 of the
kernel sources it was measured on (`kernel_sources_sha256`) and the git head; `bench.py` takes `roofline.traffic`
from it only if that digest matches the sources it runs.

Derived figures (SQ_* cycle counters tick once per 4 clocks; a 32x32x16 MFMA occupies the matrix pipe of its SIMD
for 32 clocks; every workgroup has 8 waves on the 4 SIMDs of one CU, which its LDS use fills):
  simd_clocks        = SQ_WAVE_CYCLES * 4 / waves_per_simd
  mfma_busy_pct      = 100 * SQ_INSTS_MFMA * 32 / simd_clocks
  valu_busy_pct      = 100 * SQ_ACTIVE_INST_VALU * 4 / simd_clocks
  lds_conflict_share = SQ_LDS_BANK_CONFLICT / (SQ_ACTIVE_INST_LDS * 4)
  wait_share         = SQ_WAIT_ANY / SQ_WAVE_CYCLES
"""
from __future__ import annotations

import argparse
import collections
import csv
import ctypes
import glob
import json
import os
import signal
import subprocess
import sys
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
GIB_KIB = 1 << 20   # the calibration copy reads 1 GiB and writes 1 GiB

PASSES = (
    ("trace", ["--kernel-trace", "--stats"], ["--steps", "2", "--warmup", "1"]),
    ("fetch", ["--pmc", "FETCH_SIZE"], ["--steps", "1", "--warmup", "0", "--calibrate-copy"]),
    ("write", ["--pmc", "WRITE_SIZE"], ["--steps", "1", "--warmup", "0", "--calibrate-copy"]),
    ("sq1", ["--pmc", "SQ_INSTS_VALU", "SQ_INSTS_MFMA", "SQ_VALU_MFMA_BUSY_CYCLES", "SQ_BUSY_CYCLES", "SQ_WAVE_CYCLES",
             "SQ_LDS_BANK_CONFLICT", "SQ_ACTIVE_INST_LDS", "SQ_WAIT_ANY"], ["--steps", "1", "--warmup", "0"]),
    ("sq2", ["--pmc", "SQ_INSTS_LDS", "SQ_INSTS_VMEM_RD", "SQ_INSTS_VMEM_WR", "SQ_INSTS_SALU", "SQ_ACTIVE_INST_VALU",
             "SQ_WAIT_INST_ANY", "SQ_INSTS_VALU_TRANS_F32", "SQ_WAIT_INST_LDS"], ["--steps", "1", "--warmup", "0"]),
)


TRACE_LAUNCHES = sum(int(PASSES[0][2][i + 1]) for i in (0, 2))   # --steps + --warmup of the trace pass


def run_pass(workload: str, tag: str, prof_args, bench_args, raw_dir: str, limit_s: int) -> str:
    out_dir = os.path.join(raw_dir, f"{workload}_{tag}")
    os.makedirs(out_dir, exist_ok=True)
    cmd = ["rocprofv3", *prof_args, "--output-format", "csv", "-d", out_dir, "-o", workload, "--",
           "python3", os.path.join(ROOT, "bench.py"), "--workload", workload, "--only", "--no-cpu-baseline", *bench_args]
    env = dict(os.environ, TMPDIR="/tmp")
    print("+", " ".join(cmd), flush=True)
    with open(os.path.join(out_dir, "run.log"), "w") as log:
        proc = subprocess.Popen(cmd, cwd="/tmp", env=env, stdout=log, stderr=subprocess.STDOUT, start_new_session=True)
        try:
            rc = proc.wait(timeout=limit_s)
        except subprocess.TimeoutExpired:
            os.killpg(proc.pid, signal.SIGKILL)      # the group this call started, nothing else
            proc.wait()
            raise RuntimeError(f"rocprofv3 pass {tag} of {workload} exceeded {limit_s} s; see {out_dir}/run.log")
    if rc != 0:
        raise RuntimeError(f"rocprofv3 pass {tag} of {workload} failed with exit code {rc}; see {out_dir}/run.log")
    return out_dir


def find_csv(out_dir: str, suffix: str) -> str:
    hits = glob.glob(os.path.join(out_dir, "**", f"*{suffix}"), recursive=True)
    if not hits:
        raise RuntimeError(f"no *{suffix} under {out_dir}")
    return hits[0]


def short_name(kernel_name: str) -> str:
    """ttt::ttt_mlp_bwd_split_kernel<2, true>(ttt::BwdParams) -> ttt_mlp_bwd_split_kernel<2, true>"""
    n = kernel_name.split("(")[0]
    return n.split("::")[-1].replace("void ", "").strip()


def is_ours(name: str) -> bool:
    return "ttt_mlp_fwd" in name or "ttt_mlp_bwd" in name or "ttt_mlp_export" in name


def is_copy(name: str) -> bool:
    return "copy" in name.lower() and "ttt_mlp" not in name


def kernel_stats(out_dir: str):
    rows = {}
    for r in csv.DictReader(open(find_csv(out_dir, "kernel_stats.csv"))):
        rows[r["Name"]] = dict(calls=int(r["Calls"]), avg_ns=float(r["AverageNs"]), total_ns=float(r["TotalDurationNs"]),
                               pct=float(r["Percentage"]))
    return rows


def counter_sums(out_dir: str):
    """{kernel: {counter: [value per dispatch]}} - the per-dimension rows of one dispatch are added up."""
    per_dispatch = collections.defaultdict(float)
    for r in csv.DictReader(open(find_csv(out_dir, "counter_collection.csv"))):
        per_dispatch[(r["Kernel_Name"], r["Dispatch_Id"], r["Counter_Name"])] += float(r["Counter_Value"])
    out = collections.defaultdict(lambda: collections.defaultdict(list))
    for (k, _, c), v in per_dispatch.items():
        out[k][c].append(v)
    return out


def kernel_geometry():
    lib = ctypes.CDLL(os.path.join(HERE, "libttt_mlp.so"))
    geo = {}
    for which, key in ((0, "fwd"), (1, "bwd")):
        lds, thr = ctypes.c_int(), ctypes.c_int()
        lib.ttt_mlp_kernel_info(which, ctypes.byref(lds), ctypes.byref(thr))
        geo[key] = dict(lds_bytes_per_workgroup=lds.value, threads_per_workgroup=thr.value,
                        waves_per_simd=thr.value // 64 // 4)
    return geo


# Algorithmic work of one launch: only the 64x64x256 contractions count as FLOPs (7 per mini-batch and (batch, head)
# in the forward, 21 in the backward: 7 replayed + 14 new); the bytes are the operator's inputs and outputs of a
# mini-batch (the backward's four accumulating outputs are read and written) plus the checkpoints, once per group.
G_FLOP = 2 * 64 * 64 * 256
PEAK_BF16_TFLOPS = 2516.6
PEAK_HBM_GBS = 8000.0
SHAPES = {"c2": (1, 48, 256, 16), "c3": (1, 48, 256, 16), "c4": (1, 48, 4096, 64), "c5": (8, 48, 512, 32)}   # B, NH, NC, cgs


def algorithmic(workload: str, which: str):
    B, NH, NC, cgs = SHAPES[workload]
    units = B * NH * NC
    if which == "fwd":
        return dict(units=units, flop=7 * G_FLOP * units, bytes=units * (32896 + 132352 / cgs))
    return dict(units=units, flop=21 * G_FLOP * units, bytes=units * (57600 + 24576 + 132352 / cgs))


def sources_digest() -> str:
    """sha256 over the kernel sources (the same digest bench.py checks before it quotes the traffic of a summary)."""
    import hashlib
    h = hashlib.sha256()
    csrc = os.path.join(HERE, "csrc")
    for name in sorted(os.listdir(csrc)):
        if name.endswith((".hip", ".hpp")):
            h.update(name.encode())
            with open(os.path.join(csrc, name), "rb") as f:
                h.update(f.read())
    return h.hexdigest()


def launch_summary(workload: str, kernels: dict) -> dict:
    """Roofline per launch (forward / backward): a launch may be made of two kernels (pairs beyond a multiple of the CU
    count run with more workgroups each) or of several dispatches of one (sequences cut at checkpoints), so time, bytes
    and instruction counts are summed over its kernels, each times its `dispatches_per_launch`."""
    launches = {}
    for which in ("fwd", "bwd"):
        ks = [e for k, e in kernels.items() if f"ttt_mlp_{which}" in k]
        if not ks:
            continue
        alg = algorithmic(workload, which)
        n = [e.get("dispatches_per_launch", 1) for e in ks]
        ms = sum(e["avg_ns"] * d for e, d in zip(ks, n)) / 1e6
        L = dict(kernels=[k for k in kernels if f"ttt_mlp_{which}" in k], launch_ms=ms, units=alg["units"],
                 algorithmic_flop=alg["flop"], algorithmic_bytes=alg["bytes"],
                 achieved_tflops=alg["flop"] / (ms * 1e-3) / 1e12)
        L["frac_of_bf16_mfma_peak"] = L["achieved_tflops"] / PEAK_BF16_TFLOPS
        if all("hbm_bytes" in e for e in ks):
            L["hbm_bytes"] = sum(e["hbm_bytes"] * d for e, d in zip(ks, n))
            L["hbm_bytes_per_unit"] = L["hbm_bytes"] / alg["units"]
            L["traffic_over_algorithmic"] = L["hbm_bytes"] / alg["bytes"]
            L["hbm_gbs"] = L["hbm_bytes"] / (ms * 1e6)
        if all("counters" in e for e in ks):
            for cn, label in (("SQ_INSTS_VALU", "valu_insts_per_unit"), ("SQ_INSTS_MFMA", "mfma_insts_per_unit"),
                              ("SQ_INSTS_LDS", "lds_insts_per_unit")):
                if all(cn in e["counters"] for e in ks):
                    L[label] = sum(e["counters"][cn] * d for e, d in zip(ks, n)) / alg["units"]
        launches[which] = L
    return launches


def profile(workload: str, raw_dir: str, limit_s: int):
    dirs = {tag: run_pass(workload, tag, pa, ba, raw_dir, limit_s) for tag, pa, ba in PASSES}
    stats = kernel_stats(dirs["trace"])
    fetch, write = counter_sums(dirs["fetch"]), counter_sums(dirs["write"])
    sq = counter_sums(dirs["sq1"])
    for k, v in counter_sums(dirs["sq2"]).items():
        sq[k].update(v)
    # calibration: what FETCH_SIZE / WRITE_SIZE read for a copy of 1 GiB
    cal = {}
    for label, table, counter in (("fetch", fetch, "FETCH_SIZE"), ("write", write, "WRITE_SIZE")):
        vals = [max(v[counter]) for k, v in table.items() if is_copy(k) and counter in v]
        if not vals:
            raise RuntimeError(f"calibration copy kernel not found in the {label} pass")
        cal[label] = dict(copy_kernel_kib=max(vals), factor=GIB_KIB / max(vals))
    geo = kernel_geometry()
    kernels = {}
    for name, st in stats.items():
        if not is_ours(name) or "zero_words" in name:
            continue
        key = short_name(name)
        g = geo["fwd" if "fwd" in key else "bwd"]
        # the trace pass makes TRACE_LAUNCHES forward and backward launches; a launch whose sequences are cut at
        # checkpoints dispatches the kernel several times
        e = dict(calls=st["calls"], dispatches_per_launch=max(1, round(st["calls"] / TRACE_LAUNCHES)), avg_ns=st["avg_ns"], **g)
        rd = [v["FETCH_SIZE"] for k, v in fetch.items() if short_name(k) == key and "FETCH_SIZE" in v]
        wr = [v["WRITE_SIZE"] for k, v in write.items() if short_name(k) == key and "WRITE_SIZE" in v]
        if rd and wr:
            e["hbm_read_bytes"] = sum(rd[0]) / len(rd[0]) * 1024 * cal["fetch"]["factor"]
            e["hbm_write_bytes"] = sum(wr[0]) / len(wr[0]) * 1024 * cal["write"]["factor"]
            e["hbm_bytes"] = e["hbm_read_bytes"] + e["hbm_write_bytes"]
            e["hbm_gbs"] = e["hbm_bytes"] / e["avg_ns"]
            e["hbm_frac_of_peak"] = e["hbm_gbs"] / PEAK_HBM_GBS
        c = {}
        for k, v in sq.items():
            if short_name(k) == key:
                c = {cn: sum(vals) / len(vals) for cn, vals in v.items()}
        if c:
            e["counters"] = c
            simd_clocks = c["SQ_WAVE_CYCLES"] * 4 / g["waves_per_simd"]
            e["mfma_busy_pct"] = 100 * c["SQ_INSTS_MFMA"] * 32 / simd_clocks
            e["valu_busy_pct"] = 100 * c["SQ_ACTIVE_INST_VALU"] * 4 / simd_clocks
            e["lds_conflict_share"] = c["SQ_LDS_BANK_CONFLICT"] / max(c["SQ_ACTIVE_INST_LDS"] * 4, 1)
            e["wait_share"] = c["SQ_WAIT_ANY"] / c["SQ_WAVE_CYCLES"]
        kernels[key] = e
    launches = launch_summary(workload, kernels)
    try:
        head = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], capture_output=True, text=True).stdout.strip()
    except OSError:
        head = ""
    return dict(workload=workload, launches=launches, kernel_sources_sha256=sources_digest(), git_head=head, device="MI355X (gfx950), one GPU", calibration=cal, kernels=kernels,
                commands=[" ".join(["rocprofv3", *pa, "--output-format csv -d <raw>/" + f"{workload}_{tag}", "-o", workload, "--",
                                    "python3 bench.py --workload", workload, "--only --no-cpu-baseline", *ba]) for tag, pa, ba in PASSES],
                note="each pass is its own run from /tmp with TMPDIR=/tmp; HBM bytes = counter KiB x 1024 x calibration factor")


def main():
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--workload", action="append", choices=["c2", "c3", "c4", "c5"])
    ap.add_argument("--raw", default=os.path.join(tempfile.gettempdir(), "ttt_mlp_counters"), help="where rocprofv3 writes its CSVs")
    ap.add_argument("--out", default=os.path.join(ROOT, "profiles"))
    ap.add_argument("--limit", type=int, default=170, help="seconds allowed per rocprofv3 pass")
    a = ap.parse_args()
    raw, out = os.path.abspath(a.raw), os.path.abspath(a.out)    # rocprofv3 runs from /tmp
    os.makedirs(out, exist_ok=True)
    for w in a.workload or ["c4"]:
        res = profile(w, raw, a.limit)
        path = os.path.join(out, f"ttt_mlp_{w}_counters.json")
        with open(path, "w") as f:
            json.dump(res, f, indent=1, sort_keys=True)
        print("wrote", path, flush=True)
        for k, e in res["kernels"].items():
            print(f"  {k:40s} {e['avg_ns'] / 1e6:9.3f} ms  HBM {e.get('hbm_bytes', 0) / 1e9:8.2f} GB ({e.get('hbm_gbs', 0):6.0f} GB/s)  "
                  f"MFMA {e.get('mfma_busy_pct', 0):5.1f} %  VALU {e.get('valu_busy_pct', 0):5.1f} %  "
                  f"LDS conflicts {100 * e.get('lds_conflict_share', 0):4.1f} %  waiting {100 * e.get('wait_share', 0):4.1f} %", flush=True)


if __name__ == "__main__":
    sys.exit(main())
