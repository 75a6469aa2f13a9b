#!/usr/bin/env python3
"""Benchmark of the TTT-MLP forward + remat-backward hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c4|c5|c3|c2] [--only] [--no-cpu-baseline]

A "step" is one forward + one remat backward over one batch of synthetic input that is already
resident in HBM (zero-filling the four accumulating gradient outputs is part of the step, as the
operator's contract makes the caller do it).  Prints ONE JSON line:
  value      tokens/s for forward + backward, whole job
  roofline   the dominant kernel (the backward) against the dense bf16 MFMA peak, its duration
             measured with events on the launch stream inside the timed region
  cpu_baseline  the fp32 PyTorch oracle of the same math on the host cores, on a bounded sample
  c5         (default run only) the same figures for the fill-the-chip workload, the one the 35 % target is set on
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "ttt-tk_amd"))

G_FLOP = 2 * 64 * 64 * 256                 # one 64x64x256 contraction
FWD_G, BWD_G = 7, 21                        # contractions per mini-batch per (batch, head): forward; replay 7 + reverse 14
PEAK_BF16_TFLOPS = 2516.6                   # MI355X dense bf16 MFMA: 256 CU x 4096 FLOP/clk x 2.4 GHz
WORKLOADS = {
    # name: (B, NH, NC, checkpoint_group_size, eta logit std, description); c2 is the forward alone
    "c2": (1, 48, 256, 16, 1.0, "forward only B=1 NH=48 16,384 tokens cgs=16"),
    "c3": (1, 48, 256, 16, 1.0, "fwd+bwd B=1 NH=48 16,384 tokens cgs=16"),
    "c4": (1, 48, 4096, 64, 1.0, "fwd+bwd B=1 NH=48 262,144 tokens cgs=64 (the configuration the metric is quoted on)"),
    "c5": (8, 48, 512, 32, 2.0, "fwd+bwd B=8 NH=48 32,768 tokens/sequence cgs=32 (fill-the-chip)"),
}


def measured_traffic(workload, which):
    """HBM bytes per launch of the forward (`which` = "fwd") or backward ("bwd") kernels of a workload, from the
    rocprofv3 counter summary that `ttt-tk_amd/profile_counters.py` leaves under profiles/ (FETCH_SIZE + WRITE_SIZE,
    each scaled by what the same counter reads for a copy of known size); None if that workload was not profiled."""
    path = os.path.join(ROOT, "profiles", f"ttt_mlp_{workload}_counters.json")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        summary = json.load(f)
    launch = summary.get("launches", {}).get(which)     # summed over the kernels and dispatches a launch is made of
    if launch is not None:
        return launch.get("hbm_bytes")
    vals = [k["hbm_bytes"] * k.get("dispatches_per_launch", 1) for name, k in summary["kernels"].items()
            if f"ttt_mlp_{which}" in name and "hbm_bytes" in k]
    return sum(vals) if vals else None


def make_device_inputs(B, NH, NC, eta_std, dev):
    """Synthetic inputs of the operator's shapes and dtypes, generated on the device (seed 0)."""
    import torch
    g = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *s: torch.randn(*s, generator=g, device=dev, dtype=torch.float32)
    t = {}
    for name in ("XQ", "XK", "XV", "grad_L_XQW_mini_batch"):
        t[name] = torch.empty(B, NH, NC, 64, 64, device=dev, dtype=torch.bfloat16)
        for b in range(B):                      # generated per batch element to bound the fp32 temporary
            t[name][b] = rn(NH, NC, 64, 64).to(torch.bfloat16)
    t["W1"] = rn(B, NH, 64, 256) * 0.02
    t["W2"] = rn(B, NH, 256, 64) * 0.02
    t["b1"] = torch.zeros(B, NH, 1, 256, device=dev)
    t["b2"] = torch.zeros(B, NH, 1, 64, device=dev)
    t["ttt_norm_weight"] = torch.ones(1, NH, 1, 64, device=dev)
    t["ttt_norm_bias"] = torch.zeros(1, NH, 1, 64, device=dev)
    t["last_eta"] = (torch.sigmoid(rn(B, NH, NC, 64, 1) * eta_std) / 64).to(torch.bfloat16)
    t["grad_L_W1_last"] = rn(B, NH, 64, 256) * 1e-3
    t["grad_L_b1_last"] = rn(B, NH, 1, 256) * 1e-3
    t["grad_L_W2_last"] = rn(B, NH, 256, 64) * 1e-3
    t["grad_L_b2_last"] = rn(B, NH, 1, 64) * 1e-3
    return t


def cpu_baseline(NH, cgs, nc_sample, backward=True):
    """fp32 oracle forward + backward on the host cores over the first nc_sample mini-batches."""
    import torch
    from oracle import ttt_mlp_oracle as orc
    threads = os.cpu_count() or 1
    env = os.environ.get("OMP_NUM_THREADS")
    if env and env.isdigit():
        threads = min(threads, int(env))
    torch.set_num_threads(threads)
    d = orc.make_inputs(1, NH, nc_sample, seed=0)
    keys = ("XQ", "XK", "XV", "last_eta", "ttt_norm_weight", "ttt_norm_bias", "W1", "b1", "W2", "b2")
    t0 = time.perf_counter()
    with torch.no_grad():
        _, ck, _ = orc.ttt_forward(*[d[k] for k in keys], cgs)
        if backward:
            orc.ttt_backward(d["XQ"], d["XK"], d["XV"], d["last_eta"], d["ttt_norm_weight"], d["ttt_norm_bias"], ck,
                             orc.State(d["grad_L_W1_last"], d["grad_L_b1_last"], d["grad_L_W2_last"], d["grad_L_b2_last"]),
                             d["grad_L_XQW_mini_batch"], cgs)
    dt = time.perf_counter() - t0
    return {"value": nc_sample * 64 / dt, "unit": "tokens/s", "cores": threads, "kind": "port",
            "sample": f"fp32 PyTorch oracle, {'forward + backward' if backward else 'forward'}, B=1 NH={NH} first {nc_sample} mini-batches "
                      f"({nc_sample * 64} tokens) cgs={cgs}, {dt:.1f} s"}


METRICS = {
    # the metric string follows the workload; c4's is BASELINE.json's
    "c2": "TTT-MLP forward tokens/sec on 1 MI355X (B=1,NH=48,16K tok); % bf16 MFMA peak",
    "c3": "TTT-MLP fwd+bwd tokens/sec on 1 MI355X (B=1,NH=48,16K tok); % bf16 MFMA peak",
    "c4": "TTT-MLP fwd+bwd tokens/sec on 1 MI355X (B=1,NH=48,256K tok); % bf16 MFMA peak",
    "c5": "TTT-MLP fwd+bwd tokens/sec on 1 MI355X (B=8,NH=48,32K tok/seq); % bf16 MFMA peak",
}


def kernel_sources_digest():
    """sha256 over the kernel sources the library is built from: the counter summaries under profiles/ carry the digest
    of the sources they were measured on, and a summary of other sources is not quoted."""
    import hashlib
    h = hashlib.sha256()
    csrc = os.path.join(ROOT, "ttt-tk_amd", "csrc")
    for name in sorted(os.listdir(csrc)):
        if name.endswith((".hip", ".hpp")):
            h.update(name.encode())
            with open(os.path.join(csrc, name), "rb") as f:
                h.update(f.read())
    return h.hexdigest()


def measured_traffic_checked(workload, which):
    """(bytes or None, note or None): the measured HBM bytes of profiles/ if they were taken on these kernel sources."""
    path = os.path.join(ROOT, "profiles", f"ttt_mlp_{workload}_counters.json")
    if not os.path.exists(path):
        return None, "no counter summary for this workload under profiles/"
    with open(path) as f:
        stamp = json.load(f).get("kernel_sources_sha256")
    if stamp != kernel_sources_digest():
        return None, "the counter summary under profiles/ was measured on other kernel sources (its kernel_sources_sha256 differs)"
    return measured_traffic(workload, which), None


def run_workload(name, steps, warmup, overwrite=False, no_overlap=False, calibrate_copy=False):
    """Times `steps` forward (+ backward) steps of one workload and returns the figures of its JSON block."""
    import torch
    import ttt_mlp_host as host          # fails loudly if the HIP extension is not built
    import test_time_training as ext

    dev = torch.device("cuda:0")
    B, NH, NC, cgs, eta_std, desc = WORKLOADS[name]
    t = make_device_inputs(B, NH, NC, eta_std, dev)
    t.update(host.alloc_forward_buffers(B, NH, NC, cgs, dev))
    backward = name != "c2"
    if backward:
        t.update(host.alloc_backward_buffers(B, NH, NC, cgs, dev))
    host.set_synchronize(False)           # time with events; the operator's default host sync is not part of the kernel
    ext.set_overlap(not no_overlap)
    ext.set_accumulate(not overwrite)

    def step(ev=None):
        if backward and not overwrite:
            host.zero_accumulating_grads(t)    # the operator adds to four of its outputs, as upstream does
        if ev:
            ev[0].record()
        host.forward(t, cgs)
        if ev:
            ev[1].record()
        if backward:
            host.backward(t, cgs)
        if ev:
            ev[2].record()

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    events = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    t0 = time.perf_counter()
    for i in range(steps):
        step(events[i])
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ext.check_last_status()               # raises if workgroups of an unsynchronised launch gave up waiting for each other
    host.set_synchronize(True)
    if calibrate_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).fill_(1.0)     # 1 GiB read + 1 GiB written
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    assert bool(torch.isfinite(t["Out"].float()).all())
    assert not backward or bool(torch.isfinite(t["grad_L_W1_init"]).all())

    fwd_ms = sum(e[0].elapsed_time(e[1]) for e in events) / steps
    bwd_ms = sum(e[1].elapsed_time(e[2]) for e in events) / steps
    ms_per_step = wall * 1e3 / steps
    tokens = B * NC * 64
    mb_steps = B * NH * NC
    bwd_tflops = BWD_G * G_FLOP * mb_steps / (bwd_ms * 1e-3) / 1e12 if backward else 0.0
    fwd_tflops = FWD_G * G_FLOP * mb_steps / (fwd_ms * 1e-3) / 1e12
    all_tflops = (FWD_G + (BWD_G if backward else 0)) * G_FLOP * mb_steps / (ms_per_step * 1e-3) / 1e12
    # one kernel per combination of roles: ttt_mlp_bwd_split_kernel<replaying workgroups, grad_L_XK workgroup>
    bwd_kernel = "ttt_mlp_bwd_kernel"
    fwd_kernel = "ttt_mlp_fwd_kernel" if ext.last_forward_mode() == 0 else f"ttt_mlp_fwd_split_kernel<{32 if NC >= 512 else 8}>"
    import ctypes
    lib = ctypes.CDLL(os.path.join(os.path.dirname(os.path.abspath(host.__file__)), "libttt_mlp.so"))
    cus = torch.cuda.get_device_properties(dev).multi_processor_count

    def cut(which, overlapped):   # launches of a call whose sequences are cut at checkpoints (0: they are not)
        seg, launches = ctypes.c_int(), ctypes.c_int()
        lib.ttt_mlp_segment_plan(which, ctypes.c_longlong(B * NH), cus, NC, cgs, 1 if overlapped else 0, ctypes.byref(seg), ctypes.byref(launches))
        return launches.value if seg.value > 0 else 0

    if cut(0, ext.last_forward_mode() == 1):
        fwd_kernel = f"ttt_mlp_fwd_kernel x {cut(0, ext.last_forward_mode() == 1)} (sequences cut at checkpoints)"
    if backward and cut(1, ext.last_backward_mode() == 1):
        bwd_kernel = f"ttt_mlp_bwd_kernel x {cut(1, ext.last_backward_mode() == 1)} (sequences cut at checkpoints)"
    elif backward and ext.last_backward_mode() == 1:
        one, rest, per = ctypes.c_longlong(), ctypes.c_longlong(), ctypes.c_int()
        lib.ttt_mlp_launch_plan(1, ctypes.c_longlong(B * NH), cus, ctypes.byref(one), ctypes.byref(rest), ctypes.byref(per))
        bwd_kernel = f"ttt_mlp_bwd_split_kernel<{2 if per.value >= 3 else 1}, {'true' if per.value >= 4 else 'false'}>"
        if one.value:
            bwd_kernel = "ttt_mlp_bwd_kernel + " + bwd_kernel
    traffic, note = measured_traffic_checked(name, "bwd" if backward else "fwd")
    # the dominant kernel: the backward (the forward where there is no backward)
    roofline = {"bound": "mfma", "kernel": bwd_kernel if backward else fwd_kernel,
                "achieved": bwd_tflops if backward else fwd_tflops, "peak": PEAK_BF16_TFLOPS,
                "unit": "TFLOP/s", "frac": (bwd_tflops if backward else fwd_tflops) / PEAK_BF16_TFLOPS,
                "traffic": traffic,
                "flop_per_launch": (BWD_G if backward else FWD_G) * G_FLOP * mb_steps,
                "avg_launch_ms": bwd_ms if backward else fwd_ms}
    if note:
        roofline["traffic_note"] = note
    del t
    torch.cuda.empty_cache()
    return {
        "metric": METRICS[name],
        "value": tokens / (ms_per_step * 1e-3), "unit": "tokens/s", "ms_per_step": ms_per_step,
        "config": {"workload": f"{name}: {desc}", "B": B, "NH": NH, "NC": NC, "tokens": tokens,
                   "checkpoint_group_size": cgs},
        "fwd_ms": fwd_ms, "bwd_ms": bwd_ms, "fwd_tflops": fwd_tflops, "fwd_bwd_tflops": all_tflops,
        "pct_of_bf16_mfma_peak": 100.0 * all_tflops / PEAK_BF16_TFLOPS,
        "roofline": roofline,
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--workload", choices=sorted(WORKLOADS), default="c4")   # ("custom" is what --shape registers)
    ap.add_argument("--only", action="store_true",
                    help="time the named workload alone (without this, a c4 run also times the fill-the-chip workload c5 "
                         "and reports it in a \"c5\" block of the same JSON line)")
    ap.add_argument("--shape", default=None, metavar="B,NH,NC,CGS",
                    help="time this shape instead of a named workload (implies --only; the line's metric names the shape); "
                         "for launch-plan measurements at head counts other than the benchmark's")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--overwrite", action="store_true",
                    help="let ttt_backward overwrite grad_L_XQ / XK / XV / last_eta instead of adding to them "
                         "(no zero-fill in the step; not the upstream calling convention, so not the default)")
    ap.add_argument("--no-overlap", action="store_true",
                    help="backward with one workgroup per (batch, head) even where two fit the device")
    ap.add_argument("--cpu-sample-mb", type=int, default=1536, help="mini-batches in the CPU baseline sample")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 1 GiB device copy, so that a counter run has a kernel of known traffic")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (every (batch, head) recurrence is independent and no "
                 "collective is involved); --gpus must be 1")

    import torch
    import ttt_mlp_host  # noqa: F401    fails loudly if the HIP extension is not built

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    if a.shape:
        B, NH, NC, cgs = (int(x) for x in a.shape.split(","))
        a.workload, a.only, a.no_cpu_baseline = "custom", True, True
        WORKLOADS["custom"] = (B, NH, NC, cgs, 1.0, f"fwd+bwd B={B} NH={NH} {NC * 64} tokens/sequence cgs={cgs}")
        METRICS["custom"] = f"TTT-MLP fwd+bwd tokens/sec on 1 MI355X (B={B},NH={NH},{NC * 64} tok/seq); % bf16 MFMA peak"
    res = run_workload(a.workload, a.steps, a.warmup, a.overwrite, a.no_overlap, a.calibrate_copy)
    out = {
        "metric": res["metric"], "value": res["value"], "unit": res["unit"], "n_gpus": 1, "steps": a.steps,
        "warmup": a.warmup, "ms_per_step": res["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic", "config": res["config"],
        "fwd_ms": res["fwd_ms"], "bwd_ms": res["bwd_ms"], "fwd_tflops": res["fwd_tflops"],
        "fwd_bwd_tflops": res["fwd_bwd_tflops"], "pct_of_bf16_mfma_peak": res["pct_of_bf16_mfma_peak"],
        "roofline": res["roofline"],
    }
    if a.workload == "c4" and not a.only:
        # the configuration the target (35 % of the MFMA peak) is set on, timed the same way in the same run
        out["c5"] = run_workload("c5", a.steps, a.warmup, a.overwrite, a.no_overlap)
    if not a.no_cpu_baseline:
        B, NH, NC, cgs, _, _ = WORKLOADS[a.workload]
        out["cpu_baseline"] = cpu_baseline(NH, cgs, min(a.cpu_sample_mb, NC), a.workload != "c2")
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
