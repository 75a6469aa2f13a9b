#!/usr/bin/env python3
"""Per-stage clock budget of one forward and one backward mini-batch of the TTT-MLP kernels.

    python ttt-tk_amd/build.py --stages                       # once, no GPU needed: libttt_mlp_stages.so
    python ttt-tk_amd/stage_clocks.py --workload c4 [--out profiles/ttt_mlp_c4_stage_clocks.txt]

Loads the library built with -DTTT_STAGE_CLOCKS (the product library contains no clocks), runs the forward and the
backward of the workload once each the way the operator module would (same launch plan, workspace from torch), and
prints for every kind of workgroup - forward: recurrence / output branch; backward: replay / reverse walk - the
clocks per mini-batch that its waves spent in each stage, averaged over the (batch, head) pairs: the mean over
the 8 waves and the slowest wave.  The stage names and their descriptions are read from the two enums in
csrc/ttt_mlp_kernels.hpp.  Reading the clock is a scalar-memory operation that also waits for the wave's
outstanding LDS reads, so an instrumented kernel runs some 10 % slower than the product kernel; the launch times of
both are printed side by side.
"""
from __future__ import annotations

import argparse
import ctypes
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
SLOTS = 24
WAVES = 8
WORKLOADS = {   # B, NH, NC, checkpoint_group_size, std of the eta logits
    "c3": (1, 48, 256, 16, 1.0),
    "c4": (1, 48, 4096, 64, 1.0),
    "c5": (8, 48, 512, 32, 2.0),
}


def stage_names(header_text: str, enum: str):
    """[(name, description)] of `enum` in the kernels' header, in order, without the closing *_COUNT."""
    body = re.search(r"enum\s+" + enum + r"\s*\{(.*?)\};", header_text, re.S).group(1)
    out = []
    for line in body.splitlines():
        m = re.match(r"\s*(\w+)\s*,?\s*(?://\s*(.*))?$", line)
        if m and m.group(1) and not m.group(1).endswith("_COUNT"):
            out.append((m.group(1), (m.group(2) or "").strip()))
    return out


PER_WAVE = False


def table(title, clocks, names, per_mb):
    """clocks: tensor [pairs][8 waves][SLOTS] of summed clocks; per_mb: mini-batches each wave went through."""
    mean_w = clocks.double().mean(dim=0) / per_mb          # [8][SLOTS]
    tot = mean_w.sum(dim=1)                                # per wave
    lines = [f"{title}: {tot.mean().item():9.0f} clocks per mini-batch (mean over the waves; slowest wave {tot.max().item():.0f})"]
    for i, (name, desc) in enumerate(names):
        m, mx = mean_w[:, i].mean().item(), mean_w[:, i].max().item()
        if mx <= 0:
            continue
        if PER_WAVE:
            lines.append(f"  {name:18s} {m:8.0f}   waves 0-7: " + " ".join(f"{x:6.0f}" for x in mean_w[:, i].tolist()))
        else:
            lines.append(f"  {name:18s} {m:8.0f} {100 * m / tot.mean().item():5.1f} %   slowest wave {mx:8.0f}   {desc}")
    return lines


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", choices=sorted(WORKLOADS), default="c4")
    ap.add_argument("--out", default=None, help="also write the tables to this file")
    ap.add_argument("--per-wave", action="store_true", help="every stage's clocks wave by wave instead of share and description")
    a = ap.parse_args()
    global PER_WAVE
    PER_WAVE = a.per_wave
    import torch
    sys.path.insert(0, ROOT)
    sys.path.insert(0, HERE)
    import ttt_mlp_host as host
    from bench import make_device_inputs
    from build import STAGES_LIB, LIB

    if not os.path.exists(STAGES_LIB) or os.path.getmtime(STAGES_LIB) < os.path.getmtime(LIB):
        raise SystemExit(f"{STAGES_LIB} is missing or older than the product library: run  python ttt-tk_amd/build.py --stages  first")
    header = open(os.path.join(HERE, "csrc", "ttt_mlp_kernels.hpp")).read()
    fwd_names, bwd_names = stage_names(header, "FwdStage"), stage_names(header, "BwdStage")
    B, NH, NC, cgs, eta_std = WORKLOADS[a.workload]
    BH, K = B * NH, host.num_checkpoints(NC, cgs)
    dev = torch.device("cuda:0")
    t = make_device_inputs(B, NH, NC, eta_std, dev)
    t.update(host.alloc_forward_buffers(B, NH, NC, cgs, dev))
    t.update(host.alloc_backward_buffers(B, NH, NC, cgs, dev))

    class FwdArgs(ctypes.Structure):
        _fields_ = [(n, ctypes.c_void_p) for n in host.FWD_ORDER] + [(n, ctypes.c_int32) for n in ("cgs", "B", "NH", "NC", "K")]

    class BwdArgs(ctypes.Structure):
        _fields_ = [(n, ctypes.c_void_p) for n in host.BWD_ORDER] + [(n, ctypes.c_int32) for n in ("cgs", "B", "NH", "NC", "K", "overwrite")]

    fa = FwdArgs(*[t[k].data_ptr() for k in host.FWD_ORDER], cgs, B, NH, NC, K)
    ba = BwdArgs(*[t[k].data_ptr() for k in host.BWD_ORDER], cgs, B, NH, NC, K, 0)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def launches(lib):
        lib.ttt_mlp_fwd_workspace_bytes.restype = ctypes.c_size_t
        lib.ttt_mlp_bwd_workspace_bytes.restype = ctypes.c_size_t
        nf, nb = lib.ttt_mlp_fwd_workspace_bytes(B, NH), lib.ttt_mlp_bwd_workspace_bytes(B, NH, cgs)
        wf = torch.empty(max(nf, 1), dtype=torch.uint8, device=dev)
        wb = torch.empty(max(nb, 1), dtype=torch.uint8, device=dev)

        def fwd():
            if nf:
                return lib.ttt_mlp_fwd_launch_overlapped(ctypes.byref(fa), ctypes.c_void_p(wf.data_ptr()), ctypes.c_size_t(nf), stream)
            return lib.ttt_mlp_fwd_launch(ctypes.byref(fa), stream)

        def bwd():
            if nb:
                return lib.ttt_mlp_bwd_launch_overlapped(ctypes.byref(ba), ctypes.c_void_p(wb.data_ptr()), ctypes.c_size_t(nb), stream)
            return lib.ttt_mlp_bwd_launch(ctypes.byref(ba), stream)
        return fwd, bwd, (wf, wb)

    def timed(fn):
        rc = fn()   # warm-up
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        rc |= fn()
        e1.record()
        torch.cuda.synchronize()
        if rc:
            raise SystemExit(f"launch failed: code {rc}")
        return e0.elapsed_time(e1)

    plain = ctypes.CDLL(LIB)
    pf, pb, keep0 = launches(plain)
    plain_ms = (timed(pf), timed(pb))

    lib = ctypes.CDLL(STAGES_LIB)
    cf = torch.zeros(BH, 2, WAVES, SLOTS, dtype=torch.int32, device=dev)
    cb = torch.zeros(BH, 4, WAVES, SLOTS, dtype=torch.int32, device=dev)
    lib.ttt_mlp_set_stage_clocks.restype = None
    sf, sb, keep1 = launches(lib)
    lib.ttt_mlp_set_stage_clocks(ctypes.c_void_p(0), ctypes.c_void_p(0))
    sf(); sb()   # warm-up without clocks
    lib.ttt_mlp_set_stage_clocks(ctypes.c_void_p(cf.data_ptr()), ctypes.c_void_p(cb.data_ptr()))
    torch.cuda.synchronize()
    e0, e1, e2 = (torch.cuda.Event(enable_timing=True) for _ in range(3))
    e0.record(); rc = sf(); e1.record(); rc |= sb(); e2.record()
    torch.cuda.synchronize()
    if rc:
        raise SystemExit(f"launch failed: code {rc}")
    stage_ms = (e0.elapsed_time(e1), e1.elapsed_time(e2))
    cf, cb = cf.cpu().long() & 0xFFFFFFFF, cb.cpu().long() & 0xFFFFFFFF

    props = torch.cuda.get_device_properties(0)
    out = [f"Stage clocks of the TTT-MLP kernels, workload {a.workload}: B={B} NH={NH} NC={NC} checkpoint_group_size={cgs} on {props.name} ({props.multi_processor_count} CUs)",
           f"Command: python ttt-tk_amd/build.py --stages && python ttt-tk_amd/stage_clocks.py --workload {a.workload}",
           f"Launch times: forward {plain_ms[0]:.2f} ms, backward {plain_ms[1]:.2f} ms (product library); "
           f"{stage_ms[0]:.2f} ms, {stage_ms[1]:.2f} ms with the clocks compiled in",
           "Clocks are shader clocks per mini-batch and wave, averaged over the (batch, head) pairs whose workgroup of that kind ran;",
           "a stage's share is of the workgroup's own total.  Barrier waits are part of the stage that ends with the barrier.", ""]

    def present(x):   # pairs whose workgroup of this kind wrote anything
        return x[x.sum(dim=(1, 2)) > 0]

    one_f, rec, outb = present(cf[:, 0]), None, present(cf[:, 1])
    if len(outb):   # pairs with two workgroups: slot 0 is the recurrence alone
        two = cf[:, 1].sum(dim=(1, 2)) > 0
        rec, one_f = cf[two, 0], cf[~two, 0]
        one_f = present(one_f)
    if len(one_f):
        out += table(f"forward, one workgroup per pair ({len(one_f)} pairs)", one_f, fwd_names, NC) + [""]
    if rec is not None:
        out += table(f"forward, recurrence workgroup ({len(rec)} pairs)", rec, fwd_names, NC) + [""]
        out += table(f"forward, output-branch workgroup ({len(outb)} pairs)", outb, fwd_names, NC) + [""]
    r0, r1, walk = cb[:, 0], cb[:, 1], cb[:, 2]
    has_r0, has_r1 = r0.sum(dim=(1, 2)) > 0, r1.sum(dim=(1, 2)) > 0
    single = present(walk[~has_r0])
    if len(single):
        out += table(f"backward, one workgroup per pair ({len(single)} pairs)", single, bwd_names, NC) + [""]
    if has_r0.any():
        n_rep = 2 if has_r1.any() else 1
        groups0 = (K + n_rep - 1) // n_rep   # groups (counted from the end) replayed by the first replaying workgroup
        mb0 = NC - (K - groups0) * cgs if n_rep == 1 else sum(min(cgs, NC - (K - 1 - g) * cgs) for g in range(0, K, 2))
        out += table(f"backward, replaying workgroup 0 of {n_rep} ({int(has_r0.sum())} pairs, {mb0} of the {NC} mini-batches)", r0[has_r0], bwd_names, mb0) + [""]
        out += table(f"backward, reverse-walk workgroup ({int(has_r0.sum())} pairs)", walk[has_r0], bwd_names, NC) + [""]
        fin = cb[:, 3]
        if (fin.sum(dim=(1, 2)) > 0).any():
            out += table(f"backward, grad_L_XK workgroup ({int((fin.sum(dim=(1, 2)) > 0).sum())} pairs)", present(fin), bwd_names, NC) + [""]
    text = "\n".join(out)
    print(text)
    if a.out:
        os.makedirs(os.path.dirname(os.path.abspath(a.out)), exist_ok=True)
        with open(a.out, "w") as f:
            f.write(text + "\n")
    del keep0, keep1
    return 0


if __name__ == "__main__":
    sys.exit(main())
