"""The counter harness's arithmetic on synthetic rocprofv3 CSVs (no GPU, no rocprofv3): per-dispatch sums over the
counter's dimension rows, the copy calibration, and the derived busy / conflict / wait figures."""
import csv
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "ttt-tk_amd"))

import profile_counters as pc  # noqa: E402

PKG = os.path.join(ROOT, "ttt-tk_amd")


def _write(path, header, rows):
    os.makedirs(os.path.dirname(path), exist_ok=True)
    with open(path, "w", newline="") as f:
        w = csv.writer(f)
        w.writerow(header)
        w.writerows(rows)


def test_kernel_names_are_shortened_and_classified():
    assert pc.short_name("ttt::ttt_mlp_bwd_split_kernel<2, true>(ttt::BwdParams)") == "ttt_mlp_bwd_split_kernel<2, true>"
    assert pc.is_ours("void ttt::ttt_mlp_fwd_kernel(ttt::FwdParams)") and not pc.is_ours("at::native::copy_kernel")
    assert pc.is_copy("void at::native::elementwise_kernel<direct_copy_kernel_cuda>") and not pc.is_copy("ttt_mlp_fwd_kernel")


def test_counter_rows_of_one_dispatch_are_summed_and_dispatches_kept_apart(tmp_path):
    hdr = ["Dispatch_Id", "Kernel_Name", "Counter_Name", "Counter_Value"]
    rows = [[1, "k", "FETCH_SIZE", 10], [1, "k", "FETCH_SIZE", 5], [2, "k", "FETCH_SIZE", 7], [3, "copy", "FETCH_SIZE", 4]]
    _write(str(tmp_path / "x" / "c4_counter_collection.csv"), hdr, rows)
    got = pc.counter_sums(str(tmp_path / "x"))
    assert sorted(got["k"]["FETCH_SIZE"]) == [7.0, 15.0] and got["copy"]["FETCH_SIZE"] == [4.0]


def test_kernel_stats_are_read_by_name(tmp_path):
    hdr = ["Name", "Calls", "TotalDurationNs", "AverageNs", "Percentage", "MinNs", "MaxNs", "StdDev"]
    _write(str(tmp_path / "t" / "c4_kernel_stats.csv"), hdr, [["ttt::ttt_mlp_fwd_kernel(ttt::FwdParams)", 3, 300, 100.0, 50.0, 90, 110, 1]])
    st = pc.kernel_stats(str(tmp_path / "t"))
    assert st["ttt::ttt_mlp_fwd_kernel(ttt::FwdParams)"]["avg_ns"] == 100.0


def test_stage_names_come_from_the_kernels_header_and_fit_the_slots():
    """stage_clocks.py labels the clock slots with the enum entries of csrc/ttt_mlp_kernels.hpp, in order."""
    import re
    import stage_clocks as sc
    header = open(os.path.join(PKG, "csrc", "ttt_mlp_kernels.hpp")).read()
    fwd, bwd = sc.stage_names(header, "FwdStage"), sc.stage_names(header, "BwdStage")
    assert [n for n, _ in fwd][:3] == ["FS_TOP", "FS_F1_GELU", "FS_X2_SPLIT"] and fwd[-1][0] == "FS_OUT_LN"
    assert bwd[0][0] == "BS_GROUP" and bwd[-1][0] == "BS_X_SUMS" and "BS_PUBLISH" in [n for n, _ in bwd]
    assert all(desc for _, desc in fwd + bwd), "every stage carries its description"
    slots = int(re.search(r"constexpr int STAGE_SLOTS = (\d+);", header).group(1))
    assert slots == sc.SLOTS and len(fwd) <= slots and len(bwd) <= slots
    # every stage is marked in the kernel it belongs to
    fsrc = open(os.path.join(PKG, "csrc", "ttt_mlp_fwd.hip")).read()
    bsrc = open(os.path.join(PKG, "csrc", "ttt_mlp_bwd.hip")).read()
    for n, _ in fwd:
        assert f"TTT_STAGE({n})" in fsrc, n
    for n, _ in bwd:
        assert f"TTT_STAGE({n})" in bsrc, n


def test_the_product_library_contains_no_stage_clocks():
    import ctypes
    lib = ctypes.CDLL(os.path.join(PKG, "libttt_mlp.so"))
    assert not hasattr(lib, "ttt_mlp_set_stage_clocks")
    stages = os.path.join(PKG, "libttt_mlp_stages.so")
    if os.path.exists(stages):
        assert hasattr(ctypes.CDLL(stages), "ttt_mlp_set_stage_clocks")


def test_algorithmic_work_per_launch_follows_the_shapes():
    """7 / 21 contractions of 2*64*64*256 FLOP per (batch, head, mini-batch); bytes = the operator's inputs and outputs of a
    mini-batch plus the checkpoint bytes once per group."""
    f, b = pc.algorithmic("c4", "fwd"), pc.algorithmic("c4", "bwd")
    assert f["units"] == b["units"] == 48 * 4096
    assert f["flop"] == 7 * 2097152 * 48 * 4096 and b["flop"] == 21 * 2097152 * 48 * 4096
    assert abs(f["bytes"] - 48 * 4096 * (3 * 8192 + 128 + 8192 + 132352 / 64)) < 1
    assert abs(b["bytes"] - 48 * 4096 * (4 * 8192 + 128 + 3 * 8192 + 128 + 3 * 8192 + 132352 / 64)) < 1
    assert pc.algorithmic("c5", "bwd")["units"] == 8 * 48 * 512


def test_bench_and_harness_stamp_the_same_kernel_sources():
    """bench.py quotes the measured traffic of a summary only when the digest of the kernel sources matches."""
    sys.path.insert(0, ROOT)
    import bench
    assert bench.kernel_sources_digest() == pc.sources_digest()
    assert len(pc.sources_digest()) == 64
    for w in ("c2", "c3", "c4", "c5"):
        assert w in bench.METRICS and w in pc.SHAPES
        assert bench.WORKLOADS[w][:4] == pc.SHAPES[w]


def test_launch_summary_adds_up_the_kernels_of_one_launch():
    """c5's backward is two kernels in a row (one workgroup per pair, then the rest with two each): time, bytes and
    instruction counts of a launch are their sums, the roofline figures follow from the algorithmic work."""
    kernels = {
        "ttt_mlp_bwd_kernel": dict(avg_ns=24e6, hbm_bytes=9e10, counters=dict(SQ_INSTS_VALU=5e9, SQ_INSTS_MFMA=3e8, SQ_INSTS_LDS=8e8)),
        "ttt_mlp_bwd_split_kernel<1, false>": dict(avg_ns=12e6, hbm_bytes=4.5e10, counters=dict(SQ_INSTS_VALU=3e9, SQ_INSTS_MFMA=1e8, SQ_INSTS_LDS=4e8)),
        "ttt_mlp_fwd_kernel": dict(avg_ns=10e6),
    }
    L = pc.launch_summary("c5", kernels)
    units = 8 * 48 * 512
    b = L["bwd"]
    assert b["kernels"] == ["ttt_mlp_bwd_kernel", "ttt_mlp_bwd_split_kernel<1, false>"] and b["units"] == units
    assert abs(b["launch_ms"] - 36.0) < 1e-9 and abs(b["hbm_bytes"] - 1.35e11) < 1
    assert abs(b["achieved_tflops"] - 21 * 2097152 * units / 36e-3 / 1e12) < 1e-6
    assert abs(b["frac_of_bf16_mfma_peak"] - b["achieved_tflops"] / 2516.6) < 1e-12
    assert abs(b["traffic_over_algorithmic"] - 1.35e11 / (units * (57600 + 24576 + 132352 / 32))) < 1e-9
    assert abs(b["valu_insts_per_unit"] - 8e9 / units) < 1e-6 and abs(b["mfma_insts_per_unit"] - 4e8 / units) < 1e-6
    assert abs(b["hbm_gbs"] - 1.35e11 / 36e6) < 1e-6
    f = L["fwd"]
    assert "hbm_bytes" not in f and "valu_insts_per_unit" not in f and abs(f["launch_ms"] - 10.0) < 1e-9


def test_launch_summary_counts_every_dispatch_of_a_cut_launch():
    """c5 with the sequences cut at checkpoints: a launch is three dispatches of the one-workgroup kernel, and the
    per-dispatch averages of the profiler are multiplied out."""
    kernels = {
        "ttt_mlp_bwd_kernel": dict(avg_ns=12e6, dispatches_per_launch=3, hbm_bytes=4.5e10,
                                   counters=dict(SQ_INSTS_VALU=3e9, SQ_INSTS_MFMA=1e8, SQ_INSTS_LDS=4e8)),
        "ttt_mlp_fwd_kernel": dict(avg_ns=3e6, dispatches_per_launch=3),
    }
    L = pc.launch_summary("c5", kernels)
    units = 8 * 48 * 512
    assert abs(L["bwd"]["launch_ms"] - 36.0) < 1e-9 and abs(L["bwd"]["hbm_bytes"] - 1.35e11) < 1
    assert abs(L["bwd"]["valu_insts_per_unit"] - 9e9 / units) < 1e-6
    assert abs(L["fwd"]["launch_ms"] - 9.0) < 1e-9
    assert pc.TRACE_LAUNCHES == 3


def test_bench_reads_the_traffic_of_a_whole_launch(tmp_path, monkeypatch):
    """`roofline.traffic` is per launch: where a launch is several dispatches of one kernel the per-dispatch bytes of
    the counter summary are not the figure."""
    import json
    import bench
    prof = tmp_path / "profiles"
    prof.mkdir()
    (prof / "ttt_mlp_c5_counters.json").write_text(json.dumps({
        "kernels": {"ttt_mlp_bwd_kernel": {"hbm_bytes": 4.0e10, "dispatches_per_launch": 3}},
        "launches": {"bwd": {"hbm_bytes": 1.2e11}}}))
    (prof / "ttt_mlp_c4_counters.json").write_text(json.dumps({      # a summary without the per-launch block
        "kernels": {"ttt_mlp_bwd_kernel": {"hbm_bytes": 4.0e10, "dispatches_per_launch": 3},
                    "ttt_mlp_bwd_split_kernel<1, false>": {"hbm_bytes": 1.0e10}}}))
    monkeypatch.setattr(bench, "ROOT", str(tmp_path))
    assert bench.measured_traffic("c5", "bwd") == 1.2e11
    assert bench.measured_traffic("c4", "bwd") == 1.3e11
    assert bench.measured_traffic("c5", "fwd") is None and bench.measured_traffic("c3", "bwd") is None
