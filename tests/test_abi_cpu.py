"""CPU-side checks of the drop-in boundary: the C ABI library loads and exports every symbol the
header declares, argument validation behaves, and the Python operator module mirrors the reference
interface (names, positional arity, error behaviour).  No kernel is launched here."""
import ctypes
import inspect
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "ttt-tk_amd")
LIB = os.path.join(PKG, "libttt_mlp.so")
HEADER = os.path.join(ROOT, "include", "ttt_mlp.h")


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(LIB):
        import sys
        sys.path.insert(0, ROOT)
        import __graft_entry__ as ge
        ge.build()
    return ctypes.CDLL(LIB)


def declared_functions():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(ttt_mlp_[a-z0-9_]+)\s*\(", src)))


def test_header_declares_the_expected_entry_points():
    assert declared_functions() == ["ttt_mlp_abi_version", "ttt_mlp_bwd_export_group0", "ttt_mlp_bwd_launch", "ttt_mlp_bwd_launch_overlapped",
                                    "ttt_mlp_bwd_status_offset", "ttt_mlp_bwd_workspace_bytes", "ttt_mlp_error_string",
                                    "ttt_mlp_fwd_launch", "ttt_mlp_fwd_launch_overlapped", "ttt_mlp_fwd_launch_static", "ttt_mlp_fwd_status_offset",
                                    "ttt_mlp_fwd_workspace_bytes", "ttt_mlp_kernel_info", "ttt_mlp_launch_plan", "ttt_mlp_segment_plan", "ttt_mlp_set_compute_units", "ttt_mlp_set_wait_limit",
                                    "ttt_mlp_status_accumulate"]


def test_library_exports_every_declared_symbol(lib):
    for name in declared_functions():
        assert hasattr(lib, name), name
    assert lib.ttt_mlp_abi_version() == 2


def test_kernel_info_reports_lds_within_one_cu(lib):
    for which in (0, 1):
        lds, thr = ctypes.c_int(), ctypes.c_int()
        assert lib.ttt_mlp_kernel_info(which, ctypes.byref(lds), ctypes.byref(thr)) == 0
        assert thr.value in (256, 512) and 0 < lds.value <= 160 * 1024
    assert lib.ttt_mlp_kernel_info(2, ctypes.byref(lds), ctypes.byref(thr)) != 0


class FwdArgs(ctypes.Structure):
    _fields_ = [(n, ctypes.c_void_p) for n in
                ("XQ", "XK", "XV", "last_eta", "ttt_norm_weight", "ttt_norm_bias", "W1", "b1", "W2", "b2",
                 "W1_checkpoints", "b1_checkpoints", "W2_checkpoints", "b2_checkpoints", "Out")] + \
               [(n, ctypes.c_int32) for n in ("checkpoint_group_size", "B", "NH", "NC", "K")]


def test_forward_launch_rejects_bad_arguments_before_touching_the_gpu(lib):
    lib.ttt_mlp_error_string.restype = ctypes.c_char_p
    assert lib.ttt_mlp_fwd_launch(None, None) == 1001
    a = FwdArgs()
    assert lib.ttt_mlp_fwd_launch(ctypes.byref(a), None) == 1001          # null pointers
    for f, _ in FwdArgs._fields_[:15]:
        setattr(a, f, 0x1000)
    a.B, a.NH, a.NC, a.K, a.checkpoint_group_size = 1, 2, 9, 2, 4
    assert lib.ttt_mlp_fwd_launch(ctypes.byref(a), None) == 1002          # K must be ceil(9/4) = 3
    assert b"ceil" in lib.ttt_mlp_error_string(1002)
    a.K = 3
    a.XK = 0x1008
    assert lib.ttt_mlp_fwd_launch(ctypes.byref(a), None) == 1003          # misaligned
    a.XK = 0x1000
    a.NC = 0
    assert lib.ttt_mlp_fwd_launch(ctypes.byref(a), None) == 1001
    a.NC, a.checkpoint_group_size, a.K = (1 << 18) + 1, 1, (1 << 18) + 1   # beyond the 32-bit offsets of one (batch, head)
    assert lib.ttt_mlp_fwd_launch(ctypes.byref(a), None) == 1004
    a.NC, a.checkpoint_group_size, a.K = 1 << 17, (1 << 16) + 1, 2
    assert lib.ttt_mlp_fwd_launch(ctypes.byref(a), None) == 1004
    # more checkpoints than 32-bit byte offsets of 64 KiB slots reach: NC = 2^17 with a checkpoint before every mini-batch
    a.NC, a.checkpoint_group_size, a.K = 1 << 17, 1, 1 << 17
    assert lib.ttt_mlp_fwd_launch(ctypes.byref(a), None) == 1004
    a.NC, a.checkpoint_group_size, a.K = (1 << 15) + 1, 1, (1 << 15) + 1
    assert lib.ttt_mlp_fwd_launch(ctypes.byref(a), None) == 1004
    assert b"32768 checkpoints" in lib.ttt_mlp_error_string(1004)
    assert lib.ttt_mlp_bwd_launch(None, None) == 1001


def test_overlapped_backward_needs_a_device_with_room(lib):
    """Without a GPU no device has room for two workgroups per (batch, head): the size query says 0 and
    the launcher refuses before anything is enqueued."""
    lib.ttt_mlp_bwd_workspace_bytes.restype = ctypes.c_size_t
    lib.ttt_mlp_error_string.restype = ctypes.c_char_p
    assert lib.ttt_mlp_bwd_workspace_bytes(0, 2, 4) == 0
    assert lib.ttt_mlp_bwd_workspace_bytes(1, 2, 0) == 0
    assert lib.ttt_mlp_bwd_launch_overlapped(None, None, ctypes.c_size_t(0), None) == 1001
    lib.ttt_mlp_fwd_workspace_bytes.restype = ctypes.c_size_t
    assert lib.ttt_mlp_fwd_workspace_bytes(0, 2) == 0
    assert lib.ttt_mlp_fwd_launch_overlapped(None, None, ctypes.c_size_t(0), None) == 1001
    if not torch.cuda.is_available():
        assert lib.ttt_mlp_fwd_workspace_bytes(1, 2) == 0
    if not torch.cuda.is_available():
        assert lib.ttt_mlp_bwd_workspace_bytes(1, 2, 4) == 0
    assert b"ttt_mlp_bwd_launch" in lib.ttt_mlp_error_string(1005)
    assert b"workspace" in lib.ttt_mlp_error_string(1006)


def test_struct_layout_matches_header_field_order():
    src = open(HEADER).read()
    body = src[src.index("typedef struct ttt_mlp_fwd_args"):src.index("} ttt_mlp_fwd_args;")]
    names = re.findall(r"\b(?:const\s+)?(?:uint16_t|float)\s*\*\s*(\w+);", body)
    assert names == [f for f, _ in FwdArgs._fields_[:15]]
    body = src[src.index("typedef struct ttt_mlp_bwd_args"):src.index("} ttt_mlp_bwd_args;")]
    names = re.findall(r"\b(?:const\s+)?(?:uint16_t|float)\s*\*\s*(\w+);", body)
    import sys
    sys.path.insert(0, PKG)
    import ttt_mlp_host as host
    assert tuple(names) == host.BWD_ORDER         # 42 tensors in the operator's positional order
    assert len(host.FWD_ORDER) == 15 and len(host.BWD_ORDER) == 42


def test_operator_module_mirrors_reference_interface(lib):
    import sys
    sys.path.insert(0, PKG)
    import test_time_training as ttt
    assert ttt.__doc__ == "Test Time Training Kernels"
    assert ttt.ttt_forward.__doc__.strip().endswith("TTT Forward.")
    assert ttt.ttt_backward.__doc__.strip().endswith("TTT Backward.")
    sig = ttt.ttt_forward.__doc__.splitlines()[0]
    assert sig.count("arg") == 16                  # 15 tensors + checkpoint_group_size, positional only
    sig = ttt.ttt_backward.__doc__.splitlines()[0]
    assert sig.count("arg") == 43


def test_operator_raises_on_cpu_tensors_and_bad_shapes(lib):
    import sys
    sys.path.insert(0, PKG)
    import ttt_mlp_host as host
    B, NH, NC, cgs = 1, 2, 3, 2
    from oracle import ttt_mlp_oracle as orc
    d = orc.make_inputs(B, NH, NC, seed=0, with_grads=False)
    t = dict(d)
    t.update(host.alloc_forward_buffers(B, NH, NC, cgs, "cpu"))
    with pytest.raises(RuntimeError, match="XQ"):
        host.forward(t, cgs)                       # CPU tensors: no silent fallback
    t["XQ"] = t["XQ"][..., :32]
    with pytest.raises(RuntimeError, match="XQ"):
        host.forward(t, cgs)
    t = dict(d)
    t.update(host.alloc_forward_buffers(B, NH, NC, 3, "cpu"))      # K = 1, but cgs = 2 needs 2
    with pytest.raises(RuntimeError, match="checkpoints"):
        host.forward(t, cgs)


def test_host_allocator_shapes():
    import sys
    sys.path.insert(0, PKG)
    import ttt_mlp_host as host
    assert host.num_checkpoints(9, 4) == 3 and host.num_checkpoints(8, 4) == 2
    f = host.alloc_forward_buffers(2, 3, 9, 4, "cpu")
    assert f["W1_checkpoints"].shape == (2, 3, 3, 64, 256) and f["Out"].dtype == torch.bfloat16
    b = host.alloc_backward_buffers(2, 3, 9, 4, "cpu")
    assert b["Z1_group"].shape == (2, 3, 4, 64, 256) and b["std_ln_group"].shape == (2, 3, 4, 64, 1)
    assert b["grad_L_ttt_norm_weight"].shape == (2, 3, 1, 64)      # per batch element
    for k in ("grad_L_last_eta", "grad_L_XQ", "grad_L_XK", "grad_L_XV"):
        assert b[k].abs().max() == 0


def test_host_module_offers_the_autograd_wrapper(lib):
    import inspect
    import torch
    import ttt_mlp_host as host
    assert issubclass(host.TTTMLPFunction, torch.autograd.Function)
    assert list(inspect.signature(host.ttt_mlp).parameters) == [
        "XQ", "XK", "XV", "last_eta", "ttt_norm_weight", "ttt_norm_bias", "W1", "b1", "W2", "b2", "checkpoint_group_size"]
    assert "grad_last" in inspect.signature(host.ttt_mlp_backward).parameters


def test_launch_plan_keeps_waiting_workgroups_within_the_device(lib):
    """Workgroups that wait for each other must all be resident: whatever the plan, the launch with several
    workgroups per pair never exceeds the CU count, and full rounds of the device come first."""
    def plan(which, pairs, cus):
        a, b, c = ctypes.c_longlong(), ctypes.c_longlong(), ctypes.c_int()
        assert lib.ttt_mlp_launch_plan(which, ctypes.c_longlong(pairs), cus, ctypes.byref(a), ctypes.byref(b), ctypes.byref(c)) == 0
        return a.value, b.value, c.value
    assert plan(1, 48, 256) == (0, 48, 5)          # the metric's configuration: four workgroups per pair + one that fetches ahead
    assert plan(1, 32, 256) == (0, 32, 5)
    assert plan(1, 56, 256) == (0, 56, 4)          # a fifth would not fit
    assert plan(1, 64, 256) == (0, 64, 4)          # four per pair fill the device exactly
    assert plan(1, 128, 256) == (0, 128, 2)
    assert plan(1, 44, 256) == (0, 44, 4)          # not a multiple of 8 pairs: the fifth would not share the walk's XCD
    assert plan(1, 72, 256) == (0, 72, 3)
    assert plan(1, 96, 256) == (0, 96, 2)
    assert plan(1, 200, 256) == (200, 0, 0)        # two per pair would not fit: one each
    assert plan(1, 384, 256) == (256, 128, 2)      # one full round, the rest with two each
    assert plan(1, 260, 256) == (256, 4, 4)
    assert plan(1, 264, 256) == (256, 8, 5)
    assert plan(1, 512, 256) == (512, 0, 0)
    assert plan(0, 48, 256) == (0, 48, 2)          # forward: two per pair at most
    assert plan(0, 384, 256) == (256, 128, 2)
    assert plan(0, 200, 256) == (200, 0, 0)
    assert plan(1, 48, 0) == (48, 0, 0)            # no device: nothing to overlap
    for which in (0, 1):
        for cus in (1, 8, 104, 256, 304):
            for pairs in list(range(1, 40)) + [cus - 1, cus, cus + 1, 2 * cus, 3 * cus + 5, 10 * cus + cus // 3]:
                if pairs <= 0:
                    continue
                one, rest, per = plan(which, pairs, cus)
                assert one + rest == pairs and one % cus == 0 or rest == 0
                assert rest * per <= cus
                assert per in ((0, 2) if which == 0 else (0, 2, 3, 4, 5))
    assert lib.ttt_mlp_launch_plan(2, ctypes.c_longlong(1), 1, None, None, None) == 1001


def test_export_of_group_zero_validates_like_the_backward(lib):
    assert lib.ttt_mlp_bwd_export_group0(None, None) == 1001


def test_segment_plan_cuts_sequences_where_a_last_round_would_idle(lib):
    """More pairs than CUs: the sequences are cut at checkpoint boundaries and the (segment, pair) jobs launched a
    device's worth at a time, when that is shorter than whole rounds (or than a last round with several workgroups per
    pair).  A pair's earlier segment must sit in an earlier launch, the segments are whole checkpoint groups, and the
    backward needs two mini-batch slots of x_hat_ln_group for its parked sums."""
    def plan(which, pairs, cus, NC, cgs, ws):
        a, b = ctypes.c_int(-1), ctypes.c_int(-1)
        assert lib.ttt_mlp_segment_plan(which, ctypes.c_longlong(pairs), cus, NC, cgs, ws, ctypes.byref(a), ctypes.byref(b)) == 0
        return a.value, b.value
    for which in (0, 1):
        for ws in (0, 1):
            assert plan(which, 384, 256, 512, 32, ws) == (256, 3)      # the fill-the-chip configuration: 1.5 rounds
            assert plan(which, 48, 256, 4096, 64, ws)[0] == 0         # fewer pairs than CUs: nothing to gain
            assert plan(which, 256, 256, 512, 32, ws)[0] == 0
            assert plan(which, 512, 256, 512, 32, ws)[0] == 0         # full rounds
            assert plan(which, 384, 256, 512, 512, ws)[0] == 0        # one checkpoint group: nowhere to cut
    assert plan(0, 257, 256, 512, 32, 1) == (64, 9)                   # 8 segments: 9 launches of an eighth
    assert plan(1, 384, 256, 512, 1, 0)[0] == 0                       # backward, groups of one mini-batch
    assert plan(0, 384, 256, 512, 1, 0)[0] > 0
    assert plan(0, 384, 256, 512, 32, 1) == plan(0, 384, 256, 512, 32, 0)
    assert lib.ttt_mlp_segment_plan(2, ctypes.c_longlong(8), 8, 8, 8, 0, ctypes.byref(ctypes.c_int()), ctypes.byref(ctypes.c_int())) == 1001
    assert lib.ttt_mlp_segment_plan(0, ctypes.c_longlong(8), 8, 8, 8, 0, None, None) == 1001
    for which in (0, 1):
        for cus in (2, 8, 104, 256):
            for pairs in (cus + 1, cus + cus // 2, 2 * cus - 1, 2 * cus + 1, 3 * cus + 5):
                for NC, cgs in ((512, 32), (100, 8), (90, 3), (7, 2), (4096, 64)):
                    seg, launches = plan(which, pairs, cus, NC, cgs, 1)
                    if seg == 0:
                        continue
                    assert seg % cgs == 0 and seg < NC
                    segments = -(-NC // seg)
                    assert launches == -(-segments * pairs // cus)
                    # job (segment s, pair p) has index s * pairs + p: the launch of (s, p) comes after that of (s - 1, p)
                    assert all((s * pairs + p) // cus > ((s - 1) * pairs + p) // cus for s in range(1, segments) for p in (0, pairs - 1))
