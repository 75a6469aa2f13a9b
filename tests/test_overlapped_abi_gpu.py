"""The two-workgroup launchers called directly through the C ABI (ctypes): shapes the operator module never
routes there (a single mini-batch, a single checkpoint group), the status word, and the error codes."""
import ctypes
import os

import pytest
import torch

from oracle import ttt_mlp_oracle as orc

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "ttt-tk_amd", "libttt_mlp.so")
FWD_KEYS = ("XQ", "XK", "XV", "last_eta", "ttt_norm_weight", "ttt_norm_bias", "W1", "b1", "W2", "b2")
UP_KEYS = ("grad_L_W1_last", "grad_L_b1_last", "grad_L_W2_last", "grad_L_b2_last", "grad_L_XQW_mini_batch")
SIZES = ("checkpoint_group_size", "B", "NH", "NC", "K")


def _lib():
    lib = ctypes.CDLL(LIB)
    lib.ttt_mlp_fwd_workspace_bytes.restype = ctypes.c_size_t
    lib.ttt_mlp_bwd_workspace_bytes.restype = ctypes.c_size_t
    return lib


def _args(order, t, cgs, B, NH, NC, K):
    class Args(ctypes.Structure):
        _fields_ = [(n, ctypes.c_void_p) for n in order] + [(n, ctypes.c_int32) for n in SIZES] + \
                   ([("overwrite", ctypes.c_int32)] if len(order) == 42 else [])    # the backward's struct ends with its policy flag
    return Args(*[t[k].data_ptr() for k in order], cgs, B, NH, NC, K)


# 8 pairs: the backward runs with a fifth workgroup per pair that fetches ahead of the walk (a multiple of 8 pairs)
@pytest.mark.parametrize("B,NH,NC,cgs", [(1, 2, 1, 1), (1, 3, 5, 8), (2, 2, 17, 4), (1, 8, 13, 4), (2, 4, 3, 8),
                                          (1, 16, 9, 4), (3, 8, 5, 2), (1, 48, 19, 8)])
def test_overlapped_launchers_through_ctypes(B, NH, NC, cgs):
    print(f"case B={B} NH={NH} NC={NC} cgs={cgs}", flush=True)
    import ttt_mlp_host as host
    lib = _lib()
    dev = torch.device("cuda:0")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    K = host.num_checkpoints(NC, cgs)
    d = orc.make_inputs(B, NH, NC, seed=31)
    results = []
    for overlapped in (False, True):
        t = {k: d[k].to(dev).contiguous() for k in FWD_KEYS + UP_KEYS}
        t.update(host.alloc_forward_buffers(B, NH, NC, cgs, dev))
        t.update(host.alloc_backward_buffers(B, NH, NC, cgs, dev))
        fa = _args(host.FWD_ORDER, t, cgs, B, NH, NC, K)
        ba = _args(host.BWD_ORDER, t, cgs, B, NH, NC, K)
        if not overlapped:
            assert lib.ttt_mlp_fwd_launch(ctypes.byref(fa), stream) == 0
            assert lib.ttt_mlp_bwd_launch(ctypes.byref(ba), stream) == 0
        else:
            for which, a in (("fwd", fa), ("bwd", ba)):
                nbytes = (lib.ttt_mlp_fwd_workspace_bytes(B, NH) if which == "fwd"
                          else lib.ttt_mlp_bwd_workspace_bytes(B, NH, cgs))
                assert nbytes > 0 and nbytes % 256 == 0
                ws = torch.full((nbytes + 256,), 0xA5, dtype=torch.uint8, device=dev)
                base = (ws.data_ptr() + 255) // 256 * 256
                launch = getattr(lib, f"ttt_mlp_{which}_launch_overlapped")
                # too small / misaligned / missing workspace are refused before anything is enqueued
                assert launch(ctypes.byref(a), ctypes.c_void_p(base), ctypes.c_size_t(nbytes - 1), stream) == 1006
                assert launch(ctypes.byref(a), ctypes.c_void_p(base + 16), ctypes.c_size_t(nbytes), stream) == 1003
                assert launch(ctypes.byref(a), None, ctypes.c_size_t(nbytes), stream) == 1001
                assert launch(ctypes.byref(a), ctypes.c_void_p(base), ctypes.c_size_t(nbytes), stream) == 0
                torch.cuda.synchronize()
                off_fn = getattr(lib, f"ttt_mlp_{which}_status_offset")
                off_fn.restype = ctypes.c_size_t
                assert off_fn(B, NH) == B * NH * 32 * 4
                status = ws[base - ws.data_ptr():].view(torch.int32)[off_fn(B, NH) // 4].item()
                assert status == 0, "a workgroup gave up waiting for the other"
        torch.cuda.synchronize()
        results.append({k: t[k].float().cpu() for k in ("Out", "W1_checkpoints", "b2_checkpoints") + host.GRAD_NAMES})
    for k in results[0]:
        assert torch.isfinite(results[1][k]).all(), k
        assert torch.equal(results[0][k], results[1][k]), k


@pytest.mark.parametrize("NH", [2, 8])   # 8 pairs: with the workgroup that fetches ahead of the walk
def test_a_wait_that_gives_up_is_reported_and_every_wave_exits(NH):
    """Forced from the host: with a wait limit of one clock tick the first workgroup that has to wait for its
    partner gives up at once, raises the status word, and all workgroups of the launch leave.  The operator
    (which synchronises by default) reports it; with the default limit the same call then succeeds."""
    import ttt_mlp_host as host
    import test_time_training as ext
    dev = torch.device("cuda:0")
    B, NC, cgs = 1, 24, 4
    print(f"case B={B} NH={NH} NC={NC} cgs={cgs}", flush=True)
    d = orc.make_inputs(B, NH, NC, seed=41)
    t = {k: d[k].to(dev).contiguous() for k in FWD_KEYS + UP_KEYS}
    t.update(host.alloc_forward_buffers(B, NH, NC, cgs, dev))
    t.update(host.alloc_backward_buffers(B, NH, NC, cgs, dev))
    try:
        ext.set_wait_limit(1)
        with pytest.raises(RuntimeError, match="gave up"):
            host.forward(t, cgs)
        assert ext.last_forward_mode() == 1
        ext.set_wait_limit(2_000_000_000)
        host.forward(t, cgs)              # checkpoints for the backward
        ext.set_wait_limit(1)
        with pytest.raises(RuntimeError, match="gave up"):
            host.backward(t, cgs)
        assert ext.last_backward_mode() == 1
    finally:
        ext.set_wait_limit(2_000_000_000)
    torch.cuda.synchronize()
    host.zero_accumulating_grads(t)
    host.backward(t, cgs)                 # the device is fine and the same call goes through
    assert torch.isfinite(t["grad_L_W1_init"]).all()


def test_a_wait_that_gives_up_is_reported_to_callers_that_synchronise_later():
    """With set_synchronize(False) the operator returns before the kernels have run, and its workspace (with the
    status word) goes back to the allocator: the status is folded into a device word that stays, and
    check_last_status() raises after the caller's own synchronisation - once; then the word is clear again."""
    import ttt_mlp_host as host
    import test_time_training as ext
    dev = torch.device("cuda:0")
    B, NH, NC, cgs = 1, 2, 24, 4
    d = orc.make_inputs(B, NH, NC, seed=43)
    t = {k: d[k].to(dev).contiguous() for k in FWD_KEYS + UP_KEYS}
    t.update(host.alloc_forward_buffers(B, NH, NC, cgs, dev))
    t.update(host.alloc_backward_buffers(B, NH, NC, cgs, dev))
    try:
        host.set_synchronize(False)
        host.forward(t, cgs)
        host.backward(t, cgs)
        ext.check_last_status()            # nothing gave up: no error
        ext.set_wait_limit(1)
        host.forward(t, cgs)               # gives up on the device; the call itself cannot know
        assert ext.last_forward_mode() == 1
        torch.cuda.synchronize()
        with pytest.raises(RuntimeError, match="gave up"):
            ext.check_last_status()
        ext.check_last_status()            # reported once
        ext.set_wait_limit(2_000_000_000)
        host.forward(t, cgs)
        ext.set_wait_limit(1)
        host.zero_accumulating_grads(t)
        host.backward(t, cgs)
        ext.set_wait_limit(2_000_000_000)
        host.forward(t, cgs)               # a good launch afterwards does not hide the earlier failure
        with pytest.raises(RuntimeError, match="gave up"):
            ext.check_last_status()
    finally:
        ext.set_wait_limit(2_000_000_000)
        host.set_synchronize(True)
    host.zero_accumulating_grads(t)
    host.forward(t, cgs)
    host.backward(t, cgs)
    assert torch.isfinite(t["grad_L_W1_init"]).all()
