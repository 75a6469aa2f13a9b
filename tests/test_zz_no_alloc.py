"""The forward entry point that allocates nothing (`ttt_mlp_fwd_launch_static`: its workspace is a fixed array in
the library's device memory) against the entry point it is a variant of (`ttt_mlp_fwd_launch_overlapped` with a
caller-owned workspace), through the C ABI: bit-identical Out and checkpoints on two calls in a row, the second
with a smaller input, so that whatever the first call left in the array must not matter; and the same call
replayed from a captured graph against the eager call."""
import ctypes
import os

import pytest
import torch

from oracle import ttt_mlp_oracle as orc

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "ttt-tk_amd", "libttt_mlp.so")
FWD_KEYS = ("XQ", "XK", "XV", "last_eta", "ttt_norm_weight", "ttt_norm_bias", "W1", "b1", "W2", "b2")
OUT_KEYS = ("Out", "W1_checkpoints", "b1_checkpoints", "W2_checkpoints", "b2_checkpoints")
SIZES = ("checkpoint_group_size", "B", "NH", "NC", "K")


def _args(order, t, cgs, B, NH, NC, K):
    class Args(ctypes.Structure):
        _fields_ = [(n, ctypes.c_void_p) for n in order] + [(n, ctypes.c_int32) for n in SIZES]
    return Args(*[t[k].data_ptr() for k in order], cgs, B, NH, NC, K)


def test_static_scratch_forward_matches_the_workspace_forward_twice_in_a_row():
    import ttt_mlp_host as host
    lib = ctypes.CDLL(LIB)
    lib.ttt_mlp_fwd_workspace_bytes.restype = ctypes.c_size_t
    lib.ttt_mlp_error_string.restype = ctypes.c_char_p
    dev = torch.device("cuda:0")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    sticky = torch.zeros(1, dtype=torch.int32, device=dev)
    for B, NH, NC, cgs, seed in ((2, 4, 40, 8, 51), (1, 3, 9, 4, 52)):      # 8 pairs (the maximum), then 3
        print(f"case B={B} NH={NH} NC={NC} cgs={cgs}", flush=True)
        K = host.num_checkpoints(NC, cgs)
        d = orc.make_inputs(B, NH, NC, seed=seed, with_grads=False)
        res = []
        for static in (False, True):
            t = {k: d[k].to(dev).contiguous() for k in FWD_KEYS}
            t.update(host.alloc_forward_buffers(B, NH, NC, cgs, dev))
            for k in OUT_KEYS:
                t[k].fill_(float("nan"))
            a = _args(host.FWD_ORDER, t, cgs, B, NH, NC, K)
            if static:
                rc = lib.ttt_mlp_fwd_launch_static(ctypes.byref(a), ctypes.c_void_p(sticky.data_ptr()), stream)
            else:
                nbytes = lib.ttt_mlp_fwd_workspace_bytes(B, NH)
                assert nbytes > 0
                ws = torch.empty(nbytes + 256, dtype=torch.uint8, device=dev)
                base = (ws.data_ptr() + 255) // 256 * 256
                rc = lib.ttt_mlp_fwd_launch_overlapped(ctypes.byref(a), ctypes.c_void_p(base), ctypes.c_size_t(nbytes), stream)
            assert rc == 0, lib.ttt_mlp_error_string(rc)
            torch.cuda.synchronize()
            res.append({k: t[k].float().cpu() for k in OUT_KEYS})
        assert sticky.item() == 0, "a workgroup gave up waiting for the other"
        for k in OUT_KEYS:
            assert torch.isfinite(res[1][k]).all(), k
            assert torch.equal(res[0][k], res[1][k]), k
        # and both agree with the oracle (max-rel 2e-2, cosine 0.9999)
        out, ck, _ = orc.ttt_forward(*[d[k] for k in FWD_KEYS], cgs)
        for k, r in (("Out", out), ("W1_checkpoints", ck.W1), ("W2_checkpoints", ck.W2)):
            st = orc.parity_stats(res[1][k], r)
            assert st["max_rel"] <= 2e-2 and st["cosine"] >= 0.9999, (k, st)


def test_static_scratch_forward_rejects_more_pairs_than_its_array_serves():
    import ttt_mlp_host as host
    lib = ctypes.CDLL(LIB)
    lib.ttt_mlp_error_string.restype = ctypes.c_char_p
    dev = torch.device("cuda:0")
    B, NH, NC, cgs = 1, 9, 2, 2
    d = orc.make_inputs(B, NH, NC, seed=53, with_grads=False)
    t = {k: d[k].to(dev).contiguous() for k in FWD_KEYS}
    t.update(host.alloc_forward_buffers(B, NH, NC, cgs, dev))
    t["Out"].zero_()
    a = _args(host.FWD_ORDER, t, cgs, B, NH, NC, 1)
    rc = lib.ttt_mlp_fwd_launch_static(ctypes.byref(a), None, None)
    assert rc == 1007 and b"at most 8" in lib.ttt_mlp_error_string(rc)
    torch.cuda.synchronize()
    assert t["Out"].float().abs().max() == 0          # nothing was launched
    assert lib.ttt_mlp_fwd_launch_static(None, None, None) == 1001


def test_static_scratch_forward_replayed_from_a_captured_graph():
    """A caller that captures: one ordinary call first (it looks the array's address up and loads the code), then
    the same call recorded into a graph.  The launch records kernels only (its counters are cleared by a small
    kernel, not by a memset node).  Every replay, on fresh inputs and with eager work and synchronisations in
    between, must give what the eager call gives on the same inputs."""
    import ttt_mlp_host as host
    lib = ctypes.CDLL(LIB)
    lib.ttt_mlp_error_string.restype = ctypes.c_char_p
    dev = torch.device("cuda:0")
    B, NH, NC, cgs = 1, 4, 24, 8
    K = host.num_checkpoints(NC, cgs)
    d = orc.make_inputs(B, NH, NC, seed=60, with_grads=False)
    t = {k: d[k].to(dev).contiguous() for k in FWD_KEYS}
    t.update(host.alloc_forward_buffers(B, NH, NC, cgs, dev))
    a = _args(host.FWD_ORDER, t, cgs, B, NH, NC, K)
    sticky = torch.zeros(1, dtype=torch.int32, device=dev)

    def eager():
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = lib.ttt_mlp_fwd_launch_static(ctypes.byref(a), ctypes.c_void_p(sticky.data_ptr()), stream)
        assert rc == 0, lib.ttt_mlp_error_string(rc)
        torch.cuda.synchronize()

    print("ordinary call ahead of the capture", flush=True)
    eager()
    graph = torch.cuda.CUDAGraph()
    print("capture", flush=True)
    with torch.cuda.graph(graph):
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = lib.ttt_mlp_fwd_launch_static(ctypes.byref(a), ctypes.c_void_p(sticky.data_ptr()), stream)
    assert rc == 0, lib.ttt_mlp_error_string(rc)
    for rep in range(3):
        print(f"replay {rep}", flush=True)
        d = orc.make_inputs(B, NH, NC, seed=61 + rep, with_grads=False)
        for k in FWD_KEYS:
            t[k].copy_(d[k].to(dev))
        for k in OUT_KEYS:
            t[k].fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        got = {k: t[k].float().cpu() for k in OUT_KEYS}
        for k in OUT_KEYS:
            t[k].fill_(float("nan"))
        eager()
        for k in OUT_KEYS:
            assert torch.isfinite(got[k]).all(), (rep, k)
            assert torch.equal(got[k], t[k].float().cpu()), (rep, k)
    assert sticky.item() == 0, "a workgroup gave up waiting for the other"
