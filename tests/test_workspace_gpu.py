"""A caller-owned workspace for the operator module: with `set_workspace(tensor)` the two operators allocate nothing
(the upstream operator takes every tensor, scratch included, from its caller: kernels/ttt_backward/ttt.cu:1451-1917)
and give the same results, bit for bit, as with a workspace from torch's allocator."""
import pytest
import torch

from oracle import ttt_mlp_oracle as orc

pytestmark = pytest.mark.gpu

FWD_KEYS = ("XQ", "XK", "XV", "last_eta", "ttt_norm_weight", "ttt_norm_bias", "W1", "b1", "W2", "b2")
UP_KEYS = ("grad_L_W1_last", "grad_L_b1_last", "grad_L_W2_last", "grad_L_b2_last", "grad_L_XQW_mini_batch")


def _run(host, t, cgs):
    host.zero_accumulating_grads(t)
    host.forward(t, cgs)
    host.backward(t, cgs)
    torch.cuda.synchronize()
    return {k: t[k].clone() for k in ("Out", "W1_checkpoints", "b1_checkpoints") + host.GRAD_NAMES}


def test_operators_allocate_nothing_with_a_caller_workspace():
    import test_time_training as ext
    import ttt_mlp_host as host
    dev = torch.device("cuda:0")
    B, NH, NC, cgs = 1, 8, 24, 4
    print(f"case B={B} NH={NH} NC={NC} cgs={cgs}", flush=True)
    d = orc.make_inputs(B, NH, NC, seed=5)
    t = {k: d[k].to(dev).contiguous() for k in FWD_KEYS + UP_KEYS}
    t.update(host.alloc_forward_buffers(B, NH, NC, cgs, dev))
    t.update(host.alloc_backward_buffers(B, NH, NC, cgs, dev))
    ext.set_workspace(None)
    ref = _run(host, t, cgs)                       # workspace from torch's allocator
    assert ext.last_forward_mode() == 1 and ext.last_backward_mode() == 1
    nbytes = host.workspace_bytes(B, NH, cgs)
    assert nbytes > 0
    ws = torch.full((nbytes,), 0x5A, dtype=torch.uint8, device=dev)
    try:
        host.set_workspace(ws)
        for call in range(2):
            for k in ("Out",) + host.GRAD_NAMES[:6]:
                t[k].fill_(7.0)
            host.zero_accumulating_grads(t)
            torch.cuda.synchronize()
            before, peak0 = torch.cuda.memory_allocated(dev), torch.cuda.max_memory_allocated(dev)
            torch.cuda.reset_peak_memory_stats(dev)
            host.forward(t, cgs)
            host.backward(t, cgs)
            torch.cuda.synchronize()
            assert torch.cuda.memory_allocated(dev) == before, "the operators kept memory"
            assert torch.cuda.max_memory_allocated(dev) == before, "the operators allocated during the calls"
            assert ext.last_forward_mode() == 1 and ext.last_backward_mode() == 1, "the caller's workspace was not used"
            for k, r in ref.items():
                assert torch.equal(t[k], r), (call, k)
        # a workspace that is too small for the shape: one workgroup per pair, still nothing allocated, same results
        host.set_workspace(ws[:4096])
        host.zero_accumulating_grads(t)
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated(dev)
        torch.cuda.reset_peak_memory_stats(dev)
        host.forward(t, cgs)
        host.backward(t, cgs)
        torch.cuda.synchronize()
        assert torch.cuda.max_memory_allocated(dev) == before
        assert ext.last_forward_mode() == 0 and ext.last_backward_mode() == 0
        for k, r in ref.items():
            assert torch.equal(t[k], r), ("small", k)
        with pytest.raises(RuntimeError):
            ext.set_workspace(torch.zeros(16, dtype=torch.float32, device=dev))
    finally:
        host.set_workspace(None)


def test_compute_unit_budget_turns_the_waiting_launches_off():
    """Workgroups that wait for each other must all be resident; a host that cannot promise the whole device says how
    many CUs there are, and shapes that no longer fit run with one workgroup per (batch, head) - same results."""
    import test_time_training as ext
    import ttt_mlp_host as host
    dev = torch.device("cuda:0")
    B, NH, NC, cgs = 1, 8, 12, 4
    print(f"case B={B} NH={NH} NC={NC} cgs={cgs}", flush=True)
    d = orc.make_inputs(B, NH, NC, seed=6)
    t = {k: d[k].to(dev).contiguous() for k in FWD_KEYS + UP_KEYS}
    t.update(host.alloc_forward_buffers(B, NH, NC, cgs, dev))
    t.update(host.alloc_backward_buffers(B, NH, NC, cgs, dev))
    ref = _run(host, t, cgs)
    assert ext.last_forward_mode() == 1 and ext.last_backward_mode() == 1
    try:
        ext.set_compute_units(15)             # 2 x 8 workgroups do not fit 15 CUs
        assert host.workspace_bytes(B, NH, cgs) == 0
        got = _run(host, t, cgs)
        assert ext.last_forward_mode() == 0 and ext.last_backward_mode() == 0
        for k, r in ref.items():
            assert torch.equal(got[k], r), k
        ext.set_compute_units(16)             # two per pair fit, more do not
        assert host.workspace_bytes(B, NH, cgs) > 0
        got = _run(host, t, cgs)
        assert ext.last_forward_mode() == 1 and ext.last_backward_mode() == 1
        for k, r in ref.items():
            assert torch.equal(got[k], r), k
    finally:
        ext.set_compute_units(0)
