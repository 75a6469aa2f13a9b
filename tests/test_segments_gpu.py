"""More (batch, head) pairs than CUs: the launchers cut every sequence into segments at checkpoint boundaries and
launch the (segment, pair) jobs a device's worth at a time.  A forward segment starts from the checkpoint the one
before it left; a backward segment takes the running gradients and the norm-gradient sums from where the one before it
left them.  Forced here on a few pairs by a small compute-unit budget; the results must not change by a bit - Out, all
checkpoints and all ten gradients."""
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
CK_KEYS = ("W1_checkpoints", "b1_checkpoints", "W2_checkpoints", "b2_checkpoints")


def _plan(lib, which, pairs, cus, NC, cgs, with_workspace):
    seg, launches = ctypes.c_int(-1), ctypes.c_int(-1)
    rc = lib.ttt_mlp_segment_plan(which, ctypes.c_longlong(pairs), cus, NC, cgs, with_workspace, ctypes.byref(seg), ctypes.byref(launches))
    assert rc == 0
    return seg.value, launches.value


@pytest.mark.parametrize("NC,cgs", [(96, 8), (100, 8), (90, 3)])
def test_cut_sequences_give_the_same_forward(NC, cgs):
    import test_time_training as ext
    import ttt_mlp_host as host
    lib = ctypes.CDLL(LIB)
    dev = torch.device("cuda:0")
    B, NH = 1, 3
    print(f"case B={B} NH={NH} NC={NC} cgs={cgs}", flush=True)
    d = orc.make_inputs(B, NH, NC, seed=71)
    t = {k: d[k].to(dev).contiguous() for k in FWD_KEYS + UP_KEYS}
    t.update(host.alloc_forward_buffers(B, NH, NC, cgs, dev))
    t.update(host.alloc_backward_buffers(B, NH, NC, cgs, dev))

    def run():
        for k in ("Out",) + CK_KEYS:
            t[k].fill_(float("nan"))
        host.zero_accumulating_grads(t)
        host.forward(t, cgs)
        host.backward(t, cgs)
        torch.cuda.synchronize()
        return {k: t[k].clone() for k in ("Out",) + CK_KEYS + host.GRAD_NAMES}

    ref = run()                                   # 3 pairs on the whole device: whole sequences
    for k, r in ref.items():
        assert torch.isfinite(r.float()).all(), k
    try:
        ext.set_compute_units(2)                  # 3 pairs on 2 CUs
        for overlap in (True, False):             # with the operator's workspace, and the plain launch
            for which in (0, 1):
                seg, launches = _plan(lib, which, B * NH, 2, NC, cgs, 1 if overlap else 0)
                print(f"  overlap={overlap} {('forward', 'backward')[which]}: segments of {seg} mini-batches, {launches} launches", flush=True)
                if not overlap:                   # against whole rounds a cut always pays here
                    assert seg > 0 and seg % cgs == 0 and launches >= 3, "the shape was meant to be cut"
            ext.set_overlap(overlap)
            got = run()
            for k, r in ref.items():
                assert torch.equal(got[k], r), (overlap, k)
    finally:
        ext.set_overlap(True)
        ext.set_compute_units(0)


def test_cut_backward_with_the_overwrite_policy_and_the_group_tensors():
    """The cut backward under the operator's other switches: outputs overwritten instead of added to (garbage in the
    four accumulating outputs must not matter), and the sixteen group tensors filled behind it (x_hat_ln_group carries
    the cut backward's parked sums before that kernel rewrites it)."""
    import test_time_training as ext
    import ttt_mlp_host as host
    dev = torch.device("cuda:0")
    B, NH, NC, cgs = 1, 3, 64, 8
    print(f"case B={B} NH={NH} NC={NC} cgs={cgs}", flush=True)
    d = orc.make_inputs(B, NH, NC, seed=72)
    t = {k: d[k].to(dev).contiguous() for k in FWD_KEYS + UP_KEYS}
    t.update(host.alloc_forward_buffers(B, NH, NC, cgs, dev))
    t.update(host.alloc_backward_buffers(B, NH, NC, cgs, dev))
    group_keys = [k for k in host.BWD_ORDER if k.endswith("_group")]
    assert len(group_keys) == 16

    def run(garbage):
        host.zero_accumulating_grads(t)
        if garbage:
            for k in ("grad_L_XQ", "grad_L_XK", "grad_L_XV", "grad_L_last_eta"):
                t[k].fill_(3.0)
        host.forward(t, cgs)
        host.backward(t, cgs)
        torch.cuda.synchronize()
        return {k: t[k].clone() for k in ("Out",) + host.GRAD_NAMES + tuple(group_keys)}

    try:
        host.set_fill_group_tensors(True)
        ref = run(False)                          # whole sequences, accumulation into zeros
        ext.set_compute_units(2)
        ext.set_overlap(False)
        host.set_accumulate(False)
        got = run(True)
        for k, r in ref.items():
            assert torch.equal(got[k], r), k
    finally:
        host.set_accumulate(True)
        host.set_fill_group_tensors(False)
        ext.set_overlap(True)
        ext.set_compute_units(0)
