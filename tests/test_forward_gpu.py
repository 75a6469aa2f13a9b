"""GPU parity of the forward scan against the CPU oracle (same seeded inputs).

Bar: per tensor max|hw - ref| / max|ref| <= 2e-2 and cosine >= 0.9999, reference = fp32 oracle on
the bf16-rounded inputs."""
import pytest
import torch

from oracle import ttt_mlp_oracle as orc

pytestmark = pytest.mark.gpu

MAX_REL, MIN_COS = 2e-2, 0.9999
FWD_KEYS = ("XQ", "XK", "XV", "last_eta", "ttt_norm_weight", "ttt_norm_bias", "W1", "b1", "W2", "b2")


def _run_forward(d, cgs, overlap=None):
    """overlap: None = the operator's own choice; False / True = one / two workgroups per (batch, head),
    and the mode that actually ran is asserted."""
    import ttt_mlp_host as host
    import test_time_training as ext
    dev = torch.device("cuda:0")
    B, NH, NC = d["XQ"].shape[:3]
    t = {k: d[k].to(dev).contiguous() for k in FWD_KEYS}
    t.update(host.alloc_forward_buffers(B, NH, NC, cgs, dev))
    for k in ("W1_checkpoints", "b1_checkpoints", "W2_checkpoints", "b2_checkpoints"):
        t[k].fill_(float("nan"))
    t["Out"].fill_(float("nan"))
    if overlap is not None:
        ext.set_overlap(bool(overlap))
    try:
        ret = host.forward(t, cgs)
    finally:
        ext.set_overlap(True)
    if overlap is not None:
        assert ext.last_forward_mode() == int(bool(overlap))
    assert ret.data_ptr() == t["Out"].data_ptr()
    return {k: v.float().cpu() for k, v in t.items()}


def _check(name, hw, ref):
    st = orc.parity_stats(hw, ref)
    print(f"{name:16s} max_rel={st['max_rel']:.3e} cos={st['cosine']:.6f} max_abs={st['max_abs']:.3e}", flush=True)
    assert torch.isfinite(hw).all(), name
    assert st["max_rel"] <= MAX_REL and st["cosine"] >= MIN_COS, (name, st)


@pytest.mark.parametrize("B,NH,NC,cgs,seed,rand_affine", [
    (1, 2, 4, 1, 0, False),      # the CPU-runnable reference configuration
    (1, 2, 4, 4, 1, True),
    (2, 3, 9, 4, 2, True),       # ragged last checkpoint group, biases and norm affine non-trivial
    (1, 1, 1, 1, 3, True),       # single mini-batch
    (1, 4, 32, 8, 4, False),
])
def test_forward_matches_oracle(B, NH, NC, cgs, seed, rand_affine):
    print(f"case B={B} NH={NH} NC={NC} cgs={cgs} seed={seed}", flush=True)
    d = orc.make_inputs(B, NH, NC, seed=seed, with_grads=False)
    if rand_affine:
        g = torch.Generator().manual_seed(100 + seed)
        d["b1"] = 0.02 * torch.randn(B, NH, 1, 256, generator=g)
        d["b2"] = 0.02 * torch.randn(B, NH, 1, 64, generator=g)
        d["ttt_norm_weight"] = 1 + 0.1 * torch.randn(1, NH, 1, 64, generator=g)
        d["ttt_norm_bias"] = 0.1 * torch.randn(1, NH, 1, 64, generator=g)
    hw = _run_forward(d, cgs)
    out, ck, _ = orc.ttt_forward(*[d[k] for k in FWD_KEYS], cgs)
    _check("Out", hw["Out"], out)
    for name, ref in zip(("W1_checkpoints", "b1_checkpoints", "W2_checkpoints", "b2_checkpoints"), ck):
        if name.startswith("b") and ref.abs().max() == 0:
            assert hw[name].abs().max() == 0
            continue
        _check(name, hw[name], ref)
    # slot 0 is the caller's initial state, bit for bit
    assert torch.equal(hw["W1_checkpoints"][:, :, 0], d["W1"])
    assert torch.equal(hw["W2_checkpoints"][:, :, 0], d["W2"])
    assert torch.equal(hw["b1_checkpoints"][:, :, 0], d["b1"])
    assert torch.equal(hw["b2_checkpoints"][:, :, 0], d["b2"])


@pytest.mark.parametrize("B,NH,NC,cgs", [
    (1, 2, 4, 1),        # less than one hand-over of eight mini-batches
    (2, 3, 9, 4),        # one full hand-over and a ragged one; (batch, head) count not a multiple of 8
    (1, 8, 40, 8),       # five hand-overs: both halves of the ring are reused, the recurrence waits for the output branch
    (1, 4, 33, 16),
    (2, 130, 5, 2),      # more pairs than CUs: a full round with one workgroup each, the remaining 4 pairs with two
    (1, 72, 5, 2),
])
def test_overlapped_forward_is_bit_identical(B, NH, NC, cgs):
    """Computing Out on a second workgroup changes the schedule, not one bit of the results."""
    print(f"case B={B} NH={NH} NC={NC} cgs={cgs}", flush=True)
    d = orc.make_inputs(B, NH, NC, seed=21, with_grads=False)
    g = torch.Generator().manual_seed(121)
    d["b1"] = 0.02 * torch.randn(B, NH, 1, 256, generator=g)
    d["b2"] = 0.02 * torch.randn(B, NH, 1, 64, generator=g)
    d["ttt_norm_weight"] = 1 + 0.1 * torch.randn(1, NH, 1, 64, generator=g)
    d["ttt_norm_bias"] = 0.1 * torch.randn(1, NH, 1, 64, generator=g)
    one = _run_forward(d, cgs, overlap=False)
    two = _run_forward(d, cgs, overlap=True)
    for k in ("Out", "W1_checkpoints", "b1_checkpoints", "W2_checkpoints", "b2_checkpoints"):
        assert torch.isfinite(two[k]).all(), k
        assert torch.equal(one[k], two[k]), k
