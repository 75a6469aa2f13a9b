"""The autograd wrapper around the two operators (GPU): gradients that `torch.autograd` collects through
`ttt_mlp_host.ttt_mlp` equal the oracle's, to the same bar as the operator tests."""
import pytest
import torch

from oracle import ttt_mlp_oracle as orc

pytestmark = pytest.mark.gpu

MAX_REL, MIN_COS = 2e-2, 0.9999
KEYS = ("XQ", "XK", "XV", "last_eta", "ttt_norm_weight", "ttt_norm_bias", "W1", "b1", "W2", "b2")
GRAD_OF = dict(XQ="grad_L_XQ", XK="grad_L_XK", XV="grad_L_XV", last_eta="grad_L_last_eta",
               ttt_norm_weight="grad_L_ttt_norm_weight", ttt_norm_bias="grad_L_ttt_norm_bias",
               W1="grad_L_W1_init", b1="grad_L_b1_init", W2="grad_L_W2_init", b2="grad_L_b2_init")


@pytest.mark.parametrize("B,NH,NC,cgs", [(2, 2, 5, 2), (1, 3, 8, 4)])
def test_autograd_function_matches_oracle(B, NH, NC, cgs):
    import ttt_mlp_host as host
    dev = torch.device("cuda:0")
    d = orc.make_inputs(B, NH, NC, seed=5)
    leaves = {k: d[k].to(dev).contiguous().requires_grad_(True) for k in KEYS}
    out = host.ttt_mlp(*[leaves[k] for k in KEYS], cgs)
    assert out.shape == (B, NH, NC, 64, 64) and out.dtype == torch.bfloat16
    out.backward(d["grad_L_XQW_mini_batch"].to(dev))

    ref_out, ck, _ = orc.ttt_forward(*[d[k] for k in KEYS], cgs)
    zeros = orc.State(*[torch.zeros_like(d[k]) for k in ("grad_L_W1_last", "grad_L_b1_last", "grad_L_W2_last", "grad_L_b2_last")])
    ref = orc.ttt_backward(d["XQ"], d["XK"], d["XV"], d["last_eta"], d["ttt_norm_weight"], d["ttt_norm_bias"], ck, zeros,
                           d["grad_L_XQW_mini_batch"], cgs)
    failures = []
    st = orc.parity_stats(out.detach().float().cpu(), ref_out)
    if not (st["max_rel"] <= MAX_REL and st["cosine"] >= MIN_COS):
        failures.append(("Out", st))
    for k in KEYS:
        g = leaves[k].grad
        assert g is not None and g.shape == leaves[k].shape and g.dtype == leaves[k].dtype, k
        want = ref[GRAD_OF[k]]
        if k in ("ttt_norm_weight", "ttt_norm_bias"):
            want = want.sum(dim=0, keepdim=True)       # the operator emits them per batch element
        st = orc.parity_stats(g.float().cpu(), want)
        print(f"{k:18s} max_rel={st['max_rel']:.3e} cos={st['cosine']:.6f}", flush=True)
        if not (st["max_rel"] <= MAX_REL and st["cosine"] >= MIN_COS):
            failures.append((k, st["max_rel"], st["cosine"]))
    assert not failures, failures
