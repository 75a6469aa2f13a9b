"""Pins for the CPU oracle: every function is checked against something other than its own
formula -- PyTorch library routines, torch.autograd in fp64, closed-form special cases and
finite differences -- chosen so that a dropped term, a wrong sign or a transposed operand fails."""
import math

import pytest
import torch

from oracle import ttt_mlp_oracle as orc

torch.set_default_dtype(torch.float32)
F64 = torch.float64


def _small(B=1, NH=2, NC=3, CS=8, F=8, HID=16, seed=0, bias=True):
    g = torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g, dtype=F64)
    d = dict(XQ=rn(B, NH, NC, CS, F), XK=rn(B, NH, NC, CS, F), XV=rn(B, NH, NC, CS, F),
             last_eta=torch.sigmoid(rn(B, NH, NC, CS, 1)) / CS,
             ttt_norm_weight=1.0 + 0.1 * rn(1, NH, 1, F), ttt_norm_bias=0.1 * rn(1, NH, 1, F),
             W1=0.3 * rn(B, NH, F, HID), b1=0.1 * rn(B, NH, 1, HID) * bias,
             W2=0.3 * rn(B, NH, HID, F), b2=0.1 * rn(B, NH, 1, F) * bias)
    up = dict(gO=rn(B, NH, NC, CS, F), gW1=0.1 * rn(B, NH, F, HID), gb1=0.1 * rn(B, NH, 1, HID),
              gW2=0.1 * rn(B, NH, HID, F), gb2=0.1 * rn(B, NH, 1, F))
    return d, up


FWD_KEYS = ("XQ", "XK", "XV", "last_eta", "ttt_norm_weight", "ttt_norm_bias", "W1", "b1", "W2", "b2")


def _autograd_grads(d, up):
    leaves = {k: d[k].clone().requires_grad_(True) for k in FWD_KEYS}
    out, st = orc.ttt_forward_differentiable(*[leaves[k] for k in FWD_KEYS])
    scalar = (out * up["gO"]).sum() + (st.W1 * up["gW1"]).sum() + (st.b1 * up["gb1"]).sum() \
        + (st.W2 * up["gW2"]).sum() + (st.b2 * up["gb2"]).sum()
    grads = torch.autograd.grad(scalar, [leaves[k] for k in FWD_KEYS])
    return dict(zip(FWD_KEYS, grads)), out.detach()


def _oracle_grads(d, up, cgs):
    out, ck, fin = orc.ttt_forward(*[d[k] for k in FWD_KEYS], cgs, dtype=F64)
    res = orc.ttt_backward(d["XQ"], d["XK"], d["XV"], d["last_eta"], d["ttt_norm_weight"],
                           d["ttt_norm_bias"], ck, orc.State(up["gW1"], up["gb1"], up["gW2"], up["gb2"]),
                           up["gO"], cgs, dtype=F64)
    return res, out, ck, fin


# ------------------------------------------------------------------ elementwise
def test_gelu_matches_library_routine():
    x = torch.linspace(-9, 9, 4001, dtype=F64)
    ref = torch.nn.functional.gelu(x, approximate="tanh")
    # the truncated sqrt(2/pi) differs from the library's by 8e-11
    assert (orc.gelu_tanh(x) - ref).abs().max() < 1e-8


def test_gelu_derivatives_match_autograd_of_library_routine():
    x = torch.linspace(-7, 7, 2801, dtype=F64, requires_grad=True)
    y = torch.nn.functional.gelu(x, approximate="tanh")
    d1, = torch.autograd.grad(y.sum(), x, create_graph=True)
    d2, = torch.autograd.grad(d1.sum(), x)
    xd = x.detach()
    # the reference's constants are truncated to 8-10 digits: 3*K0*K1 vs 0.1070322243
    assert (orc.gelu_tanh_d1(xd) - d1.detach()).abs().max() < 1e-7
    assert (orc.gelu_tanh_d2(xd) - d2).abs().max() < 1e-7
    # known values: gelu'(0) = 1/2, gelu''(0) = sqrt(2/pi)
    z = torch.zeros(1, dtype=F64)
    assert abs(orc.gelu_tanh_d1(z).item() - 0.5) < 1e-12
    assert abs(orc.gelu_tanh_d2(z).item() - math.sqrt(2 / math.pi)) < 1e-8


def test_layernorm_matches_library_routine():
    z = torch.randn(3, 5, 64, dtype=F64, generator=torch.Generator().manual_seed(1)) * 3 + 1
    xh, sd = orc.ln_fwd(z)
    ref = torch.nn.functional.layer_norm(z, (64,), eps=orc.LN_EPS)
    assert (xh - ref).abs().max() < 1e-12
    assert torch.allclose(sd.squeeze(-1), torch.sqrt(z.var(dim=-1, unbiased=False) + orc.LN_EPS), atol=1e-12)


def test_ln_bwd_and_fused_l2_grad_match_autograd():
    g = torch.Generator().manual_seed(2)
    z = torch.randn(4, 7, 16, dtype=F64, generator=g, requires_grad=True)
    tgt = torch.randn(4, 7, 16, dtype=F64, generator=g)
    gamma = 1 + 0.2 * torch.randn(16, dtype=F64, generator=g)
    beta = 0.3 * torch.randn(16, dtype=F64, generator=g)
    y = gamma * torch.nn.functional.layer_norm(z, (16,), eps=orc.LN_EPS) + beta
    ref, = torch.autograd.grad(0.5 * ((y - tgt) ** 2).sum(), z)
    got, xh, sd, g_out, g_xhat = orc.ln_l2_grad(z.detach(), tgt, gamma, beta)
    assert (got - ref).abs().max() < 1e-11
    assert torch.allclose(g_out, (y - tgt).detach(), atol=1e-12)
    assert torch.allclose(g_xhat, g_out * gamma, atol=1e-12)


# ---------------------------------------------------------------- forward scan
def test_weight_step_is_eta_weighted_gradient_step():
    d, _ = _small(NC=1)
    W = [d[k].clone().requires_grad_(True) for k in ("W1", "b1", "W2", "b2")]
    xk, xv, eta = d["XK"][:, :, 0], d["XV"][:, :, 0], d["last_eta"][:, :, 0]
    Z2 = torch.nn.functional.gelu(xk @ W[0] + W[1], approximate="tanh") @ W[2] + W[3]
    y = d["ttt_norm_weight"] * torch.nn.functional.layer_norm(Z2, Z2.shape[-1:], eps=orc.LN_EPS) + d["ttt_norm_bias"]
    loss_t = 0.5 * ((y - (xv - xk)) ** 2).sum(dim=-1, keepdim=True)      # per token
    grads = torch.autograd.grad((eta * loss_t).sum(), W)
    _, nxt, _ = orc.forward_step(orc.State(*[d[k] for k in ("W1", "b1", "W2", "b2")]), d["XQ"][:, :, 0], xk, xv,
                                 eta, d["ttt_norm_weight"], d["ttt_norm_bias"])
    for w, gw, n in zip(W, grads, nxt):
        assert (n - (w.detach() - gw)).abs().max() < 1e-9


def test_zero_eta_reduces_to_plain_mlp_layernorm_residual():
    d, _ = _small(NC=4)
    d["last_eta"] = torch.zeros_like(d["last_eta"])
    out, ck, fin = orc.ttt_forward(*[d[k] for k in FWD_KEYS], 2, dtype=F64)
    g = lambda z: torch.nn.functional.gelu(z, approximate="tanh")
    Z2 = g(d["XQ"] @ d["W1"].unsqueeze(2) + d["b1"].unsqueeze(2)) @ d["W2"].unsqueeze(2) + d["b2"].unsqueeze(2)
    ref = d["XQ"] + d["ttt_norm_weight"].unsqueeze(2) * torch.nn.functional.layer_norm(Z2, Z2.shape[-1:], eps=orc.LN_EPS) \
        + d["ttt_norm_bias"].unsqueeze(2)
    assert (out - ref).abs().max() < 1e-7      # truncated sqrt(2/pi) in the oracle
    for a, b in zip(fin, (d["W1"], d["b1"], d["W2"], d["b2"])):
        assert torch.equal(a, b)


@pytest.mark.parametrize("NC,cgs", [(6, 1), (6, 2), (6, 4), (5, 8), (1, 1)])
def test_checkpoints_are_states_before_each_group(NC, cgs):
    d, _ = _small(NC=NC)
    out, ck, fin = orc.ttt_forward(*[d[k] for k in FWD_KEYS], cgs, dtype=F64)
    K = math.ceil(NC / cgs)
    assert ck.W1.shape[2] == K and ck.b2.shape[2] == K
    # slot 0 is the initial state, bit for bit
    for t, k in zip(ck, ("W1", "b1", "W2", "b2")):
        assert torch.equal(t[:, :, 0], d[k])
    # restarting from slot k reproduces the tail of the scan
    for k in range(K):
        s = k * cgs
        sub = {key: (d[key][:, :, s:] if key in ("XQ", "XK", "XV", "last_eta") else d[key]) for key in FWD_KEYS}
        sub.update(W1=ck.W1[:, :, k], b1=ck.b1[:, :, k], W2=ck.W2[:, :, k], b2=ck.b2[:, :, k])
        out2, _, fin2 = orc.ttt_forward(*[sub[key] for key in FWD_KEYS], cgs, dtype=F64)
        assert (out2 - out[:, :, s:]).abs().max() < 1e-12
        assert (fin2.W1 - fin.W1).abs().max() < 1e-12


def test_forward_matches_differentiable_twin():
    d, _ = _small(NC=4)
    out, _, fin = orc.ttt_forward(*[d[k] for k in FWD_KEYS], 3, dtype=F64)
    out2, fin2 = orc.ttt_forward_differentiable(*[d[k] for k in FWD_KEYS])
    assert (out - out2).abs().max() < 1e-7
    for a, b in zip(fin, fin2):
        assert (a - b).abs().max() < 1e-7


# ------------------------------------------------------------------- backward
NAMES = {"XQ": "grad_L_XQ", "XK": "grad_L_XK", "XV": "grad_L_XV", "last_eta": "grad_L_last_eta",
         "W1": "grad_L_W1_init", "b1": "grad_L_b1_init", "W2": "grad_L_W2_init", "b2": "grad_L_b2_init"}


def _check_against_autograd(d, up, cgs, tol):
    ref, _ = _autograd_grads(d, up)
    got, *_ = _oracle_grads(d, up, cgs)
    for k, name in NAMES.items():
        scale = ref[k].abs().max().item() + 1e-30
        assert (got[name] - ref[k]).abs().max().item() / scale < tol, name
    # the operator reports norm grads per batch element; autograd gives their sum over B
    for k, name in (("ttt_norm_weight", "grad_L_ttt_norm_weight"), ("ttt_norm_bias", "grad_L_ttt_norm_bias")):
        summed = got[name].sum(dim=0, keepdim=True)
        scale = ref[k].abs().max().item() + 1e-30
        assert (summed - ref[k]).abs().max().item() / scale < tol, name


@pytest.mark.parametrize("B,NH,NC,cgs", [(1, 2, 3, 1), (2, 2, 5, 2), (2, 1, 4, 8), (1, 1, 1, 1)])
def test_all_ten_grads_match_autograd_fp64(B, NH, NC, cgs):
    d, up = _small(B=B, NH=NH, NC=NC, seed=3)
    # truncated derivative constants limit agreement to ~1e-7
    _check_against_autograd(d, up, cgs, 2e-6)


def test_all_ten_grads_match_autograd_at_kernel_tile_sizes():
    d, up = _small(B=1, NH=1, NC=2, CS=64, F=64, HID=256, seed=4)
    for k in ("W1", "W2"):
        d[k] = d[k] * (0.02 / 0.3)
    _check_against_autograd(d, up, 2, 2e-6)


def test_grads_do_not_depend_on_checkpoint_group_size():
    d, up = _small(B=1, NH=2, NC=7, seed=5)
    base, *_ = _oracle_grads(d, up, 1)
    for cgs in (2, 3, 7, 16):
        other, *_ = _oracle_grads(d, up, cgs)
        for k in base:
            assert (base[k] - other[k]).abs().max() < 1e-10, (k, cgs)


def test_grads_are_linear_in_upstream_grads_and_zero_for_zero():
    d, up = _small(B=1, NH=1, NC=3, seed=6)
    _, up2 = _small(B=1, NH=1, NC=3, seed=7)
    zero = {k: torch.zeros_like(v) for k, v in up.items()}
    g0, *_ = _oracle_grads(d, zero, 2)
    assert all(v.abs().max() == 0 for v in g0.values())
    g1, *_ = _oracle_grads(d, up, 2)
    g2, *_ = _oracle_grads(d, up2, 2)
    mix = {k: 2.0 * up[k] - 3.0 * up2[k] for k in up}
    gm, *_ = _oracle_grads(d, mix, 2)
    for k in g1:
        assert (gm[k] - (2.0 * g1[k] - 3.0 * g2[k])).abs().max() < 1e-9, k


def test_grads_match_central_finite_differences():
    d, up = _small(B=1, NH=1, NC=2, CS=4, F=4, HID=8, seed=8)
    got, *_ = _oracle_grads(d, up, 1)

    def scalar(dd):
        out, _, fin = orc.ttt_forward(*[dd[k] for k in FWD_KEYS], 1, dtype=F64)
        return ((out * up["gO"]).sum() + (fin.W1 * up["gW1"]).sum() + (fin.b1 * up["gb1"]).sum()
                + (fin.W2 * up["gW2"]).sum() + (fin.b2 * up["gb2"]).sum()).item()

    h = 1e-6
    gen = torch.Generator().manual_seed(9)
    for key, name in list(NAMES.items()) + [("ttt_norm_weight", "grad_L_ttt_norm_weight"),
                                            ("ttt_norm_bias", "grad_L_ttt_norm_bias")]:
        flat = d[key].flatten()
        for idx in torch.randperm(flat.numel(), generator=gen)[:4].tolist():
            dp = {k: v.clone() for k, v in d.items()}
            dm = {k: v.clone() for k, v in d.items()}
            dp[key].view(-1)[idx] += h
            dm[key].view(-1)[idx] -= h
            fd = (scalar(dp) - scalar(dm)) / (2 * h)
            an = got[name].sum(dim=0, keepdim=True).flatten()[idx].item() if "norm" in name \
                else got[name].flatten()[idx].item()
            assert abs(fd - an) < 1e-5 * max(1.0, abs(an)), (name, idx, fd, an)


def test_bf16_operand_variant_stays_close_to_fp32_oracle():
    d = orc.make_inputs(1, 2, 4, seed=0)
    a, cka, _ = orc.ttt_forward(*[d[k] for k in FWD_KEYS], 1)
    b, ckb, _ = orc.ttt_forward(*[d[k] for k in FWD_KEYS], 1, emulate_bf16_operands=True)
    st = orc.parity_stats(b, a)
    assert st["max_rel"] < 2e-2 and st["cosine"] > 0.9999
    assert orc.parity_stats(ckb.W1, cka.W1)["cosine"] > 0.9999


def test_operand_rounding_classes_separate_the_sources_of_error():
    """The rounding switches per operand class (weights / activations / activation gradients) that located what the
    kernels must carry in two bf16 terms: rounding nothing reproduces the oracle, rounding one class costs
    less than rounding all three, and every variant stays within the parity bar at this length."""
    d = orc.make_inputs(1, 2, 48, seed=3)
    ref, ck, _ = orc.ttt_forward(*[d[k] for k in FWD_KEYS], 8)
    up = orc.State(d["grad_L_W1_last"], d["grad_L_b1_last"], d["grad_L_W2_last"], d["grad_L_b2_last"])
    args = (d["XQ"], d["XK"], d["XV"], d["last_eta"], d["ttt_norm_weight"], d["ttt_norm_bias"])
    gref = orc.ttt_backward(*args, ck, up, d["grad_L_XQW_mini_batch"], 8)

    def err(rounding):
        out, c, _ = orc.ttt_forward(*[d[k] for k in FWD_KEYS], 8, emulate_bf16_operands=rounding)
        g = orc.ttt_backward(*args, c, up, d["grad_L_XQW_mini_batch"], 8, emulate_bf16_operands=rounding)
        worst = max(1 - orc.parity_stats(g[k], gref[k])["cosine"] for k in gref)
        return worst, out

    none, out = err(orc.OperandRounding(w=False, a=False, g=False))
    assert none < 1e-12 and torch.equal(out, ref)      # cosine of identical tensors, up to its own rounding
    all3, _ = err(orc.OperandRounding())
    assert 0 < all3 < 1e-4
    for kw in (dict(w=True, a=False, g=False), dict(w=False, a=True, g=False), dict(w=False, a=False, g=True)):
        one, _ = err(orc.OperandRounding(**kw))
        assert 0 < one < all3, kw


# ------------------------------------------------- per-group tensors (what the kernel leaves for group 0)
@pytest.mark.parametrize("NC,cgs,group", [(5, 2, 0), (5, 2, 2), (3, 4, 0), (4, 4, 0)])
def test_group_tensors_match_library_routines_and_autograd(NC, cgs, group):
    """Every slot of replay_group_tensors, rebuilt from PyTorch's own gelu / layer_norm / autograd and from the
    per-mini-batch states that ttt_forward's checkpoints give at checkpoint_group_size = 1."""
    Fn = torch.nn.functional
    d, _ = _small(NC=NC, seed=7)
    out, ck, fin = orc.ttt_forward(*[d[k] for k in FWD_KEYS], cgs, dtype=F64)
    _, ck1, _ = orc.ttt_forward(*[d[k] for k in FWD_KEYS], 1, dtype=F64)       # state before every mini-batch
    states = [orc.State(*[t[:, :, i] for t in ck1]) for i in range(NC)] + [fin]
    got = orc.replay_group_tensors(d["XQ"], d["XK"], d["XV"], d["last_eta"], d["ttt_norm_weight"], d["ttt_norm_bias"],
                                   ck, cgs, group, dtype=F64)
    gamma, beta = d["ttt_norm_weight"], d["ttt_norm_bias"]
    Fdim = d["XQ"].shape[-1]
    n = min(NC, (group + 1) * cgs) - group * cgs
    for slot in range(cgs):
        if slot >= n:
            for name, v in got.items():
                assert not v[:, :, slot].any(), name
            continue
        i = group * cgs + slot
        st, nxt = states[i], states[i + 1]
        xq, xk, xv = d["XQ"][:, :, i], d["XK"][:, :, i], d["XV"][:, :, i]
        for name, ref in zip(("W1_init_group", "b1_init_group", "W2_init_group", "b2_init_group"), st):
            assert torch.equal(got[name][:, :, slot], ref), name
        z1 = (xk @ st.W1 + st.b1).requires_grad_(True)
        x2 = Fn.gelu(z1, approximate="tanh")
        z2 = (x2 @ st.W2 + st.b2)
        z2_leaf = z2.detach().requires_grad_(True)
        xh_leaf = Fn.layer_norm(z2_leaf, (Fdim,), eps=orc.LN_EPS).detach().requires_grad_(True)
        loss_from_xh = 0.5 * ((gamma * xh_leaf + beta - (xv - xk)) ** 2).sum()
        g_xhat, = torch.autograd.grad(loss_from_xh, xh_leaf)
        loss_from_z2 = 0.5 * ((gamma * Fn.layer_norm(z2_leaf, (Fdim,), eps=orc.LN_EPS) + beta - (xv - xk)) ** 2).sum()
        g_z2, = torch.autograd.grad(loss_from_z2, z2_leaf)
        loss_from_z1 = 0.5 * ((gamma * Fn.layer_norm(z2, (Fdim,), eps=orc.LN_EPS) + beta - (xv - xk)) ** 2).sum()
        g_z1_total, = torch.autograd.grad(loss_from_z1, z1)
        z1b = xq @ nxt.W1 + nxt.b1
        x2b = Fn.gelu(z1b, approximate="tanh")
        z2b = x2b @ nxt.W2 + nxt.b2
        ref = dict(Z1_group=z1.detach(), X2_group=x2.detach(), grad_l_wrt_Z2_group=g_z2, grad_l_wrt_Z1_group=g_z1_total,
                   x_hat_fused_group=xh_leaf.detach(),
                   std_fused_group=torch.sqrt(z2.detach().var(dim=-1, unbiased=False, keepdim=True) + orc.LN_EPS),
                   grad_output_fused_group=(gamma * xh_leaf + beta - (xv - xk)).detach(), grad_x_hat_fused_group=g_xhat,
                   Z1_bar_group=z1b, X2_bar_group=x2b, x_hat_ln_group=Fn.layer_norm(z2b, (Fdim,), eps=orc.LN_EPS),
                   std_ln_group=torch.sqrt(z2b.var(dim=-1, unbiased=False, keepdim=True) + orc.LN_EPS))
        for name, r in ref.items():
            assert got[name][:, :, slot].shape == r.shape, name
            assert (got[name][:, :, slot] - r).abs().max() < 1e-8 * (1 + r.abs().max()), (name, slot)
        # and the output the forward returns is the residual on top of this slot's output LayerNorm
        assert (xq + gamma * got["x_hat_ln_group"][:, :, slot] + beta - out[:, :, i]).abs().max() < 1e-10
