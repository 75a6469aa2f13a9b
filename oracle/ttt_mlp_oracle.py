"""CPU oracle for the non-causal TTT-MLP forward scan and its remat backward.

THIS FILE IS TEST INFRASTRUCTURE.  It is a checker: only the test-suite, the
smoke check and the benchmark's ``cpu_baseline`` leg may import it.  The shipped
operator never calls anything in here and has no CPU fallback.

What it restates (reference file:line, all under the upstream repository):
  * one mini-batch step of the inner MLP, the LayerNorm-fused reconstruction
    loss gradient, the eta-scaled weight step, the post-update forward and the
    output LayerNorm + residual     -> kernels/ttt_backward/matching.py:57-171
                                       (forward-only twin kernels/ttt/matching.py:30-125)
  * tanh-GELU first / second derivative with the truncated constants
                                    -> kernels/ttt_backward/matching.py:42-55,
                                       include/common/base_ops.cuh:465-548
  * the checkpointing rule "store the state *before* mini-batch i when
    i % cgs == 0 at slot i // cgs"  -> kernels/ttt/matching.py:217-228,
                                       kernels/ttt/ttt.cu:277-294
  * the hand-derived backward of one step
                                    -> kernels/ttt_backward/matching.py:173-342
  * the group replay / reverse walk that drives it (which state is "init",
    which is "last", ragged last group)
                                    -> kernels/ttt_backward/matching.py:539-663,
                                       kernels/ttt_backward/ttt.cu:453-485,824-828

How each function is pinned (none of it by retyping its own formula):
  gelu_tanh            torch.nn.functional.gelu(approximate="tanh")   (library routine)
  gelu_tanh_d1/_d2     first / second torch.autograd derivative of that routine in fp64
  ln_fwd               torch.nn.functional.layer_norm without affine (eps inside the sqrt)
  ln_l2_grad           autograd of 0.5*||gamma*LN(z)+beta-target||^2 wrt z
  forward_step         autograd of sum_t eta_t * loss_t wrt (W1,b1,W2,b2) gives the step;
                       eta = 0 collapses to Out = XQ + LN(MLP(XQ))
  ttt_forward          checkpoint invariants + composition of the above
  replay_group_tensors the values it copies out of forward_step are the ones backward_step consumes
                       (pinned by the gradients below); slot 0 of the state tensors = the checkpoint,
                       slot i+1 = slot i after the step; x_hat rows have mean 0 / variance 1,
                       X2 = gelu(Z1); grad_l_wrt_Z2 = autograd of the loss at that slot's Z2
  backward_step /      torch.autograd straight through ``ttt_forward_differentiable`` in
  ttt_backward         fp64 (all ten gradients), invariance to checkpoint_group_size,
                       linearity in the upstream grads, finite differences at NC = 2
The upstream repository stores no golden vectors for this path, so every pin
above comes from mathematics or from PyTorch's own routines; the fixtures in
tests/golden/ were written by this file after those pins passed.

Shapes follow the operator: XQ/XK/XV [B,NH,NC,CS,F], last_eta [B,NH,NC,CS,1],
ttt_norm_weight/bias [1,NH,1,F], W1 [B,NH,F,H], b1 [B,NH,1,H], W2 [B,NH,H,F],
b2 [B,NH,1,F] with CS = F = 64 and H = 4F in the shipped kernels (the oracle
itself accepts any sizes).
"""
from __future__ import annotations

import math
from typing import Dict, NamedTuple, Optional, Tuple

import torch

# Truncated constants used by the upstream derivative formulas
# (kernels/ttt_backward/matching.py:42-55).
K0 = 0.79788456          # ~ sqrt(2/pi)
K1 = 0.044715
K2 = 0.1070322243        # 3 * K0 * K1
LN_EPS = 1e-8            # kernels/ttt_backward/matching.py:102


# --------------------------------------------------------------------------- GELU
def _tanh_arg(x):
    return K0 * x * (1.0 + K1 * x * x)


def gelu_tanh(x: torch.Tensor) -> torch.Tensor:
    """tanh-approximated GELU, 0.5*x*(1+tanh(c(x)))."""
    return 0.5 * x * (1.0 + torch.tanh(_tanh_arg(x)))


def gelu_tanh_d1(x: torch.Tensor) -> torch.Tensor:
    """d/dx gelu_tanh (kernels/ttt_backward/matching.py:42-45)."""
    t = torch.tanh(_tanh_arg(x))
    return 0.5 * x * (1.0 - t * t) * (K0 + K2 * x * x) + 0.5 * (1.0 + t)


def gelu_tanh_d2(x: torch.Tensor) -> torch.Tensor:
    """d2/dx2 gelu_tanh (kernels/ttt_backward/matching.py:47-55)."""
    t = torch.tanh(_tanh_arg(x))
    x2 = x * x
    inner = K0 + 3.0 * K0 * K1 * x2
    return (1.0 - t * t) * (K0 + 6.0 * K0 * K1 * x2 - x * t * inner * inner)


# --------------------------------------------------------------------- LayerNorm
def ln_fwd(z: torch.Tensor, eps: float = LN_EPS) -> Tuple[torch.Tensor, torch.Tensor]:
    """Row LayerNorm statistics: returns (x_hat, std) with biased variance."""
    mu = z.mean(dim=-1, keepdim=True)
    d = z - mu
    std = torch.sqrt((d * d).mean(dim=-1, keepdim=True) + eps)
    return d / std, std


def ln_bwd(g_xhat: torch.Tensor, x_hat: torch.Tensor, std: torch.Tensor) -> torch.Tensor:
    """Gradient wrt the LayerNorm input given the gradient wrt x_hat."""
    n = x_hat.shape[-1]
    s1 = g_xhat.sum(dim=-1, keepdim=True)
    s2 = (g_xhat * x_hat).sum(dim=-1, keepdim=True)
    return (n * g_xhat - s1 - x_hat * s2) / (n * std)


def ln_l2_grad(z, target, gamma, beta, eps: float = LN_EPS):
    """d/dz of 0.5*||gamma*LN(z)+beta-target||^2 and the pieces the backward re-uses."""
    x_hat, std = ln_fwd(z, eps)
    g_out = gamma * x_hat + beta - target
    g_xhat = g_out * gamma
    return ln_bwd(g_xhat, x_hat, std), x_hat, std, g_out, g_xhat


# ------------------------------------------------------------ operand rounding
def _ident(x):
    return x


def _rb(x):
    """Round to bf16 and back (models a bf16 MFMA operand with fp32 accumulate)."""
    return x.to(torch.bfloat16).to(x.dtype)


class OperandRounding:
    """Which matrix-product operands are rounded to bf16: ``w`` weights and weight gradients,
    ``a`` activations, ``g`` activation gradients.  Used to study where the operand precision matters."""

    def __init__(self, w=True, a=True, g=True):
        self.w = _rb if w else _ident
        self.a = _rb if a else _ident
        self.g = _rb if g else _ident


def _cat(rnd):
    if isinstance(rnd, OperandRounding):
        return rnd.w, rnd.a, rnd.g
    return rnd, rnd, rnd


class State(NamedTuple):
    W1: torch.Tensor
    b1: torch.Tensor
    W2: torch.Tensor
    b2: torch.Tensor


# ------------------------------------------------------------------ one step
def forward_step(state: State, xq, xk, xv, eta, gamma, beta, *, rnd=_ident,
                 gelu=gelu_tanh) -> Tuple[torch.Tensor, State, Dict[str, torch.Tensor]]:
    """One mini-batch of the scan.

    eta is the per-token step size [.., CS, 1]; gamma/beta broadcast over tokens.
    ``rnd`` is applied to every matrix-product operand (identity for the oracle
    proper, bf16 rounding for the operand-emulating variant).
    """
    W1, b1, W2, b2 = state
    T = lambda a: a.transpose(-1, -2)
    rw, ra, rg = _cat(rnd)
    Z1 = ra(xk) @ rw(W1) + b1
    X2 = gelu(Z1)
    Z2 = ra(X2) @ rw(W2) + b2
    gZ2, xhat_f, std_f, g_out, g_xhat = ln_l2_grad(Z2, xv - xk, gamma, beta)
    gZ1 = (rg(gZ2) @ T(rw(W2))) * gelu_tanh_d1(Z1)
    W1n = W1 - T(ra(xk)) @ rg(eta * gZ1)
    b1n = b1 - (eta * gZ1).sum(dim=-2, keepdim=True)
    W2n = W2 - T(ra(X2)) @ rg(eta * gZ2)
    b2n = b2 - (eta * gZ2).sum(dim=-2, keepdim=True)
    Z1b = ra(xq) @ rw(W1n) + b1n
    X2b = gelu(Z1b)
    Z2b = ra(X2b) @ rw(W2n) + b2n
    xhat_l, std_l = ln_fwd(Z2b)
    out = xq + gamma * xhat_l + beta
    saved = dict(Z1=Z1, X2=X2, xhat_f=xhat_f, std_f=std_f, g_out=g_out, g_xhat=g_xhat,
                 gZ2=gZ2, gZ1=gZ1, Z1b=Z1b, X2b=X2b, xhat_l=xhat_l, std_l=std_l)
    return out, State(W1n, b1n, W2n, b2n), saved


def _norm_params(ttt_norm_weight, ttt_norm_bias, dtype):
    # [1,NH,1,F] broadcasts against [B,NH,CS,F] as is.
    return ttt_norm_weight.to(dtype), ttt_norm_bias.to(dtype)


def _eta5(last_eta):
    return last_eta if last_eta.dim() == 5 else last_eta.unsqueeze(-1)


# -------------------------------------------------------------------- forward
def ttt_forward(XQ, XK, XV, last_eta, ttt_norm_weight, ttt_norm_bias, W1, b1, W2, b2,
                checkpoint_group_size: int, *, dtype=torch.float32, emulate_bf16_operands=False,
                gelu=gelu_tanh):
    """Forward scan.  Returns (Out [B,NH,NC,CS,F], checkpoints State of [B,NH,K,..], final State)."""
    rnd = emulate_bf16_operands if isinstance(emulate_bf16_operands, OperandRounding) else \
        (_rb if emulate_bf16_operands else _ident)
    XQ, XK, XV = XQ.to(dtype), XK.to(dtype), XV.to(dtype)
    eta = _eta5(last_eta).to(dtype)
    gamma, beta = _norm_params(ttt_norm_weight, ttt_norm_bias, dtype)
    st = State(W1.to(dtype), b1.to(dtype), W2.to(dtype), b2.to(dtype))
    NC = XQ.shape[2]
    cgs = int(checkpoint_group_size)
    ck = [[], [], [], []]
    outs = []
    for i in range(NC):
        if i % cgs == 0:
            for lst, t in zip(ck, st):
                lst.append(t)
        o, st, _ = forward_step(st, XQ[:, :, i], XK[:, :, i], XV[:, :, i], eta[:, :, i], gamma, beta,
                                rnd=rnd, gelu=gelu)
        outs.append(o)
    out = torch.stack(outs, dim=2)
    ckpt = State(*[torch.stack(l, dim=2) for l in ck])
    return out, ckpt, st


def ttt_forward_differentiable(XQ, XK, XV, last_eta, ttt_norm_weight, ttt_norm_bias, W1, b1, W2, b2):
    """The same scan with no checkpoint bookkeeping, for torch.autograd cross-checks.

    Uses torch's own tanh-GELU so that autograd differentiates the library routine.
    """
    if not W1.requires_grad:           # the inner gradient is taken with autograd even when
        W1 = W1.detach().requires_grad_(True)    # the caller wants values only
    st = State(W1, b1, W2, b2)
    eta = _eta5(last_eta)
    outs = []
    g = lambda z: torch.nn.functional.gelu(z, approximate="tanh")
    for i in range(XQ.shape[2]):
        W1_, b1_, W2_, b2_ = st
        xq, xk, xv, e = XQ[:, :, i], XK[:, :, i], XV[:, :, i], eta[:, :, i]
        Z1 = xk @ W1_ + b1_
        X2 = g(Z1)
        Z2 = X2 @ W2_ + b2_
        x_hat = torch.nn.functional.layer_norm(Z2, Z2.shape[-1:], eps=LN_EPS)
        resid = ttt_norm_weight * x_hat + ttt_norm_bias - (xv - xk)
        # The inner-loop gradient is itself differentiated, hence create_graph.
        loss = 0.5 * (resid * resid).sum()
        gZ2, = torch.autograd.grad(loss, Z2, create_graph=True)
        gZ1 = (gZ2 @ W2_.transpose(-1, -2)) * torch.autograd.grad(X2.sum(), Z1, create_graph=True)[0]
        W1n = W1_ - (e * xk).transpose(-1, -2) @ gZ1
        b1n = b1_ - (e * gZ1).sum(dim=-2, keepdim=True)
        W2n = W2_ - (e * X2).transpose(-1, -2) @ gZ2
        b2n = b2_ - (e * gZ2).sum(dim=-2, keepdim=True)
        Z2b = g(xq @ W1n + b1n) @ W2n + b2n
        outs.append(xq + ttt_norm_weight * torch.nn.functional.layer_norm(Z2b, Z2b.shape[-1:], eps=LN_EPS)
                    + ttt_norm_bias)
        st = State(W1n, b1n, W2n, b2n)
    return torch.stack(outs, dim=2), st


# ------------------------------------------------------------------- backward
def backward_step(gO, g: State, init: State, last: State, s: Dict[str, torch.Tensor], xq, xk, eta,
                  gamma, *, rnd=_ident):
    """Reverse of ``forward_step``.

    gO   upstream gradient on Out for this mini-batch
    g    gradient wrt the state *after* this mini-batch (running)
    init state before the step, last state after it
    Returns (dXQ, dXK, dXV, d_eta), gradient wrt the state before the step, (d_gamma, d_beta)
    where the norm gradients are per (batch, head): [B,NH,1,F].
    """
    T = lambda a: a.transpose(-1, -2)
    gW1, gb1, gW2, gb2 = g
    n = xq.shape[-1]
    sF = lambda a: a.sum(dim=-1, keepdim=True)     # over features
    sT = lambda a: a.sum(dim=-2, keepdim=True)     # over tokens

    # output LayerNorm + residual
    d_beta = sT(gO)
    d_gamma = sT(gO * s["xhat_l"])
    rw, ra, rg = _cat(rnd)
    gZ2b = ln_bwd(gO * gamma, s["xhat_l"], s["std_l"])
    # post-update forward
    gZ1b = (rg(gZ2b) @ T(rw(last.W2))) * gelu_tanh_d1(s["Z1b"])
    gb2 = gb2 + sT(gZ2b)
    gW2 = gW2 + T(ra(s["X2b"])) @ rg(gZ2b)
    gb1 = gb1 + sT(gZ1b)
    gW1 = gW1 + T(ra(xq)) @ rg(gZ1b)
    dXQ = gO + rg(gZ1b) @ T(rw(last.W1))
    # the weight step: W_next = W - (eta x)^T g
    d1 = gelu_tanh_d1(s["Z1"])
    ggZ1 = -(ra(eta * xk) @ rw(gW1)) - eta * gb1
    u = ggZ1 * d1
    ggZ2 = -(ra(eta * s["X2"]) @ rw(gW2)) - eta * gb2 + rg(u) @ rw(init.W2)
    P1 = rg(s["gZ1"]) @ T(rw(gW1))
    P2 = rg(s["gZ2"]) @ T(rw(gW2))
    d_eta = -sF(P2 * s["X2"]) - sF(gb2 * s["gZ2"]) - sF(P1 * xk) - sF(gb1 * s["gZ1"])
    gW2_via_gZ1 = T(rg(u)) @ rg(s["gZ2"])
    # second-order pass through the LayerNorm-fused loss gradient
    xh, sd = s["xhat_f"], s["std_f"]
    a = sF(ggZ2 * xh)
    bb = sF(s["g_xhat"] * xh)
    gg_xhat = (ggZ2 - (sF(ggZ2) + xh * a) / n) / sd
    g_y = gamma * gg_xhat
    d_gamma = d_gamma + sT(s["g_out"] * gg_xhat + g_y * xh)
    d_beta = d_beta + sT(g_y)
    gx = g_y * gamma - (s["g_xhat"] * a + ggZ2 * bb) / (n * sd)
    g_std = (-gx * xh - ggZ2 * s["gZ2"]) / sd
    dZ2 = gx / sd + (sF(g_std) * xh - sF(gx) / sd) / n
    # inner MLP
    R = rg(s["gZ2"]) @ T(rw(init.W2))              # = gZ1 before the GELU' factor
    dX2 = rg(dZ2) @ T(rw(init.W2)) - eta * P2
    dZ1 = dX2 * d1 + R * ggZ1 * gelu_tanh_d2(s["Z1"])
    dXK = g_y - eta * P1 + rg(dZ1) @ T(rw(init.W1))
    dXV = -g_y
    gW2 = gW2 + gW2_via_gZ1 + T(ra(s["X2"])) @ rg(dZ2)
    gb2 = gb2 + sT(dZ2)
    gW1 = gW1 + T(ra(xk)) @ rg(dZ1)
    gb1 = gb1 + sT(dZ1)
    return (dXQ, dXK, dXV, d_eta), State(gW1, gb1, gW2, gb2), (d_gamma, d_beta)


def ttt_backward(XQ, XK, XV, last_eta, ttt_norm_weight, ttt_norm_bias, ckpt: State,
                 grad_last: State, grad_out, checkpoint_group_size: int, *, dtype=torch.float32,
                 emulate_bf16_operands=False):
    """Remat backward: per checkpoint group (last to first) replay forward, then walk back.

    ckpt       State of [B,NH,K,..] checkpoints as written by ``ttt_forward``
    grad_last  gradient wrt the state after the last mini-batch
    grad_out   gradient wrt Out, [B,NH,NC,CS,F]
    Returns a dict with the operator's ten output gradients (norm grads per batch element,
    [B,NH,1,F]) in ``dtype``.
    """
    rnd = emulate_bf16_operands if isinstance(emulate_bf16_operands, OperandRounding) else \
        (_rb if emulate_bf16_operands else _ident)
    XQ, XK, XV, gO = XQ.to(dtype), XK.to(dtype), XV.to(dtype), grad_out.to(dtype)
    eta = _eta5(last_eta).to(dtype)
    gamma, beta = _norm_params(ttt_norm_weight, ttt_norm_bias, dtype)
    B, NH, NC, CS, F = XQ.shape
    cgs = int(checkpoint_group_size)
    K = ckpt.W1.shape[2]
    assert K == math.ceil(NC / cgs), "checkpoint count does not match NC and checkpoint_group_size"
    g = State(*[t.to(dtype) for t in grad_last])
    d_gamma = torch.zeros(B, NH, 1, F, dtype=dtype)
    d_beta = torch.zeros(B, NH, 1, F, dtype=dtype)
    dXQ, dXK, dXV = torch.zeros_like(XQ), torch.zeros_like(XQ), torch.zeros_like(XQ)
    dEta = torch.zeros_like(eta)
    for k in range(K - 1, -1, -1):
        st = State(*[t[:, :, k].to(dtype) for t in ckpt])
        inits, saves = [], []
        idx = [i for i in range(k * cgs, min(NC, (k + 1) * cgs))]
        for i in idx:
            inits.append(st)
            _, st, sv = forward_step(st, XQ[:, :, i], XK[:, :, i], XV[:, :, i], eta[:, :, i], gamma, beta,
                                     rnd=rnd)
            saves.append(sv)
        last = st
        for j in range(len(idx) - 1, -1, -1):
            i = idx[j]
            (dq, dk, dv, de), g, (dg, db) = backward_step(gO[:, :, i], g, inits[j], last, saves[j],
                                                          XQ[:, :, i], XK[:, :, i], eta[:, :, i], gamma,
                                                          rnd=rnd)
            dXQ[:, :, i], dXK[:, :, i], dXV[:, :, i], dEta[:, :, i] = dq, dk, dv, de
            d_gamma += dg
            d_beta += db
            last = inits[j]
    return dict(grad_L_ttt_norm_weight=d_gamma, grad_L_ttt_norm_bias=d_beta,
                grad_L_W1_init=g.W1, grad_L_b1_init=g.b1, grad_L_W2_init=g.W2, grad_L_b2_init=g.b2,
                grad_L_last_eta=dEta, grad_L_XQ=dXQ, grad_L_XK=dXK, grad_L_XV=dXV)


# ------------------------------------------------- per-group tensors of one checkpoint group
GROUP_TENSOR_FROM_SAVED = dict(
    Z1_group="Z1", X2_group="X2", Z1_bar_group="Z1b", X2_bar_group="X2b",
    grad_l_wrt_Z2_group="gZ2", grad_l_wrt_Z1_group="gZ1",
    x_hat_fused_group="xhat_f", std_fused_group="std_f", grad_output_fused_group="g_out",
    grad_x_hat_fused_group="g_xhat", x_hat_ln_group="xhat_l", std_ln_group="std_l")


def replay_group_tensors(XQ, XK, XV, last_eta, ttt_norm_weight, ttt_norm_bias, ckpt: State,
                         checkpoint_group_size: int, group: int = 0, *, dtype=torch.float32):
    """The sixteen ``*_group`` tensors of ``ttt_backward`` as the upstream harness fills its reference copies
    for one checkpoint group (kernels/ttt_backward/matching.py:552-590; after the call the kernel's tensors
    hold group 0, compared at :667-690): slot i = state before mini-batch i of the group and the
    intermediates of its step.  Slots past the end of the sequence stay zero.  Shapes [B,NH,cgs,..]."""
    XQ, XK, XV = XQ.to(dtype), XK.to(dtype), XV.to(dtype)
    eta = _eta5(last_eta).to(dtype)
    gamma, beta = _norm_params(ttt_norm_weight, ttt_norm_bias, dtype)
    B, NH, NC, CS, F = XQ.shape
    cgs = int(checkpoint_group_size)
    st = State(*[t[:, :, group].to(dtype) for t in ckpt])
    H = st.W1.shape[-1]
    out = dict(W1_init_group=torch.zeros(B, NH, cgs, F, H, dtype=dtype), b1_init_group=torch.zeros(B, NH, cgs, 1, H, dtype=dtype),
               W2_init_group=torch.zeros(B, NH, cgs, H, F, dtype=dtype), b2_init_group=torch.zeros(B, NH, cgs, 1, F, dtype=dtype))
    for name, key in GROUP_TENSOR_FROM_SAVED.items():
        last = 1 if key.startswith("std") else (F if key in ("gZ2", "xhat_f", "g_out", "g_xhat", "xhat_l") else H)
        out[name] = torch.zeros(B, NH, cgs, CS, last, dtype=dtype)
    for slot, i in enumerate(range(group * cgs, min(NC, (group + 1) * cgs))):
        for name, t in zip(("W1_init_group", "b1_init_group", "W2_init_group", "b2_init_group"), st):
            out[name][:, :, slot] = t
        _, st, sv = forward_step(st, XQ[:, :, i], XK[:, :, i], XV[:, :, i], eta[:, :, i], gamma, beta)
        for name, key in GROUP_TENSOR_FROM_SAVED.items():
            out[name][:, :, slot] = sv[key]
    return out


# ----------------------------------------------------------- synthetic workloads
def make_inputs(B: int, NH: int, NC: int, *, CS: int = 64, F: int = 64, HID: int = 256, seed: int = 0,
                eta_logit_std: float = 1.0, with_grads: bool = True,
                generator: Optional[torch.Generator] = None) -> Dict[str, torch.Tensor]:
    """Seeded synthetic inputs in the operator's dtypes (bf16 activations, fp32 state).

    Distributions: XQ/XK/XV ~ N(0,1); W1/W2 ~ N(0,0.02); b1/b2 = 0; norm weight 1, bias 0;
    last_eta = sigmoid(N(0, eta_logit_std)) / CS; grad_L_XQW ~ N(0,1);
    grad_L_{W1,b1,W2,b2}_last ~ N(0,1e-3).
    """
    gen = generator or torch.Generator().manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float32)
    d = {}
    for name in ("XQ", "XK", "XV"):
        d[name] = rn(B, NH, NC, CS, F).to(torch.bfloat16)
    d["W1"] = rn(B, NH, F, HID) * 0.02
    d["W2"] = rn(B, NH, HID, F) * 0.02
    d["b1"] = torch.zeros(B, NH, 1, HID)
    d["b2"] = torch.zeros(B, NH, 1, F)
    d["ttt_norm_weight"] = torch.ones(1, NH, 1, F)
    d["ttt_norm_bias"] = torch.zeros(1, NH, 1, F)
    d["last_eta"] = (torch.sigmoid(rn(B, NH, NC, CS, 1) * eta_logit_std) / CS).to(torch.bfloat16)
    if with_grads:
        d["grad_L_XQW_mini_batch"] = rn(B, NH, NC, CS, F).to(torch.bfloat16)
        d["grad_L_W1_last"] = rn(B, NH, F, HID) * 1e-3
        d["grad_L_b1_last"] = rn(B, NH, 1, HID) * 1e-3
        d["grad_L_W2_last"] = rn(B, NH, HID, F) * 1e-3
        d["grad_L_b2_last"] = rn(B, NH, 1, F) * 1e-3
    return d


# ---------------------------------------------------------------- parity metric
def parity_stats(hw: torch.Tensor, ref: torch.Tensor) -> Dict[str, float]:
    """max-abs error normalised by max-abs(ref), cosine, plus the four statistics the
    upstream harness prints (kernels/ttt_backward/matching.py:14-24)."""
    hw = hw.detach().to(torch.float64).flatten()
    ref = ref.detach().to(torch.float64).flatten()
    diff = (hw - ref).abs()
    denom = ref.abs().max().item()
    nz = ref != 0
    rel = diff[nz] / ref[nz].abs() if nz.any() else torch.tensor([float("inf")])
    cos = torch.dot(hw, ref).item() / max(hw.norm().item() * ref.norm().item(), 1e-300)
    return dict(max_rel=diff.max().item() / max(denom, 1e-300), cosine=cos,
                max_abs=diff.max().item(), median_abs=diff.median().item(),
                max_elem_rel=rel.max().item(), median_elem_rel=rel.median().item())
