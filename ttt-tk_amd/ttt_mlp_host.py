"""Host-side helpers around the `test_time_training` operator module: the caller-owned buffers the
two operators expect (checkpoints, the sixteen remat scratch tensors, zero-filled accumulating
outputs) and thin call wrappers that pass everything in the operator's positional order.

The operator itself allocates nothing (upstream README.md:22-98); this file is the allocator a
caller would otherwise write by hand (upstream kernels/ttt_backward/matching.py:393-436).
It never falls back to a CPU path: importing the module fails if the extension has not been built.
"""
from __future__ import annotations

import math
import os
import sys
from typing import Dict

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
if _HERE not in sys.path:
    sys.path.insert(0, _HERE)

import test_time_training as _ext  # noqa: E402  (hard requirement: no fallback)

CS, F, HID = 64, 64, 256

FWD_ORDER = ("XQ", "XK", "XV", "last_eta", "ttt_norm_weight", "ttt_norm_bias", "W1", "b1", "W2", "b2",
             "W1_checkpoints", "b1_checkpoints", "W2_checkpoints", "b2_checkpoints", "Out")

BWD_ORDER = ("XQ", "XK", "XV", "last_eta", "ttt_norm_weight", "ttt_norm_bias",
             "W1_checkpoints", "b1_checkpoints", "W2_checkpoints", "b2_checkpoints", "Out",
             "W1_init_group", "b1_init_group", "W2_init_group", "b2_init_group",
             "x_hat_ln_group", "std_ln_group", "X2_group", "Z1_group", "Z1_bar_group", "X2_bar_group",
             "grad_l_wrt_Z2_group", "grad_l_wrt_Z1_group", "x_hat_fused_group", "grad_x_hat_fused_group",
             "grad_output_fused_group", "std_fused_group",
             "grad_L_W1_last", "grad_L_b1_last", "grad_L_W2_last", "grad_L_b2_last", "grad_L_XQW_mini_batch",
             "grad_L_ttt_norm_weight", "grad_L_ttt_norm_bias",
             "grad_L_W1_init", "grad_L_b1_init", "grad_L_W2_init", "grad_L_b2_init",
             "grad_L_last_eta", "grad_L_XQ", "grad_L_XK", "grad_L_XV")

GRAD_NAMES = BWD_ORDER[32:]


def num_checkpoints(NC: int, cgs: int) -> int:
    return math.ceil(NC / cgs)


def alloc_forward_buffers(B: int, NH: int, NC: int, cgs: int, device) -> Dict[str, torch.Tensor]:
    """Checkpoints [B,NH,K,...] fp32 and Out [B,NH,NC,CS,F] bf16 (uninitialised)."""
    K = num_checkpoints(NC, cgs)
    f32 = dict(dtype=torch.float32, device=device)
    return dict(W1_checkpoints=torch.empty(B, NH, K, F, HID, **f32), b1_checkpoints=torch.empty(B, NH, K, 1, HID, **f32),
                W2_checkpoints=torch.empty(B, NH, K, HID, F, **f32), b2_checkpoints=torch.empty(B, NH, K, 1, F, **f32),
                Out=torch.empty(B, NH, NC, CS, F, dtype=torch.bfloat16, device=device))


def alloc_backward_buffers(B: int, NH: int, NC: int, cgs: int, device, zero_fill: bool = True) -> Dict[str, torch.Tensor]:
    """The sixteen remat scratch tensors, and the ten output gradients.  The four that `ttt_backward` adds to are
    zero-filled unless ``zero_fill`` is False (for the operator's overwrite policy, `set_accumulate(False)`)."""
    acc = torch.zeros if zero_fill else torch.empty
    f32 = dict(dtype=torch.float32, device=device)
    bf = dict(dtype=torch.bfloat16, device=device)
    G = cgs
    d = dict(
        W1_init_group=torch.empty(B, NH, G, F, HID, **f32), b1_init_group=torch.empty(B, NH, G, 1, HID, **f32),
        W2_init_group=torch.empty(B, NH, G, HID, F, **f32), b2_init_group=torch.empty(B, NH, G, 1, F, **f32),
        x_hat_ln_group=torch.empty(B, NH, G, CS, F, **bf), std_ln_group=torch.empty(B, NH, G, CS, 1, **f32),
        X2_group=torch.empty(B, NH, G, CS, HID, **bf), Z1_group=torch.empty(B, NH, G, CS, HID, **bf),
        Z1_bar_group=torch.empty(B, NH, G, CS, HID, **bf), X2_bar_group=torch.empty(B, NH, G, CS, HID, **bf),
        grad_l_wrt_Z2_group=torch.empty(B, NH, G, CS, F, **bf), grad_l_wrt_Z1_group=torch.empty(B, NH, G, CS, HID, **bf),
        x_hat_fused_group=torch.empty(B, NH, G, CS, F, **bf), grad_x_hat_fused_group=torch.empty(B, NH, G, CS, F, **bf),
        grad_output_fused_group=torch.empty(B, NH, G, CS, F, **bf), std_fused_group=torch.empty(B, NH, G, CS, 1, **f32),
        grad_L_ttt_norm_weight=torch.empty(B, NH, 1, F, **f32), grad_L_ttt_norm_bias=torch.empty(B, NH, 1, F, **f32),
        grad_L_W1_init=torch.empty(B, NH, F, HID, **f32), grad_L_b1_init=torch.empty(B, NH, 1, HID, **f32),
        grad_L_W2_init=torch.empty(B, NH, HID, F, **f32), grad_L_b2_init=torch.empty(B, NH, 1, F, **f32),
        grad_L_last_eta=acc(B, NH, NC, CS, 1, **bf), grad_L_XQ=acc(B, NH, NC, CS, F, **bf),
        grad_L_XK=acc(B, NH, NC, CS, F, **bf), grad_L_XV=acc(B, NH, NC, CS, F, **bf))
    return d


def zero_accumulating_grads(t: Dict[str, torch.Tensor]) -> None:
    for k in ("grad_L_last_eta", "grad_L_XQ", "grad_L_XK", "grad_L_XV"):
        t[k].zero_()


def forward(t: Dict[str, torch.Tensor], cgs: int) -> torch.Tensor:
    return _ext.ttt_forward(*[t[k] for k in FWD_ORDER], int(cgs))


def backward(t: Dict[str, torch.Tensor], cgs: int) -> torch.Tensor:
    return _ext.ttt_backward(*[t[k] for k in BWD_ORDER], int(cgs))


def set_synchronize(on: bool) -> None:
    _ext.set_synchronize(bool(on))


GROUP_TENSORS = ("W1_init_group", "b1_init_group", "W2_init_group", "b2_init_group", "x_hat_ln_group", "std_ln_group",
                 "X2_group", "Z1_group", "Z1_bar_group", "X2_bar_group", "grad_l_wrt_Z2_group", "grad_l_wrt_Z1_group",
                 "x_hat_fused_group", "grad_x_hat_fused_group", "grad_output_fused_group", "std_fused_group")


def set_accumulate(on: bool) -> None:
    """True (default, upstream behaviour, kernels/ttt_backward/matching.py:406-415): `ttt_backward` adds to
    grad_L_last_eta / grad_L_XQ / grad_L_XK / grad_L_XV and the caller zero-fills them.  False: it overwrites
    them; `ttt_mlp` / `ttt_mlp_backward` then allocate them without the fill."""
    _ext.set_accumulate(bool(on))


def set_fill_group_tensors(on: bool) -> None:
    """After ``ttt_backward`` leave the values of checkpoint group 0 in the sixteen ``*_group`` tensors, as the
    upstream kernel does (its harness compares them, kernels/ttt_backward/matching.py:667-690).  Off by default:
    the kernels use those tensors as workspace in their own formats, filling them costs one more kernel."""
    _ext.set_fill_group_tensors(bool(on))


class TTTMLPFunction(torch.autograd.Function):
    """`Out = ttt_mlp(XQ, XK, XV, last_eta, ttt_norm_weight, ttt_norm_bias, W1, b1, W2, b2)` with the
    remat backward, as the usage block of the upstream README (README.md:22-96) and its test harness
    (kernels/ttt_backward/matching.py:393-436, 522-523) call the two operators:
      forward  allocates the checkpoints and Out and calls `ttt_forward`; only the inputs and the
               checkpoints are kept for the backward (that is the point of the remat scheme);
      backward allocates the sixteen scratch tensors and the zero-filled accumulating outputs, calls
               `ttt_backward`, and sums the per-batch-element norm gradients over B.
    The state after the last mini-batch is not an output of `ttt_forward`, so its upstream gradient is
    zero here; `ttt_mlp_backward` below takes it explicitly.
    Shapes / dtypes are the operator's: XQ, XK, XV [B,NH,NC,64,64] bf16, last_eta [B,NH,NC,64,1] bf16,
    norm weight / bias [1,NH,1,64] fp32, W1 [B,NH,64,256], b1 [B,NH,1,256], W2 [B,NH,256,64],
    b2 [B,NH,1,64] fp32; everything contiguous and on the GPU."""

    @staticmethod
    def forward(ctx, XQ, XK, XV, last_eta, ttt_norm_weight, ttt_norm_bias, W1, b1, W2, b2, checkpoint_group_size):
        cgs = int(checkpoint_group_size)
        B, NH, NC = XQ.shape[:3]
        t = dict(XQ=XQ, XK=XK, XV=XV, last_eta=last_eta, ttt_norm_weight=ttt_norm_weight, ttt_norm_bias=ttt_norm_bias,
                 W1=W1, b1=b1, W2=W2, b2=b2)
        t = {k: v.detach().contiguous() for k, v in t.items()}
        t.update(alloc_forward_buffers(B, NH, NC, cgs, XQ.device))
        forward(t, cgs)
        ctx.cgs = cgs
        ctx.save_for_backward(t["XQ"], t["XK"], t["XV"], t["last_eta"], t["ttt_norm_weight"], t["ttt_norm_bias"],
                              t["W1_checkpoints"], t["b1_checkpoints"], t["W2_checkpoints"], t["b2_checkpoints"])
        return t["Out"]

    @staticmethod
    def backward(ctx, grad_out):
        XQ, XK, XV, last_eta, nw, nb, W1c, b1c, W2c, b2c = ctx.saved_tensors
        g = ttt_mlp_backward(XQ, XK, XV, last_eta, nw, nb, (W1c, b1c, W2c, b2c), grad_out, ctx.cgs)
        return (g["grad_L_XQ"], g["grad_L_XK"], g["grad_L_XV"], g["grad_L_last_eta"],
                g["grad_L_ttt_norm_weight"].sum(dim=0, keepdim=True), g["grad_L_ttt_norm_bias"].sum(dim=0, keepdim=True),
                g["grad_L_W1_init"], g["grad_L_b1_init"], g["grad_L_W2_init"], g["grad_L_b2_init"], None)


def ttt_mlp_backward(XQ, XK, XV, last_eta, ttt_norm_weight, ttt_norm_bias, checkpoints, grad_out, cgs, grad_last=None):
    """One `ttt_backward` call with freshly allocated workspace.  `checkpoints` = (W1, b1, W2, b2) checkpoints of the
    forward; `grad_last` = upstream gradients wrt the state after the last mini-batch (W1, b1, W2, b2 shapes), zeros
    when omitted.  Returns the ten gradients by the operator's names; the norm gradients are per batch element."""
    B, NH, NC = XQ.shape[:3]
    dev = XQ.device
    f32 = dict(dtype=torch.float32, device=dev)
    t = dict(XQ=XQ, XK=XK, XV=XV, last_eta=last_eta, ttt_norm_weight=ttt_norm_weight, ttt_norm_bias=ttt_norm_bias,
             grad_L_XQW_mini_batch=grad_out.to(torch.bfloat16).contiguous())
    for name, c in zip(("W1_checkpoints", "b1_checkpoints", "W2_checkpoints", "b2_checkpoints"), checkpoints):
        t[name] = c
    if grad_last is None:
        grad_last = (torch.zeros(B, NH, F, HID, **f32), torch.zeros(B, NH, 1, HID, **f32),
                     torch.zeros(B, NH, HID, F, **f32), torch.zeros(B, NH, 1, F, **f32))
    for name, gl in zip(("grad_L_W1_last", "grad_L_b1_last", "grad_L_W2_last", "grad_L_b2_last"), grad_last):
        t[name] = gl.to(torch.float32).contiguous()
    t["Out"] = torch.empty(B, NH, NC, CS, F, dtype=torch.bfloat16, device=dev)   # unused by the operator, must exist
    t.update(alloc_backward_buffers(B, NH, NC, cgs, dev, zero_fill=_ext.get_accumulate()))
    backward(t, cgs)
    return {k: t[k] for k in GRAD_NAMES}


def ttt_mlp(XQ, XK, XV, last_eta, ttt_norm_weight, ttt_norm_bias, W1, b1, W2, b2, checkpoint_group_size):
    """Differentiable call: see TTTMLPFunction."""
    return TTTMLPFunction.apply(XQ, XK, XV, last_eta, ttt_norm_weight, ttt_norm_bias, W1, b1, W2, b2, checkpoint_group_size)


def workspace_bytes(B: int, NH: int, cgs: int) -> int:
    """Bytes of workspace with which `ttt_forward` / `ttt_backward` of this shape can use several workgroups per
    (batch, head); 0 if the shape runs with one workgroup per pair."""
    return int(_ext.workspace_bytes(int(B), int(NH), int(cgs)))


def set_workspace(ws) -> None:
    """Hand the operators a caller-owned workspace (1-D uint8 GPU tensor, `workspace_bytes(...)` bytes or more): they
    then allocate nothing per call, like the upstream operator, whose every tensor is the caller's
    (upstream kernels/ttt_backward/ttt.cu:1451-1917).  ``None`` returns to a workspace from torch's allocator per call."""
    _ext.set_workspace(ws)
