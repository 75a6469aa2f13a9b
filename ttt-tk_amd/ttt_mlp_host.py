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


def alloc_backward_buffers(B: int, NH: int, NC: int, cgs: int, device) -> Dict[str, torch.Tensor]:
    """The sixteen remat scratch tensors, and the ten output gradients (accumulating ones zeroed)."""
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
        grad_L_last_eta=torch.zeros(B, NH, NC, CS, 1, **bf), grad_L_XQ=torch.zeros(B, NH, NC, CS, F, **bf),
        grad_L_XK=torch.zeros(B, NH, NC, CS, F, **bf), grad_L_XV=torch.zeros(B, NH, NC, CS, F, **bf))
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
