"""Writes tests/golden/c1_oracle_samples.json: known-answer samples of the oracle on the
CPU-runnable reference configuration (B=1, NH=2, NC=4, checkpoint_group_size=1, seed 0).

The upstream repository stores no golden vectors for this path, so these were produced by
oracle/ttt_mlp_oracle.py after its pins (tests/test_oracle_pins.py) passed.  Inputs are regenerated
from the seed; their checksums are stored so that a change of the random stream is detected rather
than reported as a numerical regression.  For each output: every STRIDE-th element (fp32), the sum
and the L2 norm in float64.

    python tests/golden/make_fixtures.py
"""
import json
import os
import sys

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import ttt_mlp_oracle as orc  # noqa: E402

STRIDE = 997
B, NH, NC, CGS, SEED = 1, 2, 4, 1, 0
FWD_KEYS = ("XQ", "XK", "XV", "last_eta", "ttt_norm_weight", "ttt_norm_bias", "W1", "b1", "W2", "b2")


def summarize(t):
    f = t.detach().to(torch.float64).flatten()
    return {"shape": list(t.shape), "sum": f.sum().item(), "l2": f.norm().item(),
            "samples": t.detach().to(torch.float32).flatten()[::STRIDE].tolist()}


def compute():
    d = orc.make_inputs(B, NH, NC, seed=SEED)
    out, ck, fin = orc.ttt_forward(*[d[k] for k in FWD_KEYS], CGS)
    g = orc.ttt_backward(d["XQ"], d["XK"], d["XV"], d["last_eta"], d["ttt_norm_weight"], d["ttt_norm_bias"], ck,
                         orc.State(d["grad_L_W1_last"], d["grad_L_b1_last"], d["grad_L_W2_last"], d["grad_L_b2_last"]),
                         d["grad_L_XQW_mini_batch"], CGS)
    outputs = {"Out": out, "W1_checkpoints": ck.W1, "b1_checkpoints": ck.b1, "W2_checkpoints": ck.W2,
               "b2_checkpoints": ck.b2, "W1_final": fin.W1, "W2_final": fin.W2}
    outputs.update(g)
    return d, outputs


def main():
    d, outputs = compute()
    doc = {"config": {"B": B, "NH": NH, "NC": NC, "checkpoint_group_size": CGS, "seed": SEED, "stride": STRIDE},
           "inputs": {k: {"sum": v.double().sum().item(), "l2": v.double().norm().item()} for k, v in d.items()},
           "outputs": {k: summarize(v) for k, v in outputs.items()}}
    path = os.path.join(HERE, "c1_oracle_samples.json")
    with open(path, "w") as f:
        json.dump(doc, f, indent=1)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
