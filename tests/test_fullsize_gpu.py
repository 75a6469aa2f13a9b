"""The benchmark configurations (C2 - C5) at their full sizes on the GPU.

C2/C3 (16,384 tokens, 48 heads) and C4 (262,144 tokens, 48 heads) are checked against the CPU oracle for every
head, as the upstream harness compares every head (kernels/ttt_backward/matching.py:667-705); C5 (8 x 48
recurrences) on 48 of its (batch, head) pairs, every head once and every batch element six times.  C4 and C5 are
also drawn with a second seed (8 heads / 16 pairs against the oracle).  Size-independent properties cover the rest:
exact linearity in the upstream gradients, zero gradients for zero upstream gradients, independence of heads, and
agreement between two checkpoint group sizes.

Bar, on every configuration: max|hw - ref| / max|ref| <= 2e-2 and cosine >= 0.9999 per tensor (Out,
checkpoints, ten gradients), reference = fp32 oracle on the same bf16-rounded inputs.  On C4 and C5 the tensor is
all compared (batch, head) pairs together; each pair by itself is reported too and held to 3e-2 / 0.9998.

Inputs: the benchmark's distributions, except that b1, b2 and the norm weight / bias are not the trivial
zeros / ones / zeros here (b ~ N(0, 0.02), weight ~ 1 + N(0, 0.1), bias ~ N(0, 0.1)), so that the bias and
norm-parameter paths carry signal over the whole sequence.

If the environment variable TTT_PARITY_LOG names a file, every per-tensor line is appended to it."""
import os

import pytest
import torch

from oracle import ttt_mlp_oracle as orc

pytestmark = pytest.mark.gpu

MAX_REL, MIN_COS = 2e-2, 0.9999              # the bar, per tensor
PAIR_MAX_REL, PAIR_MIN_COS = 3e-2, 0.9998    # any single (batch, head) pair of C4 / C5 taken by itself
FWD_KEYS = ("XQ", "XK", "XV", "last_eta", "ttt_norm_weight", "ttt_norm_bias", "W1", "b1", "W2", "b2")
UP_KEYS = ("grad_L_W1_last", "grad_L_b1_last", "grad_L_W2_last", "grad_L_b2_last", "grad_L_XQW_mini_batch")
GRADS = ("grad_L_ttt_norm_weight", "grad_L_ttt_norm_bias", "grad_L_W1_init", "grad_L_b1_init", "grad_L_W2_init",
         "grad_L_b2_init", "grad_L_last_eta", "grad_L_XQ", "grad_L_XK", "grad_L_XV")


def device_inputs(B, NH, NC, eta_std, seed=0):
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(seed)
    rn = lambda *s: torch.randn(*s, generator=g, device=dev, dtype=torch.float32)
    t = {}
    for name in ("XQ", "XK", "XV", "grad_L_XQW_mini_batch"):
        t[name] = torch.empty(B, NH, NC, 64, 64, device=dev, dtype=torch.bfloat16)
        for b in range(B):
            t[name][b] = rn(NH, NC, 64, 64).to(torch.bfloat16)
    t["W1"], t["W2"] = rn(B, NH, 64, 256) * 0.02, rn(B, NH, 256, 64) * 0.02
    t["b1"], t["b2"] = rn(B, NH, 1, 256) * 0.02, rn(B, NH, 1, 64) * 0.02
    t["ttt_norm_weight"], t["ttt_norm_bias"] = 1 + rn(1, NH, 1, 64) * 0.1, rn(1, NH, 1, 64) * 0.1
    t["last_eta"] = (torch.sigmoid(rn(B, NH, NC, 64, 1) * eta_std) / 64).to(torch.bfloat16)
    t["grad_L_W1_last"], t["grad_L_b1_last"] = rn(B, NH, 64, 256) * 1e-3, rn(B, NH, 1, 256) * 1e-3
    t["grad_L_W2_last"], t["grad_L_b2_last"] = rn(B, NH, 256, 64) * 1e-3, rn(B, NH, 1, 64) * 1e-3
    return t


def run(t, cgs, backward=True):
    import ttt_mlp_host as host
    B, NH, NC = t["XQ"].shape[:3]
    dev = t["XQ"].device
    r = dict(t)
    r.update(host.alloc_forward_buffers(B, NH, NC, cgs, dev))
    host.forward(r, cgs)
    if backward:
        r.update(host.alloc_backward_buffers(B, NH, NC, cgs, dev))
        host.backward(r, cgs)
    return r


def cpu_pairs(t, pairs):
    """The (b, h) recurrences of `pairs` as one CPU problem with B = 1 and one head per pair."""
    d = {}
    for k in FWD_KEYS + UP_KEYS:
        v = t[k]
        if k.startswith("ttt_norm"):
            d[k] = torch.cat([v[:, h:h + 1] for _, h in pairs], dim=1).cpu()
        else:
            d[k] = torch.cat([v[b:b + 1, h:h + 1] for b, h in pairs], dim=1).cpu()
    return d


def oracle(d, cgs, backward=True):
    out, ck, _ = orc.ttt_forward(*[d[k] for k in FWD_KEYS], cgs)
    ref = {"Out": out, "W1_checkpoints": ck.W1, "b1_checkpoints": ck.b1, "W2_checkpoints": ck.W2, "b2_checkpoints": ck.b2}
    if backward:
        ref.update(orc.ttt_backward(d["XQ"], d["XK"], d["XV"], d["last_eta"], d["ttt_norm_weight"], d["ttt_norm_bias"], ck,
                                    orc.State(d["grad_L_W1_last"], d["grad_L_b1_last"], d["grad_L_W2_last"],
                                              d["grad_L_b2_last"]), d["grad_L_XQW_mini_batch"], cgs))
    return ref


def report(line):
    print(line, flush=True)
    path = os.environ.get("TTT_PARITY_LOG")
    if path:
        with open(path, "a") as f:
            f.write(line + "\n")


def compare(tag, hw, ref, failures, bar=True):
    """One line per tensor; with `bar` a tensor outside max-rel 2e-2 / cosine 0.9999 is a failure."""
    for name, r in ref.items():
        if r.abs().max() == 0:
            assert hw[name].abs().max() == 0, name
            continue
        st = orc.parity_stats(hw[name], r)
        ok = not bar or (st["max_rel"] <= MAX_REL and st["cosine"] >= MIN_COS)
        report(f"{tag} {name:24s} max_rel={st['max_rel']:.3e} cos={st['cosine']:.6f}{'' if ok else '  <-- FAIL'}")
        if not ok:
            failures.append((tag, name, st["max_rel"], st["cosine"]))


def check_subset(case, t, r, cgs, pairs, backward=True):
    """The (batch, head) recurrences of `pairs` against the oracle.  The bar applies to each tensor as a whole (all
    compared pairs together: the statistic the parity bar is stated for, and what the upstream harness prints,
    kernels/ttt_backward/matching.py:9-40); every pair is also reported by itself, with the worst of them per tensor,
    and held to PAIR_MAX_REL / PAIR_MIN_COS: the per-head tensors of the bias and norm gradients have 64 - 256
    elements, whose cosine scatters from head to head around the whole tensor's."""
    torch.set_num_threads(min(16, os.cpu_count() or 1))
    failures = []
    ref = oracle(cpu_pairs(t, pairs), cgs, backward)
    hw_all = {k: torch.cat([r[k][b:b + 1, h:h + 1] for b, h in pairs], dim=1).float().cpu() for k in ref}
    worst = {}
    for i, (b, h) in enumerate(pairs):
        for k, v in ref.items():
            x, y = hw_all[k][:, i].flatten().double(), v[:, i].flatten().double()
            if y.abs().max() == 0:
                continue
            mr = ((x - y).abs().max() / y.abs().max()).item()
            cs = (torch.dot(x, y) / (x.norm() * y.norm())).item()
            report(f"{case} (b={b},h={h}) {k:24s} max_rel={mr:.3e} cos={cs:.6f}")
            w = worst.setdefault(k, [0.0, 1.0])
            w[0], w[1] = max(w[0], mr), min(w[1], cs)
    for k, (mr, cs) in worst.items():
        ok = mr <= PAIR_MAX_REL and cs >= PAIR_MIN_COS
        report(f"{case} worst single pair of {len(pairs)} {k:24s} max_rel={mr:.3e} cos={cs:.6f}{'' if ok else '  <-- FAIL'}")
        if not ok:
            failures.append((case, "worst pair", k, mr, cs))
    compare(f"{case} all {len(pairs)} pairs", hw_all, ref, failures)
    assert not failures, failures


def test_c2_forward_16k_tokens_all_heads():
    report("case C2: forward B=1 NH=48 NC=256 cgs=16")
    t = device_inputs(1, 48, 256, 1.0)
    r = run(t, 16, backward=False)
    d = {k: t[k].cpu() for k in FWD_KEYS}
    ref = oracle(d, 16, backward=False)
    failures = []
    compare("C2", {k: r[k].float().cpu() for k in ref}, ref, failures)
    assert not failures, failures


def test_c3_forward_backward_16k_tokens_all_heads():
    report("case C3: forward+backward B=1 NH=48 NC=256 cgs=16")
    t = device_inputs(1, 48, 256, 1.0)
    r = run(t, 16)
    d = {k: t[k].cpu() for k in FWD_KEYS + UP_KEYS}
    torch.set_num_threads(min(16, os.cpu_count() or 1))
    ref = oracle(d, 16)
    failures = []
    compare("C3", {k: r[k].float().cpu() for k in ref}, ref, failures)
    assert not failures, failures


def test_c4_long_sequence_262k_tokens():
    report("case C4: forward+backward B=1 NH=48 NC=4096 cgs=64")
    t = device_inputs(1, 48, 4096, 1.0)
    r = run(t, 64)
    for k in GRADS + ("Out",):
        assert bool(torch.isfinite(r[k].float()).all()), k
    check_subset("C4", t, r, 64, [(0, h) for h in range(48)])
    # exact linearity: doubling every upstream gradient doubles every output gradient bit for bit
    t2 = dict(t)
    for k in UP_KEYS:
        t2[k] = t[k] * 2
    r2 = run(t2, 64)
    for k in GRADS:
        assert torch.equal(r2[k].float(), r[k].float() * 2), k
    del r2, t2
    # another checkpoint group size walks the same recurrence from other restart points
    r3 = run(t, 128)
    failures = []
    compare("C4 cgs 128 vs 64", {k: r3[k].float().cpu() for k in GRADS}, {k: r[k].float().cpu() for k in GRADS}, failures)
    assert not failures, failures


def test_c5_fill_the_chip_384_recurrences():
    report("case C5: forward+backward B=8 NH=48 NC=512 cgs=32, wide eta")
    t = device_inputs(8, 48, 512, 2.0)
    r = run(t, 32)
    for k in GRADS + ("Out",):
        assert bool(torch.isfinite(r[k].float()).all()), k
    check_subset("C5", t, r, 32, [((5 * h + h // 8) % 8, h) for h in range(48)])
    # zero upstream gradients give zero gradients everywhere
    tz = dict(t)
    for k in UP_KEYS:
        tz[k] = torch.zeros_like(t[k])
    rz = run(tz, 32)
    for k in GRADS:
        assert rz[k].float().abs().max() == 0, k
    del rz, tz
    # heads are independent: reversing the head order reverses the outputs bit for bit
    tf = {k: (v.flip(1).contiguous() if v.dim() >= 2 and v.shape[1] == 48 else v) for k, v in t.items()}
    rf = run(tf, 32)
    for k in GRADS + ("Out",):
        assert torch.equal(rf[k].flip(1), r[k]), k


def test_c4_and_c5_second_seed():
    """The same two configurations drawn with another seed: the margin to the bar must not hang on one draw."""
    report("case C4 seed 1: forward+backward B=1 NH=48 NC=4096 cgs=64")
    t = device_inputs(1, 48, 4096, 1.0, seed=1)
    r = run(t, 64)
    check_subset("C4 seed 1", t, r, 64, [(0, h) for h in (1, 7, 12, 22, 28, 35, 41, 46)])
    del t, r
    report("case C5 seed 1: forward+backward B=8 NH=48 NC=512 cgs=32, wide eta")
    t = device_inputs(8, 48, 512, 2.0, seed=1)
    r = run(t, 32)
    check_subset("C5 seed 1", t, r, 32, [(i % 8, 3 * i) for i in range(16)])
