#!/usr/bin/env python3
"""Writes the golden fixtures of the MoE forward path (tests/golden/*.npz) from the pinned CPU oracle.

The reference holds no golden vectors for this path (it has no mixture-of-experts layer and no tests that
cover its building blocks with expected outputs), so the fixtures freeze what the pinned oracle computes for
  * the fp32 parity configuration (256 tokens, d=128, 8 experts, top-2, H=256) under a fixed seed, and
  * small adversarial cases: ties (all-equal gate rows, duplicated gate rows), empty experts, K == E,
    shared experts without renormalisation.
The backward pass of four of the cases is frozen the same way (bw_*.npz, see BW_CASES), and so are five steps of the
AdamW update (adamw_steps.npz).
Inputs are regenerated from the seed by the counter-based generator, so only expected outputs are stored:
routing arrays in full, the layer output as float64 checksums plus a few rows.
Run from the repository root:  python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import oracle as O  # noqa: E402
from tests.synth import C, make_inputs  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))

CASES = {
    "c1_tiny_f32_seed20251": dict(cfg=C.CONFIGS["c1_tiny_f32"], seed=20251, tweak=None),
    "ties_all_equal_gate": dict(cfg=C.MoEConfig("t", T=77, d=64, E=8, K=3, H=64, dtype="f32"), seed=9, tweak="zero_gate"),
    "ties_duplicated_gate_rows": dict(cfg=C.MoEConfig("t", T=77, d=64, E=8, K=3, H=64, dtype="f32"), seed=10, tweak="dup_rows"),
    "k_equals_e": dict(cfg=C.MoEConfig("t", T=70, d=48, E=5, K=5, H=80, renorm=False, dtype="f32"), seed=5005, tweak=None),
    "shared_no_renorm": dict(cfg=C.MoEConfig("t", T=96, d=64, E=64, K=6, H=96, Es=2, renorm=False, dtype="f32"), seed=11, tweak=None),
    "zipf_empty_experts": dict(cfg=C.MoEConfig("t", T=128, d=64, E=128, K=8, H=64, dtype="f32", zipf_bias=1.2), seed=11, tweak=None),
    "bf16_small": dict(cfg=C.MoEConfig("t", T=200, d=256, E=8, K=2, H=384, dtype="bf16"), seed=4242, tweak=None),
}


def case_inputs(spec):
    inp = make_inputs(spec["cfg"], spec["seed"])
    if spec["tweak"] == "zero_gate":
        inp["Wg"][:] = 0.0
    elif spec["tweak"] == "dup_rows":
        inp["Wg"][5] = inp["Wg"][1]
        inp["Wg"][6] = inp["Wg"][2]
    return inp


def expected(spec):
    cfg = spec["cfg"]
    inp = case_inputs(spec)
    r = O.moe_forward(inp["x"], inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm, cfg.Es,
                      bf16=cfg.dtype == "bf16")
    out64 = r["out"].astype(np.float64)
    return dict(ids=r["ids"], w=r["w"], counts=r["counts"], offsets=r["offsets"], dst=r["dst"], src_row=r["src_row"],
                out_sum=np.array(out64.sum()), out_l2=np.array(np.sqrt((out64 ** 2).sum())),
                out_abs_sum=np.array(np.abs(out64).sum()), out_head=r["out"][:4].copy(), out_tail=r["out"][-2:].copy())


# Backward pass (pinned oracle: float64 autograd, finite differences): the output gradient is drawn from the case's
# seed (stream 900); stored are the gate gradients in full, per-expert norms of the expert gradients, and rows and
# float64 checksums of the input gradient.  Files bw_<case>.npz.
BW_CASES = ("c1_tiny_f32_seed20251", "shared_no_renorm", "zipf_empty_experts", "bf16_small")


def backward_dout(spec):
    cfg = spec["cfg"]
    g = O.fill_normal(cfg.T * cfg.d, spec["seed"], 900, 1.0).reshape(cfg.T, cfg.d)
    return O.round_bf16(g) if cfg.dtype == "bf16" else g


def expected_backward(spec):
    cfg = spec["cfg"]
    inp = case_inputs(spec)
    r = O.moe_backward(inp["x"], backward_dout(spec), inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K,
                       cfg.renorm, cfg.Es, bf16=cfg.dtype == "bf16")
    dx64 = r["dx"].astype(np.float64)
    norms = np.array([[np.sqrt((r[k][g].astype(np.float64) ** 2).sum()) for g in range(cfg.E + cfg.Es)]
                      for k in ("dW1", "dW3", "dW2")])
    out = dict(dx_head=r["dx"][:4].copy(), dx_tail=r["dx"][-2:].copy(), dx_sum=np.array(dx64.sum()),
               dx_l2=np.array(np.sqrt((dx64 ** 2).sum())), dx_abs_sum=np.array(np.abs(dx64).sum()), dWg=r["dWg"],
               dW_norms=norms, dW2_first_row=r["dW2"][int(np.argmax(norms[2]))][0].copy())
    if r["dbg"] is not None:
        out["dbg"] = r["dbg"]
    return out


# AdamW (the updater oracle, pinned against torch.optim.AdamW in float64 and closed forms): 512 parameters, five steps
# with gradients whose magnitudes span six decades (and exact zeros); stored are the parameters and both moments after
# every step, bit for bit.  File adamw_steps.npz.
ADAMW = dict(n=512, steps=5, lr=3e-3, beta1=0.9, beta2=0.95, wd=1e-2, seed=77)


def adamw_inputs():
    n, seed = ADAMW["n"], ADAMW["seed"]
    w0 = O.fill_normal(n, seed, 1, 0.5)
    grads = []
    for t in range(ADAMW["steps"]):
        g = O.fill_normal(n, seed, 10 + t, 1.0) * (np.float32(10.0) ** np.floor(O.fill_normal(n, seed, 20 + t, 2.0)).clip(-4, 1))
        g = g.astype(np.float32)
        g[::17] = 0.0
        grads.append(g)
    return w0, grads


def expected_adamw():
    w, grads = adamw_inputs()
    m, v = np.zeros_like(w), np.zeros_like(w)
    out = {}
    for t, g in enumerate(grads, 1):
        w, m, v = O.adamw(w, g, m, v, ADAMW["lr"], ADAMW["beta1"], ADAMW["beta2"], ADAMW["wd"], t)
        out[f"w{t}"], out[f"m{t}"], out[f"v{t}"] = w.copy(), m.copy(), v.copy()
    return out


def main():
    np.savez_compressed(os.path.join(HERE, "adamw_steps.npz"), **expected_adamw())
    print("wrote adamw_steps")
    for name, spec in CASES.items():
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **expected(spec))
        print("wrote", name)
    for name in BW_CASES:
        np.savez_compressed(os.path.join(HERE, "bw_" + name + ".npz"), **expected_backward(CASES[name]))
        print("wrote bw_" + name)


if __name__ == "__main__":
    main()
