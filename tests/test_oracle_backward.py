"""Pins the backward oracle (CPU only): float64 autograd of the dense formulation with the routing held fixed,
central finite differences of an independent float64 NumPy forward, and closed forms."""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from oracle import oracle_np as N
from tests.synth import C, make_inputs, scaled

GRADS = ("dx", "dWg", "dbg", "dW1", "dW3", "dW2")


def _case(name, seed, **kw):
    cfg = scaled(C.CONFIGS[name], **kw)
    inp = make_inputs(cfg, seed)
    dout = O.fill_normal(cfg.T * cfg.d, seed, 900, 1.0).reshape(cfg.T, cfg.d)
    if cfg.dtype == "bf16":
        dout = O.round_bf16(dout)
    # a gate that spreads the probabilities: the synthetic 0.02 leaves the router gradient tiny
    inp["Wg"] = inp["Wg"] * np.float32(8.0)
    return cfg, inp, dout


def autograd_f64(cfg, inp, dout, ids):
    """d(sum(out*dout)) by torch autograd in float64; ids [T,K] fixed.  Dense formulation: no permutation anywhere."""
    t64 = lambda a: torch.tensor(np.asarray(a, np.float64), requires_grad=True)
    x, Wg, W1, W3, W2 = (t64(inp[k]) for k in ("x", "Wg", "W1", "W3", "W2"))
    bg = t64(inp["bg"]) if inp["bg"] is not None else None
    logits = x @ Wg.T + (bg if bg is not None else 0.0)
    p = torch.softmax(logits, dim=1)
    idt = torch.tensor(ids.astype(np.int64))
    q = torch.gather(p, 1, idt)
    w = q / q.sum(dim=1, keepdim=True) if cfg.renorm else q
    out = torch.zeros_like(x)
    for g in range(cfg.E + cfg.Es):
        y = (torch.nn.functional.silu(x @ W1[g].T) * (x @ W3[g].T)) @ W2[g].T
        if g < cfg.E:
            coef = (w * (idt == g)).sum(dim=1, keepdim=True)
            out = out + coef * y
        else:
            out = out + y
    (out * torch.tensor(dout.astype(np.float64))).sum().backward()
    r = dict(dx=x.grad, dWg=Wg.grad, dW1=W1.grad, dW3=W3.grad, dW2=W2.grad, dbg=bg.grad if bg is not None else None)
    return {k: (None if v is None else v.numpy()) for k, v in r.items()}


def forward_f64_loops(cfg, a, ids):
    """Independent float64 forward, token by token, routing fixed."""
    T = a["x"].shape[0]
    out = np.zeros((T, cfg.d))
    for t in range(T):
        xr = a["x"][t]
        lg = a["Wg"] @ xr + (a["bg"] if a["bg"] is not None else 0.0)
        e = np.exp(lg - lg.max())
        p = e / e.sum()
        q = p[ids[t]]
        w = q / q.sum() if cfg.renorm else q
        for j in range(cfg.K + cfg.Es):
            g = ids[t, j] if j < cfg.K else cfg.E + j - cfg.K
            h1, h3 = a["W1"][g] @ xr, a["W3"][g] @ xr
            y = a["W2"][g] @ (h1 / (1.0 + np.exp(-h1)) * h3)
            out[t] += (w[j] if j < cfg.K else 1.0) * y
    return out


CASES = [
    ("c1_tiny_f32", dict(T=24, d=20, H=12, E=4, K=2)),
    ("c1_tiny_f32", dict(T=19, d=16, H=24, E=6, K=3, renorm=False, Es=2)),
    ("c1_tiny_f32", dict(T=16, d=12, H=8, E=5, K=2, zipf_bias=1.2)),
    ("c1_tiny_f32", dict(T=9, d=8, H=8, E=3, K=3)),         # every expert selected by every token
]


@pytest.mark.parametrize("name,kw", CASES)
def test_backward_matches_float64_autograd(name, kw):
    cfg, inp, dout = _case(name, 5, **kw)
    fwd = O.moe_forward(inp["x"], inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm, cfg.Es)
    got = O.moe_backward(inp["x"], dout, inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm, cfg.Es)
    ref = autograd_f64(cfg, inp, dout, fwd["ids"])
    for k in GRADS:
        if ref[k] is None:
            assert got[k] is None
            continue
        assert got[k].shape == ref[k].shape, k
        assert N.rel_l2(got[k], ref[k]) < 2e-5, (k, N.rel_l2(got[k], ref[k]))


def test_backward_matches_finite_differences():
    cfg, inp, dout = _case("c1_tiny_f32", 11, T=10, d=12, H=10, E=4, K=2, Es=1, zipf_bias=1.2)
    fwd = O.moe_forward(inp["x"], inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm, cfg.Es)
    got = O.moe_backward(inp["x"], dout, inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm, cfg.Es)
    a = {k: (None if v is None else v.astype(np.float64)) for k, v in inp.items()}
    d64 = dout.astype(np.float64)
    rng = np.random.default_rng(3)
    eps = 1e-6
    for key, gk in (("x", "dx"), ("Wg", "dWg"), ("bg", "dbg"), ("W1", "dW1"), ("W3", "dW3"), ("W2", "dW2")):
        flat = a[key].reshape(-1)
        picks = rng.choice(flat.size, size=min(12, flat.size), replace=False)
        fd = np.empty(len(picks))
        for n, i in enumerate(picks):
            keep = flat[i]
            flat[i] = keep + eps
            up = (forward_f64_loops(cfg, a, fwd["ids"]) * d64).sum()
            flat[i] = keep - eps
            dn = (forward_f64_loops(cfg, a, fwd["ids"]) * d64).sum()
            flat[i] = keep
            fd[n] = (up - dn) / (2 * eps)
        an = got[gk].reshape(-1)[picks]
        scale = np.abs(got[gk]).max()
        assert np.abs(an - fd).max() < 2e-4 * scale, (gk, an, fd)


def test_backward_closed_forms():
    # one expert, K = 1, renormalised: the combine weight is exactly 1, the gate gets no gradient, the layer is the
    # dense SwiGLU MLP
    cfg, inp, dout = _case("c1_tiny_f32", 2, T=7, d=8, H=6, E=1, K=1, zipf_bias=1.2)
    got = O.moe_backward(inp["x"], dout, inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], 1, True, 0)
    assert not got["dWg"].any() and not got["dbg"].any() and not got["dlogits"].any()
    x, W1, W3, W2, g = (v.astype(np.float64) for v in (inp["x"], inp["W1"][0], inp["W3"][0], inp["W2"][0], dout))
    h1, h3 = x @ W1.T, x @ W3.T
    s = 1 / (1 + np.exp(-h1))
    da = g @ W2
    dh1, dh3 = da * h3 * s * (1 + h1 * (1 - s)), da * h1 * s
    assert N.rel_l2(got["dW2"][0], g.T @ (h1 * s * h3)) < 1e-5
    assert N.rel_l2(got["dW1"][0], dh1.T @ x) < 1e-5
    assert N.rel_l2(got["dW3"][0], dh3.T @ x) < 1e-5
    assert N.rel_l2(got["dx"], dh1 @ W1 + dh3 @ W3) < 1e-5
    # without renormalisation and K = E the softmax gradient sums to zero over the experts of every token
    cfg, inp, dout = _case("c1_tiny_f32", 3, T=6, d=8, H=6, E=3, K=3, renorm=False)
    got = O.moe_backward(inp["x"], dout, inp["Wg"], None, inp["W1"], inp["W3"], inp["W2"], 3, False, 0)
    assert np.abs(got["dlogits"].sum(axis=1)).max() < 1e-5 * np.abs(got["dlogits"]).max()
    # an expert no token selected gets zero weight gradients
    cfg, inp, dout = _case("c1_tiny_f32", 4, T=3, d=8, H=6, E=8, K=1)
    fwd = O.moe_forward(inp["x"], inp["Wg"], None, inp["W1"], inp["W3"], inp["W2"], 1, True, 0)
    got = O.moe_backward(inp["x"], dout, inp["Wg"], None, inp["W1"], inp["W3"], inp["W2"], 1, True, 0)
    for e in range(8):
        if fwd["counts"][e] == 0:
            assert not got["dW1"][e].any() and not got["dW3"][e].any() and not got["dW2"][e].any()
    # linear in dout
    got2 = O.moe_backward(inp["x"], 2 * dout, inp["Wg"], None, inp["W1"], inp["W3"], inp["W2"], 1, True, 0)
    for k in ("dx", "dW1", "dW2", "dWg"):
        assert N.rel_l2(got2[k], 2 * got[k].astype(np.float64)) < 1e-6


def test_backward_bf16_mode_close_to_float64():
    cfg, inp, dout = _case("c2_mixtral", 8, T=40, d=32, H=48, E=4, K=2)
    fwd = O.moe_forward(inp["x"], inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm, cfg.Es, True)
    got = O.moe_backward(inp["x"], dout, inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm, cfg.Es,
                         True)
    ref = autograd_f64(cfg, inp, dout, fwd["ids"])
    for k in ("dx", "dWg", "dW1", "dW3", "dW2"):
        assert N.rel_l2(got[k], ref[k]) < 1e-2, (k, N.rel_l2(got[k], ref[k]))
    assert np.array_equal(got["dx"], O.round_bf16(got["dx"]))


def test_backward_routed_equals_full_on_a_token_subset():
    # input gradient, dw and dlogits of a token depend on that token only: a subset with compacted expert indices
    # reproduces the rows of the full pass bit for bit
    cfg, inp, dout = _case("c1_tiny_f32", 21, T=30, d=16, H=12, E=6, K=2, Es=1)
    fwd = O.moe_forward(inp["x"], inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm, cfg.Es)
    full = O.moe_backward(inp["x"], dout, inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm, cfg.Es)
    tok = np.array([3, 4, 17, 29])
    need = sorted(set(fwd["ids"][tok].ravel().tolist()))
    remap = {g: i for i, g in enumerate(need)}
    wid = np.vectorize(remap.get)(fwd["ids"][tok]).astype(np.int32)
    sel = need + [cfg.E + s for s in range(cfg.Es)]
    got = O.moe_backward_routed(inp["x"][tok], dout[tok], inp["Wg"], fwd["p"][tok], fwd["ids"][tok], wid, fwd["w"][tok],
                                inp["W1"][sel], inp["W3"][sel], inp["W2"][sel], cfg.Es, cfg.renorm)
    assert np.array_equal(got["dx"], full["dx"][tok])
    assert np.array_equal(got["dw"], full["dw"][tok])
    assert np.array_equal(got["dlogits"], full["dlogits"][tok])


def _gamma(d, seed):
    return (O.fill_normal(d, seed, C.STREAM_NORM, 1.0) * np.float32(0.1) + np.float32(1.0)).astype(np.float32)


@pytest.mark.parametrize("name,kw", CASES[:3])
def test_block_backward_matches_float64_autograd(name, kw):
    cfg, inp, dout = _case(name, 9, **kw)
    gamma = _gamma(cfg.d, 9)
    fwd = O.block_forward(inp["x"], gamma, inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm, cfg.Es)
    got = O.block_backward(inp["x"], gamma, dout, inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm,
                           cfg.Es)
    t64 = lambda a: torch.tensor(np.asarray(a, np.float64), requires_grad=True)
    x, gm, Wg, W1, W3, W2 = (t64(v) for v in (inp["x"], gamma, inp["Wg"], inp["W1"], inp["W3"], inp["W2"]))
    bg = t64(inp["bg"]) if inp["bg"] is not None else None
    h = x / torch.sqrt((x * x).mean(dim=1, keepdim=True) + 1e-6) * gm
    logits = h @ Wg.T + (bg if bg is not None else 0.0)
    p = torch.softmax(logits, dim=1)
    idt = torch.tensor(fwd["ids"].astype(np.int64))
    q = torch.gather(p, 1, idt)
    w = q / q.sum(dim=1, keepdim=True) if cfg.renorm else q
    out = x
    for g in range(cfg.E + cfg.Es):
        y = (torch.nn.functional.silu(h @ W1[g].T) * (h @ W3[g].T)) @ W2[g].T
        out = out + ((w * (idt == g)).sum(dim=1, keepdim=True) * y if g < cfg.E else y)
    (out * torch.tensor(dout.astype(np.float64))).sum().backward()
    ref = dict(dx=x.grad, dgamma=gm.grad, dWg=Wg.grad, dW1=W1.grad, dW3=W3.grad, dW2=W2.grad)
    for k, v in ref.items():
        assert N.rel_l2(got[k], v.numpy()) < 2e-5, (k, N.rel_l2(got[k], v.numpy()))
    if bg is not None:
        assert N.rel_l2(got["dbg"], bg.grad.numpy()) < 2e-5


def test_rmsnorm_backward_closed_forms():
    rng = np.random.default_rng(8)
    T, d = 5, 96
    x = rng.standard_normal((T, d)).astype(np.float32)
    ones = np.ones(d, np.float32)
    _, rms = O.rmsnorm(x, ones)
    # dh orthogonal to x and gamma = 1: the rms term vanishes, dx = dh / rms
    dh = rng.standard_normal((T, d)).astype(np.float64)
    dh -= (dh * x).sum(1, keepdims=True) / (x.astype(np.float64) ** 2).sum(1, keepdims=True) * x
    dx, dg = O.rmsnorm_backward(x, dh.astype(np.float32), ones, rms)
    assert N.rel_l2(dx, dh / rms[:, None]) < 1e-5
    # dh = x: dgamma = sum_t x^2 / rms; and dx = x/rms * (1 - mean(x^2)/rms^2) = x/rms * 1e-6/rms^2 (tiny)
    dx, dg = O.rmsnorm_backward(x, x, ones, rms)
    assert N.rel_l2(dg, (x.astype(np.float64) ** 2 / rms[:, None]).sum(0)) < 1e-6
    assert np.abs(dx).max() < 1e-4
    # the residual gradient is added as it is
    r = rng.standard_normal((T, d)).astype(np.float32)
    dx2, _ = O.rmsnorm_backward(x, x, ones, rms, resid=r)
    assert N.rel_l2(dx2, dx.astype(np.float64) + r) < 1e-6
