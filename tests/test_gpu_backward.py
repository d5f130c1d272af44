"""Backward pass through the C ABI against the backward oracle (which float64 autograd and finite differences pin):
input gradient and every parameter gradient to 1e-5 (fp32) / 1e-2 (bf16) relative L2, plus accGrad / update."""
import importlib

import numpy as np
import pytest

from oracle import oracle as O
from oracle import oracle_np as N
from tests.synth import C, make_inputs, scaled

pytestmark = pytest.mark.gpu
L = importlib.import_module("omega-ai_amd._lib")


def _setup(name, kw, seed):
    from tests import gpu_util as G
    cfg = scaled(C.CONFIGS[name], **kw)
    inp = make_inputs(cfg, seed)
    inp["Wg"] = inp["Wg"] * np.float32(8.0)   # spread the probabilities: a router gradient worth checking
    dout = O.fill_normal(cfg.T * cfg.d, seed, 900, 1.0).reshape(cfg.T, cfg.d)
    if cfg.dtype == "bf16":
        dout = O.round_bf16(dout)
    layer = G.build_layer(cfg, inp)
    return G, cfg, inp, dout, layer


def _check_grads(layer, cfg, ref, tol):
    errs = {"dWg": N.rel_l2(layer.grad(L.W_GATE), ref["dWg"])}
    if ref["dbg"] is not None:
        errs["dbg"] = N.rel_l2(layer.grad(L.W_GATE_BIAS), ref["dbg"])
    for g in range(cfg.E + cfg.Es):
        for which, k in ((L.W_W1, "dW1"), (L.W_W3, "dW3"), (L.W_W2, "dW2")):
            got = layer.grad(which, g)
            if not ref[k][g].any():
                assert not got.any(), (k, g)        # an expert without rows: exact zeros
            else:
                errs[f"{k}[{g}]"] = N.rel_l2(got, ref[k][g])
    bad = {k: v for k, v in errs.items() if not v < tol}
    assert not bad, bad


CASES_F32 = [
    ("c1_tiny_f32", {}),
    ("c1_tiny_f32", dict(T=77, d=102, H=72)),                                   # nothing a multiple of the tiles
    ("c1_tiny_f32", dict(T=96, d=64, H=48, E=6, K=3, renorm=False, Es=2)),      # shared experts, no renormalisation
    ("c1_tiny_f32", dict(T=50, d=48, H=40, E=16, K=2, zipf_bias=1.2)),          # gate bias, experts without rows
    ("c1_tiny_f32", dict(T=1, d=32, H=16, E=4, K=4)),
]


@pytest.mark.parametrize("name,kw", CASES_F32)
def test_backward_fp32_matches_oracle(name, kw):
    G, cfg, inp, dout, layer = _setup(name, kw, 31)
    x = G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype)
    g = G.P.DeviceBuffer.from_numpy(G.ctx(), dout, cfg.dtype)
    with pytest.raises(RuntimeError):      # no forward yet
        layer.back(g)
    out = layer.forward(x).to_numpy()
    dx = layer.back(g).to_numpy()
    ref = O.moe_backward(inp["x"], dout, inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm, cfg.Es)
    assert N.rel_l2(dx, ref["dx"]) < 1e-5, N.rel_l2(dx, ref["dx"])
    _check_grads(layer, cfg, ref, 1e-5)
    # the forward output is untouched and a second backward gives the same bits (gradients are overwritten, not added)
    assert np.array_equal(layer.getOutput().to_numpy(), out)
    w1 = layer.grad(L.W_W1, 0)
    assert np.array_equal(layer.back(g).to_numpy(), dx)
    assert np.array_equal(layer.grad(L.W_W1, 0), w1)
    layer.close()


def test_acc_grad_and_update_fp32():
    G, cfg, inp, dout, layer = _setup("c1_tiny_f32", dict(T=40, d=32, H=24, E=4, K=2, zipf_bias=1.2), 5)
    x = G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype)
    g1 = G.P.DeviceBuffer.from_numpy(G.ctx(), dout, cfg.dtype)
    g2 = G.P.DeviceBuffer.from_numpy(G.ctx(), (0.5 * dout).astype(np.float32), cfg.dtype)
    layer.forward(x)
    layer.back(g1)
    a = {k: layer.grad(w, 1) for k, w in (("W1", L.W_W1), ("W2", L.W_W2))}
    a["Wg"], a["bg"] = layer.grad(L.W_GATE), layer.grad(L.W_GATE_BIAS)
    layer.freeze = True                     # a frozen layer's update() does nothing (FullyLayer.update)
    w_frozen = layer._download_weight(L.W_W1, 1, (cfg.H, cfg.d))
    layer.update(0.25)
    layer.updateAdamW(0.25, 1)
    assert np.array_equal(layer._download_weight(L.W_W1, 1, (cfg.H, cfg.d)), w_frozen)
    layer.freeze = False
    layer.accGrad(1.0)                      # first call: copy
    layer.back(g2)
    layer.accGrad(2.0)                      # then acc += 2 * grad(0.5 dout) = 2 * grad(dout) in total
    before = {k: layer._download_weight(w, 1, s) for k, w, s in (("W1", L.W_W1, (cfg.H, cfg.d)), ("W2", L.W_W2, (cfg.d, cfg.H)))}
    before["Wg"] = layer._download_weight(L.W_GATE, 0, (cfg.E, cfg.d))
    before["bg"] = layer._download_weight(L.W_GATE_BIAS, 0, (cfg.E,))
    layer.update(0.25)
    after = {k: layer._download_weight(w, 1, s) for k, w, s in (("W1", L.W_W1, (cfg.H, cfg.d)), ("W2", L.W_W2, (cfg.d, cfg.H)))}
    after["Wg"] = layer._download_weight(L.W_GATE, 0, (cfg.E, cfg.d))
    after["bg"] = layer._download_weight(L.W_GATE_BIAS, 0, (cfg.E,))
    for k in ("W1", "W2", "Wg", "bg"):
        want = before[k].astype(np.float64) - 0.25 * 2.0 * a[k].astype(np.float64)
        assert N.rel_l2(after[k], want) < 1e-6, k
    # the accumulators were cleared: the next update uses the plain gradient of the next backward
    layer.forward(x)
    layer.back(g1)
    gW = layer.grad(L.W_W1, 1)
    layer.update(1.0)
    assert N.rel_l2(layer._download_weight(L.W_W1, 1, (cfg.H, cfg.d)), after["W1"].astype(np.float64) - gW) < 1e-6
    layer.close()


CASES_BF16 = [
    ("c2_mixtral", dict(T=300, d=256, H=384)),                          # H = 128 mod 256: ragged last column tile
    ("c4_finegrained", dict(T=200, d=256, H=256, E=16, K=4, Es=2)),     # experts far below one k-space minimum, shared experts
    ("c5_skewed", dict(T=257, d=512, H=256, E=32, K=4)),                # gate bias, experts without rows
    ("c2_mixtral", dict(T=1200, d=256, H=512, E=4, K=2)),               # several row tiles per expert
    ("c2_mixtral", dict(T=1, d=256, H=256, E=8, K=2)),
]


@pytest.mark.parametrize("name,kw", CASES_BF16)
def test_backward_bf16_matches_oracle(name, kw):
    G, cfg, inp, dout, layer = _setup(name, kw, 47)
    x = G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype)
    g = G.P.DeviceBuffer.from_numpy(G.ctx(), dout, cfg.dtype)
    out = layer.forward(x).to_numpy()
    dx = layer.back(g).to_numpy()
    ref = O.moe_backward(inp["x"], dout, inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm, cfg.Es,
                         bf16=True)
    assert N.rel_l2(dx, ref["dx"]) < 1e-2, N.rel_l2(dx, ref["dx"])
    _check_grads(layer, cfg, ref, 1e-2)
    # forward output and routing untouched; a second backward gives the same bits; a forward after it still matches
    assert np.array_equal(layer.getOutput().to_numpy(), out)
    w2 = layer.grad(L.W_W2, 0)
    assert np.array_equal(layer.back(g).to_numpy(), dx)
    assert np.array_equal(layer.grad(L.W_W2, 0), w2)
    assert np.array_equal(layer.forward(x).to_numpy(), out)
    # training mode: the forward pass keeps h1 / h3, the backward pass skips their recomputation - same bits
    w13 = (layer.grad(L.W_W1, cfg.E - 1), layer.grad(L.W_W3, 0))
    layer.set_training(True)
    assert np.array_equal(layer.forward(x).to_numpy(), out)
    assert np.array_equal(layer.back(g).to_numpy(), dx)
    assert np.array_equal(layer.grad(L.W_W2, 0), w2)
    assert np.array_equal(layer.grad(L.W_W1, cfg.E - 1), w13[0]) and np.array_equal(layer.grad(L.W_W3, 0), w13[1])
    layer.set_training(False)
    # new weights invalidate the transposed copies the pass keeps: gradients follow the new weights
    W2n = O.round_bf16(inp["W2"][0] * np.float32(0.5))
    layer.set_expert(0, inp["W1"][0], inp["W3"][0], W2n)
    inp["W2"][0] = W2n
    layer.forward(x)
    dx2 = layer.back(g).to_numpy()
    ref2 = O.moe_backward(inp["x"], dout, inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm, cfg.Es,
                          bf16=True)
    assert N.rel_l2(dx2, ref2["dx"]) < 1e-2
    layer.close()


@pytest.mark.parametrize("name,kw,block", [
    ("c2_mixtral", dict(T=300, d=256, H=384), False),
    ("c4_finegrained", dict(T=200, d=256, H=256, E=16, K=4, Es=2), True),     # shared experts, block form
    ("c5_skewed", dict(T=257, d=512, H=256, E=32, K=4), False),               # experts without rows
])
def test_backward_bf16_same_bits_in_both_gather_modes(name, kw, block):
    """A backward pass needs the gathered rows of x.  When the forward pass left them to the loads of the up product
    (omega_moe_set_gather_mode ON_LOAD) the copy is made on demand: input gradient and every parameter gradient carry
    the same bits as after a forward pass that wrote the copy itself, in the plain and in the block form."""
    G, cfg, inp, dout, layer = _setup(name, kw, 53)
    if block:
        layer.set_norm((1.0 + 0.1 * O.fill_normal(cfg.d, 17, 901, 1.0)).astype(np.float32))
    x = G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype)
    g = G.P.DeviceBuffer.from_numpy(G.ctx(), dout, cfg.dtype)
    got = {}
    for mode in (1, 2):
        layer.set_gather_mode(mode)
        out = (layer.forward_block(x) if block else layer.forward(x)).to_numpy()
        assert layer.gather_on_load() == (mode == 2)
        dx = (layer.back_block(g) if block else layer.back(g)).to_numpy()
        got[mode] = [out, dx] + _all_grads(layer, cfg, block)
    assert len(got[1]) == len(got[2])
    for a, b in zip(got[1], got[2]):
        assert np.array_equal(a, b)
    layer.close()


def test_backward_full_size_mixtral():
    """C2 at full size.  Rows of a token depend on that token only: input gradient and dlogits of sampled tokens against
    the oracle (with the experts those tokens use).  Weight gradients of every expert through bilinear probes:
    u^T dW v = sum_r (delta_r . u)(input_r . v) over the expert's rows, with delta and input taken from the workspace
    (dy is recomputed on the host from dout, the combine weights and the permutation)."""
    from tests import gpu_util as G
    P = G.P
    cfg = C.CONFIGS["c2_mixtral"]
    T, d, H, E, K = cfg.T, cfg.d, cfg.H, cfg.E, cfg.K
    layer = P.MoELayer(d, H, E, K, renorm=cfg.renorm, nShared=cfg.Es, bias=cfg.has_gate_bias, ctx=G.ctx(), dtype=cfg.dtype,
                       router_mode="exact", T_max=T)
    layer.init_synthetic(77, C, cfg)
    x = P.DeviceBuffer(G.ctx(), (T, d), cfg.dtype)
    x.fill_normal(77, C.STREAM_X, C.tensor_std(cfg, "x"))
    g = P.DeviceBuffer(G.ctx(), (T, d), cfg.dtype)
    g.fill_normal(77, 900, 1.0)
    layer.forward(x)
    dx = layer.back(g).to_numpy()
    assert np.isfinite(dx).all()
    xh, gh = x.to_numpy(), g.to_numpy()
    r = layer.routing()
    Wg = layer._download_weight(L.W_GATE, 0, (E, d))
    p = O.softmax(O.gate(xh, Wg, None))
    # ---- sampled tokens against the oracle
    tok = np.unique(np.linspace(0, T - 1, 5).astype(np.int64))
    need = sorted(set(r["ids"][tok].ravel().tolist()))
    remap = {e: i for i, e in enumerate(need)}
    wid = np.vectorize(remap.get)(r["ids"][tok]).astype(np.int32)
    W1 = np.stack([layer._download_weight(L.W_W1, e, (H, d)) for e in need])
    W3 = np.stack([layer._download_weight(L.W_W3, e, (H, d)) for e in need])
    W2 = np.stack([layer._download_weight(L.W_W2, e, (d, H)) for e in need])
    ref = O.moe_backward_routed(xh[tok], gh[tok], Wg, p[tok], r["ids"][tok], wid, r["w"][tok], W1, W3, W2, 0, cfg.renorm,
                                bf16=True)
    del W1, W3, W2
    assert N.rel_l2(dx[tok], ref["dx"]) < 1e-2, N.rel_l2(dx[tok], ref["dx"])
    dlog = layer.workspace("dlogits", T)
    assert N.rel_l2(dlog[tok], ref["dlogits"]) < 1e-2
    # ---- gate weight gradient: all tokens
    rng = np.random.default_rng(5)
    u, v = rng.standard_normal((4, E)), rng.standard_normal((4, d))
    dWg = layer.grad(L.W_GATE).astype(np.float64)
    want = np.array([((dlog @ u[i]) * (xh @ v[i])).sum() for i in range(4)])
    got = np.array([u[i] @ dWg @ v[i] for i in range(4)])
    assert N.rel_l2(got, want) < 1e-3, (got, want)
    # ---- expert weight gradients: every expert, all its rows
    a = layer.workspace("a", T)            # [P,H]
    xg = layer.workspace("xg", T)          # [P,d]
    dh = layer.workspace("dh", T)          # [P,2H]
    dy = np.empty((T * K, d), np.float32)  # dy[dst[p]] = bf16(w[p] * dout[t])
    wflat = r["w"].reshape(-1)
    dy[r["dst"]] = O.round_bf16(wflat[:, None] * np.repeat(gh, K, axis=0))
    off = r["offsets"]
    ud, vH = rng.standard_normal(d), rng.standard_normal(H)
    uH, vd = rng.standard_normal(H), rng.standard_normal(d)
    got2, want2, got1, want1, got3, want3 = [], [], [], [], [], []
    for e in range(E):
        rows = slice(off[e], off[e + 1])
        dW2 = layer.grad(L.W_W2, e)
        got2.append(ud @ (dW2.astype(np.float64) @ vH))
        want2.append(((dy[rows].astype(np.float64) @ ud) * (a[rows].astype(np.float64) @ vH)).sum())
        xv = xg[rows].astype(np.float64) @ vd
        dW1 = layer.grad(L.W_W1, e)
        got1.append(uH @ (dW1.astype(np.float64) @ vd))
        want1.append(((dh[rows, :H].astype(np.float64) @ uH) * xv).sum())
        dW3 = layer.grad(L.W_W3, e)
        got3.append(uH @ (dW3.astype(np.float64) @ vd))
        want3.append(((dh[rows, H:].astype(np.float64) @ uH) * xv).sum())
    for gt, wt, nm in ((got2, want2, "dW2"), (got1, want1, "dW1"), (got3, want3, "dW3")):
        assert N.rel_l2(np.array(gt), np.array(wt)) < 1e-3, (nm, gt, wt)
    layer.close()


def test_backward_call_order_and_growth():
    """Error paths and workspace growth: a backward pass must follow a plain forward of the same T; a larger batch after a
    smaller one regrows both workspaces, in training mode too."""
    G, cfg, inp, dout, layer = _setup("c2_mixtral", dict(T=64, d=256, H=256, E=4, K=2), 3)
    P = G.P
    x = P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype)
    g = P.DeviceBuffer.from_numpy(G.ctx(), dout, cfg.dtype)
    layer.set_norm(np.ones(cfg.d, np.float32))
    layer.forward_block(x)
    with pytest.raises(RuntimeError):          # the block form has no backward pass
        layer.back(g)
    layer.forward(x)
    layer.stage("router", x)
    with pytest.raises(RuntimeError):          # a stage run on its own invalidates the forward
        layer.back(g)
    layer.forward(x)
    dx_small = layer.back(g).to_numpy()
    # a batch four times as large (new workspace), training mode on, then the small one again
    cfg2 = scaled(cfg, T=256)
    inp2 = make_inputs(cfg2, 4)
    dout2 = O.round_bf16(O.fill_normal(cfg2.T * cfg2.d, 4, 900, 1.0).reshape(cfg2.T, cfg2.d))
    x2 = P.DeviceBuffer.from_numpy(G.ctx(), inp2["x"], cfg.dtype)
    g2 = P.DeviceBuffer.from_numpy(G.ctx(), dout2, cfg.dtype)
    layer.set_training(True)
    layer.forward(x2)
    dx2 = layer.back(g2).to_numpy()
    ref2 = O.moe_backward(inp2["x"], dout2, inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm, cfg.Es,
                          bf16=True)
    assert N.rel_l2(dx2, ref2["dx"]) < 1e-2
    assert N.rel_l2(layer.grad(L.W_W2, 1), ref2["dW2"][1]) < 1e-2
    layer.forward(x)
    assert np.array_equal(layer.back(g).to_numpy(), dx_small)
    # an empty batch is a no-op for every pass (and leaves the saved forward alone)
    assert layer.lib.omega_moe_forward(layer.handle, None, 0, None) == 0
    assert layer.lib.omega_moe_backward(layer.handle, None, None, 0, None) == 0
    assert layer.lib.omega_moe_backward_block(layer.handle, None, None, 0, None) == 0
    assert np.array_equal(layer.back(g).to_numpy(), dx_small)
    layer.close()


def test_update_bf16_keeps_fp32_masters():
    """Two plain updates of a bf16 layer: the weights are the re-rounded fp32 masters w0 - lr*g1 - lr*g2, not a chain of
    bf16 roundings; a backward pass straight after an update raises (the forward pass must run again); new weights
    restart the masters."""
    G, cfg, inp, dout, layer = _setup("c2_mixtral", dict(T=96, d=256, H=256, E=4, K=2), 13)
    P = G.P
    x = P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype)
    g = P.DeviceBuffer.from_numpy(G.ctx(), dout, cfg.dtype)
    lr = 0.37
    shapes = {"W1": (L.W_W1, (cfg.H, cfg.d)), "W3": (L.W_W3, (cfg.H, cfg.d)), "W2": (L.W_W2, (cfg.d, cfg.H))}
    w0 = {k: layer._download_weight(w, 2, s) for k, (w, s) in shapes.items()}
    w0["Wg"] = layer._download_weight(L.W_GATE, 0, (cfg.E, cfg.d))
    grads = []
    for step in range(2):
        layer.forward(x)
        layer.back(g)
        gr = {k: layer.grad(w, 2) for k, (w, s) in shapes.items()}
        gr["Wg"] = layer.grad(L.W_GATE)
        grads.append(gr)
        layer.update(lr)
        with pytest.raises(RuntimeError):
            layer.back(g)
    for k in ("W1", "W3", "W2", "Wg"):
        got = layer._download_weight(*((shapes[k][0], 2, shapes[k][1]) if k != "Wg" else (L.W_GATE, 0, (cfg.E, cfg.d))))
        m = w0[k].copy()
        for gr in grads:
            m = (np.float32(-lr) * gr[k] + m).astype(np.float32)     # one rounding per step: fused multiply-add
        want = O.round_bf16(m)
        chain = O.round_bf16(O.round_bf16(w0[k] - np.float32(lr) * grads[0][k]) - np.float32(lr) * grads[1][k])
        # fused vs unfused multiply-add may move a value by one bf16 step when it sits on a rounding boundary
        close = np.abs(got - want) <= np.abs(want) * 2.0 ** -7
        assert close.all() and (got == want).mean() > 0.999, (k, (got == want).mean())
        assert (got == want).mean() > (got == chain).mean()          # masters, not re-rounded bf16 weights
    # the next forward / backward uses the updated weights (transposed copies rebuilt)
    for e in range(cfg.E):
        for k, (w, s) in shapes.items():
            inp[k][e] = layer._download_weight(w, e, s)
    inp["Wg"] = layer._download_weight(L.W_GATE, 0, (cfg.E, cfg.d))
    layer.forward(x)
    dx = layer.back(g).to_numpy()
    ref = O.moe_backward(inp["x"], dout, inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm, cfg.Es,
                         bf16=True)
    assert N.rel_l2(dx, ref["dx"]) < 1e-2
    assert N.rel_l2(layer.grad(L.W_W1, 0), ref["dW1"][0]) < 1e-2
    # setting a weight restarts the masters from the weights
    layer.set_expert(2, inp["W1"][2], inp["W3"][2], w0["W2"])
    layer.forward(x)
    layer.back(g)
    g2 = layer.grad(L.W_W2, 2)
    layer.update(lr)
    got = layer._download_weight(L.W_W2, 2, (cfg.d, cfg.H))
    want = O.round_bf16((np.float32(-lr) * g2 + w0["W2"]).astype(np.float32))
    assert (got == want).mean() > 0.999
    layer.close()


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_sgd_steps_reduce_a_regression_loss(dtype):
    """forward -> back(out - target) -> update, a few times: the squared error to a fixed target goes down
    (the layer trains with the plain update, fp32 and bf16 with master weights)."""
    G, cfg, inp, _, layer = _setup("c2_mixtral", dict(T=128, d=256, H=256, E=4, K=2, dtype=dtype), 23)
    P = G.P
    bf = dtype == "bf16"
    x = P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype)
    target = O.fill_normal(cfg.T * cfg.d, 23, 901, 0.5).reshape(cfg.T, cfg.d)
    losses = []
    layer.set_training(True)
    for step in range(8):
        out = layer.forward(x).to_numpy()
        diff = (out - target).astype(np.float32)
        losses.append(float(0.5 * (diff.astype(np.float64) ** 2).sum()))
        g = P.DeviceBuffer.from_numpy(G.ctx(), O.round_bf16(diff) if bf else diff, cfg.dtype)
        layer.back(g)
        layer.update(2e-3)
        g.free()
    assert all(b < a for a, b in zip(losses, losses[1:])), losses
    assert losses[-1] < 0.8 * losses[0], losses
    layer.close()


def _all_grads(layer, cfg, with_norm):
    out = [layer.grad(L.W_GATE)]
    if cfg.zipf_bias:
        out.append(layer.grad(L.W_GATE_BIAS))
    if with_norm:
        out.append(layer.grad(L.W_NORM))
    for g in range(cfg.E + cfg.Es):
        out += [layer.grad(L.W_W1, g), layer.grad(L.W_W3, g), layer.grad(L.W_W2, g)]
    return out


@pytest.mark.parametrize("name,kw,block", [
    ("c1_tiny_f32", dict(T=50, d=48, H=40, E=16, K=2, zipf_bias=1.2), False),
    ("c1_tiny_f32", dict(T=96, d=64, H=48, E=6, K=3, renorm=False, Es=2), True),
    ("c2_mixtral", dict(T=300, d=256, H=384), True),
])
def test_grad_norm_and_clipping(name, kw, block):
    """The layer's part of Network.clipGradNorm: its sum of squares against float64 over every gradient tensor read
    back one by one, the same bits twice, and the scaling exact (one fp32 product per element), on the gradients and,
    once accGrad has run, on the accumulators."""
    G, cfg, inp, dout, layer = _setup(name, kw, 17)
    x = G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype)
    g = G.P.DeviceBuffer.from_numpy(G.ctx(), dout, cfg.dtype)
    with pytest.raises(RuntimeError):
        layer.gradSumSq()                     # no backward yet
    if block:
        layer.set_norm((1.0 + 0.1 * O.fill_normal(cfg.d, 17, 901, 1.0)).astype(np.float32))
        layer.forward_block(x)
        layer.back_block(g)
    else:
        layer.forward(x)
        layer.back(g)
    grads = _all_grads(layer, cfg, block)
    want = sum(float((a.astype(np.float64) ** 2).sum()) for a in grads)
    got = layer.gradSumSq()
    assert abs(got - want) <= 2e-6 * want, (got, want)
    assert layer.gradSumSq() == got
    # a clip below the norm: coefficient as Network.clipGradNorm forms it, every tensor scaled by exactly that float
    clip = 0.5 * np.sqrt(want)
    coef = layer.clipGradNorm(clip)
    expect = np.float32(clip / (np.sqrt(np.float64(np.float32(got))) + np.float64(np.float32(1e-6))))
    assert coef == float(expect) and 0.49 < coef < 0.51
    after = _all_grads(layer, cfg, block)
    for a, b in zip(grads, after):
        assert np.array_equal(b, a * np.float32(coef))
    assert abs(layer.gradSumSq() - coef * coef * want) <= 1e-5 * want
    # a clip above the norm leaves everything alone
    assert layer.clipGradNorm(10.0 * np.sqrt(want)) == 1.0
    assert all(np.array_equal(a, b) for a, b in zip(after, _all_grads(layer, cfg, block)))
    # with accumulators the norm and the scaling are theirs: acc = grad, then acc += 1 * grad -> 4 x the sum of squares
    layer.accGrad(1.0)
    layer.accGrad(1.0)
    s_acc = layer.gradSumSq()
    assert abs(s_acc - 4 * coef * coef * want) <= 1e-5 * 4 * want
    layer.scaleGrad(0.5)
    assert abs(layer.gradSumSq() - coef * coef * want) <= 1e-5 * want
    assert all(np.array_equal(a, b) for a, b in zip(after, _all_grads(layer, cfg, block)))   # the plain gradients were not touched
    layer.close()


def test_empty_expert_gradients_stay_zero_across_passes_bf16():
    """An expert without rows has zero weight gradients.  The backward pass zeroes such a block once and then leaves
    it alone for as long as the expert stays empty; whatever writes the block in between - the expert getting rows
    again, update() bringing the accumulators in - must make the next pass zero it again."""
    G, cfg, inp, dout, layer = _setup("c2_mixtral", dict(T=96, d=256, H=256, E=4, K=2, zipf_bias=1.2), 41)
    x = G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype)
    g = G.P.DeviceBuffer.from_numpy(G.ctx(), dout, cfg.dtype)
    shut = inp["bg"].copy()
    shut[3] = -1e4                       # expert 3 never wins
    open_ = inp["bg"].copy()
    open_[:] = 0.0

    def run(bias):
        layer.set_gate(inp["Wg"], bias)
        layer.forward(x)
        layer.back(g)
        return int(layer.routing()["counts"][3]), layer.grad(L.W_W1, 3), layer.grad(L.W_W2, 3)

    n, g1, g2 = run(shut)
    assert n == 0 and not g1.any() and not g2.any()
    n, g1, g2 = run(shut)                # still empty: the block is left alone, and is still zero
    assert n == 0 and not g1.any() and not g2.any()
    n, g1, g2 = run(open_)               # rows again: real gradients
    assert n > 0 and g1.any() and g2.any()
    n, g1, g2 = run(shut)                # empty again: zero again
    assert n == 0 and not g1.any() and not g2.any()
    # accumulators: a pass with rows, then an empty one; update() copies the accumulated (non-zero) gradients into the
    # gradient block, so the next empty pass has to zero it afresh
    run(open_)
    layer.accGrad(1.0)
    n, g1, _ = run(shut)
    assert n == 0 and not g1.any()
    layer.accGrad(1.0)
    layer.update(1e-3)
    assert layer.grad(L.W_W1, 3).any()   # the block now holds the accumulated gradient of the pass with rows
    n, g1, g2 = run(shut)
    assert n == 0 and not g1.any() and not g2.any()
    layer.close()
