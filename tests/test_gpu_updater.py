"""AdamW update through the C ABI against the updater oracle (which torch.optim.AdamW in float64 and closed forms pin):
every parameter tensor after each of several steps, bit for bit - the step is a fixed sequence of IEEE operations
(fused multiply-add, multiply, divide, square root), the same on both machines.  bf16 layers: the step is taken on
fp32 masters and the weights read back are the masters re-rounded."""
import importlib

import numpy as np
import pytest

from oracle import oracle as O
from oracle import oracle_np as N
from tests.synth import C, make_inputs, scaled

pytestmark = pytest.mark.gpu
L = importlib.import_module("omega-ai_amd._lib")


def _tensors(cfg, block):
    t = [("Wg", L.W_GATE, 0, (cfg.E, cfg.d))]
    if cfg.zipf_bias:
        t.append(("bg", L.W_GATE_BIAS, 0, (cfg.E,)))
    if block:
        t.append(("gamma", L.W_NORM, 0, (cfg.d,)))
    for g in range(cfg.E + cfg.Es):
        t += [(f"W1[{g}]", L.W_W1, g, (cfg.H, cfg.d)), (f"W3[{g}]", L.W_W3, g, (cfg.H, cfg.d)), (f"W2[{g}]", L.W_W2, g, (cfg.d, cfg.H))]
    return t


@pytest.mark.parametrize("name,kw,block", [
    ("c1_tiny_f32", dict(T=50, d=48, H=40, E=6, K=2, zipf_bias=1.2), False),
    ("c1_tiny_f32", dict(T=64, d=64, H=48, E=4, K=2, Es=1, renorm=False), True),
    ("c2_mixtral", dict(T=200, d=256, H=384, E=4, K=2), False),
    ("c5_skewed", dict(T=150, d=256, H=256, E=8, K=3, Es=1), True),
])
def test_adamw_steps_match_oracle(name, kw, block):
    from tests import gpu_util as G
    cfg = scaled(C.CONFIGS[name], **kw)
    bf = cfg.dtype == "bf16"
    inp = make_inputs(cfg, 23)
    inp["Wg"] = inp["Wg"] * np.float32(8.0)
    layer = G.build_layer(cfg, inp)
    gamma0 = (1.0 + 0.1 * O.fill_normal(cfg.d, 23, 901, 1.0)).astype(np.float32)
    if block:
        layer.set_norm(gamma0)
    x = G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype)
    tensors = _tensors(cfg, block)
    with pytest.raises(RuntimeError):
        layer.updateAdamW(1e-2, 1)                       # no backward yet
    # the oracle's state: masters (= the weights as the layer holds them at the start), moments
    master = {k: layer._download_weight(w, g, s) for k, w, g, s in tensors}
    mom = {k: (np.zeros(s, np.float32), np.zeros(s, np.float32)) for k, _, _, s in tensors}
    lr, b1, b2, wd = 3e-3, 0.9, 0.95, 1e-2
    first = {k: v.copy() for k, v in master.items()}
    for t in (1, 2, 3):
        dout = O.fill_normal(cfg.T * cfg.d, 23, 900 + t, 1.0).reshape(cfg.T, cfg.d)
        if bf:
            dout = O.round_bf16(dout)
        g = G.P.DeviceBuffer.from_numpy(G.ctx(), dout, cfg.dtype)
        if block:
            layer.forward_block(x)
            layer.back_block(g)
        else:
            layer.forward(x)
            layer.back(g)
        grads = {k: layer.grad(w, e) for k, w, e, _ in tensors}
        layer.updateAdamW(lr, t, b1, b2, wd)
        with pytest.raises(RuntimeError):                # the forward pass must run again
            layer.back(g)
        for k, w, e, s in tensors:
            master[k], m, v = O.adamw(master[k], grads[k], *mom[k], lr, b1, b2, wd, t)
            mom[k] = (m, v)
            got = layer._download_weight(w, e, s)
            # the gate bias and the norm weight are fp32 in bf16 layers too
            want = O.round_bf16(master[k]) if bf and w not in (L.W_GATE_BIAS, L.W_NORM) else master[k]
            assert np.array_equal(got, want), (k, t, float(np.abs(got - want).max()))
    # three steps of at most lr each (plus decay) moved the parameters, and in fp32 by about lr per step
    if not bf:
        moved = np.abs(master["W1[0]"] - first["W1[0]"])
        assert 0.5 * lr < np.median(moved) <= 3.2 * lr
    layer.close()


def test_adamw_uses_accumulated_gradients_and_rejects_bad_arguments():
    from tests import gpu_util as G
    cfg = scaled(C.CONFIGS["c1_tiny_f32"], T=40, d=32, H=24, E=4, K=2)
    inp = make_inputs(cfg, 29)
    layer = G.build_layer(cfg, inp)
    x = G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype)
    dout = O.fill_normal(cfg.T * cfg.d, 29, 900, 1.0).reshape(cfg.T, cfg.d)
    g = G.P.DeviceBuffer.from_numpy(G.ctx(), dout, cfg.dtype)
    layer.forward(x)
    layer.back(g)
    gW = layer.grad(L.W_W2, 1)
    w0 = layer._download_weight(L.W_W2, 1, (cfg.d, cfg.H))
    layer.accGrad(1.0)
    layer.accGrad(0.5)                                    # acc = 1.5 * grad
    for bad in (dict(train_time=0), dict(train_time=1, beta1=1.0), dict(train_time=1, beta2=-0.1)):
        with pytest.raises(RuntimeError):
            layer.updateAdamW(1e-2, **bad)
    layer.updateAdamW(1e-2, 1, weight_decay=0.0)
    acc = (np.float32(0.5) * gW + gW).astype(np.float32)
    want, _, _ = O.adamw(w0, acc, np.zeros_like(w0), np.zeros_like(w0), 1e-2, 0.9, 0.95, 0.0, 1)
    assert np.array_equal(layer._download_weight(L.W_W2, 1, (cfg.d, cfg.H)), want)
    layer.close()


def test_adamw_training_reduces_a_regression_loss_bf16():
    """A few AdamW steps on a fixed batch towards a target: the loss falls (the whole chain forward -> back ->
    updateAdamW -> forward on bf16 weights re-rounded from the masters works together)."""
    from tests import gpu_util as G
    cfg = scaled(C.CONFIGS["c2_mixtral"], T=128, d=256, H=256, E=4, K=2)
    inp = make_inputs(cfg, 37)
    layer = G.build_layer(cfg, inp)
    layer.set_training(True)
    x = G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype)
    target = O.round_bf16(O.fill_normal(cfg.T * cfg.d, 37, 950, 0.5).reshape(cfg.T, cfg.d))
    losses = []
    for t in range(1, 9):
        out = layer.forward(x).to_numpy()
        diff = (out - target).astype(np.float32)
        losses.append(float((diff.astype(np.float64) ** 2).mean()))
        g = G.P.DeviceBuffer.from_numpy(G.ctx(), O.round_bf16(diff * np.float32(2.0 / diff.size * cfg.T)), cfg.dtype)
        layer.back(g)
        layer.updateAdamW(2e-3, t, weight_decay=0.0)
        g.free()
    assert losses[-1] < 0.8 * losses[0] and all(np.isfinite(losses)), losses
    layer.close()
