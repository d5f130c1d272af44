"""Seeded random sweep over small layer shapes (both dtypes, E from 1 to 130, K up to 8, shared experts, token counts
around the tile sizes, skewed and uniform gates): routing bit for bit, outputs within tolerance, reruns identical."""
import numpy as np
import pytest

from oracle import oracle_np as N
from tests.synth import C, make_inputs

pytestmark = pytest.mark.gpu


def _cases(seed, n):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(n):
        bf = rng.random() < 0.75
        E = int(rng.choice([1, 2, 3, 8, 16, 40, 64, 130]))
        K = int(rng.integers(1, min(E, 8) + 1))
        cfg = C.MoEConfig("r", T=int(rng.choice([1, 2, 31, 33, 255, 257, 700, 1500, 3000])),
                          d=int(rng.choice([256, 512])) if bf else int(rng.choice([64, 100, 256])), E=E, K=K,
                          H=int(rng.choice([256, 384, 640])) if bf else int(rng.choice([48, 128, 200])),
                          Es=int(rng.choice([0, 0, 1, 2])), renorm=bool(rng.random() < 0.5),
                          dtype="bf16" if bf else "f32", zipf_bias=1.2 if rng.random() < 0.3 else 0.0)
        out.append((cfg, int(rng.integers(1, 1 << 30))))
    return out


@pytest.mark.parametrize("cfg,seed", _cases(2025, 24), ids=lambda v: f"{v.dtype}-T{v.T}-d{v.d}-E{v.E}-K{v.K}-H{v.H}-Es{v.Es}" if hasattr(v, "dtype") else str(v))
def test_random_shape(cfg, seed):
    from tests import gpu_util as G
    inp = make_inputs(cfg, seed)
    layer = G.build_layer(cfg, inp)
    x = G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype)
    out = layer.forward(x).to_numpy()
    ref = G.oracle_forward(cfg, inp)
    G.assert_routing_bit_exact(layer.routing(), ref)
    assert N.rel_l2(out, ref["out"]) < (1e-2 if cfg.dtype == "bf16" else 1e-5)
    assert np.array_equal(layer.forward(x).to_numpy(), out)
    layer.close()
    x.free()


def _bw_cases(seed, n):
    rng = np.random.default_rng(seed)
    out = []
    while len(out) < n:
        bf = rng.random() < 0.7
        E = int(rng.choice([1, 2, 5, 8, 24, 64]))
        K = int(rng.integers(1, min(E, 4) + 1))
        Es = int(rng.choice([0, 0, 1, 2]))
        T = int(rng.choice([1, 2, 33, 100, 257, 400]))
        if T * (K + Es) > 1300:
            continue
        cfg = C.MoEConfig("rb", T=T, d=int(rng.choice([256, 512])) if bf else int(rng.choice([30, 64, 100])), E=E, K=K,
                          H=int(rng.choice([256, 384, 512])) if bf else int(rng.choice([24, 48, 96])), Es=Es,
                          renorm=bool(rng.random() < 0.5), dtype="bf16" if bf else "f32",
                          zipf_bias=1.2 if rng.random() < 0.3 else 0.0)
        out.append((cfg, int(rng.integers(1, 1 << 30)), bool(rng.random() < 0.5)))
    return out


@pytest.mark.parametrize("cfg,seed,training", _bw_cases(77, 16),
                         ids=lambda v: f"{v.dtype}-T{v.T}-d{v.d}-E{v.E}-K{v.K}-H{v.H}-Es{v.Es}" if hasattr(v, "dtype") else str(v))
def test_random_shape_backward(cfg, seed, training):
    import importlib
    from oracle import oracle as O
    from tests import gpu_util as G
    L = importlib.import_module("omega-ai_amd._lib")
    inp = make_inputs(cfg, seed)
    inp["Wg"] = inp["Wg"] * np.float32(8.0)
    bf = cfg.dtype == "bf16"
    dout = O.fill_normal(cfg.T * cfg.d, seed, 900, 1.0).reshape(cfg.T, cfg.d)
    if bf:
        dout = O.round_bf16(dout)
    layer = G.build_layer(cfg, inp)
    layer.set_training(training)
    x = G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype)
    g = G.P.DeviceBuffer.from_numpy(G.ctx(), dout, cfg.dtype)
    layer.forward(x)
    dx = layer.back(g).to_numpy()
    ref = O.moe_backward(inp["x"], dout, inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm, cfg.Es,
                         bf16=bf)
    tol = 1e-2 if bf else 1e-5
    assert N.rel_l2(dx, ref["dx"]) < tol
    assert N.rel_l2(layer.grad(L.W_GATE), ref["dWg"]) < tol
    if ref["dbg"] is not None:
        assert N.rel_l2(layer.grad(L.W_GATE_BIAS), ref["dbg"]) < tol
    for e in range(cfg.E + cfg.Es):
        for which, k in ((L.W_W1, "dW1"), (L.W_W3, "dW3"), (L.W_W2, "dW2")):
            got = layer.grad(which, e)
            if not ref[k][e].any():
                assert not got.any(), (k, e)
            else:
                assert N.rel_l2(got, ref[k][e]) < tol, (k, e)
    layer.close()
    x.free()
    g.free()
