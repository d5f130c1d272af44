"""The layer at the limits the library accepts (E = 256 routed experts, K = 64 slots, Es = 64 shared experts) and just
past them (refused with a message), forward and backward, against the oracle."""
import importlib

import numpy as np
import pytest

from oracle import oracle as O
from oracle import oracle_np as N
from tests.synth import C, make_inputs

pytestmark = pytest.mark.gpu
L = importlib.import_module("omega-ai_amd._lib")

CASES = [
    C.MoEConfig("lim", T=9, d=32, E=256, K=64, H=16, Es=0, dtype="f32"),
    C.MoEConfig("lim", T=5, d=24, E=12, K=3, H=8, Es=64, renorm=False, dtype="f32"),
    C.MoEConfig("lim", T=40, d=256, E=256, K=16, H=256, Es=1, dtype="bf16", zipf_bias=1.2),
    C.MoEConfig("lim", T=700, d=256, E=2, K=2, H=256, Es=3, dtype="bf16"),       # K = E: every expert takes every token
]


@pytest.mark.parametrize("cfg", CASES, ids=lambda c: f"{c.dtype}-E{c.E}-K{c.K}-Es{c.Es}")
def test_limits_forward_and_backward(cfg):
    from tests import gpu_util as G
    bf = cfg.dtype == "bf16"
    inp = make_inputs(cfg, 3)
    inp["Wg"] = inp["Wg"] * np.float32(8.0)
    dout = O.fill_normal(cfg.T * cfg.d, 3, 900, 1.0).reshape(cfg.T, cfg.d)
    if bf:
        dout = O.round_bf16(dout)
    layer = G.build_layer(cfg, inp)
    x = G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype)
    g = G.P.DeviceBuffer.from_numpy(G.ctx(), dout, cfg.dtype)
    out = layer.forward(x).to_numpy()
    ref = G.oracle_forward(cfg, inp)
    G.assert_routing_bit_exact(layer.routing(), ref)
    tol = 1e-2 if bf else 1e-5
    assert N.rel_l2(out, ref["out"]) < tol
    dx = layer.back(g).to_numpy()
    bw = O.moe_backward(inp["x"], dout, inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm, cfg.Es,
                        bf16=bf)
    assert N.rel_l2(dx, bw["dx"]) < tol
    assert N.rel_l2(layer.grad(L.W_GATE), bw["dWg"]) < tol
    for e in (0, cfg.E - 1, cfg.E + cfg.Es - 1):
        for which, k in ((L.W_W1, "dW1"), (L.W_W3, "dW3"), (L.W_W2, "dW2")):
            got = layer.grad(which, e)
            if bw[k][e].any():
                assert N.rel_l2(got, bw[k][e]) < tol, (k, e)
            else:
                assert not got.any(), (k, e)
    layer.close()


def test_past_the_limits_is_refused():
    from tests import gpu_util as G
    for kw in (dict(nExperts=257, topK=2), dict(nExperts=100, topK=65), dict(nExperts=8, topK=2, nShared=65),
               dict(nExperts=8, topK=9)):
        a = dict(embedDim=32, hidden=16, nExperts=8, topK=2, nShared=0)
        a.update(kw)
        with pytest.raises(RuntimeError, match="Error code"):
            G.P.MoELayer(a["embedDim"], a["hidden"], a["nExperts"], a["topK"], nShared=a["nShared"], ctx=G.ctx())
