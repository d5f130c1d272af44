"""JSON weight import into the real layer: weights read back byte for byte, forward and block form equal to the oracle."""
import importlib
import json

import numpy as np
import pytest

from oracle import oracle as O
from oracle import oracle_np as N
from tests.synth import C, make_inputs, scaled

pytestmark = pytest.mark.gpu
W = importlib.import_module("omega-ai_amd.weights_json")
L = importlib.import_module("omega-ai_amd._lib")


@pytest.mark.parametrize("name,kw,scheme", [("c1_tiny_f32", dict(T=64), "mixtral"),
                                            ("c4_finegrained", dict(T=96, d=256, H=256, E=8, K=3, Es=2), "deepseek"),
                                            ("c4_finegrained", dict(T=64, d=128, H=64, E=4, K=2, Es=1, dtype="f32"), "omega")])
def test_layer_loaded_from_json(name, kw, scheme, tmp_path):
    from tests import gpu_util as G
    cfg = scaled(C.CONFIGS[name], **kw)
    bf = cfg.dtype == "bf16"
    inp = make_inputs(cfg, 5)
    gamma = (O.fill_normal(cfg.d, 5, C.STREAM_NORM, 1.0) * np.float32(0.1) + np.float32(1.0)).astype(np.float32)
    path = tmp_path / "layer.json"
    path.write_text(json.dumps(W.export_moe_weights(dict(inp, bg=None), layer_index=3, scheme=scheme, gamma=gamma)))
    layer = G.P.MoELayer(cfg.d, cfg.H, cfg.E, cfg.K, renorm=cfg.renorm, nShared=cfg.Es, bias=False, ctx=G.ctx(),
                         dtype=cfg.dtype)
    assert layer.loadJson(str(path), layer_index=3, scheme=scheme) == []
    for g in range(cfg.E + cfg.Es):    # what the layer holds is what the file held (bf16 inputs are bf16-exact already)
        assert np.array_equal(layer._download_weight(L.W_W1, g, (cfg.H, cfg.d)), inp["W1"][g])
        assert np.array_equal(layer._download_weight(L.W_W2, g, (cfg.d, cfg.H)), inp["W2"][g])
    assert np.array_equal(layer._download_weight(L.W_GATE, 0, (cfg.E, cfg.d)), inp["Wg"])
    x = G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype)
    out = layer.forward(x).to_numpy()
    ref = O.moe_forward(inp["x"], inp["Wg"], None, inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm, cfg.Es, bf)
    G.assert_routing_bit_exact(layer.routing(), ref)
    assert N.rel_l2(out, ref["out"]) < (1e-2 if bf else 1e-5)
    blk = O.block_forward(inp["x"], gamma, inp["Wg"], None, inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm, cfg.Es, bf)
    assert N.rel_l2(layer.forward_block(x).to_numpy(), blk["out"]) < (1e-2 if bf else 1e-5)   # the norm weight came from the file
    layer.close()


def test_java_seeded_init_runs_through_the_layer():
    """initJava(seed): the weights RandomUtils.setSeed(seed) + the house-style initialisation would draw, set through the
    C ABI and read back bit for bit; the forward pass on them equals the oracle's."""
    import importlib
    from oracle import oracle as O
    from tests import gpu_util as G
    JR = importlib.import_module("omega-ai_amd.java_random")
    L = importlib.import_module("omega-ai_amd._lib")
    cfg = C.MoEConfig("j", T=50, d=32, E=4, K=2, H=24, Es=1, dtype="f32")
    layer = G.P.MoELayer(cfg.d, cfg.H, cfg.E, cfg.K, renorm=True, nShared=cfg.Es, ctx=G.ctx(), dtype="f32")
    arrays = layer.initJava(2024)
    flat = JR.JavaRandom(2024).normal_(cfg.E * cfg.d + 3 * (cfg.E + cfg.Es) * cfg.H * cfg.d, 0.01, 0.02)
    assert np.array_equal(layer._download_weight(L.W_GATE, 0, (cfg.E, cfg.d)).ravel(), flat[:cfg.E * cfg.d])
    o = cfg.E * cfg.d + 3 * cfg.H * cfg.d * 2            # expert 2: linear1, linear2, linear3
    n = cfg.H * cfg.d
    assert np.array_equal(layer._download_weight(L.W_W1, 2, (cfg.H, cfg.d)).ravel(), flat[o:o + n])
    assert np.array_equal(layer._download_weight(L.W_W2, 2, (cfg.d, cfg.H)).ravel(), flat[o + n:o + 2 * n])
    assert np.array_equal(layer._download_weight(L.W_W3, 2, (cfg.H, cfg.d)).ravel(), flat[o + 2 * n:o + 3 * n])
    x = O.fill_normal(cfg.T * cfg.d, 1, C.STREAM_X, 1.0).reshape(cfg.T, cfg.d)
    out = layer.forward(G.P.DeviceBuffer.from_numpy(G.ctx(), x, "f32")).to_numpy()
    ref = O.moe_forward(x, arrays["Wg"], None, arrays["W1"], arrays["W3"], arrays["W2"], cfg.K, True, cfg.Es)
    G.assert_routing_bit_exact(layer.routing(), ref)
    assert N.rel_l2(out, ref["out"]) < 1e-5
    layer.close()
