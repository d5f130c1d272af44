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
