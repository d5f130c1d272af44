"""JSON weight import (host logic, CPU only): names of the three schemes, layout, error behaviour."""
import importlib
import json

import numpy as np
import pytest

W = importlib.import_module("omega-ai_amd.weights_json")


class FakeLayer:
    """Records what the loader hands to the layer."""

    def __init__(self, d, H, E, Es, bias=False):
        self.embedDim, self.hidden, self.nExperts, self.nShared, self.hasBias = d, H, E, Es, bias
        self.gate = self.bias = self.norm = None
        self.experts = {}

    def set_gate(self, Wg, bg=None):
        self.gate, self.bias = Wg, bg

    def set_expert(self, g, W1, W3, W2):
        self.experts[g] = (W1, W3, W2)

    def set_norm(self, gamma):
        self.norm = gamma


def _arrays(d, H, E, Es, bias, seed=0):
    r = np.random.default_rng(seed)
    f = lambda *s: r.standard_normal(s).astype(np.float32)
    return dict(Wg=f(E, d), bg=f(E) if bias else None, W1=f(E + Es, H, d), W3=f(E + Es, H, d), W2=f(E + Es, d, H))


@pytest.mark.parametrize("scheme,Es,bias", [("omega", 2, True), ("omega", 0, False), ("mixtral", 0, False),
                                            ("deepseek", 2, True), ("deepseek", 0, False)])
def test_round_trip_through_json_text(scheme, Es, bias, tmp_path):
    d, H, E = 6, 4, 3
    a = _arrays(d, H, E, Es, bias)
    gamma = np.linspace(0.5, 1.5, d).astype(np.float32)
    p = tmp_path / "w.json"
    p.write_text(json.dumps(W.export_moe_weights(a, layer_index=5, scheme=scheme, gamma=gamma)))
    lay = FakeLayer(d, H, E, Es, bias)
    missing = W.load_moe_weights(lay, str(p), layer_index=5, scheme=scheme)
    assert missing == []
    assert np.array_equal(lay.gate, a["Wg"]) and np.array_equal(lay.norm, gamma)
    assert (lay.bias is None) == (not bias) and (not bias or np.array_equal(lay.bias, a["bg"]))
    assert sorted(lay.experts) == list(range(E + Es))
    for g in range(E + Es):          # [out,in] row-major, float32, exactly the exported values
        for got, want in zip(lay.experts[g], (a["W1"][g], a["W3"][g], a["W2"][g])):
            assert got.dtype == np.float32 and got.flags["C_CONTIGUOUS"] and np.array_equal(got, want)


def test_hf_names_and_fused_shared_split():
    d, H, E, Es = 4, 2, 2, 2
    a = _arrays(d, H, E, Es, False, seed=3)
    m = W.export_moe_weights(a, layer_index=1, scheme="deepseek")
    assert "model.layers.1.mlp.gate.weight" in m and "model.layers.1.mlp.experts.1.down_proj.weight" in m
    fused = np.asarray(m["model.layers.1.mlp.shared_experts.gate_proj.weight"])
    assert fused.shape == (Es * H, d)
    assert np.asarray(m["model.layers.1.mlp.shared_experts.down_proj.weight"]).shape == (d, Es * H)
    lay = FakeLayer(d, H, E, Es)
    W.load_moe_weights(lay, m, layer_index=1, scheme="deepseek", strict=False)
    assert np.array_equal(lay.experts[E + 1][0], a["W1"][E + 1]) and np.array_equal(lay.experts[E + 1][2], a["W2"][E + 1])
    mx = W.export_moe_weights(_arrays(d, H, E, 0, False), layer_index=0, scheme="mixtral")
    assert "model.layers.0.block_sparse_moe.experts.0.w3.weight" in mx


def test_dense_llama_names_for_a_single_expert():
    # the names Llama3Test uses for the dense FFN (J/example/transformer/test/Llama3Test.java:677-681)
    d, H = 4, 3
    a = _arrays(d, H, 1, 0, False, seed=5)
    m = {"layers.2.feed_forward.gate.weight": a["Wg"].tolist(), "layers.2.feed_forward.w1.weight": a["W1"][0].tolist(),
         "layers.2.feed_forward.w3.weight": a["W3"][0].tolist(), "layers.2.feed_forward.w2.weight": a["W2"][0].tolist(),
         "layers.2.ffn_norm.weight": [1.0] * d}
    lay = FakeLayer(d, H, 1, 0)
    assert W.load_moe_weights(lay, m, layer_index=2, scheme="omega") == []
    assert np.array_equal(lay.experts[0][2], a["W2"][0]) and np.array_equal(lay.norm, np.ones(d, np.float32))


def test_errors():
    d, H, E = 4, 2, 2
    a = _arrays(d, H, E, 0, False)
    m = W.export_moe_weights(a, scheme="mixtral")
    del m["model.layers.0.block_sparse_moe.experts.1.w2.weight"]
    with pytest.raises(RuntimeError, match="experts.1.w2.weight is null"):
        W.load_moe_weights(FakeLayer(d, H, E, 0), m, scheme="mixtral")
    lay = FakeLayer(d, H, E, 0)
    missing = W.load_moe_weights(lay, m, scheme="mixtral", strict=False)     # the reference's report-and-go-on
    assert "model.layers.0.block_sparse_moe.experts.1.w2.weight" in missing and 1 not in lay.experts and 0 in lay.experts
    assert "model.layers.0.post_attention_layernorm.weight" in missing       # optional: only the block form needs it
    m2 = W.export_moe_weights(a, scheme="mixtral")
    m2["model.layers.0.block_sparse_moe.gate.weight"] = a["Wg"].T.tolist()    # transposed: wrong layout must not pass
    with pytest.raises(RuntimeError, match="is not shape"):
        W.load_moe_weights(FakeLayer(d, H, E, 0), m2, scheme="mixtral")
    with pytest.raises(RuntimeError, match="shared"):
        W.load_moe_weights(FakeLayer(d, H, E, 1), W.export_moe_weights(a, scheme="mixtral"), scheme="mixtral")
    m3 = W.export_moe_weights(a, scheme="deepseek")
    m3["model.layers.0.mlp.shared_expert_gate.weight"] = [[0.0] * d]
    with pytest.raises(RuntimeError, match="shared_expert_gate"):
        W.load_moe_weights(FakeLayer(d, H, E, 0), m3, scheme="deepseek")
    with pytest.raises(ValueError):
        W.load_moe_weights(FakeLayer(d, H, E, 0), {}, scheme="nope")


def test_fused_w12_form_of_the_dit_ffn():
    """DiTSwiGLUFFN's parameters: w12 [2H, d] = [SiLU branch; multiplier], down projection named w3 [d, H]; for routed
    and shared experts and, with E == 1, under the dense names."""
    d, H, E, Es = 6, 4, 3, 1
    a = _arrays(d, H, E, Es, False, seed=9)
    m = W.export_moe_weights(a, layer_index=2, scheme="omega", fused12=True)
    k12 = "layers.2.feed_forward.experts.1.w12.weight"
    assert np.asarray(m[k12]).shape == (2 * H, d) and "layers.2.feed_forward.experts.1.w1.weight" not in m
    assert np.asarray(m["layers.2.feed_forward.experts.1.w3.weight"]).shape == (d, H)
    lay = FakeLayer(d, H, E, Es)
    assert W.load_moe_weights(lay, m, layer_index=2, scheme="omega") == ["layers.2.ffn_norm.weight"]
    for g in range(E + Es):
        for got, want in zip(lay.experts[g], (a["W1"][g], a["W3"][g], a["W2"][g])):
            assert got.flags["C_CONTIGUOUS"] and np.array_equal(got, want)
    # the halves are not interchangeable: the first H rows are the SiLU branch
    assert np.array_equal(np.asarray(m[k12], np.float32)[:H], a["W1"][1])
    # a down projection of the wrong shape (the separate form's w3 [H, d]) is refused
    bad = dict(m)
    bad["layers.2.feed_forward.experts.0.w3.weight"] = a["W3"][0].tolist()
    with pytest.raises(RuntimeError, match="Error code"):
        W.load_moe_weights(FakeLayer(d, H, E, Es), bad, layer_index=2, scheme="omega")
    # dense names with one expert
    a1 = _arrays(d, H, 1, 0, False, seed=10)
    dense = {"layers.0.feed_forward.gate.weight": a1["Wg"].tolist(),
             "layers.0.feed_forward.w12.weight": np.concatenate([a1["W1"][0], a1["W3"][0]]).tolist(),
             "layers.0.feed_forward.w3.weight": a1["W2"][0].tolist()}
    lay1 = FakeLayer(d, H, 1, 0)
    W.load_moe_weights(lay1, dense, strict=False)
    assert np.array_equal(lay1.experts[0][0], a1["W1"][0]) and np.array_equal(lay1.experts[0][2], a1["W2"][0])
    with pytest.raises(ValueError):
        W.export_moe_weights(a, scheme="mixtral", fused12=True)
