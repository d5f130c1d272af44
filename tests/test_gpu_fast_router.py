"""FAST router mode on the matrix cores (bf16 layers with more than 16 experts): logits within fp32 summation-order
noise of the oracle's, the same experts for all but near-tied tokens, exact dispatch of the ids it chose, output within
tolerance."""
import numpy as np
import pytest

from oracle import oracle as O
from oracle import oracle_np as N
from tests.synth import C, make_inputs, scaled

pytestmark = pytest.mark.gpu

CASES = [
    ("c4_finegrained", dict(T=300, d=256, H=256, E=32, K=4, Es=0)),      # one expert block, k split four ways, d = 256
    ("c4_finegrained", dict(T=257, d=768, H=256, E=64, K=6, Es=1)),      # two blocks, k split two ways, odd trip count
    ("c5_skewed", dict(T=1000, d=512, H=256, E=128, K=8)),                # four blocks, gate bias
    ("c5_skewed", dict(T=65, d=256, H=256, E=200, K=5)),                  # eight blocks (E padded to 256), ragged tile
    ("c4_finegrained", dict(T=33, d=256, H=256, E=17, K=2, Es=0)),        # just above the threshold
]


@pytest.mark.parametrize("name,kw", CASES)
def test_fast_router_on_matrix_cores(name, kw):
    from tests import gpu_util as G
    cfg = scaled(C.CONFIGS[name], **kw)
    inp = make_inputs(cfg, 91)
    layer = G.build_layer(cfg, inp, router_mode="fast")
    x = G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype)
    logits, probs = layer.router_probs(x, cfg.T)
    ref = G.oracle_forward(cfg, inp)
    assert N.rel_l2(logits, ref["logits"]) < 1e-5 and N.rel_l2(probs, ref["p"]) < 1e-5
    out = layer.forward(x).to_numpy()
    r = layer.routing()
    agree = (r["ids"] == ref["ids"]).all(axis=1).mean()
    assert agree >= 0.99, agree
    # weights of the tokens that agree, and the dispatch of whatever was chosen
    same = (r["ids"] == ref["ids"]).all(axis=1)
    assert np.allclose(r["w"][same], ref["w"][same], rtol=1e-4, atol=1e-7)
    c2, o2, d2, s2 = N.dispatch_argsort(r["ids"], cfg.E)
    assert np.array_equal(r["counts"], c2) and np.array_equal(r["dst"], d2) and np.array_equal(r["src_row"], s2)
    assert N.rel_l2(out, ref["out"]) <= 1e-2
    assert np.array_equal(layer.forward(x).to_numpy(), out)          # fixed summation order: reproducible
    layer.close()
