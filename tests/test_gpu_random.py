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
