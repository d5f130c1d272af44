"""Block form through the C ABI: out = x + layer(rmsnorm(x)) against the oracle.

Row statistics, routing of the normalised rows (ids, weights, counts, offsets, permutation) and the gathered
normalised rows are compared bit for bit; outputs to 1e-5 (fp32) / 1e-2 (bf16) relative L2.  The plain forward of the
same layer must be unaffected by a block call before it."""
import numpy as np
import pytest

from oracle import oracle as O
from oracle import oracle_np as N
from tests.synth import C, make_inputs, scaled

pytestmark = pytest.mark.gpu

SEED = 20251


def _gamma(d, seed):
    return (O.fill_normal(d, seed, C.STREAM_NORM, 1.0) * np.float32(0.1) + np.float32(1.0)).astype(np.float32)


CASES = [
    ("c1_tiny_f32", {}),
    ("c1_tiny_f32", dict(T=77, d=102, H=72)),                      # unaligned rows: element-wise paths
    ("c4_finegrained", dict(T=96, d=128, H=64, E=8, K=3, Es=2, dtype="f32")),   # shared experts read the normalised rows
    ("c2_mixtral", dict(T=300, d=256, H=384)),
    ("c4_finegrained", dict(T=200, d=256, H=256, E=16, K=4, Es=2)),
    ("c5_skewed", dict(T=257, d=512, H=256, E=32, K=4)),
]


@pytest.mark.parametrize("name,kw", CASES)
def test_block_forward_matches_oracle(name, kw):
    from tests import gpu_util as G
    cfg = scaled(C.CONFIGS[name], **kw)
    bf = cfg.dtype == "bf16"
    inp = make_inputs(cfg, 77)
    gamma = _gamma(cfg.d, 77)
    layer = G.build_layer(cfg, inp)
    with pytest.raises(RuntimeError):  # the norm weight has not been set yet
        layer.forward_block(G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype))
    layer.set_norm(gamma)
    x = G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype)
    out = layer.forward_block(x).to_numpy()
    ref = O.block_forward(inp["x"], gamma, inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm,
                          cfg.Es, bf)
    assert np.array_equal(layer.norm_rms().view(np.uint32), ref["rms"].view(np.uint32))
    r = layer.routing()
    G.assert_routing_bit_exact(r, ref)
    assert np.array_equal(layer.workspace("xg", cfg.T), ref["h"][ref["src_row"]])
    err = N.rel_l2(out, ref["out"])
    assert err < (1e-2 if bf else 1e-5), err
    # the same call again gives the same bits, and the plain forward is what it was
    assert np.array_equal(layer.forward_block(x).to_numpy(), out)
    plain = layer.forward(x).to_numpy()
    pref = G.oracle_forward(cfg, inp)
    G.assert_routing_bit_exact(layer.routing(), pref)
    assert N.rel_l2(plain, pref["out"]) < (1e-2 if bf else 1e-5)
    layer.close()


def test_block_forward_full_size_mixtral():
    """C2 at full size: statistics and routing of all tokens bit for bit, output on sampled tokens."""
    from tests import gpu_util as G
    P, L = G.P, __import__("importlib").import_module("omega-ai_amd._lib")
    cfg = C.CONFIGS["c2_mixtral"]
    layer = P.MoELayer(cfg.d, cfg.H, cfg.E, cfg.K, renorm=cfg.renorm, nShared=cfg.Es, bias=cfg.has_gate_bias,
                       ctx=G.ctx(), dtype=cfg.dtype, router_mode="exact", T_max=cfg.T)
    layer.init_synthetic(SEED, C, cfg)
    x = P.DeviceBuffer(G.ctx(), (cfg.T, cfg.d), cfg.dtype)
    x.fill_normal(SEED, C.STREAM_X, C.tensor_std(cfg, "x"))
    layer.fill_workspace("a", 0xFF)        # NaN: a valid row that the forward does not write cannot pass
    layer.fill_workspace("y", 0xFF)
    out = layer.forward_block(x).to_numpy()
    xh = x.to_numpy()
    gamma = _gamma(cfg.d, SEED)
    h, rms = O.rmsnorm(xh, gamma, True)
    assert np.array_equal(layer.norm_rms().view(np.uint32), rms.view(np.uint32))
    Wg = layer._download_weight(L.W_GATE, 0, (cfg.E, cfg.d))
    ids, w = O.topk(O.softmax(O.gate(h, Wg, None)), cfg.K, cfg.renorm)
    r = layer.routing()
    assert np.array_equal(r["ids"], ids)
    assert np.array_equal(r["w"].view(np.uint32), w.view(np.uint32))
    counts, offsets, dst, src = N.dispatch_argsort(ids, cfg.E)
    for k, v in (("counts", counts), ("offsets", offsets), ("dst", dst), ("src_row", src)):
        assert np.array_equal(r[k], v), k
    assert np.array_equal(layer.workspace("xg", cfg.T), h[src])
    # every work item of the two products (float64 spot checks on every 32-row block), then the oracle on a token
    # sample that touches every row tile
    assert G.check_products_every_block(layer, cfg, cfg.T, r, h) > 0
    tok = np.union1d(G.row_tile_tokens(r, cfg, cfg.T), np.linspace(0, cfg.T - 1, 6).astype(np.int32)).astype(np.int32)
    W1 = np.stack([layer._download_weight(L.W_W1, g, (cfg.H, cfg.d)) for g in range(cfg.E)])
    W3 = np.stack([layer._download_weight(L.W_W3, g, (cfg.H, cfg.d)) for g in range(cfg.E)])
    W2 = np.stack([layer._download_weight(L.W_W2, g, (cfg.d, cfg.H)) for g in range(cfg.E)])
    ref = G.oracle_tokens_parallel(
        lambda part: O.block_tokens(xh, h, r["ids"], r["w"], W1, W3, W2, cfg.E, 0, part, bf16=True), tok)
    del W1, W3, W2
    G.assert_rows_close(out[tok], ref, 1e-2, 2e-2, "oracle sample")
    assert np.isfinite(out).all()
    # residual identity on the whole batch: out - x is the layer applied to h, whose plain forward we can run
    hbuf = P.DeviceBuffer.from_numpy(G.ctx(), h, cfg.dtype)
    lay = layer.forward(hbuf).to_numpy()
    assert N.rel_l2(out.astype(np.float64) - xh, lay) < 5e-2
    layer.close()


BW_CASES = [
    ("c1_tiny_f32", {}, False),
    ("c1_tiny_f32", dict(T=77, d=102, H=72), False),
    ("c4_finegrained", dict(T=96, d=128, H=64, E=8, K=3, Es=2, dtype="f32"), False),
    ("c2_mixtral", dict(T=300, d=256, H=384), False),
    ("c4_finegrained", dict(T=200, d=256, H=256, E=16, K=4, Es=2), True),
    ("c5_skewed", dict(T=257, d=512, H=256, E=32, K=4), True),
]


@pytest.mark.parametrize("name,kw,training", BW_CASES)
def test_block_backward_matches_oracle(name, kw, training):
    """back_block: the layer's backward on the normalised rows, the norm backward and the residual gradient; input
    gradient, norm weight gradient and the layer's parameter gradients against the oracle."""
    import importlib
    from tests import gpu_util as G
    L = importlib.import_module("omega-ai_amd._lib")
    cfg = scaled(C.CONFIGS[name], **kw)
    bf = cfg.dtype == "bf16"
    inp = make_inputs(cfg, 61)
    inp["Wg"] = inp["Wg"] * np.float32(8.0)
    gamma = _gamma(cfg.d, 61)
    dout = O.fill_normal(cfg.T * cfg.d, 61, 900, 1.0).reshape(cfg.T, cfg.d)
    if bf:
        dout = O.round_bf16(dout)
    layer = G.build_layer(cfg, inp)
    layer.set_norm(gamma)
    layer.set_training(training)
    x = G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype)
    g = G.P.DeviceBuffer.from_numpy(G.ctx(), dout, cfg.dtype)
    layer.forward(x)
    with pytest.raises(RuntimeError):      # the last forward was the plain one
        layer.back_block(g)
    out = layer.forward_block(x).to_numpy()
    with pytest.raises(RuntimeError):      # ... and now it was the block form
        layer.back(g)
    dx = layer.back_block(g).to_numpy()
    ref = O.block_backward(inp["x"], gamma, dout, inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm,
                           cfg.Es, bf)
    tol = 1e-2 if bf else 1e-5
    assert N.rel_l2(dx, ref["dx"]) < tol, N.rel_l2(dx, ref["dx"])
    assert N.rel_l2(layer.grad(L.W_NORM), ref["dgamma"]) < tol
    assert N.rel_l2(layer.grad(L.W_GATE), ref["dWg"]) < tol
    for e in (0, cfg.E + cfg.Es - 1):
        for which, k in ((L.W_W1, "dW1"), (L.W_W3, "dW3"), (L.W_W2, "dW2")):
            if ref[k][e].any():
                assert N.rel_l2(layer.grad(which, e), ref[k][e]) < tol, (k, e)
    assert np.array_equal(layer.getOutput().to_numpy(), out)
    assert np.array_equal(layer.back_block(g).to_numpy(), dx)       # reproducible: no atomics anywhere
    # a plain backward afterwards leaves a zero norm gradient
    layer.forward(x)
    layer.back(g)
    assert not layer.grad(L.W_NORM).any()
    layer.close()


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_block_checkpoint_round_trip(dtype):
    """saveModelBlock / loadModelBlock: norm weight first, then the layer, raw little-endian float32, byte-exact; a layer
    loaded from it gives the same block output bit for bit."""
    import importlib
    import io
    from tests import gpu_util as G
    L = importlib.import_module("omega-ai_amd._lib")
    cfg = scaled(C.CONFIGS["c2_mixtral"], T=40, d=256, H=256, E=4, K=2, Es=1, dtype=dtype)
    inp = make_inputs(cfg, 71)
    gamma = _gamma(cfg.d, 71)
    layer = G.build_layer(cfg, inp)
    layer.set_norm(gamma)
    f = io.BytesIO()
    layer.saveModelBlock(f)
    raw = f.getvalue()
    rnd = O.round_bf16 if dtype == "bf16" else (lambda a: a)
    expect = np.concatenate([gamma.ravel(), rnd(inp["Wg"]).ravel()] +
                            [np.concatenate([rnd(inp["W1"][g]).ravel(), rnd(inp["W3"][g]).ravel(), rnd(inp["W2"][g]).ravel()])
                             for g in range(cfg.E + cfg.Es)]).astype("<f4").tobytes()
    assert raw == expect
    other = G.P.MoELayer(cfg.d, cfg.H, cfg.E, cfg.K, cfg.renorm, cfg.Es, False, ctx=G.ctx(), dtype=dtype)
    other.loadModelBlock(io.BytesIO(raw))
    x = G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype)
    assert np.array_equal(other.forward_block(x).to_numpy(), layer.forward_block(x).to_numpy())
    with pytest.raises(RuntimeError, match="Error code"):
        other.loadModelBlock(io.BytesIO(raw[:cfg.d * 4 - 8]))
    with pytest.raises(RuntimeError, match="Error code"):
        other.loadModelBlock(io.BytesIO(raw[:cfg.d * 4 + 100]))
    layer.close()
    other.close()
