"""GPU parity tests: the HIP path through the C ABI against the CPU oracle on the same seeded inputs.

Bars: expert ids, per-expert counts, offsets and the permutation bit-exact (exact router mode);
layer output within 1e-5 relative L2 in fp32 and within 1e-2 relative L2 in bf16 (fp32 accumulate).
"""
import io

import numpy as np
import pytest

from oracle import oracle as O
from oracle import oracle_np as N
from tests.synth import C, make_inputs, scaled

pytestmark = pytest.mark.gpu

F32_TOL = 1e-5
BF16_TOL = 1e-2


@pytest.fixture(scope="module")
def G():
    from tests import gpu_util
    return gpu_util


def test_device_generator_matches_oracle_bitwise(G):
    P = G.P
    for dtype, n, seed, stream, std, first in (("f32", 300001, 7, 0, 1.0, 0), ("f32", 4097, 2**63 + 9, 33, 0.02, 2**34),
                                               ("bf16", 100000, 5, 18, 1 / 64.0, 12345)):
        b = P.DeviceBuffer(G.ctx(), (n,), dtype)
        b.fill_normal(seed, stream, std, first)
        got = b.to_numpy()
        ref = O.fill_normal(n, seed, stream, std, first)
        if dtype == "bf16":
            ref = O.round_bf16(ref)
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
        b.free()


def test_c1_tiny_fp32_full_parity(G):
    cfg = C.CONFIGS["c1_tiny_f32"]
    layer, x, out, r, ref, inp = G.run_case(cfg, seed=20251)
    G.assert_routing_bit_exact(r, ref)
    lg, p = layer.router_probs(x, cfg.T)
    assert np.array_equal(lg.view(np.uint32), ref["logits"].view(np.uint32))
    assert np.array_equal(p.view(np.uint32), ref["p"].view(np.uint32))
    assert np.array_equal(layer.workspace("xg", cfg.T), inp["x"][ref["src_row"]])
    assert N.rel_l2(out, ref["out"]) <= F32_TOL
    # dense-MoE identity, independent of any permutation
    dense = N.dense_moe_fp64(inp["x"], r["ids"], r["w"], inp["W1"], inp["W3"], inp["W2"], cfg.E)
    assert N.rel_l2(out, dense) <= F32_TOL
    layer.close()


@pytest.mark.parametrize("T", [1, 2, 31, 33, 100, 257])
def test_fp32_ragged_token_counts(G, T):
    cfg = scaled(C.CONFIGS["c1_tiny_f32"], T=T)
    layer, x, out, r, ref, inp = G.run_case(cfg, seed=3 + T)
    G.assert_routing_bit_exact(r, ref)
    assert N.rel_l2(out, ref["out"]) <= F32_TOL
    layer.close()


@pytest.mark.parametrize("E,K,Es,renorm,d,H,T", [
    (1, 1, 0, True, 64, 96, 40),       # single expert == plain SwiGLU MLP
    (5, 5, 0, False, 48, 80, 70),      # K == E, odd sizes (scalar fallbacks)
    (16, 4, 1, True, 128, 192, 130),
    (64, 6, 2, False, 64, 128, 200),   # fine-grained + shared experts, no renorm
    (128, 8, 0, True, 64, 64, 300),
    (200, 8, 0, True, 32, 64, 90),     # more experts than lanes in a wave, not a power of two
])
def test_fp32_shapes(G, E, K, Es, renorm, d, H, T):
    cfg = C.MoEConfig("t", T=T, d=d, E=E, K=K, H=H, Es=Es, renorm=renorm, dtype="f32")
    layer, x, out, r, ref, inp = G.run_case(cfg, seed=E * 1000 + K)
    G.assert_routing_bit_exact(r, ref)
    assert N.rel_l2(out, ref["out"]) <= F32_TOL
    layer.close()


def test_fp32_ties_and_empty_experts(G):
    """All-equal gate rows: every token ties across all experts -> experts 0..K-1; the rest stay empty."""
    cfg = C.MoEConfig("t", T=77, d=64, E=8, K=3, H=64, dtype="f32")
    inp = make_inputs(cfg, seed=9)
    inp["Wg"][:] = 0.0
    layer = G.build_layer(cfg, inp)
    x = G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], "f32")
    out = layer.forward(x).to_numpy()
    r = layer.routing()
    ref = G.oracle_forward(cfg, inp)
    G.assert_routing_bit_exact(r, ref)
    assert r["ids"].tolist() == [[0, 1, 2]] * 77
    assert r["counts"].tolist() == [77, 77, 77, 0, 0, 0, 0, 0]
    assert N.rel_l2(out, ref["out"]) <= F32_TOL
    # duplicated gate rows: pairwise ties between experts (1,5) and (2,6)
    inp = make_inputs(cfg, seed=10)
    inp["Wg"][5] = inp["Wg"][1]
    inp["Wg"][6] = inp["Wg"][2]
    layer2 = G.build_layer(cfg, inp)
    x2 = G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], "f32")
    out2 = layer2.forward(x2).to_numpy()
    ref2 = G.oracle_forward(cfg, inp)
    G.assert_routing_bit_exact(layer2.routing(), ref2)
    assert N.rel_l2(out2, ref2["out"]) <= F32_TOL
    layer.close()
    layer2.close()


def test_zipf_bias_skewed_fp32(G):
    cfg = scaled(C.CONFIGS["c5_skewed"], T=600, d=64, H=64, dtype="f32")
    layer, x, out, r, ref, inp = G.run_case(cfg, seed=77)
    G.assert_routing_bit_exact(r, ref)
    assert (r["counts"] == 0).any()
    assert N.rel_l2(out, ref["out"]) <= F32_TOL
    layer.close()


@pytest.mark.parametrize("name,kw", [
    ("c2_mixtral", dict(T=512, d=512, H=1024)),
    ("c2_mixtral", dict(T=1000, d=256, H=384)),        # ragged row tiles
    ("c3_decode", dict(T=64, d=512, H=1024)),
    ("c4_finegrained", dict(T=512, d=256, H=384)),     # 64 experts, 2 shared, no renorm
    ("c5_skewed", dict(T=1024, d=256, H=256)),         # 128 experts, Zipf bias, empty experts
])
def test_bf16_scaled_configs(G, name, kw):
    cfg = scaled(C.CONFIGS[name], **kw)
    layer, x, out, r, ref, inp = G.run_case(cfg, seed=4242)
    G.assert_routing_bit_exact(r, ref)
    assert np.array_equal(layer.workspace("xg", cfg.T), inp["x"][ref["src_row"]])
    err = N.rel_l2(out, ref["out"])
    assert err <= BF16_TOL, err
    # against the unrounded fp64 dense identity as well (looser: bf16 rounding of a and out)
    dense = N.dense_moe_fp64(inp["x"], r["ids"], r["w"], inp["W1"], inp["W3"], inp["W2"], cfg.E, cfg.Es)
    assert N.rel_l2(out, dense) <= BF16_TOL
    layer.close()


@pytest.mark.parametrize("name,kw", [
    ("c2_mixtral", dict(T=1000, d=256, H=384)),        # ragged row tiles, rows that share a line with another tile's
    ("c2_mixtral", dict(T=37, d=512, H=512)),          # a small batch (k slices of the down product)
    ("c4_finegrained", dict(T=515, d=256, H=384)),     # shared experts (their rows are the tokens themselves), odd T
    ("c5_skewed", dict(T=1024, d=256, H=256)),         # empty experts, K = 8
])
def test_bf16_gather_modes_agree(G, name, kw):
    """The rows of x reach the experts either as a gathered copy written by the dispatch stage or through the loads of
    the up product (omega_moe_set_gather_mode): the same bits either way, against the oracle, and the gathered rows
    asked for afterwards are x[src_row] in both.  A second forward with fewer tokens in each mode (the row -> token
    table then holds stale entries behind the valid rows)."""
    cfg = scaled(C.CONFIGS[name], **kw)
    inp = make_inputs(cfg, 31337)
    ref = G.oracle_forward(cfg, inp)
    x = G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype)
    T2 = max(1, cfg.T // 3)
    cfg2 = scaled(cfg, T=T2)
    inp2 = {**inp, "x": inp["x"][:T2]}
    ref2 = G.oracle_forward(cfg2, inp2)
    x2 = G.P.DeviceBuffer.from_numpy(G.ctx(), inp2["x"], cfg.dtype)
    outs = {}
    for mode in (1, 2):
        layer = G.build_layer(cfg, inp)
        layer.set_gather_mode(mode)
        out = layer.forward(x).to_numpy()
        G.assert_routing_bit_exact(layer.routing(), ref)
        assert N.rel_l2(out, ref["out"]) <= BF16_TOL
        assert np.array_equal(layer.workspace("xg", cfg.T), inp["x"][ref["src_row"]])
        out2 = layer.forward(x2).to_numpy()
        G.assert_routing_bit_exact(layer.routing(), ref2)
        assert N.rel_l2(out2, ref2["out"]) <= BF16_TOL
        assert np.array_equal(layer.workspace("xg", T2), inp2["x"][ref2["src_row"]])
        assert np.array_equal(layer.forward(x).to_numpy(), out)
        outs[mode] = (out, out2)
        layer.close()
    assert np.array_equal(outs[1][0], outs[2][0]) and np.array_equal(outs[1][1], outs[2][1])
    layer = G.build_layer(cfg, inp)
    with pytest.raises(RuntimeError):
        layer.set_gather_mode(3)
    layer.close()


@pytest.mark.parametrize("T,d,H,E,K,Es", [
    (1, 512, 1024, 8, 2, 0),      # two experts with one row each: 32 k steps in 4 slices (no slice under 8 steps)
    (3, 256, 2048, 8, 2, 0),      # 8 slices of 8 steps
    (5, 512, 896, 8, 2, 0),       # 28 k steps in 3 uneven slices (9, 9, 10)
    (17, 256, 640, 4, 2, 1),      # shared expert rows among the sliced tiles, 20 k steps in 2 slices
    (64, 512, 1024, 8, 2, 0),     # every expert has rows: 2 slices
    (40, 1024, 512, 16, 4, 0),    # 16 experts x 4 column tiles: 2 slices
])
def test_bf16_small_batches_slice_the_down_product(G, T, d, H, E, K, Es):
    """Small batches: the down product's k range is cut into slices whose partial results are added up behind it.
    Output and the y buffer against the oracle, the same bits on a second call, and a large batch on the same layer
    in between (which takes the unsliced path) leaves the small one unchanged."""
    cfg = scaled(C.CONFIGS["c2_mixtral"], T=T, d=d, H=H, E=E, K=K, Es=Es)
    layer, x, out, r, ref, inp = G.run_case(cfg, seed=777)
    G.assert_routing_bit_exact(r, ref)
    assert N.rel_l2(out, ref["out"]) <= BF16_TOL
    y = layer.workspace("y", cfg.T)
    a = layer.workspace("a", cfg.T)
    # y = a . W2^T row by row in float64 from the rows the layer itself holds (pins the sum of the partial results)
    g_of_row = np.repeat(np.arange(E), r["counts"])
    for row in range(0, T * K, max(1, T * K // 7)):
        want = inp["W2"][g_of_row[row]].astype(np.float64) @ a[row].astype(np.float64)
        assert N.rel_l2(y[row], want) < 1e-5, row
    big = make_inputs(scaled(cfg, T=900), 778)
    xb = G.P.DeviceBuffer.from_numpy(G.ctx(), big["x"], cfg.dtype)
    ob = layer.forward(xb).to_numpy()
    refb = G.oracle_forward(scaled(cfg, T=900), {**big, **{k: inp[k] for k in ("Wg", "bg", "W1", "W3", "W2")}})
    assert N.rel_l2(ob, refb["out"]) <= BF16_TOL
    assert np.array_equal(layer.forward(x).to_numpy(), out)
    layer.close()


@pytest.mark.parametrize("T,d,E,K,zipf", [
    (37, 1536, 8, 2, 0.0),     # ragged tile whose second wave holds no token, three chunks of 512 k (odd count)
    (16, 512, 5, 2, 1.1),      # fewer experts than lanes across them, gate bias, a single chunk
    (130, 1024, 12, 3, 0.7),   # 12 of 16 expert lanes, bias, two tokens in the last tile
    (4096, 512, 16, 4, 0.0),   # one tile per compute unit: the largest batch of the small-batch kernel
    (4112, 512, 8, 2, 0.0),    # one tile more: the same layer through the general kernel
])
def test_bf16_small_batch_router_bit_exact(G, T, d, E, K, zipf):
    """bf16 layers with at most 16 experts and at most one 16-token tile per compute unit route through a kernel of
    their own (staging waves feed the waves that form the sums): logits, probabilities and the routing against the
    oracle, bit for bit, and the fast router mode gives the same bits (its terms are exact products either way)."""
    cfg = scaled(C.CONFIGS["c2_mixtral"], T=T, d=d, H=256, E=E, K=K, zipf_bias=zipf)
    layer, x, out, r, ref, inp = G.run_case(cfg, seed=9000 + T)
    G.assert_routing_bit_exact(r, ref)
    lg, p = layer.router_probs(x, T)
    assert np.array_equal(lg.view(np.uint32), ref["logits"].view(np.uint32))
    assert np.array_equal(p.view(np.uint32), ref["p"].view(np.uint32))
    assert N.rel_l2(out, ref["out"]) <= BF16_TOL
    layer.close()
    fast = G.build_layer(cfg, inp, "fast")
    fast.forward(x)
    lgf, pf = fast.router_probs(x, T)
    assert np.array_equal(lgf.view(np.uint32), lg.view(np.uint32))
    assert np.array_equal(pf.view(np.uint32), p.view(np.uint32))
    fast.close()


def test_bf16_fast_router_agrees(G):
    cfg = scaled(C.CONFIGS["c2_mixtral"], T=512, d=512, H=1024)
    layer, x, out, r, ref, inp = G.run_case(cfg, seed=4242, router_mode="fast")
    agree = (r["ids"] == ref["ids"]).all(axis=1).mean()
    assert agree >= 0.995
    c2, o2, d2, s2 = N.dispatch_argsort(r["ids"], cfg.E)          # dispatch stays exact for the ids it got
    assert np.array_equal(r["counts"], c2) and np.array_equal(r["dst"], d2) and np.array_equal(r["src_row"], s2)
    assert N.rel_l2(out, ref["out"]) <= BF16_TOL
    layer.close()


def test_stage_entry_points_match_forward(G):
    cfg = scaled(C.CONFIGS["c4_finegrained"], T=300, d=256, H=384)
    inp = make_inputs(cfg, 5)
    layer = G.build_layer(cfg, inp)
    x = G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype)
    full = layer.forward(x).to_numpy().copy()
    out2 = G.P.DeviceBuffer(G.ctx(), (cfg.T, cfg.d), cfg.dtype)
    for st in ("router", "dispatch", "experts", "combine"):
        layer.stage(st, x=x, out=out2)
    assert np.array_equal(out2.to_numpy(), full)
    # repeating dispatch alone is idempotent
    before = layer.routing()
    layer.stage("dispatch", x=x)
    after = layer.routing()
    for k in before:
        assert np.array_equal(before[k], after[k])
    # growing and shrinking the batch on one layer
    for T in (64, 700, 5):
        i2 = make_inputs(cfg, 6, T)
        xb = G.P.DeviceBuffer.from_numpy(G.ctx(), i2["x"], cfg.dtype)
        o = layer.forward(xb).to_numpy()
        i2.update({k: inp[k] for k in ("Wg", "bg", "W1", "W3", "W2")})
        ref = G.oracle_forward(cfg, i2)
        G.assert_routing_bit_exact(layer.routing(), ref)
        assert N.rel_l2(o, ref["out"]) <= BF16_TOL
    layer.close()


def test_checkpoint_round_trip_and_errors(G):
    cfg = C.MoEConfig("t", T=16, d=64, E=4, K=2, H=128, Es=1, dtype="f32", zipf_bias=1.2)
    inp = make_inputs(cfg, 1)
    layer = G.build_layer(cfg, inp)
    f = io.BytesIO()
    layer.saveModel(f)
    raw = f.getvalue()
    expect = np.concatenate([inp["Wg"].ravel(), inp["bg"].ravel()] +
                            [np.concatenate([inp["W1"][g].ravel(), inp["W3"][g].ravel(), inp["W2"][g].ravel()])
                             for g in range(5)]).astype("<f4").tobytes()
    assert raw == expect                                   # byte-exact, order gate, bias, (w1,w3,w2) per expert
    other = G.P.MoELayer(cfg.d, cfg.H, cfg.E, cfg.K, True, cfg.Es, True, ctx=G.ctx(), dtype="f32")
    other.loadModel(io.BytesIO(raw))
    x = G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], "f32")
    assert np.array_equal(other.forward(x).to_numpy(), layer.forward(x).to_numpy())
    with pytest.raises(RuntimeError, match="Error code"):
        other.loadModel(io.BytesIO(raw[:100]))
    with pytest.raises(RuntimeError, match="Error code"):
        G.P.MoELayer(64, 64, 4, 5, ctx=G.ctx())            # K > E
    with pytest.raises(RuntimeError, match="Error code"):
        G.P.MoELayer(100, 64, 4, 2, ctx=G.ctx(), dtype="bf16")   # unsupported bf16 width
    with pytest.raises(RuntimeError, match="Error code"):
        layer.forward(G.P.DeviceBuffer(G.ctx(), (4, 32), "f32"))
    layer.close()
    other.close()
