"""Pins the C oracle against independent restatements, closed forms and brute force (CPU only)."""
import math

import numpy as np
import pytest

from oracle import oracle as O
from oracle import oracle_np as N
from tests.synth import C, make_inputs, scaled


# ---------------------------------------------------------------- generator
@pytest.mark.parametrize("seed,stream,std,first", [(1, 0, 1.0, 0), (2**63 + 5, 17, 0.02, 12345), (77, 400, 1 / 64.0, 2**33)])
def test_generator_c_equals_numpy_bitwise(seed, stream, std, first):
    a = O.fill_normal(50000, seed, stream, std, first)
    b = N.fill_normal(50000, seed, stream, std, first)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_generator_is_counter_based_and_normal():
    a = O.fill_normal(1 << 20, 9, 3, 1.0)
    assert np.array_equal(a[1000:1100], O.fill_normal(100, 9, 3, 1.0, first=1000))
    assert not np.array_equal(a[:100], O.fill_normal(100, 9, 4, 1.0))
    assert not np.array_equal(a[:100], O.fill_normal(100, 10, 3, 1.0))
    a = a.astype(np.float64)
    n = a.size
    assert abs(a.mean()) < 5 / math.sqrt(n)
    assert abs(a.var() - 1) < 5 * math.sqrt(2 / n)
    assert abs((a**3).mean()) < 5 * math.sqrt(15 / n)
    assert abs((a**4).mean() - 3) < 5 * math.sqrt(96 / n)
    # tail mass beyond 3 sigma = 0.0026998
    assert abs((np.abs(a) > 3).mean() - 0.0026998) < 5 * math.sqrt(0.0027 / n)


def test_bf16_rounding_known_values():
    v = np.array([1.0, 1.0 + 2**-8, 1.0 + 3 * 2**-8, 1.0 + 2**-8 + 2**-20, -2.5, 3.4028235e38, 0.0], np.float32)
    exp = np.array([1.0, 1.0, 1.0 + 2**-6, 1.0 + 2**-7, -2.5, np.inf, 0.0], np.float32)
    assert np.array_equal(O.round_bf16(v), exp)
    r = np.random.default_rng(0).standard_normal(10000).astype(np.float32)
    assert np.array_equal(O.round_bf16(r), N.round_bf16(r))
    assert np.array_equal(O.round_bf16(O.round_bf16(r)), O.round_bf16(r))
    assert np.all(np.abs(O.round_bf16(r) - r) <= np.abs(r) * 2**-8)


# ---------------------------------------------------------------- gate / GEMM
def test_gate_closed_form_and_fp64():
    x = np.ones((3, 64), np.float32)
    Wg = np.ones((5, 64), np.float32)
    assert np.array_equal(O.gate(x, Wg), np.full((3, 5), 64, np.float32))      # all-ones => k
    rng = np.random.default_rng(1)
    x = rng.standard_normal((37, 300)).astype(np.float32)
    Wg = rng.standard_normal((11, 300)).astype(np.float32)
    bg = rng.standard_normal(11).astype(np.float32)
    ref = x.astype(np.float64) @ Wg.astype(np.float64).T + bg
    assert N.rel_l2(O.gate(x, Wg, bg), ref) < 1e-6
    # layout: W is [out,in]; a transposed operand must fail this check
    assert N.rel_l2(O.gate(x, Wg, None), x.astype(np.float64) @ Wg.astype(np.float64).T) < 1e-6
    # sequential, unfused summation: reproduce one entry by hand
    acc = np.float32(0)
    for k in range(300):
        acc = np.float32(acc + np.float32(x[5, k] * Wg[7, k]))
    assert O.gate(x, Wg)[5, 7] == acc


def test_cpu_sgemm_restatement_kat():
    # the reference's own known answer: all-ones 64^3 => 64
    A = np.ones((64, 64), np.float32)
    assert np.array_equal(O.cpu_sgemm_tn(A, A, 2), np.full((64, 64), 64, np.float32))
    rng = np.random.default_rng(2)
    W = rng.standard_normal((19, 45)).astype(np.float32)   # [out,in]
    X = rng.standard_normal((13, 45)).astype(np.float32)   # [T,in]
    assert N.rel_l2(O.cpu_sgemm_tn(W, X, 3), X.astype(np.float64) @ W.astype(np.float64).T) < 1e-6


# ---------------------------------------------------------------- softmax
def test_softmax_against_kernel_text_twin():
    rng = np.random.default_rng(3)
    for E in (1, 2, 8, 64, 128):
        z = (rng.standard_normal((500, E)) * 3).astype(np.float32)
        p = O.softmax(z)
        q = N.softmax_3pass(z)
        assert np.array_equal(p.view(np.uint32), q.view(np.uint32))
        assert np.all(np.abs(p.astype(np.float64).sum(1) - 1) < 1e-6)
        assert np.array_equal(p.argmax(1), z.argmax(1)) or E == 1
        # shift invariance: an integer shift of integer-valued logits leaves every z - max exact
        zi = np.round(z)
        assert np.array_equal(O.softmax(zi), O.softmax(zi + 7))
    z = np.array([[0.0, math.log(3.0)]], np.float32)
    assert np.allclose(O.softmax(z), [[0.25, 0.75]], atol=1e-7)
    z = np.array([[-1e30, 0.0, -1e30]], np.float32)
    assert np.array_equal(O.softmax(z), np.array([[0, 1, 0]], np.float32))
    z = np.full((4, 8), 2.5, np.float32)
    assert np.array_equal(O.softmax(z), np.full((4, 8), 0.125, np.float32))


# ---------------------------------------------------------------- silu / swiglu
SILU_KAT_IN = [1, 2, 3, 4, -5, 6, -7, -8, 9, 10, 11, -12, 13, 14, 15, -16]   # literal input of SiLUKernel.main


def test_silu_closed_forms_via_swiglu():
    # d=1,H=n with W1=I-like: a row x=[1], W1[h]=v_h, W3[h]=1, W2 = e_h picks silu(v_h)
    v = np.array(SILU_KAT_IN + [0.0], np.float32)
    n = len(v)
    W1 = v.reshape(n, 1).copy()
    W3 = np.ones((n, 1), np.float32)
    out = np.empty(n, np.float32)
    for h in range(n):
        W2 = np.zeros((1, n), np.float32)
        W2[0, h] = 1
        out[h] = O.swiglu_rows(np.ones((1, 1), np.float32), W1, W3, W2)[0, 0]
    ref = v.astype(np.float64) / (1 + np.exp(-v.astype(np.float64)))
    assert np.allclose(out, ref, rtol=2e-7, atol=1e-12)
    assert out[-1] == 0.0                                   # silu(0)=0
    # silu(x) - silu(-x) = x for the +-pairs we can form
    W1b = np.array([[3.0], [-3.0]], np.float32)
    a = [O.swiglu_rows(np.ones((1, 1), np.float32), W1b, np.ones((2, 1), np.float32),
                       np.eye(2, dtype=np.float32)[i:i + 1])[0, 0] for i in range(2)]
    assert abs((a[0] - a[1]) - 3.0) < 1e-6
    assert abs(out[10] - 11.0) < 2e-4 and abs(out[15]) < 2e-6   # limits x>>0, x<<0


def test_swiglu_fp64_and_bf16_mode():
    rng = np.random.default_rng(4)
    d, H, rows = 96, 160, 9
    xg = rng.standard_normal((rows, d)).astype(np.float32)
    W1 = (rng.standard_normal((H, d)) / math.sqrt(d)).astype(np.float32)
    W3 = (rng.standard_normal((H, d)) / math.sqrt(d)).astype(np.float32)
    W2 = (rng.standard_normal((d, H)) / math.sqrt(H)).astype(np.float32)
    x64 = xg.astype(np.float64)
    a = N.silu64(x64 @ W1.astype(np.float64).T) * (x64 @ W3.astype(np.float64).T)
    assert N.rel_l2(O.swiglu_rows(xg, W1, W3, W2), a @ W2.astype(np.float64).T) < 1e-6
    # swapping W1 and W3 must be visible
    assert N.rel_l2(O.swiglu_rows(xg, W3, W1, W2), a @ W2.astype(np.float64).T) > 1e-2
    # bf16 mode = same with `a` rounded to bf16
    a32 = (N.silu64((x64 @ W1.astype(np.float64).T)) * (x64 @ W3.astype(np.float64).T)).astype(np.float32)
    yb = N.round_bf16(a32).astype(np.float64) @ W2.astype(np.float64).T
    assert N.rel_l2(O.swiglu_rows(xg, W1, W3, W2, bf16=True), yb) < 2e-3
    assert N.rel_l2(O.swiglu_rows(xg, W1, W3, W2, bf16=True), O.swiglu_rows(xg, W1, W3, W2)) > 1e-5


# ---------------------------------------------------------------- top-k
def test_topk_brute_force_and_ties():
    rng = np.random.default_rng(5)
    for E, K in ((8, 2), (64, 6), (128, 8), (5, 5), (3, 1)):
        p = O.softmax((rng.standard_normal((400, E)) * 2).astype(np.float32))
        for renorm in (0, 1):
            ids, w = O.topk(p, K, renorm)
            ids2, w2 = N.topk_stable(p, K, renorm)
            assert np.array_equal(ids, ids2)
            assert np.array_equal(w.view(np.uint32), w2.view(np.uint32))
            if renorm:
                assert np.all(np.abs(w.astype(np.float64).sum(1) - 1) < 1e-6)
    p = np.full((3, 8), 0.125, np.float32)                   # all equal -> 0..K-1
    ids, w = O.topk(p, 3, 0)
    assert np.array_equal(ids, np.tile(np.arange(3, dtype=np.int32), (3, 1)))
    p = np.array([[0.1, 0.3, 0.3, 0.1, 0.2]], np.float32)    # duplicated maxima -> lowest index first
    ids, w = O.topk(p, 3, 0)
    assert ids.tolist() == [[1, 2, 4]]
    # quantised probabilities: many ties
    q = (rng.integers(0, 4, (500, 16)) / 4.0).astype(np.float32)
    assert np.array_equal(O.topk(q, 4, 0)[0], N.topk_stable(q, 4, 0)[0])


# ---------------------------------------------------------------- dispatch
def test_dispatch_brute_force_and_invariants():
    rng = np.random.default_rng(6)
    for T, K, E in ((1, 1, 1), (7, 2, 8), (300, 6, 64), (513, 8, 128)):
        ids = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.int32)
        counts, offsets, dst, src = O.dispatch(ids, E)
        c2, o2, d2, s2 = N.dispatch_argsort(ids, E)
        for a, b in ((counts, c2), (offsets, o2), (dst, d2), (src, s2)):
            assert np.array_equal(a, b)
        P = T * K
        assert counts.sum() == P and offsets[-1] == P
        assert np.array_equal(np.sort(dst), np.arange(P))    # bijection
        inv = np.empty(P, np.int64)
        inv[dst] = np.arange(P)
        for e in range(E):
            seg = inv[offsets[e]:offsets[e + 1]]
            assert np.all(np.diff(seg) > 0)                   # stable
            assert np.all(ids.reshape(-1)[seg] == e)
    # empty experts and a single hot expert
    ids = np.zeros((50, 1), np.int32) + 5
    counts, offsets, dst, src = O.dispatch(ids, 8)
    assert counts.tolist() == [0, 0, 0, 0, 0, 50, 0, 0] and np.array_equal(dst, np.arange(50))


# ---------------------------------------------------------------- whole layer
@pytest.mark.parametrize("name,kw", [
    ("c1_tiny_f32", {}),
    ("c4_finegrained", dict(T=96, d=64, H=96, dtype="f32")),
    ("c5_skewed", dict(T=128, d=64, H=64, dtype="f32")),
])
def test_forward_equals_dense_identity(name, kw):
    cfg = scaled(C.CONFIGS[name], **kw)
    inp = make_inputs(cfg, seed=11)
    r = O.moe_forward(inp["x"], inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm, cfg.Es)
    dense = N.dense_moe_fp64(inp["x"], r["ids"], r["w"], inp["W1"], inp["W3"], inp["W2"], cfg.E, cfg.Es)
    assert N.rel_l2(r["out"], dense) < 1e-6
    # routing pieces agree with the independent restatements
    z = inp["x"].astype(np.float64) @ inp["Wg"].astype(np.float64).T + (0 if inp["bg"] is None else inp["bg"])
    assert N.rel_l2(r["logits"], z) < 1e-6
    assert np.array_equal(r["p"], N.softmax_3pass(r["logits"]))
    ids2, w2 = N.topk_stable(r["p"], cfg.K, cfg.renorm)
    assert np.array_equal(r["ids"], ids2) and np.array_equal(r["w"], w2)
    # selecting on probabilities or on logits coincides on these inputs (no rounding-made ties)
    ids_logit = np.argsort(-r["logits"].astype(np.float64), axis=1, kind="stable")[:, :cfg.K]
    assert (ids_logit != r["ids"]).any(axis=1).sum() == 0
    c2, o2, d2, s2 = N.dispatch_argsort(r["ids"], cfg.E)
    assert np.array_equal(r["counts"], c2) and np.array_equal(r["dst"], d2) and np.array_equal(r["src_row"], s2)
    # token-subset entry point agrees with the full path
    tok = np.array([0, 5, cfg.T - 1], np.int32)
    sub = O.moe_tokens(inp["x"], r["ids"], r["w"], inp["W1"], inp["W3"], inp["W2"], cfg.E, cfg.Es, tok)
    assert np.array_equal(sub, r["out"][tok])
    if cfg.zipf_bias:
        assert (r["counts"] == 0).any() or r["counts"].max() > 8 * max(1, np.median(r["counts"]))


def test_single_expert_reduces_to_swiglu_mlp():
    cfg = scaled(C.CONFIGS["c1_tiny_f32"], T=16, E=1, K=1)
    inp = make_inputs(cfg, seed=3)
    r = O.moe_forward(inp["x"], inp["Wg"], None, inp["W1"], inp["W3"], inp["W2"], 1, True)
    assert np.array_equal(r["w"], np.ones((16, 1), np.float32))
    assert np.array_equal(r["out"], O.swiglu_rows(inp["x"], inp["W1"][0], inp["W3"][0], inp["W2"][0]))


def test_cpu_baseline_matches_oracle():
    cfg = scaled(C.CONFIGS["c4_finegrained"], T=40, d=48, H=56, E=8, K=3, dtype="f32")
    inp = make_inputs(cfg, seed=5)
    r = O.moe_forward(inp["x"], inp["Wg"], None, inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm, cfg.Es)
    secs, out = O.cpu_baseline_forward(inp["x"], inp["Wg"], None, inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm, cfg.Es, 4)
    assert secs > 0 and N.rel_l2(out, r["out"]) < 1e-6


def test_zipf_bias_shape():
    cfg = C.CONFIGS["c5_skewed"]
    bg = C.zipf_gate_bias(cfg, 1)
    w = np.exp(bg.astype(np.float64) / 2)
    assert abs(w.sum() - 1) < 1e-5
    ranks = np.sort(w)[::-1]
    assert np.allclose(ranks[0] / ranks[1], 2 ** 1.2, rtol=1e-5)
    assert not np.array_equal(bg, C.zipf_gate_bias(cfg, 2))


# ---------------------------------------------------------------- block form: pre-norm and residual
@pytest.mark.parametrize("T,d", [(7, 128), (3, 100), (2, 33), (4, 4096)])
@pytest.mark.parametrize("bf16", [False, True])
def test_rmsnorm_against_kernel_text_twin(T, d, bf16):
    rng = np.random.default_rng(T * 1000 + d)
    x = (rng.standard_normal((T, d)) * 3).astype(np.float32)
    g = rng.standard_normal(d).astype(np.float32)
    if bf16:
        x = O.round_bf16(x)
    h, rms = O.rmsnorm(x, g, bf16)
    h2, rms2 = N.rmsnorm_lanes(x, g, bf16)
    assert np.array_equal(rms.view(np.uint32), rms2.view(np.uint32))
    assert np.array_equal(h.view(np.uint32), h2.view(np.uint32))
    # the definition in fp64: x / sqrt(mean(x^2) + 1e-6) * g
    x64 = x.astype(np.float64)
    ref = x64 / np.sqrt((x64**2).mean(1, keepdims=True) + 1e-6) * g.astype(np.float64)
    tol = 1e-2 if bf16 else 1e-6
    assert N.rel_l2(h, ref) < tol


def test_rmsnorm_closed_forms_and_lane_order():
    d = 256
    g = np.linspace(-1, 1, d).astype(np.float32)
    # a row of ones: every lane holds d/32 exactly, the sum is exactly d, rms = sqrt(1 + 1e-6)
    h, rms = O.rmsnorm(np.ones((1, d), np.float32), g)
    r = np.sqrt(np.float32(1.0) + np.float32(1e-6)).astype(np.float32)
    assert rms[0] == r
    assert np.array_equal(h[0], (np.float32(1.0) / r * g).astype(np.float32))
    # a row of zeros: rms = sqrt(1e-6), output exactly zero (no NaN)
    h, rms = O.rmsnorm(np.zeros((1, d), np.float32), g)
    assert rms[0] == np.sqrt(np.float32(1e-6)) and not h.any()
    # doubling the row doubles rms up to the 1e-6 term
    x = np.random.default_rng(3).standard_normal((1, d)).astype(np.float32)
    _, r1 = O.rmsnorm(x, g)
    _, r2 = O.rmsnorm(2 * x, g)
    assert abs(r2[0] / r1[0] - 2) < 1e-5
    # the order of the additions is part of the definition: a plain left-to-right sum of squares gives other bits
    # on some rows, so a restatement that ignored the 32-lane structure would fail the twin test above
    X = (np.random.default_rng(4).standard_normal((64, 4096)) * 3).astype(np.float32)
    _, rms = O.rmsnorm(X, np.ones(4096, np.float32))
    seq = np.zeros(64, np.float32)
    for i in range(4096):
        seq = (seq + X[:, i] * X[:, i]).astype(np.float32)
    naive = np.sqrt((seq / np.float32(4096)).astype(np.float32) + np.float32(1e-6)).astype(np.float32)
    assert (naive != rms).any()
    assert np.allclose(naive, rms, rtol=1e-5)


@pytest.mark.parametrize("name,kw", [("c1_tiny_f32", {}), ("c4_finegrained", dict(T=48, d=64, H=32, E=8, K=3, Es=2, dtype="f32")),
                                     ("c2_mixtral", dict(T=40, d=64, H=64))])
def test_block_is_layer_on_normalised_rows_plus_residual(name, kw):
    cfg = scaled(C.CONFIGS[name], **kw)
    inp = make_inputs(cfg, 31)
    bf = cfg.dtype == "bf16"
    gamma = O.fill_normal(cfg.d, 31, C.STREAM_NORM, 1.0) * np.float32(0.1) + np.float32(1.0)
    blk = O.block_forward(inp["x"], gamma, inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm,
                          cfg.Es, bf)
    h, rms = O.rmsnorm(inp["x"], gamma, bf)
    assert np.array_equal(blk["h"], h) and np.array_equal(blk["rms"], rms)
    lay = O.moe_forward(h, inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm, cfg.Es, bf)
    for k in ("ids", "w", "counts", "offsets", "dst", "src_row", "logits", "p"):
        assert np.array_equal(blk[k], lay[k]), k
    if not bf:  # fp32: the layer output is the unrounded sum, so the residual identity is exact
        assert np.array_equal(blk["out"], (lay["out"] + inp["x"]).astype(np.float32))
    else:       # bf16: one rounding of (sum + x) against rounding the sum first
        assert N.rel_l2(blk["out"], lay["out"].astype(np.float64) + inp["x"]) < 1e-2
    tok = np.array([0, 5, cfg.T - 1], np.int32)
    sub = O.block_tokens(inp["x"], h, blk["ids"], blk["w"], inp["W1"], inp["W3"], inp["W2"], cfg.E, cfg.Es, tok, bf)
    assert np.array_equal(sub, blk["out"][tok])
