"""The every-work-item check that the full-size GPU tests rely on (tests/gpu_util.check_products_every_block and
row_tile_tokens), exercised on the CPU against a stand-in layer whose buffers come from NumPy: it must accept a correct
layer and must catch a row left unwritten (NaN poison), a 32-row block of `a` or `y` computed from the wrong rows, a
wrong column tile and a single wrong element at a block edge."""
import importlib

import numpy as np
import pytest

from oracle import oracle as O
from tests.synth import C, make_inputs

L = importlib.import_module("omega-ai_amd._lib")


class _FakeLayer:
    def __init__(self, cfg, inp, r):
        P = cfg.T * cfg.K
        self.cfg, self.inp = cfg, inp
        xg = inp["x"][r["src_row"]]
        A = np.concatenate([xg] + [inp["x"]] * cfg.Es)
        grp = np.concatenate([np.repeat(np.arange(cfg.E), r["counts"])] +
                             [np.full(cfg.T, cfg.E + s) for s in range(cfg.Es)])
        a = np.empty((len(A), cfg.H), np.float32)
        y = np.empty((len(A), cfg.d), np.float32)
        for g in range(cfg.E + cfg.Es):
            m = grp == g
            h1 = A[m].astype(np.float64) @ inp["W1"][g].T.astype(np.float64)
            h3 = A[m].astype(np.float64) @ inp["W3"][g].T.astype(np.float64)
            a[m] = O.round_bf16((h1 / (1 + np.exp(-h1)) * h3).astype(np.float32))
            y[m] = (a[m].astype(np.float64) @ inp["W2"][g].T.astype(np.float64)).astype(np.float32)
        self.buf = {"xg": xg, "a": a, "y": y}
        assert len(xg) == P

    def workspace(self, which, T):
        return self.buf[which].copy()

    def _download_weight(self, which, g, shape):
        return {L.W_W1: self.inp["W1"], L.W_W3: self.inp["W3"], L.W_W2: self.inp["W2"]}[which][g]


@pytest.fixture(scope="module")
def case():
    cfg = C.MoEConfig("chk", T=700, d=256, E=4, K=2, H=384, Es=1, dtype="bf16")
    inp = make_inputs(cfg, 4)
    inp["Wg"] = inp["Wg"] * np.float32(8.0)
    ids, w = O.topk(O.softmax(O.gate(inp["x"], inp["Wg"], None)), cfg.K, cfg.renorm)
    counts, offsets, dst, src = O.dispatch(ids, cfg.E)
    r = dict(ids=ids, w=w, counts=counts, offsets=offsets, dst=dst, src_row=src)
    return cfg, inp, r


def test_accepts_a_correct_layer(case):
    from tests import gpu_util as G
    cfg, inp, r = case
    assert G.check_products_every_block(_FakeLayer(cfg, inp, r), cfg, cfg.T, r, inp["x"]) > 1000


@pytest.mark.parametrize("what", ["nan_a", "nan_y", "a_block_wrong_rows", "y_block_wrong_rows", "y_column_tile", "a_edge",
                                  "shared_block"])
def test_catches(case, what):
    from tests import gpu_util as G
    cfg, inp, r = case
    lay = _FakeLayer(cfg, inp, r)
    e = int(np.argmax(r["counts"]))
    l0, n = int(r["offsets"][e]), int(r["counts"][e])
    blk = l0 + 32 * ((n // 32) // 2)                      # a block in the middle of the busiest expert
    if what == "nan_a":
        lay.buf["a"][l0 + n - 1, 5] = np.nan                # one element of the expert's last row
    elif what == "nan_y":
        lay.buf["y"][blk + 7] = np.nan                      # a row in the middle of a block
    elif what == "a_block_wrong_rows":
        lay.buf["a"][blk:blk + 32] = lay.buf["a"][blk - 32:blk]
        lay.buf["y"][blk:blk + 32] = lay.buf["y"][blk - 32:blk]   # consistent with the wrong a: only a's check can see it
    elif what == "y_block_wrong_rows":
        lay.buf["y"][blk:blk + 32] = lay.buf["y"][blk - 32:blk]
    elif what == "y_column_tile":
        lay.buf["y"][l0:l0 + n, 128:256] = 0.0              # a column tile of one expert left at zero
    elif what == "a_edge":
        lay.buf["a"][blk + 31, :] *= np.float32(1.05)       # last row of a block, 5 % off
    elif what == "shared_block":
        P = cfg.T * cfg.K
        lay.buf["y"][P + 64:P + 96] = lay.buf["y"][P:P + 32]
    with pytest.raises(AssertionError):
        G.check_products_every_block(lay, cfg, cfg.T, r, inp["x"])


def test_row_tile_tokens_touch_every_row_tile(case):
    from tests import gpu_util as G
    cfg, inp, r = case
    tok = G.row_tile_tokens(r, cfg, cfg.T)
    rows_of = {int(t): set() for t in tok}
    for p, row in enumerate(r["dst"]):
        t = p // cfg.K
        if t in rows_of:
            rows_of[t].add(int(row))
    touched = set().union(*rows_of.values())
    for e in range(cfg.E):
        n, l0 = int(r["counts"][e]), int(r["offsets"][e])
        Mg, nblk = -(-n // 256), -(-n // 32)
        qb, nhi = divmod(nblk, Mg)
        for mt in range(Mg):
            lo, hi = l0 + 32 * (mt * qb + min(mt, nhi)), l0 + min(32 * ((mt + 1) * qb + min(mt + 1, nhi)), n)
            assert any(lo <= q < hi for q in touched), (e, mt)
    assert 0 in tok and cfg.T - 1 in tok                # shared experts: first and last row tile
