"""Helpers shared by the GPU parity tests: build a layer from host arrays, run the oracle beside it."""
import importlib

import numpy as np

from oracle import oracle as O
from oracle import oracle_np as N
from tests.synth import C, make_inputs

P = importlib.import_module("omega-ai_amd")

_ctx = None


def ctx():
    global _ctx
    if _ctx is None:
        _ctx = P.Context(0)
    return _ctx


def build_layer(cfg, inp, router_mode="exact", T_max=0):
    layer = P.MoELayer(cfg.d, cfg.H, cfg.E, cfg.K, renorm=cfg.renorm, nShared=cfg.Es, bias=inp["bg"] is not None,
                       ctx=ctx(), dtype=cfg.dtype, router_mode=router_mode, T_max=T_max)
    layer.set_gate(inp["Wg"], inp["bg"])
    for g in range(cfg.E + cfg.Es):
        layer.set_expert(g, inp["W1"][g], inp["W3"][g], inp["W2"][g])
    return layer


def oracle_forward(cfg, inp):
    return O.moe_forward(inp["x"], inp["Wg"], inp["bg"], inp["W1"], inp["W3"], inp["W2"], cfg.K, cfg.renorm, cfg.Es,
                         bf16=cfg.dtype == "bf16")


def run_case(cfg, seed, router_mode="exact", T=None):
    """Returns (layer, x buffer, gpu out [T,d] fp32, gpu routing dict, oracle dict, inputs)."""
    inp = make_inputs(cfg, seed, T)
    layer = build_layer(cfg, inp, router_mode)
    x = P.DeviceBuffer.from_numpy(ctx(), inp["x"], cfg.dtype)
    out = layer.forward(x).to_numpy()
    r = layer.routing()
    ref = oracle_forward(cfg, inp)
    return layer, x, out, r, ref, inp


def assert_routing_bit_exact(r, ref):
    for k in ("ids", "counts", "offsets", "dst", "src_row"):
        assert np.array_equal(r[k], ref[k]), k
    assert np.array_equal(r["w"].view(np.uint32), ref["w"].view(np.uint32)), "w"


# ---- full-size checks that cover every work item of the grouped products ----

def row_tile_tokens(r, cfg, T, bm=256):
    """One token per row tile of every group (its first row; for a group's last tile also its last row), so that a
    token sample touches every row tile the grouped products schedule.  Row tiles of a group are its 32-row blocks
    dealt evenly to ceil(rows / bm) tiles, the taller tiles first."""
    toks = set()
    for e in range(cfg.E):
        n, l0 = int(r["counts"][e]), int(r["offsets"][e])
        if n == 0:
            continue
        Mg, nblk = -(-n // bm), -(-n // 32)
        qb, nhi = divmod(nblk, Mg)                   # the first nhi row tiles hold qb + 1 blocks of 32 rows, the others qb
        for mt in range(Mg):
            toks.add(int(r["src_row"][l0 + 32 * (mt * qb + min(mt, nhi))]))
        toks.add(int(r["src_row"][l0 + n - 1]))
    if cfg.Es > 0:                                   # shared experts: row t of a shared group is token t
        toks.update(range(0, T, bm))
        toks.add(T - 1)
    return np.array(sorted(toks), np.int32)


def oracle_tokens_parallel(fn, tokens, workers=8):
    """fn(token_subset) -> rows, evaluated on slices of `tokens` by a few threads (the C oracle releases the GIL)."""
    from concurrent.futures import ThreadPoolExecutor
    parts = [p for p in np.array_split(tokens, min(workers, len(tokens))) if len(p)]
    with ThreadPoolExecutor(len(parts)) as ex:
        return np.concatenate(list(ex.map(fn, parts)))


def check_products_every_block(layer, cfg, T, r, xh, seed=7):
    """After a forward over buffers that were poisoned with NaN: every valid row of a and y is finite, and for the
    first and the last row of EVERY 32-row block of every group (work items - row tiles, their row slices, k slices -
    are made of such blocks) two columns of every 128-column group of a and of y equal float64 dot products formed
    from the layer's own gathered rows / a rows and its downloaded weights.  Returns the number of elements checked."""
    import importlib
    L = importlib.import_module("omega-ai_amd._lib")
    d, H, E, K, Es = cfg.d, cfg.H, cfg.E, cfg.K, cfg.Es
    P = T * K
    a = layer.workspace("a", T)
    assert np.isfinite(a).all(), "a: a valid row was not written"
    y = layer.workspace("y", T)
    assert np.isfinite(y).all(), "y: a valid row was not written"
    xg = layer.workspace("xg", T)
    rng = np.random.default_rng(seed)

    def cols_of(width):
        return np.concatenate([g0 + rng.choice(min(128, width - g0), 2, replace=False) for g0 in range(0, width, 128)])

    checked = 0
    for g in range(E + Es):
        n = int(r["counts"][g]) if g < E else T
        if n == 0:
            continue
        l0 = int(r["offsets"][g]) if g < E else P + (g - E) * T
        first = np.arange(0, n, 32)
        rows = np.unique(np.concatenate([first, np.minimum(first + 31, n - 1)]))
        A = (xg[l0 + rows] if g < E else xh[rows]).astype(np.float64)
        ch, cd = cols_of(H), cols_of(d)
        W1 = layer._download_weight(L.W_W1, g, (H, d))[ch].astype(np.float64)
        W3 = layer._download_weight(L.W_W3, g, (H, d))[ch].astype(np.float64)
        h1, h3 = A @ W1.T, A @ W3.T
        ref_a = h1 / (1.0 + np.exp(-h1)) * h3
        got_a = a[l0 + rows][:, ch].astype(np.float64)
        # bf16 storage: half an ulp is 2^-9 relative; the sums are fp32
        bad = np.abs(got_a - ref_a) > 2.0 ** -8 * np.abs(ref_a) + 2e-5
        assert not bad.any(), ("a", g, rows[np.argwhere(bad)[0][0]], ch[np.argwhere(bad)[0][1]])
        W2 = layer._download_weight(L.W_W2, g, (d, H))[cd].astype(np.float64)
        ref_y = a[l0 + rows].astype(np.float64) @ W2.T
        got_y = y[l0 + rows][:, cd].astype(np.float64)
        scale = np.sqrt((ref_y ** 2).mean()) + 1e-30
        bad = np.abs(got_y - ref_y) > 1e-4 * (np.abs(ref_y) + scale)
        assert not bad.any(), ("y", g, rows[np.argwhere(bad)[0][0]], cd[np.argwhere(bad)[0][1]])
        checked += ref_a.size + ref_y.size
    return checked


def f32_twin(layer, cfg):
    """An fp32 layer holding the same (bf16-representable) weights as the bf16 layer `layer`: its products run on
    the fp32 tile kernel, a different code path that is pinned to the oracle at 1e-5.  The router forms the same sums
    bit for bit (products of bf16 values are exact in fp32), so both layers route alike."""
    import importlib
    L = importlib.import_module("omega-ai_amd._lib")
    c = ctx()
    twin = P.MoELayer(cfg.d, cfg.H, cfg.E, cfg.K, renorm=cfg.renorm, nShared=cfg.Es, bias=cfg.has_gate_bias, ctx=c,
                      dtype="f32", router_mode="exact", T_max=cfg.T)
    n = max(cfg.H * cfg.d, cfg.E * cfg.d)
    t16, t32 = P.DeviceBuffer(c, (n,), "bf16"), P.DeviceBuffer(c, (n,), "f32")
    items = [(L.W_GATE, 0, cfg.E * cfg.d)]
    for g in range(cfg.E + cfg.Es):
        items += [(L.W_W1, g, cfg.H * cfg.d), (L.W_W3, g, cfg.H * cfg.d), (L.W_W2, g, cfg.H * cfg.d)]
    for which, g, cnt in items:
        c.check(c.lib.omega_moe_get_weights(layer.handle, which, g, t16.ptr, 1))
        c.check(c.lib.omega_hip_convert(c.handle, t32.ptr, L.DTYPE_F32, t16.ptr, L.DTYPE_BF16, cnt))
        c.check(c.lib.omega_moe_set_weights(twin.handle, which, g, t32.ptr, 1))
    if cfg.has_gate_bias:
        twin._upload(L.W_GATE_BIAS, 0, layer._download_weight(L.W_GATE_BIAS, 0, (cfg.E,)))
    t16.free()
    t32.free()
    return twin


def f32_copy(buf):
    """fp32 device copy of a bf16 device buffer."""
    import importlib
    L = importlib.import_module("omega-ai_amd._lib")
    c = ctx()
    out = P.DeviceBuffer(c, buf.shape, "f32")
    c.check(c.lib.omega_hip_convert(c.handle, out.ptr, L.DTYPE_F32, buf.ptr, L.DTYPE_BF16, int(np.prod(buf.shape))))
    return out


def assert_rows_close(got, ref, tol_all, tol_row, what):
    """Relative L2 of the whole tensor within tol_all and of every single row within tol_row."""
    assert N.rel_l2(got, ref) <= tol_all, what
    num = np.sqrt(((got.astype(np.float64) - ref) ** 2).sum(axis=1))
    den = np.sqrt((ref.astype(np.float64) ** 2).sum(axis=1)) + 1e-30
    worst = int(np.argmax(num / den))
    assert (num / den)[worst] <= tol_row, (what, "row", worst, float((num / den)[worst]))
