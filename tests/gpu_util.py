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
