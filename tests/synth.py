"""Host-side synthetic inputs for the parity tests, drawn with the C oracle's generator."""
import importlib

import numpy as np

from oracle import oracle as O

C = importlib.import_module("omega-ai_amd.configs")


def make_inputs(cfg, seed, T=None):
    """Returns dict x[T,d], Wg[E,d], bg[E]|None, W1,W3[E+Es,H,d], W2[E+Es,d,H] as fp32 arrays
    (rounded to bf16-representable values when cfg.dtype == 'bf16')."""
    T = cfg.T if T is None else T
    G = cfg.E + cfg.Es
    r = {}
    r["x"] = O.fill_normal(T * cfg.d, seed, C.STREAM_X, C.tensor_std(cfg, "x")).reshape(T, cfg.d)
    r["Wg"] = O.fill_normal(cfg.E * cfg.d, seed, C.STREAM_WG, C.tensor_std(cfg, "Wg")).reshape(cfg.E, cfg.d)
    r["bg"] = C.zipf_gate_bias(cfg, seed)
    for which, shape in (("W1", (cfg.H, cfg.d)), ("W3", (cfg.H, cfg.d)), ("W2", (cfg.d, cfg.H))):
        r[which] = np.stack([O.fill_normal(cfg.H * cfg.d, seed, C.expert_stream(g, which),
                                           C.tensor_std(cfg, which)).reshape(shape) for g in range(G)])
    if cfg.dtype == "bf16":
        for k in ("x", "Wg", "W1", "W3", "W2"):
            r[k] = O.round_bf16(r[k])
    return r


def scaled(cfg, **kw):
    """A copy of cfg with some dimensions replaced (CPU-sized variants of the big configs)."""
    import dataclasses
    return dataclasses.replace(cfg, **kw)
