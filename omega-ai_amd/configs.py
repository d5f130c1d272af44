"""The five workload configurations and the layout of the seeded synthetic tensors.

One 64-bit seed fixes every tensor: tensor `name` is stream STREAMS[name] of the counter-based
normal generator (see csrc/fill.hip); element i of a tensor is element i of its stream in
row-major order.  x ~ N(0,1); W1,W3 ~ N(0,1/sqrt(d)); W2 ~ N(0,1/sqrt(H)); Wg ~ N(0,0.02).
Expert g (routed 0..E-1, then shared E..E+Es-1) uses streams 16+3g (W1), 17+3g (W3), 18+3g (W2).
"""
import math
from dataclasses import dataclass

import numpy as np

STREAM_X = 0
STREAM_WG = 1
STREAM_BG_PERM = 2
STREAM_NORM = 3       # gamma of the RMSNorm in front of the layer (block form): 1 + 0.1 * N(0,1)
STREAM_EXPERT0 = 16


@dataclass(frozen=True)
class MoEConfig:
    name: str
    T: int
    d: int
    E: int
    K: int
    H: int
    Es: int = 0
    renorm: bool = True
    dtype: str = "bf16"          # "f32" | "bf16"
    zipf_bias: float = 0.0       # exponent s of the Zipf gate bias (0 = no bias)
    batch: int = 1
    seq: int = 1

    @property
    def P(self):
        return self.T * self.K

    @property
    def has_gate_bias(self):
        return self.zipf_bias != 0.0

    def expert_flops(self):
        return 6 * self.d * self.H * (self.P + self.T * self.Es)

    def weight_bytes(self):
        b = 2 if self.dtype == "bf16" else 4
        return 3 * self.d * self.H * b * (self.E + self.Es)


CONFIGS = {
    "c1_tiny_f32": MoEConfig("c1_tiny_f32", T=256, d=128, E=8, K=2, H=256, dtype="f32", batch=4, seq=64),
    "c2_mixtral": MoEConfig("c2_mixtral", T=4096, d=4096, E=8, K=2, H=14336, batch=8, seq=512),
    "c3_decode": MoEConfig("c3_decode", T=64, d=4096, E=8, K=2, H=14336, batch=64, seq=1),
    "c4_finegrained": MoEConfig("c4_finegrained", T=8192, d=2048, E=64, K=6, H=1408, Es=2, renorm=False),
    "c5_skewed": MoEConfig("c5_skewed", T=16384, d=2048, E=128, K=8, H=768, zipf_bias=1.2),
}


def tensor_std(cfg, which):
    return {"x": 1.0, "Wg": 0.02, "W1": 1.0 / math.sqrt(cfg.d), "W3": 1.0 / math.sqrt(cfg.d),
            "W2": 1.0 / math.sqrt(cfg.H)}[which]


def expert_stream(g, which):
    return STREAM_EXPERT0 + 3 * g + {"W1": 0, "W3": 1, "W2": 2}[which]


def zipf_gate_bias(cfg, seed):
    """bg[e] = 2*log(rank_e^-s / sum_r r^-s) over a seeded permutation of the experts (host, fp64 -> fp32).
    The permutation sorts the experts by a SplitMix64 hash of (seed, stream 2, e)."""
    if not cfg.has_gate_bias:
        return None
    E = cfg.E
    m1, m2 = 0xBF58476D1CE4E5B9, 0x94D049BB133111EB
    mask = (1 << 64) - 1

    def mix(z):
        z = ((z ^ (z >> 30)) * m1) & mask
        z = ((z ^ (z >> 27)) * m2) & mask
        return z ^ (z >> 31)

    key = mix(seed ^ mix((STREAM_BG_PERM * 0xD1342543DE82EF95 + 1) & mask))
    h = [mix((key + 0x9E3779B97F4A7C15 * (e + 1)) & mask) for e in range(E)]
    order = sorted(range(E), key=lambda e: h[e])          # order[r] = expert with rank r+1
    wts = np.array([(r + 1) ** (-cfg.zipf_bias) for r in range(E)], np.float64)
    wts /= wts.sum()
    bg = np.empty(E, np.float64)
    for r, e in enumerate(order):
        bg[e] = 2.0 * math.log(wts[r])
    return bg.astype(np.float32)
