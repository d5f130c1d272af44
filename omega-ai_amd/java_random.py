"""java.util.Random through the library's host-side implementation (omega_jrandom_*), for initialising a layer with the
numbers a Java run of the reference draws.

RandomUtils keeps ONE java.util.Random (RandomUtils.setSeed / getInstance, J/common/utils/RandomUtils.java:18-28);
RandomUtils.normal_(n, mean, std) fills n floats with (float)(std * nextGaussian() + mean) (RandomUtils.java:697-703).
LlamaMLPLayer.initLayers draws linear1, linear2, linear3 in that order, each normal_(n, 0.01f, 0.02f)
(J/engine/nn/layer/llama/LlamaMLPLayer.java:68-90; the kaiming_uniform of the FullyLayer constructors before them uses
Math.random(), another generator, and is overwritten).
"""
import ctypes as C

import numpy as np

from . import _lib as L


class JRandomStruct(C.Structure):
    _fields_ = [("state", C.c_int64), ("next_gaussian", C.c_double), ("have_next_gaussian", C.c_int32)]


class JavaRandom:
    """new java.util.Random(seed)."""

    def __init__(self, seed):
        self.lib = L.load_library()
        self.r = JRandomStruct()
        self.setSeed(seed)

    def setSeed(self, seed):
        self.lib.omega_jrandom_seed(C.byref(self.r), int(seed))

    def nextInt(self):
        return self.lib.omega_jrandom_next_int(C.byref(self.r))

    def nextDouble(self):
        return self.lib.omega_jrandom_next_double(C.byref(self.r))

    def nextGaussian(self):
        return self.lib.omega_jrandom_next_gaussian(C.byref(self.r))

    def normal_(self, n, mean, std):
        """RandomUtils.normal_: n float32 values."""
        out = np.empty(int(n), np.float32)
        self.lib.omega_jrandom_normal(C.byref(self.r), out.ctypes.data, int(n), float(mean), float(std))
        return out


def init_layer(layer, rng, mean=0.01, std=0.02):
    """Weights in the house style of LlamaMLPLayer.initLayers from the shared generator `rng`: the gate [E,d] first
    (the reference has no gate; it is drawn like the other weights), then per expert, routed before shared, linear1
    (W1 [H,d]), linear2 (W2 [d,H]), linear3 (W3 [H,d]) in the order the reference constructs them.  Returns the arrays."""
    d, H, E, G = layer.embedDim, layer.hidden, layer.nExperts, layer.nExperts + layer.nShared
    Wg = rng.normal_(E * d, mean, std).reshape(E, d)
    layer.set_gate(Wg, np.zeros(E, np.float32) if layer.hasBias else None)
    W1, W2, W3 = [], [], []
    for g in range(G):
        W1.append(rng.normal_(H * d, mean, std).reshape(H, d))
        W2.append(rng.normal_(d * H, mean, std).reshape(d, H))
        W3.append(rng.normal_(H * d, mean, std).reshape(H, d))
        layer.set_expert(g, W1[-1], W3[-1], W2[-1])
    return dict(Wg=Wg, W1=np.stack(W1), W3=np.stack(W3), W2=np.stack(W2))
