"""The entry point that allocates nothing (omega_moe_get_router_probs_noalloc) against the entry point it is a variant
of (omega_moe_get_router_probs): logits, probabilities and the routing state it leaves, bit for bit, on two calls in a
row - the second on a smaller batch, so that whatever the first call left in the shared static scratch is still there -
and the refusals (batch above the workspace, T*E above the scratch)."""
import importlib

import numpy as np
import pytest

from tests.synth import C, make_inputs

pytestmark = pytest.mark.gpu
L = importlib.import_module("omega-ai_amd._lib")


def free_device_bytes():
    """hipMemGetInfo through the runtime the library itself is linked against."""
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    free, total = ctypes.c_size_t(), ctypes.c_size_t()
    assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return free.value


@pytest.mark.parametrize("dtype,E,K,d", [("bf16", 8, 2, 512), ("f32", 12, 3, 96), ("bf16", 128, 8, 256)])
def test_noalloc_router_probs_matches_the_allocating_entry_point(dtype, E, K, d):
    from tests import gpu_util as G
    P = G.P
    cfg = C.MoEConfig("na", T=700, d=d, E=E, K=K, H=256, dtype=dtype, zipf_bias=1.2 if E == 128 else 0.0)
    inp = make_inputs(cfg, 11)
    layer = G.build_layer(cfg, inp, T_max=cfg.T)
    x = P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], dtype)
    for T in (cfg.T, 257):                                   # two calls in a row, the second with a smaller input
        lg0, p0 = layer.router_probs(x, T)                   # the existing entry point (stages in hipMalloc'ed memory)
        r0 = layer.routing(T)
        G.ctx().sync()
        free0 = free_device_bytes()
        lg1, p1 = layer.router_probs_noalloc(x, T)
        assert free_device_bytes() == free0, "the entry point allocated (or freed) device memory"
        r1 = layer.routing(T)
        assert np.array_equal(lg0.view(np.uint32), lg1.view(np.uint32)), T
        assert np.array_equal(p0.view(np.uint32), p1.view(np.uint32)), T
        assert np.array_equal(r0["ids"], r1["ids"]) and np.array_equal(r0["w"].view(np.uint32), r1["w"].view(np.uint32))
        assert np.isfinite(p1).all() and np.allclose(p1.sum(axis=1), 1.0, atol=1e-5)
    # the routing it leaves is what dispatch continues from, as after omega_moe_router
    layer.number = 257
    layer.stage("dispatch", x)
    assert layer.routing(257)["counts"].sum() == 257 * K
    layer.close()
    x.free()


def test_noalloc_router_probs_refusals():
    from tests import gpu_util as G
    P = G.P
    cfg = C.MoEConfig("na", T=64, d=256, E=8, K=2, H=256, dtype="bf16")
    inp = make_inputs(cfg, 12)
    lib, hctx = G.ctx().lib, G.ctx().handle
    # a layer without a workspace (T_max = 0), then one whose workspace is too small: never grown by this entry point
    for T_max in (0, 32):
        layer = G.build_layer(cfg, inp, T_max=T_max)
        x = P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], "bf16")
        buf = np.empty((cfg.T, cfg.E), np.float32)
        st = lib.omega_moe_get_router_probs_noalloc(layer.handle, x.ptr, cfg.T, buf.ctypes.data, buf.ctypes.data)
        assert st == L.ERR_INVALID_ARG and b"never allocates" in lib.omega_hip_last_error(hctx)
        layer.close()
        x.free()
    # T*E above the static scratch: 16384 tokens x 128 experts
    big = C.MoEConfig("na", T=16384, d=256, E=128, K=8, H=256, dtype="bf16")
    layer = P.MoELayer(big.d, big.H, big.E, big.K, ctx=G.ctx(), dtype="bf16", T_max=big.T)
    x = P.DeviceBuffer(G.ctx(), (big.T, big.d), "bf16")
    x.fill_normal(1, 0, 1.0)
    buf = np.empty((big.T, big.E), np.float32)
    st = lib.omega_moe_get_router_probs_noalloc(layer.handle, x.ptr, big.T, buf.ctypes.data, buf.ctypes.data)
    assert st == L.ERR_UNSUPPORTED and b"static scratch" in lib.omega_hip_last_error(hctx)
    # ... and half of that batch fits exactly (8192 x 128 = 2^20)
    lg, p = layer.router_probs_noalloc(x, 8192)
    lg0, p0 = layer.router_probs(x, 8192)
    assert np.array_equal(lg.view(np.uint32), lg0.view(np.uint32)) and np.array_equal(p.view(np.uint32), p0.view(np.uint32))
    layer.close()
    x.free()
