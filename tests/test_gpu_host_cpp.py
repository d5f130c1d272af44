"""The C++ host mirror of the layer (omega-ai_amd/host/MoELayer.hpp) driven as a transformer block drives its
FFN slot, checked against the CPU oracle.  The demo binary is built by __graft_entry__.build()."""
import os
import subprocess
import tempfile

import numpy as np
import pytest

from oracle import oracle as O
from oracle import oracle_np as N
from tests.synth import C, make_inputs

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEMO = os.path.join(ROOT, "omega-ai_amd", "host", "moe_host_demo")


@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_cpp_layer_forward_and_checkpoint(dtype):
    assert os.path.exists(DEMO), "build omega-ai_amd/host/moe_host_demo first (__graft_entry__.build())"
    cfg = C.MoEConfig("t", T=200, d=256, E=8, K=2, H=384, Es=1, renorm=True, dtype=dtype)
    inp = make_inputs(cfg, 17)
    G = cfg.E + cfg.Es
    with tempfile.TemporaryDirectory() as td:
        inp["x"].astype("<f4").tofile(os.path.join(td, "x.bin"))
        model = np.concatenate([inp["Wg"].ravel()] + [np.concatenate([inp["W1"][g].ravel(), inp["W3"][g].ravel(),
                                                                     inp["W2"][g].ravel()]) for g in range(G)])
        model.astype("<f4").tofile(os.path.join(td, "model.bin"))
        gamma = (O.fill_normal(cfg.d, 17, C.STREAM_NORM, 1.0) * np.float32(0.1) + np.float32(1.0)).astype(np.float32)
        gamma.astype("<f4").tofile(os.path.join(td, "gamma.bin"))
        dout = O.fill_normal(cfg.T * cfg.d, 17, 900, 1.0).reshape(cfg.T, cfg.d)
        if dtype == "bf16":
            dout = O.round_bf16(dout)
        dout.astype("<f4").tofile(os.path.join(td, "dout.bin"))
        r = subprocess.run([DEMO, td, str(cfg.T), str(cfg.d), str(cfg.E), str(cfg.K), str(cfg.H), str(cfg.Es), "1",
                            "1" if dtype == "bf16" else "0"], capture_output=True, text=True, timeout=100)
        assert r.returncode == 0, r.stderr
        assert "layerType=feed_forward" in r.stdout
        out = np.fromfile(os.path.join(td, "out.bin"), "<f4").reshape(cfg.T, cfg.d)
        ids = np.fromfile(os.path.join(td, "ids.bin"), "<i4").reshape(cfg.T, cfg.K)
        saved = np.fromfile(os.path.join(td, "model_saved.bin"), "<f4")
        out_block = np.fromfile(os.path.join(td, "out_block.bin"), "<f4").reshape(cfg.T, cfg.d)
        dx = np.fromfile(os.path.join(td, "dx.bin"), "<f4").reshape(cfg.T, cfg.d)
        dW2_last = np.fromfile(os.path.join(td, "dW2_last.bin"), "<f4").reshape(cfg.d, cfg.H)
        dWg = np.fromfile(os.path.join(td, "dWg.bin"), "<f4").reshape(cfg.E, cfg.d)
        dx_block = np.fromfile(os.path.join(td, "dx_block.bin"), "<f4").reshape(cfg.T, cfg.d)
        dgamma = np.fromfile(os.path.join(td, "dgamma.bin"), "<f4")
        sumsq = float(np.fromfile(os.path.join(td, "gradsumsq.bin"), "<f4")[0])
        stepped = np.fromfile(os.path.join(td, "model_step.bin"), "<f4")
    ref = O.moe_forward(inp["x"], inp["Wg"], None, inp["W1"], inp["W3"], inp["W2"], cfg.K, True, cfg.Es, bf16=dtype == "bf16")
    assert np.array_equal(ids, ref["ids"])
    assert N.rel_l2(out, ref["out"]) <= (1e-2 if dtype == "bf16" else 1e-5)
    assert np.array_equal(saved, model.astype(np.float32))      # checkpoint round trip is byte-exact
    blk = O.block_forward(inp["x"], gamma, inp["Wg"], None, inp["W1"], inp["W3"], inp["W2"], cfg.K, True, cfg.Es,
                          bf16=dtype == "bf16")
    assert N.rel_l2(out_block, blk["out"]) <= (1e-2 if dtype == "bf16" else 1e-5)   # forwardBlock of the C++ layer
    bw = O.moe_backward(inp["x"], dout, inp["Wg"], None, inp["W1"], inp["W3"], inp["W2"], cfg.K, True, cfg.Es,
                        bf16=dtype == "bf16")
    tol = 1e-2 if dtype == "bf16" else 1e-5
    assert N.rel_l2(dx, bw["dx"]) <= tol                                            # back(Tensor) of the C++ layer
    assert N.rel_l2(dW2_last, bw["dW2"][cfg.E - 1]) <= tol and N.rel_l2(dWg, bw["dWg"]) <= tol
    bb = O.block_backward(inp["x"], gamma, dout, inp["Wg"], None, inp["W1"], inp["W3"], inp["W2"], cfg.K, True, cfg.Es,
                          bf16=dtype == "bf16")
    assert N.rel_l2(dx_block, bb["dx"]) <= tol and N.rel_l2(dgamma, bb["dgamma"]) <= tol     # backBlock of the C++ layer
    # gradSumSq / scaleGrad / updateAdamW / saveModelBlock of the C++ layer, on the gradients of its block backward:
    # the layer's term of the global norm against the oracle's gradients, and one AdamW step (train_time 1, no decay),
    # which moves every parameter by lr * g / (|g| + eps): against the sign of its gradient, by at most lr
    grads = [bb["dgamma"], bb["dWg"]] + [a for g in range(G) for a in (bb["dW1"][g], bb["dW3"][g], bb["dW2"][g])]
    want_ss = sum(float((a.astype(np.float64) ** 2).sum()) for a in grads)
    assert abs(sumsq - want_ss) <= 4 * tol * want_ss, (sumsq, want_ss)
    before = np.concatenate([gamma, model.astype(np.float32)])
    gflat = np.concatenate([a.ravel() for a in grads])
    assert stepped.shape == before.shape == gflat.shape
    move = stepped.astype(np.float64) - before
    lr = 2e-3
    assert np.abs(move).max() <= lr * 1.01 + (2.0 ** -8 * np.abs(before).max() if dtype == "bf16" else 0.0)
    clear = np.abs(gflat) > 1e-3 * np.abs(gflat).max()          # gradients whose sign the tolerance cannot flip
    assert clear.mean() > 0.3
    agree = np.sign(move[clear]) == -np.sign(gflat[clear])
    # (a bf16 weight moves only if the step crosses half a unit in the last place: most do at this step size)
    assert agree.mean() > (0.9 if dtype == "bf16" else 0.999), agree.mean()
