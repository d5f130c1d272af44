"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py from the pinned oracle).

CPU: the oracle still reproduces every fixture bit for bit (guards the oracle against drift).
GPU: the HIP path reproduces the routing arrays bit for bit and the output within tolerance."""
import importlib.util
import os

import numpy as np
import pytest

from oracle import oracle_np as N

HERE = os.path.dirname(os.path.abspath(__file__))
spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(HERE, "golden", "make_fixtures.py"))
MF = importlib.util.module_from_spec(spec)
spec.loader.exec_module(MF)


def load(name):
    return dict(np.load(os.path.join(HERE, "golden", name + ".npz")))


@pytest.mark.parametrize("name", sorted(MF.CASES))
def test_oracle_reproduces_fixture(name):
    want, got = load(name), MF.expected(MF.CASES[name])
    assert sorted(want) == sorted(got)
    for k in want:
        assert np.array_equal(want[k], got[k]), (name, k)


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(MF.CASES))
def test_hip_path_reproduces_fixture(name):
    from tests import gpu_util as G
    case = MF.CASES[name]
    cfg, want = case["cfg"], load(name)
    inp = MF.case_inputs(case)
    layer = G.build_layer(cfg, inp)
    x = G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype)
    out = layer.forward(x).to_numpy()
    r = layer.routing()
    for k in ("ids", "counts", "offsets", "dst", "src_row"):
        assert np.array_equal(r[k], want[k]), (name, k)
    assert np.array_equal(r["w"].view(np.uint32), want["w"].view(np.uint32))
    tol = 1e-2 if cfg.dtype == "bf16" else 1e-5
    assert N.rel_l2(out[:4], want["out_head"]) <= tol and N.rel_l2(out[-2:], want["out_tail"]) <= tol
    o64 = out.astype(np.float64)
    assert abs(np.sqrt((o64 ** 2).sum()) - want["out_l2"]) <= tol * want["out_l2"]
    assert abs(o64.sum() - want["out_sum"]) <= tol * want["out_abs_sum"]
    layer.close()


@pytest.mark.parametrize("name", sorted(MF.BW_CASES))
def test_oracle_reproduces_backward_fixture(name):
    want, got = load("bw_" + name), MF.expected_backward(MF.CASES[name])
    assert sorted(want) == sorted(got)
    for k in want:
        assert np.array_equal(want[k], got[k]), (name, k)


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(MF.BW_CASES))
def test_hip_path_reproduces_backward_fixture(name):
    import importlib
    from tests import gpu_util as G
    L = importlib.import_module("omega-ai_amd._lib")
    case = MF.CASES[name]
    cfg, want = case["cfg"], load("bw_" + name)
    inp = MF.case_inputs(case)
    layer = G.build_layer(cfg, inp)
    x = G.P.DeviceBuffer.from_numpy(G.ctx(), inp["x"], cfg.dtype)
    g = G.P.DeviceBuffer.from_numpy(G.ctx(), MF.backward_dout(case), cfg.dtype)
    layer.forward(x)
    dx = layer.back(g).to_numpy()
    tol = 1e-2 if cfg.dtype == "bf16" else 1e-5
    assert N.rel_l2(dx[:4], want["dx_head"]) <= tol and N.rel_l2(dx[-2:], want["dx_tail"]) <= tol
    d64 = dx.astype(np.float64)
    assert abs(np.sqrt((d64 ** 2).sum()) - want["dx_l2"]) <= tol * want["dx_l2"]
    assert abs(d64.sum() - want["dx_sum"]) <= tol * want["dx_abs_sum"]
    assert N.rel_l2(layer.grad(L.W_GATE), want["dWg"]) <= tol
    if "dbg" in want:
        assert N.rel_l2(layer.grad(L.W_GATE_BIAS), want["dbg"]) <= tol
    for i, which in enumerate((L.W_W1, L.W_W3, L.W_W2)):
        for e in range(cfg.E + cfg.Es):
            n = np.sqrt((layer.grad(which, e).astype(np.float64) ** 2).sum())
            assert abs(n - want["dW_norms"][i, e]) <= tol * max(want["dW_norms"][i, e], 1e-30), (i, e)
    e = int(np.argmax(want["dW_norms"][2]))
    assert N.rel_l2(layer.grad(L.W_W2, e)[0], want["dW2_first_row"]) <= tol
    layer.close()



def test_oracle_reproduces_adamw_fixture():
    want, got = load("adamw_steps"), MF.expected_adamw()
    assert sorted(want) == sorted(got) and len(want) == 3 * MF.ADAMW["steps"]
    for k in want:
        assert np.array_equal(want[k].view(np.uint32), got[k].view(np.uint32)), k
    # the frozen run did something: every parameter with a non-zero first gradient moved by about lr at step 1
    w0, grads = MF.adamw_inputs()
    moved = np.abs(want["w1"].astype(np.float64) - w0)
    nz = grads[0] != 0
    assert nz.sum() > 400 and np.all(moved[nz] > 0.5 * MF.ADAMW["lr"]) and np.all(moved[~nz] < 0.1 * MF.ADAMW["lr"])
