"""Pins the AdamW oracle (oracle/omega_updater.c) without the reference running: torch.optim.AdamW in float64 (an
independent implementation of the same algebra), the closed form of the first step, and pure decay at zero gradient."""
import numpy as np
import torch

from oracle import oracle as O


def _torch_adamw(w0, grads, lr, b1, b2, wd, eps=1e-8):
    p = torch.nn.Parameter(torch.tensor(w0, dtype=torch.float64))
    opt = torch.optim.AdamW([p], lr=lr, betas=(b1, b2), eps=eps, weight_decay=wd)
    for g in grads:
        p.grad = torch.tensor(g, dtype=torch.float64)
        opt.step()
    return p.detach().numpy()


def test_adamw_matches_torch_float64():
    rng = np.random.default_rng(3)
    n = 4096
    w0 = rng.standard_normal(n).astype(np.float32)
    grads = [(rng.standard_normal(n) * 10.0 ** rng.uniform(-4, 1, n)).astype(np.float32) for _ in range(12)]
    # float32 views of the hyper-parameters, as the reference passes them
    lr, b1, b2, wd = (float(np.float32(v)) for v in (2e-3, 0.9, 0.95, 1e-2))
    w, m, v = w0.copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    for t, g in enumerate(grads, 1):
        w, m, v = O.adamw(w, g, m, v, lr, b1, b2, wd, t)
    want = _torch_adamw(w0, grads, lr, b1, b2, wd)
    # torch adds eps to sqrt(v)/sqrt(1-b2^t), the reference to sqrt(v/(1-b2^t)): the same number
    assert np.max(np.abs(w - want)) < 2e-6 * max(1.0, np.max(np.abs(want)))
    # the moments are plain exponential averages
    mm, ma, vv = np.zeros(n), np.zeros(n), np.zeros(n)
    for g in grads:
        mm = b1 * mm + (1 - b1) * g.astype(np.float64)
        ma = b1 * ma + (1 - b1) * np.abs(g.astype(np.float64))      # the scale the float32 roundings of m live on
        vv = b2 * vv + (1 - b2) * g.astype(np.float64) ** 2
    assert np.all(np.abs(m - mm) <= 1e-6 * ma) and np.allclose(v, vv, rtol=2e-6, atol=0)


def test_adamw_first_step_closed_form():
    # step 1: m_hat = g and v_hat = g^2, so w1 = w0 - lr * (g / (|g| + eps) + wd * w0)
    w0 = np.array([1.0, -2.0, 0.5, 3.0], np.float32)
    g = np.array([0.3, -7.0, 1e-3, 0.0], np.float32)
    lr, wd = 0.125, 0.25                      # powers of two: the expected values are exact in float32
    w, m, v = O.adamw(w0, g, np.zeros(4, np.float32), np.zeros(4, np.float32), lr, 0.9, 0.95, wd, 1)
    g64 = g.astype(np.float64)
    want = w0.astype(np.float64) - lr * (g64 / (np.abs(g64) + 1e-8) + wd * w0.astype(np.float64))
    assert np.allclose(w, want, rtol=0, atol=3e-7)
    assert w[3] == np.float32(3.0 - 0.125 * 0.25 * 3.0)          # zero gradient: decay only, exact
    assert np.allclose(m, 0.1 * g, rtol=1e-6) and np.allclose(v, 0.05 * g.astype(np.float64) ** 2, rtol=1e-6)


def test_adamw_correction_is_the_host_side_double_power():
    # (float)(1.0f - Math.pow(beta, t)) with beta a float promoted to double
    for beta in (0.9, 0.95, 0.999):
        for t in (1, 2, 10, 1000):
            want = np.float32(1.0 - float(np.float32(beta)) ** t)
            assert O.lib().orc_adamw_correction(beta, t) == want


def test_adamw_without_decay_moves_against_the_gradient_by_at_most_lr_over_correction():
    rng = np.random.default_rng(5)
    w0 = rng.standard_normal(1000).astype(np.float32)
    g = rng.standard_normal(1000).astype(np.float32)
    w, _, _ = O.adamw(w0, g, np.zeros(1000, np.float32), np.zeros(1000, np.float32), 1e-2, 0.9, 0.95, 0.0, 1)
    step = w.astype(np.float64) - w0
    assert np.all(np.sign(step) == -np.sign(g)) and np.all(np.abs(step) <= 1e-2 * (1 + 1e-5))
