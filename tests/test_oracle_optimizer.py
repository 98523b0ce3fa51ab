"""CPU-only: pins the oracle's restatement of the reference's weight update
(optimizers/SteepestDescentOptimizer.cu) against PyTorch's optimizers and closed forms in float64."""
import numpy as np
import torch

import oracle_lib as O


def _data(n=4000, seed=3):
    rng = np.random.default_rng(seed)
    w = rng.standard_normal(n).astype(np.float32)
    grads = [(rng.standard_normal(n) * 3).astype(np.float32) for _ in range(6)]
    return w, grads


def test_sgd_momentum_matches_torch_sgd():
    w0, grads = _data()
    lr, mom = 1e-3, 0.9
    w = w0.copy(); deltas = np.zeros_like(w)
    tw = torch.tensor(w0, dtype=torch.float64, requires_grad=True)
    opt = torch.optim.SGD([tw], lr=lr, momentum=mom)
    for g in grads:
        cur = np.empty_like(g)
        O.opt_accumulate(g, cur, add=False)
        O.opt_update_weights(w, cur, deltas, None, lr, mom)
        tw.grad = torch.tensor(g, dtype=torch.float64)
        opt.step()
    # tolerance: fp32 accumulation of 6 steps against float64
    assert np.max(np.abs(w - tw.detach().numpy())) < 1e-5


def test_adam_matches_torch_adam():
    w0, grads = _data()
    lr, frac = 1e-2, 37.0
    w = w0.copy(); deltas = np.zeros_like(w); stats = np.zeros(2 * w.size, np.float32)
    b1 = b2 = 1.0
    tw = torch.tensor(w0, dtype=torch.float64, requires_grad=True)
    opt = torch.optim.Adam([tw], lr=lr, betas=(0.9, 0.999), eps=1e-8)
    for g in grads:
        cur = g.copy()
        b1 = O.opt_next_beta_accum(b1, 1); b2 = O.opt_next_beta_accum(b2, 2)
        O.opt_adjust_gradient(5, cur, stats, None, frac, b1, b2)
        O.opt_update_weights(w, cur, deltas, None, lr, 0.0)
        tw.grad = torch.tensor(g, dtype=torch.float64) / frac
        opt.step()
    assert abs(b1 - 0.9 ** 6) < 1e-6 and abs(b2 - 0.999 ** 6) < 1e-6
    # fp32 moments against float64: a few 1e-7 per step relative to |update| = lr
    assert np.max(np.abs(w - tw.detach().numpy())) < 2e-5


def test_adagrad_and_averaging_closed_forms():
    w0, grads = _data()
    frac = 12.0
    stats = np.full(w0.size, 1e-6, np.float32)
    acc = np.full(w0.size, 1e-6, np.float64)
    for g in grads:
        cur = g.copy()
        O.opt_adjust_gradient(1, cur, stats, None, frac)
        ave = g.astype(np.float64) / frac
        acc += ave * ave
        assert np.max(np.abs(cur - ave / np.sqrt(acc))) < 1e-5
    assert np.max(np.abs(stats - acc) / acc) < 1e-5
    # stochastic AdaGrad only accumulates the statistics, the gradient is untouched
    cur = grads[0].copy(); st2 = np.full(w0.size, 1e-6, np.float32)
    O.opt_adjust_gradient(3, cur, st2, None, frac)
    assert np.array_equal(cur, grads[0])
    assert np.max(np.abs(st2 - (1e-6 + (grads[0].astype(np.float64) / frac) ** 2))) < 1e-6
    # option 2 divides by the fraction length, nothing else
    cur = grads[1].copy()
    O.opt_adjust_gradient(2, cur, None, None, frac)
    assert np.array_equal(cur, grads[1] / np.float32(frac))


def test_nan_inf_zeroing_mask_and_accumulate():
    n = 64
    g = np.arange(n, dtype=np.float32) - 20
    g[3] = np.nan; g[7] = np.inf; g[9] = -np.inf
    w = np.ones(n, np.float32); deltas = np.full(n, 0.5, np.float32)
    mask = np.ones(n, np.float32); mask[::4] = 0.0
    cur = g.copy()
    O.opt_update_weights(w, cur, deltas, mask, 0.1, 0.5)
    assert cur[3] == 0 and cur[7] == 0 and cur[9] == 0          # written back, as the reference does
    exp_delta = 0.5 * 0.5 - np.float32(0.1) * np.where(np.isfinite(g), g, 0)
    assert np.allclose(deltas, exp_delta, rtol=1e-6)
    assert np.allclose(w, (1 + exp_delta) * mask, rtol=1e-6) and np.all(w[::4] == 0)
    # masked weights are skipped by the adaptive adjustments (after the NaN zeroing)
    st = np.zeros(2 * n, np.float32); cur = g.copy()
    O.opt_adjust_gradient(5, cur, st, mask, 1.0, 0.9, 0.999)
    assert np.all(st.reshape(n, 2)[::4] == 0) and cur[0] == g[0] and np.all(st.reshape(n, 2)[1] != 0)
    # accumulate
    a = np.arange(8, dtype=np.float32); c = np.ones(8, np.float32)
    O.opt_accumulate(a, c, add=True)
    assert np.array_equal(c, a + 1)
    O.opt_accumulate(a, c, add=False)
    assert np.array_equal(c, a)
