"""Pins the CPU oracle's LSTM against independent statements: torch.nn.LSTM (library routine,
peepholes off), and float64 autograd of a hand-written graph (peepholes, masking, both directions)."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle_lib as O
from torch_models import lstm_forward_torch, make_pat_types


def relerr(a, b):
    a = np.asarray(a, dtype=np.float64).ravel()
    b = np.asarray(b, dtype=np.float64).ravel()
    return np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30)


def run_oracle(P, L, bidir, S, T, lengths, W, x, outerr, bias=1.0):
    nd = 2 if bidir else 1
    H = L // nd
    N = T * S
    pat = make_pat_types(lengths, T)
    desc = O.LstmDesc(P, L, int(bidir), S, T, min(lengths), bias)
    fw = O.LstmState(H, N)
    bw = O.LstmState(H, N) if bidir else None
    out = np.zeros(L * N, dtype=np.float32)
    O.lstm_forward(desc, W, pat, x, fw, bw, out)
    ex = np.zeros(P * N, dtype=np.float32)
    dW = np.zeros_like(W)
    O.lstm_backward(desc, W, pat, x, outerr, fw, bw, ex, dW)
    return out, ex, dW, fw, bw, pat


def case(P, L, bidir, S, T, lengths, seed, wscale=0.3, escale=0.1):
    rng = np.random.default_rng(seed)
    nW = O.lib().orc_lstm_weight_count(P, L, int(bidir))
    W = rng.uniform(-wscale, wscale, nW).astype(np.float32)
    x = rng.standard_normal((T, S, P)).astype(np.float32)
    outerr = (escale * rng.standard_normal((T, S, L))).astype(np.float32)
    for s, n in enumerate(lengths):
        x[n:, s] = 0
        outerr[n:, s] = 0
    return W, x.reshape(-1), outerr.reshape(-1)


@pytest.mark.parametrize("bidir,lengths", [(False, [7, 7, 7]), (False, [7, 4, 6]), (True, [6, 6]), (True, [8, 3, 5, 8])])
def test_lstm_matches_autograd(bidir, lengths):
    P, H = 5, 4
    L = H * (2 if bidir else 1)
    S, T = len(lengths), max(lengths)
    W, x, outerr = case(P, L, bidir, S, T, lengths, seed=11 + len(lengths))
    out, ex, dW, fw, bw, pat = run_oracle(P, L, bidir, S, T, lengths, W, x, outerr, bias=1.0)
    # the clip must be inactive for the autograd comparison to be meaningful
    for st in [fw] + ([bw] if bidir else []):
        for k in ("dni", "dig", "dfg", "dog"):
            assert np.abs(st[k]).max() < 0.999

    Wt = torch.tensor(W, dtype=torch.float64, requires_grad=True)
    xt = torch.tensor(x.reshape(T, S, P), dtype=torch.float64, requires_grad=True)
    o = lstm_forward_torch(Wt, xt, lengths, P, L, bidir, S, T, 1.0)
    assert relerr(out, o.detach().numpy()) < 2e-6
    loss = (o * torch.tensor(outerr.reshape(T, S, L), dtype=torch.float64)).sum()
    loss.backward()
    assert relerr(ex, xt.grad.numpy()) < 1e-5
    assert relerr(dW, Wt.grad.numpy()) < 1e-5
    # every weight class separately, so that a wrong block cannot hide in the norm
    nd = 2 if bidir else 1
    o_b, o_i, o_p = 4 * P * L, 4 * P * L + 4 * L, 4 * P * L + 4 * L + 4 * L * (L // nd)
    g = Wt.grad.numpy()
    for lo, hi in [(0, o_b), (o_b, o_i), (o_i, o_p), (o_p, len(W))]:
        assert relerr(dW[lo:hi], g[lo:hi]) < 1e-5
    # masking: dummy slots carry exact zeros
    Hh = L // nd
    dummy = (pat == 0)
    if dummy.any():
        for st in [fw] + ([bw] if bidir else []):
            for k in ("dni", "dig", "dfg", "dog", "cerr", "h"):
                assert not st[k].reshape(-1, Hh)[dummy].any()
        assert not ex.reshape(-1, P)[dummy].any()


def test_bias_scale_enters_forward_and_gradient():
    P, L, S, T = 3, 4, 2, 5
    lengths = [5, 5]
    W, x, outerr = case(P, L, False, S, T, lengths, seed=5)
    out, ex, dW, *_ = run_oracle(P, L, False, S, T, lengths, W, x, outerr, bias=0.5)
    Wt = torch.tensor(W, dtype=torch.float64, requires_grad=True)
    xt = torch.tensor(x.reshape(T, S, P), dtype=torch.float64)
    o = lstm_forward_torch(Wt, xt, lengths, P, L, False, S, T, 0.5)
    (o * torch.tensor(outerr.reshape(T, S, L), dtype=torch.float64)).sum().backward()
    assert relerr(out, o.detach().numpy()) < 2e-6
    assert relerr(dW, Wt.grad.numpy()) < 1e-5


def test_forward_equals_torch_nn_lstm_without_peepholes():
    """Library-routine check: with zero peepholes and bias input 1 the layer is a textbook LSTM."""
    P, H, S, T = 6, 5, 3, 9
    lengths = [T] * S
    W, x, outerr = case(P, H, False, S, T, lengths, seed=3)
    o_b = 4 * P * H
    o_i = o_b + 4 * H
    o_p = o_i + 4 * H * H
    W[o_p:] = 0
    out, ex, dW, *_ = run_oracle(P, H, False, S, T, lengths, W, x, outerr)
    lstm = torch.nn.LSTM(P, H, bias=True).double()
    # reference gate order ni, ig, fg, og  ->  torch order i, f, g, o
    order = [1, 2, 0, 3]
    Wd = torch.tensor(W, dtype=torch.float64)
    w_ih = torch.cat([Wd[g * P * H:(g + 1) * P * H].reshape(H, P) for g in order], 0)
    w_hh = torch.cat([Wd[o_i + g * H * H: o_i + (g + 1) * H * H].reshape(H, H) for g in order], 0)
    b = torch.cat([Wd[o_b + g * H: o_b + (g + 1) * H] for g in order], 0)
    with torch.no_grad():
        lstm.weight_ih_l0.copy_(w_ih)
        lstm.weight_hh_l0.copy_(w_hh)
        lstm.bias_ih_l0.copy_(b)
        lstm.bias_hh_l0.zero_()
    xt = torch.tensor(x.reshape(T, S, P), dtype=torch.float64, requires_grad=True)
    o, _ = lstm(xt)
    assert relerr(out, o.detach().numpy()) < 2e-6
    (o * torch.tensor(outerr.reshape(T, S, H), dtype=torch.float64)).sum().backward()
    assert relerr(ex, xt.grad.numpy()) < 1e-5
    gW = torch.cat([lstm.weight_ih_l0.grad[k * H:(k + 1) * H].reshape(-1) for k in [2, 0, 1, 3]])
    assert relerr(dW[:o_b], gW.numpy()) < 1e-5
    gI = torch.cat([lstm.weight_hh_l0.grad[k * H:(k + 1) * H].reshape(-1) for k in [2, 0, 1, 3]])
    assert relerr(dW[o_i:o_p], gI.numpy()) < 1e-5


def test_clip_and_stored_output_gate_delta():
    """Large errors: stored deltas are clipped to [-1,1] while the cell error is not; a second backward
    without clearing the output-gate deltas adds the stored value (read-modify-write)."""
    P, L, S, T = 3, 4, 2, 6
    lengths = [6, 4]
    W, x, outerr = case(P, L, False, S, T, lengths, seed=9, wscale=1.0, escale=30.0)
    out, ex, dW, fw, _, pat = run_oracle(P, L, False, S, T, lengths, W, x, outerr)
    for k in ("dni", "dig", "dfg", "dog"):
        assert np.abs(fw[k]).max() <= 1.0
    assert max(np.abs(fw[k]).max() for k in ("dni", "dig", "dfg", "dog")) == 1.0
    assert np.abs(fw["cerr"]).max() > 1.0
    # hand check of the last processed... first processed step (t=T-1, s=0): no recurrent terms
    t, s, H = T - 1, 0, L
    o_p = 4 * P * L + 4 * L + 4 * L * L
    for j in range(H):
        i = (t * S + s) * H + j
        og, c, e = fw["og"][i], fw["c"][i], outerr[i]
        tc = np.tanh(np.float64(c))
        d_og = og * (1 - og) * tc * e
        ce = og * (1 - tc * tc) * e + W[o_p + 2 * L + j] * d_og
        assert abs(fw["cerr"][i] - ce) <= 1e-4 * max(1.0, abs(ce))
        assert abs(fw["dog"][i] - np.clip(d_og, -1, 1)) <= 1e-5
    # second call: the stale output-gate delta is added
    dog_before = fw["dog"].copy()
    N = T * S
    desc = O.LstmDesc(P, L, 0, S, T, min(lengths), 1.0)
    ex2 = np.zeros(P * N, dtype=np.float32)
    dW2 = np.zeros_like(W)
    O.lstm_backward(desc, W, pat, x, outerr, fw, None, ex2, dW2)
    i = (t * S + s) * H
    og, c, e = fw["og"][i], fw["c"][i], outerr[i]
    expect = np.clip(og * (1 - og) * np.tanh(np.float64(c)) * e + dog_before[i], -1, 1)
    assert abs(fw["dog"][i] - expect) <= 1e-5


def test_scalar_semantics():
    L = O.lib()
    assert L.orc_logistic(100.0) == 1.0 and L.orc_logistic(-100.0) == 0.0
    assert abs(L.orc_logistic(0.3) - 1 / (1 + np.exp(-0.3))) < 1e-7
    assert abs(L.orc_tanh(0.7) - np.tanh(0.7)) < 2e-7
    assert L.orc_tanh(60.0) == 1.0 and L.orc_tanh(-60.0) == -1.0
    assert L.orc_safe_exp(-2e30) == 0.0 and L.orc_safe_exp(89.0) == np.float32(3.4028235e38)
    assert L.orc_safe_log(1e-39) == np.float32(-1e30)
    assert abs(L.orc_log_add(-1.0, -2.0) - np.logaddexp(-1.0, -2.0)) < 1e-6
    assert L.orc_log_add(-1.0, -80.0) == -1.0
    assert L.orc_log_add(-1e10, -2e10) == np.float32(-1e30)


def test_mat_product_matches_numpy():
    rng = np.random.default_rng(0)
    m, n, k = 5, 4, 7
    for tA, tB in [(0, 0), (1, 0), (0, 1)]:
        A = rng.standard_normal((k, m) if not tA else (m, k)).astype(np.float32)  # column-major storage
        B = rng.standard_normal((n, k) if not tB else (k, n)).astype(np.float32)
        Cm = np.ones(m * n, dtype=np.float32)
        O.mat_product(Cm, m, n, k, A.reshape(-1), tA, B.reshape(-1), tB, 1)
        Am = A.T if not tA else A  # m x k
        Bm = B.T if not tB else B  # k x n
        want = 1 + (Am.astype(np.float64) @ Bm.astype(np.float64))
        assert relerr(Cm.reshape(n, m).T, want) < 1e-6


def test_oracle_thread_count_does_not_change_results():
    """Threads share out whole output elements; every sum stays sequential, so results are bit-identical."""
    P, L, lengths = 40, 128, [30, 22, 30, 9]
    S, T = len(lengths), max(lengths)
    H, N = L // 2, T * S
    rng = np.random.default_rng(9)
    W = rng.uniform(-0.1, 0.1, O.lib().orc_lstm_weight_count(P, L, 1)).astype(np.float32)
    x = rng.standard_normal(T * S * P).astype(np.float32)
    outerr = (0.1 * rng.standard_normal(T * S * L)).astype(np.float32)
    pat = make_pat_types(lengths, T)
    results = []
    for threads in (1, 4):
        O.set_threads(threads)
        desc = O.LstmDesc(P, L, 1, S, T, min(lengths), 1.0)
        fw, bw = O.LstmState(H, N), O.LstmState(H, N)
        out = np.zeros(L * N, dtype=np.float32)
        O.lstm_forward(desc, W, pat, x, fw, bw, out)
        ex = np.zeros(P * N, dtype=np.float32)
        dW = np.zeros_like(W)
        O.lstm_backward(desc, W, pat, x, outerr, fw, bw, ex, dW)
        results.append((out, ex, dW))
    O.set_threads(1)
    for a, b in zip(*results):
        assert np.array_equal(a, b)
