"""Pins the CPU oracle's WaveNet blocks: the 1-D dilated convolution against torch conv1d + autograd
(per sequence, zero padding), the conditioned gated activation against float64 autograd, and the
index-only helpers (context up-sampling, frame-rate gradient sum, skip fan-out) against brute force."""
import numpy as np
import torch

import oracle_lib as O
from test_oracle_lstm import relerr
from torch_models import make_pat_types


def cnn_case(P, hw, inter, lengths, causal, out_tanh, seed):
    D = len(hw)
    S, T = len(lengths), max(lengths)
    N = T * S
    rng = np.random.default_rng(seed)
    Lw = O.cnn_total_width(hw)
    W = rng.uniform(-0.3, 0.3, P * Lw + D).astype(np.float32)
    x = rng.standard_normal((T, S, P)).astype(np.float32)
    err = rng.standard_normal((T, S, D)).astype(np.float32)
    pat = make_pat_types(lengths, T)
    for s, n in enumerate(lengths):
        x[n:, s] = 0
        err[n:, s] = 0
    return D, S, T, N, Lw, W, x, err, pat


def torch_cnn(W, x, lengths, P, hw, inter, causal, out_tanh, bias, Lw):
    """Per sequence conv1d; returns outputs (T,S,D) with zeros on padding."""
    D, (T, S) = len(hw), x.shape[:2]
    cum = np.concatenate([[0], np.cumsum(2 * hw + 1)])
    Wm = W[:P * Lw].reshape(Lw, P)  # column-major P x Lw  ->  [col][p]
    b = W[P * Lw:]
    out = torch.zeros(T, S, D, dtype=W.dtype)
    for s, n in enumerate(lengths):
        xs = x[:n, s].T.unsqueeze(0)  # 1 x P x n
        for d in range(D):
            taps = range(-hw[d], (0 if causal else hw[d]) + 1)
            w = torch.stack([Wm[cum[d] + hw[d] + k] for k in taps], dim=1).unsqueeze(0)  # 1 x P x taps
            dil = int(inter[d])
            left = hw[d] * dil
            right = 0 if causal else hw[d] * dil
            xp = torch.nn.functional.pad(xs, (left, right))
            y = torch.nn.functional.conv1d(xp, w, dilation=dil)[0, 0] + b[d] * bias
            out[:n, s, d] = torch.tanh(y) if out_tanh else y
    return out


def run_cnn(P, hw, inter, lengths, causal, out_tanh, seed, bias=1.0):
    hw = np.asarray(hw, dtype=np.int32)
    inter = np.asarray(inter, dtype=np.int32)
    D, S, T, N, Lw, W, x, err, pat = cnn_case(P, hw, inter, lengths, causal, out_tanh, seed)
    con = np.zeros(Lw * N, dtype=np.float32)
    out = np.zeros(D * N, dtype=np.float32)
    O.cnn_forward(P, D, S, T, causal, out_tanh, bias, hw, inter, pat, W, x.reshape(-1), con, out)
    e = err.reshape(-1).copy()
    ex = np.zeros(P * N, dtype=np.float32)
    dW = np.zeros_like(W)
    O.cnn_backward(P, D, S, T, causal, out_tanh, bias, hw, inter, pat, W, x.reshape(-1), out, e, con, ex, dW)

    Wt = torch.tensor(W, dtype=torch.float64, requires_grad=True)
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    o = torch_cnn(Wt, xt, lengths, P, hw, inter, causal, out_tanh, bias, Lw)
    (o * torch.tensor(err, dtype=torch.float64)).sum().backward()
    assert relerr(out.reshape(T, S, D), o.detach().numpy()) < 2e-6
    assert relerr(ex.reshape(T, S, P), xt.grad.numpy()) < 1e-5
    assert relerr(dW, Wt.grad.numpy()) < 1e-5
    return dW, Lw, hw


def test_cnn_causal_dilated_kernel2_matches_conv1d():
    # the WaveNet setting: half width 1 (three columns per filter), causal, one dilation for all filters
    dW, Lw, hw = run_cnn(5, [1] * 6, [4] * 6, [17, 9, 14], causal=1, out_tanh=1, seed=1)
    # the future tap (third column of every filter) receives no gradient at all
    P = 5
    cols = dW[:P * Lw].reshape(Lw, P)
    assert not cols[2::3].any()
    assert cols[0::3].any() and cols[1::3].any()


def test_cnn_noncausal_mixed_filters_matches_conv1d():
    run_cnn(4, [1, 1, 2, 0, 2], [1, 3, 2, 1, 1], [12, 12], causal=0, out_tanh=0, seed=2, bias=0.5)


def test_cnn_dilation_longer_than_sequence():
    run_cnn(3, [1, 1], [16, 16], [10, 6], causal=1, out_tanh=1, seed=3)


def test_wavnetc_matches_autograd():
    D, Cdim, lengths = 4, 3, [7, 5, 7]
    S, T = len(lengths), max(lengths)
    N = S * T
    rng = np.random.default_rng(5)
    pat = make_pat_types(lengths, T)
    W = rng.uniform(-0.5, 0.5, Cdim * 2 * D).astype(np.float32)
    ctx = rng.standard_normal((N, Cdim)).astype(np.float32)
    ctx[pat == 0] = 0
    conv = rng.standard_normal((N, 2 * D)).astype(np.float32)
    err = rng.standard_normal((N, D)).astype(np.float32)
    core = np.zeros(2 * D * N, dtype=np.float32)
    cth = np.zeros_like(core)
    out = np.zeros(D * N, dtype=np.float32)
    O.wavnetc_forward(D, Cdim, N, pat, W, ctx.reshape(-1), conv.reshape(-1), core, cth, out)
    prev = np.zeros_like(core)
    dW = np.zeros_like(W)
    cg = np.ones(Cdim * N, dtype=np.float32)  # W*g is ADDED to the existing content
    O.wavnetc_backward(D, Cdim, N, pat, W, ctx.reshape(-1), core, cth, err.reshape(-1), prev, dW, cg)

    Wt = torch.tensor(W.reshape(2 * D, Cdim), dtype=torch.float64, requires_grad=True)  # [unit][c]
    ct = torch.tensor(ctx, dtype=torch.float64, requires_grad=True)
    cv = torch.tensor(conv, dtype=torch.float64, requires_grad=True)
    Y = cv + torch.tanh(ct @ Wt.T)
    z = torch.tanh(Y[:, :D]) * torch.sigmoid(Y[:, D:])
    valid = torch.tensor((pat != 0).astype(np.float64)).unsqueeze(1)
    z = z * valid
    (z * torch.tensor(err, dtype=torch.float64)).sum().backward()
    assert relerr(out.reshape(N, D), z.detach().numpy()) < 2e-6
    assert relerr(prev.reshape(N, 2 * D), cv.grad.numpy()) < 1e-5
    assert relerr(dW, Wt.grad.numpy().reshape(-1)) < 1e-5
    assert relerr(cg.reshape(N, Cdim) - 1.0, ct.grad.numpy()) < 1e-5
    assert not prev.reshape(N, 2 * D)[pat == 0].any() and not out.reshape(N, D)[pat == 0].any()
    # unconditioned twin: same gate gradient from given pre-activations
    prev2 = np.zeros_like(core)
    O.gated_backward(D, N, pat, core, err.reshape(-1), prev2)
    assert np.array_equal(prev2, prev)
    out2 = np.zeros_like(out)
    O.gated_forward(D, N, pat, core, out2)
    assert np.array_equal(out2, out)


def test_context_upsampling_and_frame_gradient_sum():
    Cdim, S, res, lengths = 3, 2, 4, [11, 7]  # samples per sequence; frames = ceil(len / res)
    T = max(lengths)
    N = T * S
    pat = make_pat_types(lengths, T)
    nfr = [-(-n // res) for n in lengths]
    Tf = max(nfr)
    rng = np.random.default_rng(6)
    src = rng.standard_normal((Tf, S, Cdim)).astype(np.float32)
    fidx = np.array([[t // res for s in range(S)] for t in range(T)], dtype=np.float32).reshape(-1)
    mv = np.concatenate([rng.standard_normal(Cdim), [0.5, 2.0, 1e-7]]).astype(np.float32)
    ctx = np.full(Cdim * N, 9, dtype=np.float32)
    O.wavnetc_load_context(Cdim, S, N, Tf, False, src.reshape(-1), fidx, mv, pat, ctx)
    want = np.zeros((T, S, Cdim), dtype=np.float32)
    for t in range(T):
        for s in range(S):
            if t < lengths[s]:
                sd = np.where(mv[Cdim:] < 1e-5, 1.0, mv[Cdim:])
                want[t, s] = (src[t // res, s] - mv[:Cdim]) / sd
    assert relerr(ctx.reshape(T, S, Cdim), want) < 1e-6
    assert not ctx.reshape(T, S, Cdim)[pat.reshape(T, S) == 0].any()
    # frame-rate gradient = sum of the sample-rate gradients of the frame's valid samples
    g = rng.standard_normal((T, S, Cdim)).astype(np.float32)
    pat_f = make_pat_types(nfr, Tf)
    fg = np.full(Tf * S * Cdim, 5, dtype=np.float32)
    O.wavnetc_sum_context_grad(Cdim, S, res, Tf * S, N, pat_f, pat, g.reshape(-1), fg)
    want = np.zeros((Tf, S, Cdim))
    for f in range(Tf):
        for s in range(S):
            if f < nfr[s]:
                for i in range(res):
                    t = f * res + i
                    if t < lengths[s]:
                        want[f, s] += g[t, s]
    assert relerr(fg.reshape(Tf, S, Cdim), want) < 1e-6


def test_skipadd_sum_and_fanout():
    rng = np.random.default_rng(7)
    n = 50
    a, b = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    out, e, es = np.zeros(n, np.float32), np.ones(n, np.float32), np.ones(n, np.float32)
    O.skipadd_forward([a, b], out, e, es)
    assert np.array_equal(out, a + b) and not e.any() and not es.any()
    e = rng.standard_normal(n).astype(np.float32)
    es = rng.standard_normal(n).astype(np.float32)
    t_skip = np.ones(n, np.float32)
    t_plain = np.full(n, 3, np.float32)
    e0, es0 = e.copy(), es.copy()
    O.skipadd_backward(e, es, [t_skip, t_plain], [1, 0])
    assert np.array_equal(e, es0 + e0)
    assert np.array_equal(t_skip, 1 + e) and np.array_equal(t_plain, e)
