"""Shared GPU-vs-oracle parity drivers.  Each function builds seeded inputs, runs the CPU oracle and the
HIP library (through its C ABI) on the same data and returns the worst L2-normalised error over all
compared tensors; index / masking properties are asserted bit-exactly on the way."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
for _d in (os.path.dirname(os.path.abspath(__file__)), os.path.join(ROOT, "oracle"), os.path.join(ROOT, "bench")):
    if _d not in sys.path:
        sys.path.insert(0, _d)

import oracle_lib as O  # noqa: E402
from torch_models import make_pat_types  # noqa: E402


def pkg():
    from __graft_entry__ import load_package

    return load_package()


def networks():
    """The tests' layer-by-layer walks over the C ABI (tests/networks.py)."""
    import networks as N

    return N


def relerr(a, b):
    a = np.asarray(a, dtype=np.float64).ravel()
    b = np.asarray(b, dtype=np.float64).ravel()
    d = np.linalg.norm(b)
    if d == 0:
        return float(np.linalg.norm(a))
    return float(np.linalg.norm(a - b) / d)


def dev(a):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def lstm_inputs(P, L, bidir, S, T, lengths, seed, wscale=0.1, escale=0.1):
    rng = np.random.default_rng(seed)
    nW = O.lib().orc_lstm_weight_count(P, L, int(bidir))
    W = rng.uniform(-wscale, wscale, nW).astype(np.float32)
    x = rng.standard_normal((T, S, P)).astype(np.float32)
    outerr = (escale * rng.standard_normal((T, S, L))).astype(np.float32)
    for s, n in enumerate(lengths):
        x[n:, s] = 0
        outerr[n:, s] = 0
    return W, x.reshape(-1), outerr.reshape(-1)


def run_lstm_case(P, L, bidir, lengths, seed, wscale=0.1, escale=0.1, bias=1.0, repeat_backward=False,
                  tol=1e-4, verbose=False):
    import torch

    capi = pkg().capi
    S, T = len(lengths), max(lengths)
    nd = 2 if bidir else 1
    H = L // nd
    N = T * S
    W, x, outerr = lstm_inputs(P, L, bidir, S, T, lengths, seed, wscale, escale)
    pat = make_pat_types(lengths, T)

    # ---- oracle
    desc = O.LstmDesc(P, L, int(bidir), S, T, min(lengths), bias)
    fw = O.LstmState(H, N)
    bw = O.LstmState(H, N) if bidir else None
    out_o = np.zeros(L * N, dtype=np.float32)
    O.lstm_forward(desc, W, pat, x, fw, bw, out_o)
    ex_o = np.zeros(P * N, dtype=np.float32)
    dW_o = np.zeros_like(W)
    O.lstm_backward(desc, W, pat, x, outerr, fw, bw, ex_o, dW_o)
    if repeat_backward:
        O.lstm_backward(desc, W, pat, x, outerr, fw, bw, ex_o, dW_o)

    # ---- HIP library
    Wd, xd, pd = dev(W), dev(x), dev(pat)
    out_d = torch.zeros(L * N, dtype=torch.float32, device="cuda")
    err_d = dev(outerr)
    ex_d = torch.full((P * N,), 7.0, dtype=torch.float32, device="cuda")  # must be overwritten
    dW_d = torch.full((len(W),), 7.0, dtype=torch.float32, device="cuda")
    layer = capi.Lstm(P, L, bidir, S, T, bias)
    layer.load_sequences(pd, T, min(lengths))
    layer.forward(Wd, xd, out_d)
    layer.check()
    layer.backward(Wd, xd, out_d, err_d, ex_d, dW_d)
    layer.check()
    if repeat_backward:
        # no load_sequences in between: the stored output-gate deltas are added (read-modify-write)
        err_d = dev(outerr)
        layer.backward(Wd, xd, out_d, err_d, ex_d, dW_d)
        layer.check()
    torch.cuda.synchronize()

    worst = 0.0
    report = {}

    def cmp(name, got, want):
        nonlocal worst
        e = relerr(got, want)
        report[name] = e
        worst = max(worst, e)

    cmp("outputs", out_d.cpu().numpy(), out_o)
    cmp("prev_errors", ex_d.cpu().numpy(), ex_o)
    dW_g = dW_d.cpu().numpy()
    o_b = 4 * P * L
    o_i = o_b + 4 * L
    o_p = o_i + 4 * L * H
    for nm, lo, hi in [("dW_input", 0, o_b), ("dW_bias", o_b, o_i), ("dW_internal", o_i, o_p),
                       ("dW_peephole", o_p, len(W))]:
        cmp(nm, dW_g[lo:hi], dW_o[lo:hi])
    dummy = (pat == 0)
    for d, st in enumerate([fw] + ([bw] if bidir else [])):
        for k in ("ni", "ig", "fg", "og", "c", "h", "dni", "dig", "dfg", "dog", "cerr"):
            got = layer.state(d, k).cpu().numpy()
            want = st[k]
            if k in ("ni", "ig", "fg", "og", "c"):
                # padding slots hold leftovers of the projection in both implementations; compare valid slots
                got = got.reshape(N, H)[~dummy]
                want = want.reshape(N, H)[~dummy]
            cmp("dir%d.%s" % (d, k), got, want)
        # masking is exact: padding slots hold exact zeros in outputs, deltas and cell errors
        if dummy.any():
            for k in ("h", "dni", "dig", "dfg", "dog", "cerr"):
                assert not layer.state(d, k).cpu().numpy().reshape(N, H)[dummy].any(), "mask leak in " + k
    if dummy.any():
        assert not out_d.cpu().numpy().reshape(N, L)[dummy].any()
        assert not ex_d.cpu().numpy().reshape(N, P)[dummy].any()
    if not bidir:
        # the recurrent terms are left in the caller's error buffer, as the reference's swap leaves them
        cmp("output_errors_inplace", err_d.cpu().numpy(), fw["herr"])
    layer.close()
    if verbose or worst > tol:
        for k, v in sorted(report.items(), key=lambda kv: -kv[1])[:8]:
            print("   %-26s %.3e" % (k, v))
    return worst


def run_lstm_two_recursions(P, L, bidir, lengths, seed, wscale=0.1, escale=0.1, bias=1.0):
    """Both GPU implementations of the recursion on the same inputs: the persistent kernels and the step-by-step
    schedule (a handle created while CNT_LSTM_STEPWISE is set).  No oracle run, so full-size fractions finish in
    a second.  Returns the worst L2-normalised difference over outputs, errors, weight updates and state."""
    import torch

    capi = pkg().capi
    S, T = len(lengths), max(lengths)
    nd = 2 if bidir else 1
    N = T * S
    W, x, outerr = lstm_inputs(P, L, bidir, S, T, lengths, seed, wscale, escale)
    pat = make_pat_types(lengths, T)
    Wd, xd, pd = dev(W), dev(x), dev(pat)
    results = []
    for stepwise in (False, True):
        if stepwise:
            os.environ["CNT_LSTM_STEPWISE"] = "1"
        try:
            layer = capi.Lstm(P, L, bidir, S, T, bias)
        finally:
            os.environ.pop("CNT_LSTM_STEPWISE", None)
        out_d = torch.zeros(L * N, dtype=torch.float32, device="cuda")
        err_d = dev(outerr)
        ex_d = torch.full((P * N,), 7.0, dtype=torch.float32, device="cuda")
        dW_d = torch.full((len(W),), 7.0, dtype=torch.float32, device="cuda")
        layer.load_sequences(pd, T, min(lengths))
        layer.forward(Wd, xd, out_d)
        layer.check()
        layer.backward(Wd, xd, out_d, err_d, ex_d, dW_d)
        layer.check()
        torch.cuda.synchronize()
        r = {"outputs": out_d.cpu().numpy(), "prev_errors": ex_d.cpu().numpy(), "dW": dW_d.cpu().numpy()}
        for d in range(nd):
            for k in ("h", "dni", "dig", "dfg", "dog", "cerr"):
                r["dir%d.%s" % (d, k)] = layer.state(d, k).cpu().numpy()
        layer.close()
        results.append(r)
    dummy = (pat == 0)
    if dummy.any():
        for r in results:
            assert not r["outputs"].reshape(N, L)[dummy].any()
            assert not r["prev_errors"].reshape(N, P)[dummy].any()
    worst = 0.0
    for k in results[0]:
        e = relerr(results[0][k], results[1][k])
        if e > 1e-5:
            print("   %-26s %.3e" % (k, e))
        worst = max(worst, e)
    return worst


def run_gemm_case(m, n, k, tA, tB, accumulate, seed):
    import torch

    capi = pkg().capi
    rng = np.random.default_rng(seed)
    A = rng.standard_normal(m * k).astype(np.float32)
    B = rng.standard_normal(k * n).astype(np.float32)
    C0 = rng.standard_normal(m * n).astype(np.float32)
    want = C0.copy()
    O.mat_product(want, m, n, k, A, tA, B, tB, accumulate)
    Cd = dev(C0)
    capi.matrix_product(Cd, m, n, k, dev(A), tA, dev(B), tB, accumulate)
    torch.cuda.synchronize()
    return relerr(Cd.cpu().numpy(), want)


def run_dense_case(P, D, N, act, bias, seed, lengths_frac=0.8):
    import torch

    capi = pkg().capi
    rng = np.random.default_rng(seed)
    W = rng.uniform(-0.1, 0.1, P * D + D).astype(np.float32)
    x = rng.standard_normal(P * N).astype(np.float32)
    err = (0.1 * rng.standard_normal(D * N)).astype(np.float32)
    y_o = np.zeros(D * N, dtype=np.float32)
    O.dense_forward(P, D, N, act, bias, W, x, y_o)
    err_o = err.copy()
    ex_o = np.zeros(P * N, dtype=np.float32)
    dW_o = np.zeros_like(W)
    O.dense_backward(P, D, N, act, bias, W, x, y_o, err_o, ex_o, dW_o)

    Wd, xd = dev(W), dev(x)
    y_d = torch.zeros(D * N, dtype=torch.float32, device="cuda")
    capi.dense_forward(P, D, N, act, bias, Wd, xd, y_d)
    err_d = dev(err)
    ex_d = torch.full((P * N,), 3.0, dtype=torch.float32, device="cuda")
    dW_d = torch.full((len(W),), 3.0, dtype=torch.float32, device="cuda")
    capi.dense_backward(P, D, N, act, bias, Wd, xd, y_d, err_d, ex_d, dW_d)
    torch.cuda.synchronize()
    worst = 0.0
    for got, want in [(y_d, y_o), (err_d, err_o), (ex_d, ex_o), (dW_d[:P * D], dW_o[:P * D]), (dW_d[P * D:], dW_o[P * D:])]:
        worst = max(worst, relerr(got.cpu().numpy(), want))
    return worst


def run_sse_case(D, lengths, seed):
    import torch

    capi = pkg().capi
    S, T = len(lengths), max(lengths)
    N = T * S
    rng = np.random.default_rng(seed)
    y = rng.standard_normal(D * N).astype(np.float32)
    tgt = rng.standard_normal(D * N).astype(np.float32)
    pat = make_pat_types(lengths, T)
    err_o = np.zeros(D * N, dtype=np.float32)
    O.sse_backward(D, N, pat, y, tgt, err_o)
    e_o = O.sse_error(D, N, pat, y, tgt)
    err_d = torch.full((D * N,), 5.0, dtype=torch.float32, device="cuda")
    res = torch.zeros(1, dtype=torch.float32, device="cuda")
    capi.sse_backward(D, N, dev(pat), dev(y), dev(tgt), err_d)
    capi.sse_error(D, N, dev(pat), dev(y), dev(tgt), res)
    torch.cuda.synchronize()
    # elementwise subtraction and masking are exact
    assert np.array_equal(err_d.cpu().numpy(), err_o)
    return abs(float(res.item()) - e_o) / max(abs(e_o), 1e-30)


def run_mdn_mixture_case(lengths, M, D, extra, seed, var_floor=0.0, maxT=None, one_call=False):
    """Mixture unit at column `extra` of the feeding layer; returns worst error over parameters,
    log-likelihoods, loss and gradients.  Padding handling (exact zeros, the index collision) is part of
    the gradient comparison because the oracle reproduces the reference's sequential outcome."""
    import torch

    capi = pkg().capi
    S, T = len(lengths), max(lengths)
    maxT = maxT or T
    F = T * S
    Lp = extra + M + 2 * M * D
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((F, Lp)).astype(np.float32)
    x[:, extra + M + M * D:] *= 0.5
    tgt = rng.standard_normal((F, D)).astype(np.float32)
    pat = make_pat_types(lengths, T)
    para_o = np.zeros(F * M * (1 + 2 * D), dtype=np.float32)
    tmp_o = np.zeros(F * M + F, dtype=np.float32)
    err_o = np.zeros(maxT * S * Lp, dtype=np.float32)
    O.mdn_mixture_forward(F, Lp, extra, M, D, var_floor, pat, x.reshape(-1), para_o)
    nll_o = O.mdn_mixture_error(F, D, 0, M, D, pat, tgt.reshape(-1), para_o, tmp_o)
    O.mdn_mixture_backward(F, Lp, D, extra, 0, M, D, var_floor, pat, tgt.reshape(-1), para_o, tmp_o, err_o)

    layer = capi.Mdn(Lp, D, S, maxT, [1, extra, Lp, 0, D, M])
    layer.set_var_floor(0, var_floor)
    pd, xd, td = dev(pat), dev(x.reshape(-1)), dev(tgt.reshape(-1))
    res = torch.zeros(1, dtype=torch.float32, device="cuda")
    err_d = torch.full((maxT * S * Lp,), 9.0, dtype=torch.float32, device="cuda")
    layer.load_sequences(pd, T)
    layer.forward(xd)
    if one_call:
        layer.error_backward(td, res, err_d)   # cnt_mdn_error_backward: both steps, one pass where the unit allows it
    else:
        layer.calculate_error(td, res)
        layer.backward(td, err_d)
    torch.cuda.synchronize()
    valid = np.repeat(pat != 0, 1)
    para_d = layer.unit_buffer(0, 0).cpu().numpy()
    tmp_d = layer.unit_buffer(0, 1).cpu().numpy()
    worst = 0.0
    # weights and std: all frames (padding frames hold the skip marker in both); means: valid frames only
    worst = max(worst, relerr(para_d[:F * M], para_o[:F * M]))
    worst = max(worst, relerr(para_d[F * M * (1 + D):], para_o[F * M * (1 + D):]))
    worst = max(worst, relerr(para_d[F * M:F * M * (1 + D)].reshape(F, -1)[valid], para_o[F * M:F * M * (1 + D)].reshape(F, -1)[valid]))
    worst = max(worst, relerr(tmp_d[:F * M], tmp_o[:F * M]))
    worst = max(worst, relerr(tmp_d[F * M:][valid], tmp_o[F * M:][valid]))
    worst = max(worst, abs(float(res.item()) - nll_o) / abs(nll_o))
    got = err_d.cpu().numpy()
    worst = max(worst, relerr(got, err_o))
    # exact zeros wherever the oracle has exact zeros (padding frames, collisions, untouched columns, tail)
    # (a gradient that underflows may flush to zero on the GPU only: allowed below 1e-30)
    assert np.all(got[err_o == 0.0] == 0.0), "a structural zero of the gradient is not zero"
    assert np.all(np.abs(err_o[got == 0.0]) < 1e-30), "the gradient has a zero where the oracle has a value"
    layer.close()
    return worst


def run_softmax_case(lengths, K, extra, seed):
    import torch

    capi = pkg().capi
    S, T = len(lengths), max(lengths)
    F = T * S
    Lp = extra + K
    rng = np.random.default_rng(seed)
    x = (2 * rng.standard_normal((F, Lp))).astype(np.float32)
    tgt = rng.integers(0, K, size=F).astype(np.float32)
    pat = make_pat_types(lengths, T)
    prob_o = np.zeros(F * K, dtype=np.float32)
    err_o = np.zeros(F * Lp, dtype=np.float32)
    O.softmax_forward(F, Lp, extra, K, 1.0, pat, x.reshape(-1), prob_o)
    nll_o = O.softmax_error(F, 1, 0, K, F * K, pat, tgt, prob_o)
    O.softmax_backward(F, Lp, 1, extra, 0, K, pat, tgt, prob_o, err_o)

    layer = capi.Mdn(Lp, 1, S, T, [1, extra, Lp, 0, 1, -1])
    res = torch.zeros(1, dtype=torch.float32, device="cuda")
    err_d = torch.full((F * Lp,), 9.0, dtype=torch.float32, device="cuda")
    pd, xd, td = dev(pat), dev(x.reshape(-1)), dev(tgt)
    layer.load_sequences(pd, T)
    layer.forward(xd)
    layer.calculate_error(td, res)
    layer.backward(td, err_d)
    torch.cuda.synchronize()
    worst = relerr(layer.unit_buffer(0, 0).cpu().numpy(), prob_o)
    worst = max(worst, abs(float(res.item()) - nll_o) / abs(nll_o))
    got = err_d.cpu().numpy()
    worst = max(worst, relerr(got, err_o))
    assert np.all(got[err_o == 0.0] == 0.0) and np.all(np.abs(err_o[got == 0.0]) < 1e-30)
    # the one-hot position is an index property: the entry below zero sits exactly at the target class
    gv = got.reshape(F, Lp)[pat != 0][:, extra:]
    assert np.array_equal(np.argmin(gv, axis=1), tgt[pat != 0].astype(np.int64))
    layer.close()
    return worst


def run_sigmoid_case(lengths, K, extra, continuous, seed, with_softmax=False):
    """MDN sigmoid unit (optionally next to a softmax unit in the same layer) against the oracle."""
    import torch

    capi = pkg().capi
    S, T = len(lengths), max(lengths)
    F = T * S
    Ks = 5 if with_softmax else 0
    Lp = extra + K + Ks
    Lt = K + (1 if with_softmax else 0)
    rng = np.random.default_rng(seed)
    x = (2 * rng.standard_normal((F, Lp))).astype(np.float32)
    tgt = np.zeros((F, Lt), dtype=np.float32)
    tgt[:, :K] = rng.uniform(0, 1, (F, K)) if continuous else (rng.uniform(0, 1, (F, K)) > 0.5)
    if with_softmax:
        tgt[:, K] = rng.integers(0, Ks, size=F)
    pat = make_pat_types(lengths, T)
    prob_o = np.zeros(F * K, dtype=np.float32)
    err_o = np.zeros(F * Lp, dtype=np.float32)
    O.sigmoid_forward(F, Lp, extra, K, pat, x.reshape(-1), prob_o)
    loss_o = O.sigmoid_error(F, Lt, 0, K, continuous, pat, tgt.reshape(-1), prob_o)
    O.sigmoid_backward(F, Lp, Lt, extra, 0, K, continuous, pat, tgt.reshape(-1), prob_o, err_o)
    config = [1, extra, extra + K, 0, K, 0]
    if with_softmax:
        sm_o = np.zeros(F * Ks, dtype=np.float32)
        O.softmax_forward(F, Lp, extra + K, Ks, 1.0, pat, x.reshape(-1), sm_o)
        loss_o += O.softmax_error(F, Lt, K, Ks, F * Ks, pat, tgt.reshape(-1), sm_o)
        O.softmax_backward(F, Lp, Lt, extra + K, K, Ks, pat, tgt.reshape(-1), sm_o, err_o)
        config = [2, extra, extra + K, 0, K, 0, extra + K, Lp, K, K + 1, -1]

    layer = capi.Mdn(Lp, Lt, S, T, config, sigmoid_continuous=continuous)
    res = torch.zeros(1, dtype=torch.float32, device="cuda")
    err_d = torch.full((F * Lp,), 9.0, dtype=torch.float32, device="cuda")
    pd, xd, td = dev(pat), dev(x.reshape(-1)), dev(tgt.reshape(-1))
    layer.load_sequences(pd, T)
    layer.forward(xd)
    layer.calculate_error(td, res)
    layer.backward(td, err_d)
    torch.cuda.synchronize()
    worst = relerr(layer.unit_buffer(0, 0).cpu().numpy(), prob_o)
    worst = max(worst, abs(float(res.item()) - loss_o) / abs(loss_o))
    got = err_d.cpu().numpy()
    worst = max(worst, relerr(got, err_o))
    # padding frames and the columns no unit owns are exactly zero
    g2, o2 = got.reshape(F, Lp), err_o.reshape(F, Lp)
    assert np.all(g2[pat == 0] == 0.0) and np.all(g2[:, :extra] == 0.0) and np.all(o2[:, :extra] == 0.0)
    layer.close()
    return worst


def run_cnn_case(P, half_width, interval, lengths, causal, out_tanh, seed, bias=1.0, maxT=None):
    """1-D convolution layer forward + backward against the oracle (which scatters into a real column buffer)."""
    import torch

    capi = pkg().capi
    hw = np.asarray(half_width, dtype=np.int32)
    it = np.asarray(interval, dtype=np.int32)
    D = len(hw)
    S, T = len(lengths), max(lengths)
    maxT = maxT or T
    N = T * S
    rng = np.random.default_rng(seed)
    Lw = O.cnn_total_width(hw)
    W = rng.uniform(-0.1, 0.1, P * Lw + D).astype(np.float32)
    x = rng.standard_normal((T, S, P)).astype(np.float32)
    err = rng.standard_normal((T, S, D)).astype(np.float32)
    pat = make_pat_types(lengths, T)
    stale = rng.standard_normal(D * N).astype(np.float32)  # outputs keep their old content on padding slots
    con = np.zeros(Lw * N, dtype=np.float32)
    out_o = stale.copy()
    O.cnn_forward(P, D, S, T, causal, out_tanh, bias, hw, it, pat, W, x.reshape(-1), con, out_o)
    err_o = err.reshape(-1).copy()
    ex_o = np.zeros(P * maxT * S, dtype=np.float32)
    dW_o = np.zeros_like(W)
    O.cnn_backward(P, D, S, T, causal, out_tanh, bias, hw, it, pat, W, x.reshape(-1), out_o, err_o, con, ex_o[:P * N], dW_o)

    layer = capi.Cnn(P, hw, it, S, maxT, causal, out_tanh, bias)
    assert layer.weight_count == len(W)
    pd, Wd, xd = dev(pat), dev(W), dev(x.reshape(-1))
    out_d = dev(stale)
    layer.forward(pd, T, Wd, xd, out_d)
    err_d = dev(err.reshape(-1))
    ex_d = torch.full((P * maxT * S,), 4.0, dtype=torch.float32, device="cuda")
    dW_d = torch.full((len(W),), 4.0, dtype=torch.float32, device="cuda")
    layer.backward(pd, T, Wd, xd, out_d, err_d, ex_d, dW_d)
    torch.cuda.synchronize()
    worst = 0.0
    got_out = out_d.cpu().numpy()
    worst = max(worst, relerr(got_out, out_o))
    dummy = (pat == 0)
    if dummy.any():  # untouched means bit-identical to what was there
        assert np.array_equal(got_out.reshape(N, D)[dummy], stale.reshape(N, D)[dummy])
    worst = max(worst, relerr(err_d.cpu().numpy(), err_o))
    got_ex = ex_d.cpu().numpy()
    worst = max(worst, relerr(got_ex, ex_o))
    assert not got_ex[P * N:].any()
    if dummy.any():
        assert not got_ex[:P * N].reshape(N, P)[dummy].any()
    got_dW = dW_d.cpu().numpy()
    worst = max(worst, relerr(got_dW[:P * Lw], dW_o[:P * Lw]))
    worst = max(worst, relerr(got_dW[P * Lw:], dW_o[P * Lw:]))
    # dilation / tap indexing: weight columns that get no signal are exactly zero in both
    cols_g = got_dW[:P * Lw].reshape(Lw, P)
    cols_o = dW_o[:P * Lw].reshape(Lw, P)
    assert np.array_equal(np.abs(cols_g).sum(1) == 0, np.abs(cols_o).sum(1) == 0)
    layer.close()
    return worst


def run_wavnetc_case(D, Cdim, lengths, seed, with_ctx_grad=True):
    import torch

    capi = pkg().capi
    S, T = len(lengths), max(lengths)
    N = S * T
    rng = np.random.default_rng(seed)
    pat = make_pat_types(lengths, T)
    W = rng.uniform(-0.3, 0.3, max(Cdim, 1) * 2 * D).astype(np.float32)
    ctx = rng.standard_normal((N, max(Cdim, 1))).astype(np.float32)
    ctx[pat == 0] = 0
    conv = rng.standard_normal((N, 2 * D)).astype(np.float32)
    err = rng.standard_normal((N, D)).astype(np.float32)
    core_o = np.zeros(2 * D * N, dtype=np.float32)
    cth_o = np.zeros_like(core_o)
    out_o = np.zeros(D * N, dtype=np.float32)
    O.wavnetc_forward(D, Cdim, N, pat, W, ctx.reshape(-1), conv.reshape(-1), core_o, cth_o, out_o)
    prev_o = np.zeros_like(core_o)
    dW_o = np.zeros_like(W)
    cg0 = rng.standard_normal(max(Cdim, 1) * N).astype(np.float32)
    cg_o = cg0.copy()
    core_keep = core_o.copy()
    O.wavnetc_backward(D, Cdim, N, pat, W, ctx.reshape(-1), core_o, cth_o, err.reshape(-1), prev_o, dW_o,
                       cg_o if with_ctx_grad else None)

    pd, Wd, cd, cvd = dev(pat), dev(W), dev(ctx.reshape(-1)), dev(conv.reshape(-1))
    core_d = torch.full((2 * D * N,), 3.0, dtype=torch.float32, device="cuda")
    cth_d = torch.full((2 * D * N,), 3.0, dtype=torch.float32, device="cuda")
    out_d = torch.full((D * N,), 3.0, dtype=torch.float32, device="cuda")
    capi.wavnetc_forward(D, Cdim, N, pd, Wd, cd, cvd, core_d, cth_d, out_d)
    torch.cuda.synchronize()
    worst = relerr(core_d.cpu().numpy(), core_keep)
    worst = max(worst, relerr(out_d.cpu().numpy(), out_o))
    prev_d = torch.full((2 * D * N,), 3.0, dtype=torch.float32, device="cuda")
    dW_d = torch.full((len(W),), 3.0, dtype=torch.float32, device="cuda")
    cg_d = dev(cg0)
    capi.wavnetc_backward(D, Cdim, N, pd, Wd, cd, core_d, cth_d, dev(err.reshape(-1)), prev_d, dW_d,
                          cg_d if with_ctx_grad else None)
    torch.cuda.synchronize()
    worst = max(worst, relerr(prev_d.cpu().numpy(), prev_o))
    dummy = (pat == 0)
    if dummy.any():
        assert not prev_d.cpu().numpy().reshape(N, 2 * D)[dummy].any()
        assert not out_d.cpu().numpy().reshape(N, D)[dummy].any()
    if Cdim > 0:
        worst = max(worst, relerr(cth_d.cpu().numpy(), cth_o))
        worst = max(worst, relerr(dW_d.cpu().numpy(), dW_o))
        if with_ctx_grad:
            worst = max(worst, relerr(cg_d.cpu().numpy(), cg_o))
    # the unconditioned layer type on the same pre-activations
    out2 = torch.zeros(D * N, dtype=torch.float32, device="cuda")
    prev2 = torch.zeros(2 * D * N, dtype=torch.float32, device="cuda")
    capi.gatedact_forward(D, N, pd, core_d, out2)
    capi.gatedact_backward(D, N, pd, core_d, dev(err.reshape(-1)), prev2)
    torch.cuda.synchronize()
    assert torch.equal(out2, out_d) and torch.equal(prev2, prev_d)
    return worst


def run_context_case(Cdim, res, lengths, seed, use_mean_std):
    import torch

    capi = pkg().capi
    S, T = len(lengths), max(lengths)
    N = T * S
    pat = make_pat_types(lengths, T)
    nfr = [-(-n // res) for n in lengths]
    Tf = max(nfr)
    rng = np.random.default_rng(seed)
    src = rng.standard_normal(Tf * S * Cdim).astype(np.float32)
    fidx = np.array([[t // res for s in range(S)] for t in range(T)], dtype=np.float32).reshape(-1)
    mv = np.concatenate([rng.standard_normal(Cdim), rng.uniform(0.5, 2.0, Cdim)]).astype(np.float32)
    mv[-1] = 1e-7
    ctx_o = np.zeros(Cdim * N, dtype=np.float32)
    O.wavnetc_load_context(Cdim, S, N, Tf, False, src, fidx, mv if use_mean_std else None, pat, ctx_o)
    ctx_d = torch.full((Cdim * N,), 2.0, dtype=torch.float32, device="cuda")
    capi.wavnetc_load_context(Cdim, S, N, Tf, False, dev(src), dev(fidx), dev(mv) if use_mean_std else None, dev(pat), ctx_d)
    g = rng.standard_normal(Cdim * N).astype(np.float32)
    pat_f = make_pat_types(nfr, Tf)
    fg_o = np.zeros(Tf * S * Cdim, dtype=np.float32)
    O.wavnetc_sum_context_grad(Cdim, S, res, Tf * S, N, pat_f, pat, g, fg_o)
    fg_d = torch.full((Tf * S * Cdim,), 2.0, dtype=torch.float32, device="cuda")
    capi.wavnetc_sum_context_grad(Cdim, S, res, Tf * S, N, dev(pat_f), dev(pat), dev(g), fg_d)
    torch.cuda.synchronize()
    if not use_mean_std:  # a pure gather: bit-exact
        assert np.array_equal(ctx_d.cpu().numpy(), ctx_o)
    return max(relerr(ctx_d.cpu().numpy(), ctx_o), relerr(fg_d.cpu().numpy(), fg_o))


def run_skipadd_case(n, seed):
    import torch

    capi = pkg().capi
    rng = np.random.default_rng(seed)
    ins = [rng.standard_normal(n).astype(np.float32) for _ in range(3)]
    out_o, e_o, es_o = np.zeros(n, np.float32), np.ones(n, np.float32), np.ones(n, np.float32)
    O.skipadd_forward(ins, out_o, e_o, es_o)
    out_d = torch.ones(n, device="cuda")
    e_d = torch.ones(n, device="cuda")
    es_d = torch.ones(n, device="cuda")
    capi.skipadd_forward([dev(a) for a in ins], out_d, e_d, es_d)
    torch.cuda.synchronize()
    assert np.array_equal(out_d.cpu().numpy(), out_o) and not e_d.any() and not es_d.any()
    e = rng.standard_normal(n).astype(np.float32)
    es = rng.standard_normal(n).astype(np.float32)
    tg = [rng.standard_normal(n).astype(np.float32) for _ in range(3)]
    flags = [1, 0, 1]
    e_o, tg_o = e.copy(), [t.copy() for t in tg]
    O.skipadd_backward(e_o, es, tg_o, flags)
    e_d, tg_d = dev(e), [dev(t) for t in tg]
    capi.skipadd_backward(e_d, dev(es), tg_d, flags)
    torch.cuda.synchronize()
    assert np.array_equal(e_d.cpu().numpy(), e_o)
    for a, b in zip(tg_d, tg_o):
        assert np.array_equal(a.cpu().numpy(), b)
    return 0.0


def run_dft_case(resolutions, max_len, lengths, seed, gamma=1.0, dis_type=0, zeta=0.0):
    """Multi-resolution DFT loss: per-resolution losses and the summed gradient against the oracle."""
    import torch

    capi = pkg().capi
    rng = np.random.default_rng(seed)
    W = len(lengths)
    src = (0.3 * rng.standard_normal((W, max_len))).astype(np.float32)
    tgt = (0.3 * rng.standard_normal((W, max_len))).astype(np.float32)
    err_o = np.zeros((2 if zeta > 0 else 1, W, len(resolutions)))
    grad_o = np.zeros((W, max_len), dtype=np.float64)
    for w in range(W):
        for r, (N, Nw, Hs) in enumerate(resolutions):
            g = np.zeros(max_len, dtype=np.float32)
            err_o[0, w, r] = O.dft_spectral_loss(dis_type, N, Nw, Hs, 0, max_len, lengths[w], gamma, 1e-5, src[w].copy(),
                                              tgt[w].copy(), g)
            g[lengths[w]:] = 0  # the layer only passes on the first `length` samples
            grad_o[w] += g
            if zeta > 0:
                err_o[1, w, r] = O.dft_phase_loss(N, Nw, Hs, 0, max_len, lengths[w], zeta, src[w].copy(), tgt[w].copy(), g)
                g[lengths[w]:] = 0
                grad_o[w] += g
    layer = capi.Dft(resolutions, max_len, W, gamma=gamma, spec_dis_type=dis_type, zeta=zeta)
    err_d = torch.full((err_o.size,), 7.0, dtype=torch.float32, device="cuda")
    prev_d = torch.full((W * max_len,), 7.0, dtype=torch.float32, device="cuda")
    layer.forward(lengths, dev(src.reshape(-1)), dev(tgt.reshape(-1)), err_d)
    layer.backward(prev_d)
    torch.cuda.synchronize()
    got_g = prev_d.cpu().numpy().reshape(W, max_len)
    got_e = err_d.cpu().numpy().reshape(err_o.shape)
    worst = max(relerr(got_e[i], err_o[i]) for i in range(err_o.shape[0]))
    for w in range(W):
        worst = max(worst, relerr(got_g[w], grad_o[w]))
        assert not got_g[w, lengths[w]:].any()
    layer.close()
    return worst
