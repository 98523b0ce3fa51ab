"""Pins the CPU oracle's mixture-density and softmax units against closed forms in float64 PyTorch
(logsumexp Gaussian-mixture likelihood, cross entropy) and against a hand-built case of the
padding-frame index collision."""
import math

import numpy as np
import torch

import oracle_lib as O
from test_oracle_lstm import relerr
from torch_models import make_pat_types

PI_REF = 3.141215


def mixture_case(lengths, M, D, extra=0, seed=0):
    S, T = len(lengths), max(lengths)
    F = T * S
    Lp = extra + M + 2 * M * D
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((F, Lp)).astype(np.float32)
    x[:, extra + M + M * D:] *= 0.5
    tgt = rng.standard_normal((F, D)).astype(np.float32)
    pat = make_pat_types(lengths, T)
    return F, Lp, x, tgt, pat


def run_mixture(F, Lp, startD, M, D, x, tgt, pat, var_floor=0.0):
    para = np.zeros(F * M * (1 + 2 * D), dtype=np.float32)
    tmp = np.zeros(F * M + F, dtype=np.float32)
    err = np.zeros(F * Lp, dtype=np.float32)
    O.mdn_mixture_forward(F, Lp, startD, M, D, var_floor, pat, x.reshape(-1), para)
    nll = O.mdn_mixture_error(F, D, 0, M, D, pat, tgt.reshape(-1), para, tmp)
    O.mdn_mixture_backward(F, Lp, D, startD, 0, M, D, var_floor, pat, tgt.reshape(-1), para, tmp, err)
    return para, tmp, err.reshape(F, Lp), nll


def torch_mixture_nll(x, tgt, valid, startD, M, D):
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    t = torch.tensor(tgt, dtype=torch.float64)
    logw = torch.log_softmax(xt[:, startD:startD + M], dim=1)
    mu = xt[:, startD + M: startD + M + M * D].reshape(-1, M, D)
    ls = xt[:, startD + M + M * D: startD + M + 2 * M * D].reshape(-1, M, D)
    z = (t[:, None, :] - mu) / torch.exp(ls)
    logp = logw - 0.5 * (z * z).sum(2) - ls.sum(2) - D * math.log(2 * PI_REF) / 2
    nll = -(torch.logsumexp(logp, dim=1) * torch.tensor(valid, dtype=torch.float64)).sum()
    nll.backward()
    return float(nll.detach()), xt.grad.numpy()


def test_mixture_matches_closed_form_all_valid():
    M, D = 4, 6
    F, Lp, x, tgt, pat = mixture_case([5, 5, 5], M, D, extra=3, seed=1)
    para, tmp, err, nll = run_mixture(F, Lp, 3, M, D, x, tgt, pat)
    ref_nll, ref_grad = torch_mixture_nll(x, tgt, np.ones(F), 3, M, D)
    assert abs(nll - ref_nll) <= 1e-5 * abs(ref_nll)
    assert relerr(err[:, 3:], ref_grad[:, 3:]) < 1e-5
    assert not err[:, :3].any()
    # forward parameters: softmax weights, copied means, exp'd std
    w = torch.softmax(torch.tensor(x[:, 3:3 + M], dtype=torch.float64), 1).numpy()
    assert relerr(para[:F * M], w) < 1e-6
    assert np.array_equal(para[F * M:F * M * (1 + D)], x[:, 3 + M:3 + M + M * D].reshape(-1))
    assert relerr(para[F * M * (1 + D):], np.exp(x[:, 3 + M + M * D:].astype(np.float64))) < 1e-6


def test_mixture_padding_and_index_collision():
    """Variable lengths, unit starting at column 0.  With M=2 and Lp=10 the padding frame f_d=15 writes its
    zero to index 30 and 31 = frame 3, columns 0..1: a VALID frame's mixture-weight gradient is wiped."""
    M, D = 2, 2
    lengths = [6, 3, 6]  # S=3, T=6: frame index f = t*3+s; s=1 is padding for t>=3 -> f=10,13,16
    F, Lp, x, tgt, pat = mixture_case(lengths, M, D, extra=0, seed=2)
    assert Lp == 10
    para, tmp, err, nll = run_mixture(F, Lp, 0, M, D, x, tgt, pat)
    valid = (pat != 0).astype(np.float64)
    ref_nll, ref_grad = torch_mixture_nll(x, tgt, valid, 0, M, D)
    assert abs(nll - ref_nll) <= 1e-5 * abs(ref_nll)
    expect = ref_grad.copy()
    wiped = []
    for fd in np.nonzero(pat == 0)[0]:
        for m in range(M):
            idx = fd * M + m
            fv, col = divmod(idx, Lp)
            if col < M:  # lands on a mixture-weight slot: the zero is written after the value
                expect[fv, col] = 0.0
                if pat[fv] != 0:
                    wiped.append((fv, col))
    assert wiped, "the case must exercise the collision"
    assert relerr(err, expect) < 1e-5
    for fv, col in wiped:
        assert err[fv, col] == 0.0 and ref_grad[fv, col] != 0.0
    # padding frames: exact zeros in every slot of the unit
    assert not err[pat == 0].any()


def test_mixture_variance_floor_blocks_std_gradient():
    M, D = 2, 3
    F, Lp, x, tgt, pat = mixture_case([4, 4], M, D, seed=3)
    x[:, M + M * D:] = -3.0  # exp(-3) = 0.0498 below the floor
    para, tmp, err, nll = run_mixture(F, Lp, 0, M, D, x, tgt, pat, var_floor=0.1)
    assert np.all(para[F * M * (1 + D):] == np.float32(0.1))
    assert not err[:, M + M * D:].any()
    assert err[:, M:M + M * D].any()


def test_softmax_unit_matches_cross_entropy():
    K, lengths = 7, [5, 3, 5]
    S, T = len(lengths), max(lengths)
    F, Lp, startD = S * T, K + 2, 2
    rng = np.random.default_rng(4)
    x = rng.standard_normal((F, Lp)).astype(np.float32) * 2
    cls = rng.integers(0, K, size=F)
    tgt = cls.astype(np.float32).reshape(F, 1)
    pat = make_pat_types(lengths, T)
    prob = np.zeros(F * K, dtype=np.float32)
    O.softmax_forward(F, Lp, startD, K, 1.0, pat, x.reshape(-1), prob)
    nll = O.softmax_error(F, 1, 0, K, F * K, pat, tgt.reshape(-1), prob)
    err = np.zeros(F * Lp, dtype=np.float32)
    O.softmax_backward(F, Lp, 1, startD, 0, K, pat, tgt.reshape(-1), prob, err)
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    valid = torch.tensor(pat != 0)
    loss = torch.nn.functional.cross_entropy(xt[valid][:, startD:], torch.tensor(cls)[valid], reduction="sum")
    loss.backward()
    assert abs(nll - float(loss)) <= 1e-5 * float(loss)
    assert relerr(err.reshape(F, Lp), xt.grad.numpy()) < 1e-5
    p = prob.reshape(F, K)
    assert np.all(p[pat == 0] == np.float32(3.4028235e38))  # the reference's skip marker
    assert relerr(p[pat != 0], torch.softmax(xt[valid][:, startD:], 1).detach().numpy()) < 1e-6


def test_sigmoid_unit_matches_binary_cross_entropy_autograd():
    """Forward = logistic, error = BCE summed over elements and divided by the number of non-padding frames,
    gradient = d(sum BCE)/d(logit) = p - t (not divided): float64 autograd on the unnormalised sum."""
    import torch

    rng = np.random.default_rng(4)
    lengths, K, extra = [7, 4, 7], 5, 2
    S, T = len(lengths), max(lengths)
    F, Lp = S * T, extra + K
    pat = make_pat_types(lengths, T)
    x = rng.standard_normal((F, Lp)).astype(np.float32)
    for continuous in (False, True):
        tgt = (rng.uniform(0, 1, (F, K)).astype(np.float32) if continuous
               else (rng.uniform(0, 1, (F, K)) > 0.4).astype(np.float32))
        prob = np.zeros(F * K, np.float32); err = np.full(F * Lp, 5.0, np.float32)
        O.sigmoid_forward(F, Lp, extra, K, pat, x.reshape(-1), prob)
        loss = O.sigmoid_error(F, K, 0, K, continuous, pat, tgt.reshape(-1), prob)
        O.sigmoid_backward(F, Lp, K, extra, 0, K, continuous, pat, tgt.reshape(-1), prob, err)
        xt = torch.tensor(x[:, extra:], dtype=torch.float64, requires_grad=True)
        valid = torch.tensor(pat != 0)
        bce = torch.nn.functional.binary_cross_entropy_with_logits(xt, torch.tensor(tgt, dtype=torch.float64), reduction="none")
        total = (bce * valid[:, None]).sum()
        total.backward()
        assert abs(loss - float(total) / int(valid.sum())) < 1e-5 * max(1.0, abs(loss))
        e = err.reshape(F, Lp)
        assert np.max(np.abs(e[:, extra:] - xt.grad.numpy())) < 1e-6
        assert np.all(e[:, :extra] == 5.0)                       # columns outside the unit are not touched
        assert np.all(e[pat == 0][:, extra:] == 0.0) and np.all(prob.reshape(F, K)[pat == 0] == 0.0)
