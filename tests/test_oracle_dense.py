"""Pins the CPU oracle's feed-forward and SSE layers against independent statements:

* `orc_dense_forward` / `orc_dense_backward` against float64 `torch.nn.functional.linear` + autograd for the
  four activations, bias values other than 1, and padding slots (the reference applies the activation
  derivative on every slot, padding included: FeedForwardLayer.cu:105-116; weight matrix P x D column-major and
  bias update = sum of bias * delta: FeedForwardLayer.cu:118-138, 1633-1738);
* `orc_sse_error` / `orc_sse_backward` against a masked closed form over ragged sequence lengths
  (SsePostOutputLayer.cu:94-136: 0.5 * sum (t - y)^2 over non-padding slots, error y - t, zero on padding).
"""
import numpy as np
import pytest
import torch

import oracle_lib as O
from test_oracle_lstm import relerr
from torch_models import make_pat_types

ACTS = {0: lambda a: a, 1: torch.tanh, 2: torch.sigmoid, 3: torch.relu}


def dense_case(P, D, N, act, bias, seed):
    rng = np.random.default_rng(seed)
    W = rng.uniform(-0.4, 0.4, P * D + D).astype(np.float32)
    x = rng.standard_normal((N, P)).astype(np.float32)
    err = rng.standard_normal((N, D)).astype(np.float32)
    return W, x, err


@pytest.mark.parametrize("act", [0, 1, 2, 3])
@pytest.mark.parametrize("P,D,N,bias", [(7, 5, 11, 1.0), (33, 18, 40, 0.5), (64, 96, 23, -1.5), (3, 1, 9, 2.0)])
def test_dense_forward_backward_against_autograd(P, D, N, act, bias):
    W, x, err = dense_case(P, D, N, act, bias, seed=100 * act + P)
    y = np.zeros(D * N, dtype=np.float32)
    O.dense_forward(P, D, N, act, bias, W, x.reshape(-1), y)

    # independent statement: y = act(x Wm^T + bias * b) with Wm[d][p] = W[d*P + p]
    Wt = torch.tensor(W[:P * D].reshape(D, P), dtype=torch.float64, requires_grad=True)
    bt = torch.tensor(W[P * D:], dtype=torch.float64, requires_grad=True)
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    yt = ACTS[act](torch.nn.functional.linear(xt, Wt, bias * bt))
    assert relerr(y.reshape(N, D), yt.detach().numpy()) < 2e-6

    # backward: the oracle takes the derivative from ITS output y, so compare on the same forward values
    (yt * torch.tensor(err, dtype=torch.float64)).sum().backward()
    e = err.reshape(-1).copy()
    ex = np.zeros(P * N, dtype=np.float32)
    dW = np.full(P * D + D, 7.0, dtype=np.float32)  # must be overwritten, not accumulated
    O.dense_backward(P, D, N, act, bias, W, x.reshape(-1), y, e, ex, dW)
    assert relerr(ex.reshape(N, P), xt.grad.numpy()) < 5e-6
    assert relerr(dW[:P * D].reshape(D, P), Wt.grad.numpy()) < 5e-6
    assert relerr(dW[P * D:], bt.grad.numpy()) < 5e-6
    # the error buffer now holds the deltas act'(y) * err (in place, FeedForwardLayer.cu:105-116)
    with torch.no_grad():
        pre = torch.nn.functional.linear(xt, Wt, bias * bt)
    pre.requires_grad_(True)
    ACTS[act](pre).backward(torch.tensor(err, dtype=torch.float64))
    assert relerr(e.reshape(N, D), pre.grad.numpy()) < 5e-6


def test_dense_deltas_are_computed_on_padding_slots_too():
    """The delta functor runs over every slot; nothing in the layer looks at the pattern types."""
    P, D, N = 6, 4, 10
    W, x, err = dense_case(P, D, N, 1, 1.0, seed=5)
    y = np.zeros(D * N, dtype=np.float32)
    O.dense_forward(P, D, N, 1, 1.0, W, x.reshape(-1), y)
    e = err.reshape(-1).copy()
    dW = np.zeros(P * D + D, dtype=np.float32)
    O.dense_backward(P, D, N, 1, 1.0, W, x.reshape(-1), y, e, None, dW)
    expect = (1.0 - y.astype(np.float64) ** 2) * err.reshape(-1)
    assert relerr(e, expect) < 1e-6
    # hand-computed bias update of unit 2: the plain sum of its deltas
    assert abs(dW[P * D + 2] - expect.reshape(N, D)[:, 2].sum()) < 1e-5


def test_dense_weight_layout_single_entry():
    """One non-zero weight W[p=2 -> d=1] sits at index d*P + p and nowhere else."""
    P, D, N = 4, 3, 2
    W = np.zeros(P * D + D, dtype=np.float32)
    W[1 * P + 2] = 3.0
    W[P * D + 0] = 0.25  # bias weight of unit 0
    x = np.arange(N * P, dtype=np.float32).reshape(N, P)
    y = np.zeros(D * N, dtype=np.float32)
    O.dense_forward(P, D, N, 0, 2.0, W, x.reshape(-1), y)
    expect = np.zeros((N, D), dtype=np.float32)
    expect[:, 1] = 3.0 * x[:, 2]
    expect[:, 0] = 2.0 * 0.25
    assert np.array_equal(y.reshape(N, D), expect)


@pytest.mark.parametrize("lengths,D", [([5, 3, 4], 4), ([7, 7], 3), ([1, 6, 2, 6], 9), ([4], 1)])
def test_sse_masked_closed_form(lengths, D):
    S, T = len(lengths), max(lengths)
    N = T * S
    rng = np.random.default_rng(sum(lengths) + D)
    y = rng.standard_normal((T, S, D)).astype(np.float32)
    tgt = rng.standard_normal((T, S, D)).astype(np.float32)
    pat = make_pat_types(lengths, T)
    mask = np.zeros((T, S, 1), dtype=np.float64)
    for s, n in enumerate(lengths):
        mask[:n, s] = 1.0
    # pattern types agree with the mask (first / normal / last are all "valid")
    assert np.array_equal(pat.reshape(T, S) != 0, mask[:, :, 0] == 1.0)

    got = O.sse_error(D, N, pat, y.reshape(-1), tgt.reshape(-1))
    expect = 0.5 * (mask * (tgt.astype(np.float64) - y) ** 2).sum()
    assert abs(got - expect) <= 2e-6 * max(1.0, expect)

    err = np.full(D * N, 9.0, dtype=np.float32)
    O.sse_backward(D, N, pat, y.reshape(-1), tgt.reshape(-1), err)
    expect_err = (mask * (y.astype(np.float64) - tgt)).astype(np.float32)
    assert np.array_equal(err.reshape(T, S, D), (y - tgt) * mask.astype(np.float32))
    assert relerr(err.reshape(T, S, D), expect_err) < 1e-7
    # the gradient of the error with respect to y, by autograd
    yt = torch.tensor(y, dtype=torch.float64, requires_grad=True)
    (0.5 * (torch.tensor(mask) * (torch.tensor(tgt, dtype=torch.float64) - yt) ** 2).sum()).backward()
    assert relerr(err.reshape(T, S, D), yt.grad.numpy()) < 1e-7
