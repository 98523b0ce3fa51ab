"""GPU: the HIP library, through the C ABI, on the inputs of the committed golden fixtures (tests/golden/*.npz)
against the outputs stored there; fp32 tensors to 1e-4 of the L2 norm, padding slots exactly zero."""
import os

import numpy as np
import pytest

import parity_cases as PC

pytestmark = pytest.mark.gpu
TOL = 1e-4
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False)


@pytest.mark.parametrize("name", ["lstm_blstm_128", "lstm_uni_64", "lstm_blstm_stepwise_24"])
def test_lstm_fixture(name):
    import torch

    print("golden", name, flush=True)
    f = load(name)
    capi = PC.pkg().capi
    P, L, bidir = int(f["P"]), int(f["L"]), bool(f["bidir"])
    lengths = [int(v) for v in f["lengths"]]
    S, T = len(lengths), max(lengths)
    N = S * T
    layer = capi.Lstm(P, L, bidir, S, T, 1.0)
    W, x, pat = PC.dev(f["weights"]), PC.dev(f["x"]), PC.dev(f["patTypes"])
    out = torch.zeros(L * N, dtype=torch.float32, device="cuda")
    ex = torch.full((P * N,), 5.0, dtype=torch.float32, device="cuda")
    dW = torch.full((f["weights"].size,), 5.0, dtype=torch.float32, device="cuda")
    layer.load_sequences(pat, T, min(lengths))
    layer.forward(W, x, out)
    layer.backward(W, x, out, PC.dev(f["output_errors"]), ex, dW)
    layer.check()
    torch.cuda.synchronize()
    assert PC.relerr(out.cpu().numpy(), f["outputs"]) < TOL
    assert PC.relerr(ex.cpu().numpy(), f["prev_errors"]) < TOL
    assert PC.relerr(dW.cpu().numpy(), f["weight_updates"]) < TOL
    dummy = f["patTypes"] == 0
    assert not out.cpu().numpy().reshape(N, L)[dummy].any()
    layer.close()


def test_dense_sse_fixture():
    import torch

    print("golden dense_tanh_sse", flush=True)
    f = load("dense_tanh_sse")
    capi = PC.pkg().capi
    P, D, act = int(f["P"]), int(f["D"]), int(f["act"])
    N = f["patTypes"].size
    W, x, tgt, pat = PC.dev(f["weights"]), PC.dev(f["x"]), PC.dev(f["targets"]), PC.dev(f["patTypes"])
    y = torch.zeros(D * N, dtype=torch.float32, device="cuda")
    err = torch.zeros(D * N, dtype=torch.float32, device="cuda")
    ex = torch.zeros(P * N, dtype=torch.float32, device="cuda")
    dW = torch.zeros(f["weights"].size, dtype=torch.float32, device="cuda")
    loss = torch.zeros(1, dtype=torch.float32, device="cuda")
    capi.dense_forward(P, D, N, act, 1.0, W, x, y)
    capi.sse_error(D, N, pat, y, tgt, loss)
    capi.sse_backward(D, N, pat, y, tgt, err)
    torch.cuda.synchronize()
    assert PC.relerr(y.cpu().numpy(), f["outputs"]) < TOL
    assert abs(float(loss.item()) - float(f["loss"])) <= TOL * abs(float(f["loss"]))
    got = err.cpu().numpy()
    assert PC.relerr(got, f["sse_errors"]) < TOL
    assert not got.reshape(N, D)[f["patTypes"] == 0].any()
    capi.dense_backward(P, D, N, act, 1.0, W, x, y, err, ex, dW)
    torch.cuda.synchronize()
    assert PC.relerr(ex.cpu().numpy(), f["prev_errors"]) < TOL
    assert PC.relerr(dW.cpu().numpy(), f["weight_updates"]) < TOL


def test_mixture_fixture():
    import torch

    print("golden mdn_mixture_4x3", flush=True)
    f = load("mdn_mixture_4x3")
    capi = PC.pkg().capi
    M, D = int(f["M"]), int(f["D"])
    lengths = [int(v) for v in f["lengths"]]
    S, T = len(lengths), max(lengths)
    Lp = M + 2 * M * D
    layer = capi.Mdn(Lp, D, S, T, [1, 0, Lp, 0, D, M])
    tgt = PC.dev(f["targets"])
    res = torch.zeros(1, dtype=torch.float32, device="cuda")
    err = torch.full((S * T * Lp,), 3.0, dtype=torch.float32, device="cuda")
    layer.load_sequences(PC.dev(f["patTypes"]), T)
    layer.forward(PC.dev(f["x"]))
    layer.calculate_error(tgt, res)
    layer.backward(tgt, err)
    torch.cuda.synchronize()
    assert abs(float(res.item()) - float(f["nll"])) <= TOL * abs(float(f["nll"]))
    assert PC.relerr(err.cpu().numpy(), f["errors"]) < TOL
    layer.close()


@pytest.mark.parametrize("name", ["dft_logamp_two_resolutions", "dft_kld_with_phase"])
def test_dft_fixture(name):
    import torch

    print("golden", name, flush=True)
    f = load(name)
    capi = PC.pkg().capi
    res = [tuple(int(v) for v in r) for r in f["resolutions"]]
    max_len, length, zeta = int(f["max_length"]), int(f["length"]), float(f["zeta"])
    layer = capi.Dft(res, max_len, 1, gamma=float(f["gamma"]), spec_dis_type=int(f["dis_type"]), zeta=zeta)
    errs = torch.zeros(f["errors"].size, dtype=torch.float32, device="cuda")
    prev = torch.full((max_len,), 2.0, dtype=torch.float32, device="cuda")
    layer.forward([length], PC.dev(f["source"]), PC.dev(f["target"]), errs)
    layer.backward(prev)
    torch.cuda.synchronize()
    assert PC.relerr(errs.cpu().numpy(), f["errors"]) < TOL
    got = prev.cpu().numpy()
    assert PC.relerr(got, f["prev_errors"]) < TOL
    assert not got[length:].any()
    layer.close()
