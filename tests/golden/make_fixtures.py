#!/usr/bin/env python3
"""Writes the golden fixtures of this directory: for a few small cases, the inputs and what the CPU oracle
(oracle/, pinned by tests/test_oracle_*.py) computes from them.  The reference holds no vectors for this path, so
these freeze the oracle: tests/test_golden.py checks that the oracle still reproduces them (a change of the
restatement shows up there, not as a silent shift of every parity test), tests/test_gpu_golden.py runs the HIP
library on the stored inputs.  Plain .npz files (arrays only, loaded with allow_pickle=False).

Run from the repository root after building the oracle:  python tests/golden/make_fixtures.py"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
for _d in (os.path.dirname(HERE), os.path.join(ROOT, "oracle"), os.path.join(ROOT, "bench")):
    if _d not in sys.path:
        sys.path.insert(0, _d)

import oracle_lib as O  # noqa: E402
from torch_models import make_pat_types  # noqa: E402


def lstm_case(P, L, bidir, lengths, seed):
    S, T = len(lengths), max(lengths)
    H, N = L // (2 if bidir else 1), S * max(lengths)
    rng = np.random.default_rng(seed)
    W = rng.uniform(-0.2, 0.2, O.lib().orc_lstm_weight_count(P, L, int(bidir))).astype(np.float32)
    x = rng.standard_normal((T, S, P)).astype(np.float32)
    e = (0.3 * rng.standard_normal((T, S, L))).astype(np.float32)
    for s, n in enumerate(lengths):
        x[n:, s] = 0
        e[n:, s] = 0
    pat = make_pat_types(lengths, T)
    desc = O.LstmDesc(P, L, int(bidir), S, T, min(lengths), 1.0)
    fw, bw = O.LstmState(H, N), (O.LstmState(H, N) if bidir else None)
    out, ex, dW = np.zeros(L * N, np.float32), np.zeros(P * N, np.float32), np.zeros_like(W)
    O.lstm_forward(desc, W, pat, x.reshape(-1), fw, bw, out)
    O.lstm_backward(desc, W, pat, x.reshape(-1), e.reshape(-1), fw, bw, ex, dW)
    return dict(P=P, L=L, bidir=int(bidir), lengths=np.asarray(lengths), weights=W, x=x.reshape(-1),
                output_errors=e.reshape(-1), patTypes=pat, outputs=out, prev_errors=ex, weight_updates=dW)


def dense_sse_case(P, D, act, lengths, seed):
    S, T = len(lengths), max(lengths)
    N = S * T
    rng = np.random.default_rng(seed)
    W = rng.uniform(-0.3, 0.3, P * D + D).astype(np.float32)
    pat = make_pat_types(lengths, T)
    x = rng.standard_normal(P * N).astype(np.float32)
    tgt = rng.standard_normal(D * N).astype(np.float32)
    y, err, ex, dW = np.zeros(D * N, np.float32), np.zeros(D * N, np.float32), np.zeros(P * N, np.float32), np.zeros_like(W)
    O.dense_forward(P, D, N, act, 1.0, W, x, y)
    loss = O.sse_error(D, N, pat, y, tgt)
    O.sse_backward(D, N, pat, y, tgt, err)
    delta = err.copy()
    O.dense_backward(P, D, N, act, 1.0, W, x, y, delta, ex, dW)
    return dict(P=P, D=D, act=act, lengths=np.asarray(lengths), weights=W, x=x, targets=tgt, patTypes=pat, outputs=y,
                loss=np.float32(loss), sse_errors=err, prev_errors=ex, weight_updates=dW)


def mixture_case(M, D, lengths, seed):
    S, T = len(lengths), max(lengths)
    F, Lp = S * T, M + 2 * M * D
    rng = np.random.default_rng(seed)
    x = rng.standard_normal(F * Lp).astype(np.float32)
    tgt = rng.standard_normal(F * D).astype(np.float32)
    pat = make_pat_types(lengths, T)
    para, tmp, err = np.zeros(F * M * (1 + 2 * D), np.float32), np.zeros(F * M + F, np.float32), np.zeros(F * Lp, np.float32)
    O.mdn_mixture_forward(F, Lp, 0, M, D, 0.0, pat, x, para)
    nll = O.mdn_mixture_error(F, D, 0, M, D, pat, tgt, para, tmp)
    O.mdn_mixture_backward(F, Lp, D, 0, 0, M, D, 0.0, pat, tgt, para, tmp, err)
    return dict(M=M, D=D, lengths=np.asarray(lengths), x=x, targets=tgt, patTypes=pat, nll=np.float32(nll), errors=err)


def dft_case(resolutions, dis_type, gamma, zeta, max_len, length, seed):
    rng = np.random.default_rng(seed)
    src = (0.3 * rng.standard_normal(max_len)).astype(np.float32)
    tgt = (0.3 * rng.standard_normal(max_len)).astype(np.float32)
    errs, grad = [], np.zeros(max_len, np.float64)
    for (N, Nw, Hs) in resolutions:
        g = np.zeros(max_len, np.float32)
        errs.append(O.dft_spectral_loss(dis_type, N, Nw, Hs, 0, max_len, length, gamma, 1e-5, src.copy(), tgt.copy(), g))
        g[length:] = 0
        grad += g
    for (N, Nw, Hs) in resolutions:
        if zeta > 0:
            g = np.zeros(max_len, np.float32)
            errs.append(O.dft_phase_loss(N, Nw, Hs, 0, max_len, length, zeta, src.copy(), tgt.copy(), g))
            g[length:] = 0
            grad += g
    return dict(resolutions=np.asarray(resolutions), dis_type=dis_type, gamma=np.float32(gamma), zeta=np.float32(zeta),
                max_length=max_len, length=length, source=src, target=tgt, errors=np.asarray(errs, np.float32),
                prev_errors=grad.astype(np.float32))


CASES = {
    "lstm_blstm_128": lambda: lstm_case(10, 128, True, [9, 6, 9, 4], 101),
    "lstm_uni_64": lambda: lstm_case(7, 64, False, [8, 8, 5], 102),
    "lstm_blstm_stepwise_24": lambda: lstm_case(5, 24, True, [7, 3], 103),
    "dense_tanh_sse": lambda: dense_sse_case(9, 6, 1, [12, 7, 10], 104),
    "mdn_mixture_4x3": lambda: mixture_case(4, 3, [10, 6, 10], 105),
    "dft_logamp_two_resolutions": lambda: dft_case([(64, 64, 16), (128, 100, 25)], 0, 0.8, 0.0, 600, 520, 106),
    "dft_kld_with_phase": lambda: dft_case([(64, 40, 10)], 1, 1.0, 0.5, 300, 300, 107),
}


def main():
    for name, make in CASES.items():
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **make())
        print("wrote", name)


if __name__ == "__main__":
    main()
