"""Pins the CPU oracle's DFT loss: transforms against numpy.fft and a brute-force DFT, the loss against
numpy, and the (deliberately non-analytic) gradient against float64 autograd of an equivalent surrogate:
the reference's gradient equals d/dx of  1/(4*B*K) * sum_k sum_b c_b d^2  with c_b = 1 for the DC and Nyquist
bins and 2 for the others (its inverse transform counts interior bins twice and its per-bin term lacks the
factor 4).  The other distance types are pinned the same way; the factor between the reference's per-bin
gradient and the true derivative of its per-bin distance is 1/4 for types 0, 2, 5, 1/2 for types 3, 4 and 1 for
types 1, 6 (derived by hand from the distance definitions, not read off the oracle)."""
import numpy as np
import torch

import oracle_lib as O
from test_oracle_lstm import relerr

PI_REF = 3.141215


def crel(a, b):
    a = np.asarray(a, dtype=np.complex128).ravel()
    b = np.asarray(b, dtype=np.complex128).ravel()
    return float(np.linalg.norm(a - b) / np.linalg.norm(b))


def test_r2c_c2r_follow_cufft_conventions():
    rng = np.random.default_rng(0)
    for n in (8, 16, 128, 512):
        x = rng.standard_normal(n).astype(np.float32)
        X = O.dft_r2c(x)
        assert crel(X, np.fft.rfft(x.astype(np.float64))) < 1e-6
        G = (rng.standard_normal(n // 2 + 1) + 1j * rng.standard_normal(n // 2 + 1)).astype(np.complex64)
        y = O.dft_c2r(G, n)
        assert relerr(y, np.fft.irfft(G.astype(np.complex128), n=n) * n) < 1e-6
    # brute force on n = 8, including the ignored imaginary parts of DC and Nyquist
    n = 8
    x = rng.standard_normal(n)
    j = np.arange(n)
    brute = np.array([np.sum(x * np.exp(-2j * np.pi * j * b / n)) for b in range(n // 2 + 1)])
    assert crel(O.dft_r2c(x.astype(np.float32)), brute) < 1e-6
    G = rng.standard_normal(5) + 1j * rng.standard_normal(5)
    full = np.zeros(n, dtype=complex)
    full[0], full[4] = G[0].real, G[4].real
    for b in (1, 2, 3):
        full[b], full[n - b] = G[b], np.conj(G[b])
    brute = np.array([np.sum(full * np.exp(2j * np.pi * np.arange(n) * t / n)) for t in range(n)]).real
    assert relerr(O.dft_c2r(G.astype(np.complex64), n), brute) < 1e-6


def bin_distance64(dis_type, S, T, floor):
    """Per-bin distance of every type in float64 torch, and the factor kappa with
    reference gradient = kappa * true derivative."""
    s2, t2 = S.abs() ** 2, T.abs() ** 2
    if dis_type == 1:
        s, t = torch.sqrt(s2 + 1e-5), torch.sqrt(t2 + 1e-5)
        return t * torch.log(t / s) - t + s, 1.0
    if dis_type == 2:
        return (s2 - t2) ** 2, 0.25
    if dis_type == 3:
        return torch.log((S - T).abs() ** 2 + 1.0), 0.5
    if dis_type == 4:
        return (S - T).abs() ** 2, 0.5
    if dis_type == 5:
        return ((s2 + 1e-5) / (t2 + 1e-5) - 1.0) ** 2, 0.25
    if dis_type == 6:
        r = torch.sqrt(t2 + 1e-5) / torch.sqrt(s2 + 1e-5)
        return r - torch.log(r) - 1.0, 1.0
    if dis_type == "phase":
        # 1 - cos(arg S - arg T); the reference divides its gradient by |S|^2 + 1e-5 where the derivative has
        # |S|^2, which the detached weight restores
        e = 1.0 - (S.real * T.real + S.imag * T.imag) / (S.abs() * T.abs())
        return e, (s2 / (s2 + 1e-5)).detach()
    return (torch.log(s2 + floor) - torch.log(t2 + floor)) ** 2, 0.25


def surrogate(src, tgt, N, Nw, Hs, length, gamma, floor, dis_type=0):
    """float64 torch statement of the loss and of the surrogate whose autograd equals the reference gradient."""
    K = 1 if length < Nw else 1 + (length - Nw) // Hs
    B = N // 2 + 1
    w = 0.5 * (1 - torch.cos(2.0 * PI_REF * torch.arange(Nw, dtype=torch.float64) / (Nw - 1)))
    x = torch.tensor(src[:length], dtype=torch.float64, requires_grad=True)
    t = torch.tensor(tgt[:length], dtype=torch.float64)

    def frames(sig):
        pad = torch.zeros(max(0, (K - 1) * Hs + Nw - length), dtype=torch.float64)
        s = torch.cat([sig, pad])
        f = torch.stack([s[k * Hs:k * Hs + Nw] * w for k in range(K)])
        return torch.fft.rfft(torch.nn.functional.pad(f, (0, N - Nw)), n=N)

    S, T = frames(x), frames(t)
    e, kappa = bin_distance64(dis_type, S, T, floor)
    loss = e.sum() / (B * K)
    c = torch.full((B,), 2.0, dtype=torch.float64)
    c[0] = c[-1] = 1.0
    sur = gamma * (kappa * c * e).sum() / (B * K)
    sur.backward()
    return float(loss.detach()), x.grad.numpy()


def run(N, Nw, Hs, max_len, length, gamma=1.0, seed=0):
    rng = np.random.default_rng(seed)
    src = (0.3 * rng.standard_normal(max_len)).astype(np.float32)
    tgt = (0.3 * rng.standard_normal(max_len)).astype(np.float32)
    grad = np.zeros(max_len, dtype=np.float32)
    err = O.dft_logamp_loss(N, Nw, Hs, 0, max_len, length, gamma, 1e-5, src, tgt, grad)
    ref_err, ref_grad = surrogate(src, tgt, N, Nw, Hs, length, gamma, 1e-5)
    assert abs(err - ref_err) <= 2e-5 * abs(ref_err)
    assert relerr(grad[:length], ref_grad) < 2e-5
    return grad


def test_loss_and_gradient_match_surrogate_autograd():
    run(16, 16, 4, 64, 64)
    run(128, 128, 40, 1000, 1000, gamma=0.7, seed=1)
    run(512, 512, 80, 2000, 2000, seed=2)


def test_frame_shorter_than_fft_and_partial_last_frame():
    run(32, 20, 5, 203, 203, seed=3)   # zero padding inside every frame; 203 leaves samples after the last frame
    g = run(64, 64, 16, 400, 250, seed=4)  # current waveform shorter than the buffer
    assert not g[250:].any()              # nothing flows to samples beyond the last valid frame
    K = 1 + (250 - 64) // 16
    assert not g[(K - 1) * 16 + 64:].any()


def test_equal_signals_give_zero():
    rng = np.random.default_rng(5)
    x = rng.standard_normal(300).astype(np.float32)
    g = np.ones(300, dtype=np.float32)
    assert O.dft_logamp_loss(64, 64, 16, 0, 300, 300, 1.0, 1e-5, x, x.copy(), g) == 0.0
    assert not g.any()


def run_type(dis_type, N, Nw, Hs, max_len, length, gamma=1.0, seed=0, tol=5e-5):
    rng = np.random.default_rng(seed)
    src = (0.3 * rng.standard_normal(max_len)).astype(np.float32)
    tgt = (0.3 * rng.standard_normal(max_len)).astype(np.float32)
    grad = np.zeros(max_len, dtype=np.float32)
    err = O.dft_spectral_loss(dis_type, N, Nw, Hs, 0, max_len, length, gamma, 1e-5, src, tgt, grad)
    ref_err, ref_grad = surrogate(src, tgt, N, Nw, Hs, length, gamma, 1e-5, dis_type)
    assert abs(err - ref_err) <= tol * abs(ref_err), (dis_type, err, ref_err)
    assert relerr(grad[:length], ref_grad) < tol, (dis_type, relerr(grad[:length], ref_grad))
    assert not grad[length:].any()


def test_every_distance_type_matches_its_surrogate():
    for dis_type in range(7):
        run_type(dis_type, 16, 16, 4, 64, 64, seed=10 + dis_type)
        run_type(dis_type, 128, 100, 40, 1000, 900, gamma=0.7, seed=20 + dis_type)
        run_type(dis_type, 512, 512, 80, 2000, 2000, seed=30 + dis_type)


def test_type_zero_is_the_log_amplitude_loss():
    rng = np.random.default_rng(40)
    src, tgt = rng.standard_normal(500).astype(np.float32), rng.standard_normal(500).astype(np.float32)
    g0, g1 = np.zeros(500, dtype=np.float32), np.zeros(500, dtype=np.float32)
    e0 = O.dft_logamp_loss(64, 64, 16, 0, 500, 400, 0.5, 1e-5, src, tgt, g0)
    e1 = O.dft_spectral_loss(0, 64, 64, 16, 0, 500, 400, 0.5, 1e-5, src, tgt, g1)
    assert e0 == e1 and np.array_equal(g0, g1)


def test_equal_signals_give_zero_for_every_type():
    rng = np.random.default_rng(41)
    x = rng.standard_normal(300).astype(np.float32)
    for dis_type in (1, 2, 4, 5, 6):  # type 3 is log(0 + 1) = 0 as well, checked apart for its gradient
        g = np.ones(300, dtype=np.float32)
        assert abs(O.dft_spectral_loss(dis_type, 64, 64, 16, 0, 300, 300, 1.0, 1e-5, x, x.copy(), g)) < 1e-7
        assert np.abs(g).max() < 1e-6
    g = np.ones(300, dtype=np.float32)
    assert O.dft_spectral_loss(3, 64, 64, 16, 0, 300, 300, 1.0, 1e-5, x, x.copy(), g) == 0.0 and not g.any()


def test_cosine_phase_distance_matches_its_surrogate():
    for N, Nw, Hs, max_len, length, zeta, seed in ((16, 16, 4, 64, 64, 1.0, 50), (128, 100, 40, 1000, 900, 0.6, 51),
                                                  (512, 512, 80, 2000, 2000, 2.0, 52)):
        rng = np.random.default_rng(seed)
        src = (0.3 * rng.standard_normal(max_len)).astype(np.float32)
        tgt = (0.3 * rng.standard_normal(max_len)).astype(np.float32)
        grad = np.zeros(max_len, dtype=np.float32)
        err = O.dft_phase_loss(N, Nw, Hs, 0, max_len, length, zeta, src, tgt, grad)
        ref_err, ref_grad = surrogate(src, tgt, N, Nw, Hs, length, zeta, 0.0, "phase")
        assert abs(err - ref_err) <= 5e-5 * abs(ref_err)
        assert relerr(grad[:length], ref_grad) < 5e-5
    # opposite signals: every bin has distance 1 - cos(pi) = 2, and the gradient vanishes
    x = np.random.default_rng(53).standard_normal(300).astype(np.float32)
    g = np.ones(300, dtype=np.float32)
    assert abs(O.dft_phase_loss(64, 64, 16, 0, 300, 300, 1.0, x, -x, g) - 2.0) < 1e-5
    assert np.abs(g).max() < 1e-5
