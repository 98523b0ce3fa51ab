"""GPU parity (through the C ABI) of the multi-resolution DFT spectral loss (distance types 0..6) with the in-house FFT against
the oracle's double-precision DFT: 1e-4 L2-normalised for losses and gradients; exact zeros beyond each
waveform's length."""
import pytest

import parity_cases as PC

pytestmark = pytest.mark.gpu
TOL = 1e-4


@pytest.mark.parametrize("res,max_len,lengths", [
    ([(32, 32, 8)], 200, [200]),
    ([(64, 40, 10)], 333, [333, 120]),                       # zero padding inside the frames, ragged lengths
    ([(512, 512, 80), (128, 128, 40), (2048, 2048, 640)], 16000, [16000, 9000]),  # benchmark config 5 resolutions
    ([(1024, 800, 200), (4096, 4096, 1024)], 6000, [6000, 5000, 4097]),
    ([(128, 128, 40)], 300, [60]),                           # waveform shorter than one frame
    # eight waveforms of very different lengths, a long and a short transform: workgroups of the short one make
    # several passes of sixteen frames, and how many depends on the waveform
    ([(2048, 2048, 512), (64, 64, 16)], 6000, [6000, 130, 2500, 64, 5999, 1000, 300, 2049]),
])
def test_dft_loss(res, max_len, lengths):
    print("dft case", res, max_len, lengths, flush=True)
    assert PC.run_dft_case(res, max_len, lengths, seed=len(res) + max_len, gamma=0.8) < TOL


def test_dft_loss_config5_full_size():
    """benchmark config 5 at its size: 8 waveforms x 16000 samples (two of them shorter), the three resolutions."""
    print("dft config 5 full size", flush=True)
    res = [(512, 512, 80), (128, 128, 40), (2048, 2048, 640)]
    lengths = [16000, 16000, 12345, 16000, 16000, 16000, 8000, 16000]
    assert PC.run_dft_case(res, 16000, lengths, seed=55, gamma=1.0) < TOL


@pytest.mark.parametrize("dis_type", [1, 2, 3, 4, 5, 6])
@pytest.mark.parametrize("res,max_len,lengths", [
    ([(64, 40, 10)], 333, [333, 120]),
    ([(512, 512, 80), (128, 128, 40), (2048, 2048, 640)], 8000, [8000, 4500]),
])
def test_dft_other_distance_types(dis_type, res, max_len, lengths):
    print("dft case", dis_type, res, max_len, lengths, flush=True)
    assert PC.run_dft_case(res, max_len, lengths, seed=7 * dis_type + max_len, gamma=0.8, dis_type=dis_type) < TOL


@pytest.mark.parametrize("dis_type,gamma,zeta", [(0, 0.8, 0.5), (4, 1.0, 2.0), (0, 0.0, 1.0)])
@pytest.mark.parametrize("res,max_len,lengths", [
    ([(64, 40, 10)], 333, [333, 120]),
    ([(512, 512, 80), (128, 128, 40), (2048, 2048, 640)], 8000, [8000, 4500]),
])
def test_dft_with_phase_distance(dis_type, gamma, zeta, res, max_len, lengths):
    print("dft phase case", dis_type, gamma, zeta, res, max_len, lengths, flush=True)
    assert PC.run_dft_case(res, max_len, lengths, seed=3 + max_len, gamma=gamma, dis_type=dis_type, zeta=zeta) < TOL


def test_dft_equal_signals_and_rejections():
    import torch

    capi = PC.pkg().capi
    gen = torch.Generator(device="cuda").manual_seed(11)
    x = torch.randn(1000, device="cuda", generator=gen)
    other = torch.randn(1000, device="cuda", generator=gen)
    layer = capi.Dft([(128, 128, 40)], 1000, 1)
    err, err_other = torch.ones(1, device="cuda"), torch.ones(1, device="cuda")
    g, g_other = torch.ones(1000, device="cuda"), torch.ones(1000, device="cuda")
    layer.forward([1000], x, x.clone(), err)
    layer.backward(g)
    layer.forward([1000], x, other, err_other)
    layer.backward(g_other)
    torch.cuda.synchronize()
    # source and target spectra come out of ONE complex transform, so identical signals agree to rounding only:
    # loss and gradient are not exactly zero, but vanish against those of two unrelated signals
    assert float(err.item()) < 1e-8 * float(err_other.item())
    print("equal signals: loss", float(err.item()), "of", float(err_other.item()), "gradient", float(g.abs().max()), "of",
          float(g_other.abs().max()), flush=True)
    assert float(g.abs().max()) < 1e-4 * float(g_other.abs().max())
    with pytest.raises(RuntimeError):
        capi.Dft([(100, 100, 25)], 1000, 1)          # not a power of two
    with pytest.raises(RuntimeError):
        capi.Dft([(128, 128, 40)], 1000, 1, spec_dis_type=7)   # no such amplitude distance
    with pytest.raises(RuntimeError):
        capi.Dft([(128, 128, 40)], 1000, 1, zeta=1.0, phase_dis_type=1)   # instantaneous phase is not built
