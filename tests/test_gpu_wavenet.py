"""GPU parity (through the C ABI) of the WaveNet blocks: dilated causal convolution layer, conditioned and
plain gated activation, context up-sampling / frame-rate gradient sum, skip-add.  Floating point: 1e-4
L2-normalised per tensor.  Masking, dilation and tap indexing: exact (zeros, untouched slots, dead taps)."""
import pytest

import parity_cases as PC

pytestmark = pytest.mark.gpu
TOL = 1e-4


@pytest.mark.parametrize("P,hw,it,lengths,causal,tanh", [
    (5, [1] * 6, [4] * 6, [17, 9, 14], 1, 1),
    (4, [1, 1, 2, 0, 2], [1, 3, 2, 1, 1], [12, 12], 0, 0),
    (3, [1, 1], [16, 16], [10, 6], 1, 1),                      # dilation longer than the sequences
    (64, [1] * 128, [1] * 128, [300, 220], 1, 1),              # WaveNet block geometry (64 -> 128), dilation 1
    (64, [1] * 128, [512] * 128, [700, 650], 1, 0),            # largest dilation of the stack, no tanh
    (64, [1] * 128, [512] * 128, [16000, 15100], 1, 1),        # benchmark config 4: one layer at full length
    (382, [2] * 40 + [1] * 30, [1] * 40 + [2] * 30, [33, 40, 21], 0, 1),
    (32, [1] * 24 + [0] * 40, [3] * 24 + [1] * 40, [400, 333, 150], 1, 1),   # two filter groups, ragged lengths
    (16, [0] * 32, [1] * 32, [200, 90], 0, 0),                              # width-1 filters (one tap), not causal
])
def test_cnn_layer(P, hw, it, lengths, causal, tanh):
    print("cnn case", P, len(hw), lengths, causal, tanh, flush=True)
    assert PC.run_cnn_case(P, hw, it, lengths, causal, tanh, seed=P + len(hw)) < TOL


def test_cnn_layer_short_fraction_clears_tail():
    print("cnn short fraction", flush=True)
    assert PC.run_cnn_case(6, [1] * 4, [2] * 4, [9, 5], 1, 1, seed=9, bias=0.5, maxT=15) < TOL


def test_cnn_rejects_too_many_taps():
    capi = PC.pkg().capi
    with pytest.raises(RuntimeError):
        capi.Cnn(4, [9, 9], [1, 1], 2, 10, 1, 1)


@pytest.mark.parametrize("D,C,lengths,cg", [(4, 3, [7, 5, 7], True), (64, 80, [200, 150], True), (64, 80, [90, 90], False),
                                            (16, 0, [30, 11], False)])
def test_wavnetc_and_gatedact(D, C, lengths, cg):
    print("wavnetc case", D, C, lengths, cg, flush=True)
    assert PC.run_wavnetc_case(D, C, lengths, seed=D + C, with_ctx_grad=cg) < TOL


@pytest.mark.parametrize("mv", [False, True])
def test_context_upsampling_and_gradient_sum(mv):
    print("context case", mv, flush=True)
    assert PC.run_context_case(80, 80, [400, 250], seed=3, use_mean_std=mv) < 1e-5


def test_skipadd():
    print("skipadd case", flush=True)
    assert PC.run_skipadd_case(64 * 1000 + 7, seed=1) == 0.0
