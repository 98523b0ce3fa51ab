"""GPU parity (through the C ABI) of the mixture-density layer: flat softmax unit and untied-variance
mixture unit, forward parameters, negative log-likelihood and gradients; 1e-4 L2-normalised per tensor,
zero patterns (padding frames, the reference's index collision) exact."""
import pytest

import parity_cases as PC

pytestmark = pytest.mark.gpu
TOL = 1e-4


@pytest.mark.parametrize("lengths,M,D,extra", [
    ([5, 5, 5], 4, 6, 0),
    ([6, 3, 6], 2, 2, 0),          # Lp=10: padding frames collide with valid mixture-weight slots
    ([9, 4, 7, 9], 3, 5, 7),       # unit does not start at column 0, leading columns stay zero
    ([40, 25, 33, 40, 12, 40, 40, 31, 40, 20], 16, 60, 0),  # benchmark config 3 geometry, shortened
    ([600, 431, 377, 512, 300, 598, 465, 349, 553, 420], 16, 60, 0),  # benchmark config 3 at full size
    ([12, 7, 12], 8, 12, 4),       # every size a multiple of four behind four leading columns: the 16-byte path
    ([12, 7, 12], 8, 12, 2),       # the same unit two columns further on: not aligned, scalar path
])
@pytest.mark.parametrize("one_call", [False, True])
def test_mixture_unit(lengths, M, D, extra, one_call):
    # one_call: error and gradient through cnt_mdn_error_backward (one pass over the parameters for the units of at most
    # sixteen components whose data is 16-byte aligned, the two kernels in turn for the others)
    print("mdn mixture case", lengths, M, D, extra, one_call, flush=True)
    assert PC.run_mdn_mixture_case(lengths, M, D, extra, seed=M + D, one_call=one_call) < TOL


@pytest.mark.parametrize("M,D,one_call", [(3, 4, False), (3, 4, True), (4, 8, True)])
def test_mixture_unit_variance_floor_and_short_fraction(M, D, one_call):
    print("mdn floor case", M, D, one_call, flush=True)
    assert PC.run_mdn_mixture_case([7, 5], M, D, 0, seed=3, var_floor=0.8, maxT=12, one_call=one_call) < TOL


@pytest.mark.parametrize("lengths,K,extra", [([6, 6], 10, 0), ([9, 5, 7], 257, 3), ([30, 17], 1024, 0)])
def test_softmax_unit(lengths, K, extra):
    print("mdn softmax case", lengths, K, extra, flush=True)
    assert PC.run_softmax_case(lengths, K, extra, seed=K) < TOL


def test_unsupported_units_are_rejected():
    capi = PC.pkg().capi
    with pytest.raises(RuntimeError):
        capi.Mdn(10, 2, 2, 4, [1, 0, 10, 0, 2, 0])      # sigmoid unit
    with pytest.raises(RuntimeError):
        capi.Mdn(10, 2, 2, 4, [1, 0, 10, 0, 2, 2], tie_variance=True)
    with pytest.raises(RuntimeError):
        capi.Mdn(10, 2, 2, 4, [2, 0, 10, 0, 2, 2])      # length does not match the unit count


@pytest.mark.parametrize("lengths,K,extra,continuous,with_softmax", [
    ([9, 5, 9], 7, 0, False, False), ([12, 12], 3, 4, True, False), ([20, 11, 20, 3], 16, 2, False, True),
    ([6], 1, 0, True, False),
])
def test_sigmoid_unit(lengths, K, extra, continuous, with_softmax):
    print("mdn sigmoid case", lengths, K, extra, continuous, with_softmax, flush=True)
    assert PC.run_sigmoid_case(lengths, K, extra, continuous, seed=K + extra, with_softmax=with_softmax) < TOL
