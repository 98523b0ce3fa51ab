"""GPU parity tests (through the C ABI) for the matrix product seam, dense / SSE layers and the LSTM.
Tolerance: 1e-4 on the L2-normalised difference per tensor (fp32, different summation order);
masking and indexing are asserted bit-exactly inside parity_cases."""
import pytest

import parity_cases as PC

pytestmark = pytest.mark.gpu
TOL = 1e-4


@pytest.mark.parametrize("m,n,k,tA,tB,acc", [
    (128, 128, 64, 0, 0, 0), (128, 128, 64, 1, 0, 0), (128, 128, 64, 0, 1, 0),
    (382, 800, 256, 0, 0, 1), (256, 800, 382, 1, 0, 0), (382, 256, 800, 0, 1, 0),
    (187, 333, 77, 0, 0, 0), (5, 3, 2, 1, 0, 1), (1, 1, 1, 0, 0, 0), (130, 129, 17, 0, 1, 1),
])
def test_matrix_product(m, n, k, tA, tB, acc):
    print("gemm case", m, n, k, tA, tB, acc, flush=True)
    assert PC.run_gemm_case(m, n, k, tA, tB, acc, seed=m + n + k) < TOL


def test_matrix_product_rejects_double_transpose():
    import torch

    capi = PC.pkg().capi
    a = torch.zeros(4, device="cuda")
    with pytest.raises(RuntimeError):
        capi.matrix_product(a, 2, 2, 2, a, 1, a, 1, 0)


@pytest.mark.parametrize("P,D,N,act", [(382, 512, 600, 1), (512, 187, 600, 0), (33, 65, 130, 2), (64, 64, 256, 3)])
def test_dense(P, D, N, act):
    print("dense case", P, D, N, act, flush=True)
    assert PC.run_dense_case(P, D, N, act, 1.0, seed=P + D) < TOL


def test_sse():
    print("sse case", flush=True)
    assert PC.run_sse_case(187, [40, 33, 40, 12], seed=2) < 1e-5


@pytest.mark.parametrize("P,L,bidir,lengths", [
    (24, 64, False, [9, 9, 9]),
    (24, 64, False, [12, 7, 12, 5]),
    (40, 128, True, [10, 10]),
    (40, 128, True, [14, 6, 11, 14, 3]),
    (50, 256, False, [20, 20, 20, 15]),
    (48, 512, True, [16, 9, 13, 16, 16, 5, 16, 12, 10, 16]),
    (33, 256, True, [1]),
    (33, 128, False, [6] * 20),
    (32, 512, False, [8, 8, 5, 8]),        # 512 cells per direction: the largest recursion kernel
    (32, 1024, True, [7, 5, 7]),
    (20, 256, False, [5] * 24),            # more than 16 parallel sequences with 256 cells
    (16, 128, True, [1, 1]),               # a single time step, two sequences
])
def test_lstm(P, L, bidir, lengths):
    print("lstm case", P, L, bidir, lengths, flush=True)
    assert PC.run_lstm_case(P, L, bidir, lengths, seed=len(lengths) + L) < TOL


def test_lstm_clip_and_repeat_backward():
    """Large errors activate the [-1,1] clip; a second backward without load_sequences adds the stored
    output-gate deltas, as in the reference."""
    print("lstm clip case", flush=True)
    assert PC.run_lstm_case(24, 64, False, [10, 6, 10], seed=4, wscale=0.5, escale=20.0) < TOL
    assert PC.run_lstm_case(24, 128, True, [10, 6, 10], seed=5, wscale=0.5, escale=20.0, repeat_backward=True) < TOL


def test_lstm_config1_unidirectional():
    """BASELINE config 1: P=382, H=256, T=200, S=4 with one sequence of 150 frames."""
    print("lstm config 1", flush=True)
    assert PC.run_lstm_case(382, 256, False, [200, 200, 200, 150], seed=1) < TOL


def test_lstm_unsupported_geometry_is_an_error():
    capi = PC.pkg().capi
    with pytest.raises(RuntimeError):
        capi.Lstm(10, 100, False, 4, 10)
    with pytest.raises(RuntimeError):
        capi.Lstm(10, 129, True, 4, 10)
