"""GPU test of cnt_dense_backward_weights_static, the entry point that allocates nothing: its split partial products
go through an array inside the library's code object instead of a buffer from hipMalloc.  Compared with
cnt_dense_backward_weights (and the CPU oracle) on two calls in a row, the second with a smaller layer and input, to
the tolerance of every other fp32 product here: 1e-4 L2-normalised."""
import numpy as np
import pytest

import oracle_lib as O
import parity_cases as PC

pytestmark = pytest.mark.gpu
TOL = 1e-4


def _one_call(capi, P, D, N, bias, seed):
    import torch

    rng = np.random.default_rng(seed)
    x = rng.standard_normal(P * N).astype(np.float32)
    err = rng.standard_normal(D * N).astype(np.float32)
    xd, ed = PC.dev(x), PC.dev(err)
    want = torch.full((P * D + D,), 7.0, dtype=torch.float32, device="cuda")
    got = torch.full((P * D + D,), -3.0, dtype=torch.float32, device="cuda")
    capi.dense_backward_weights(P, D, N, bias, xd, ed, want)
    capi.dense_backward_weights_static(P, D, N, bias, xd, ed, got)
    torch.cuda.synchronize()
    g, w = got.cpu().numpy(), want.cpu().numpy()
    assert PC.relerr(g[:P * D], w[:P * D]) < TOL
    assert PC.relerr(g[P * D:], w[P * D:]) < TOL
    # and against the oracle's sequential sums
    dW = np.zeros(P * D + D, dtype=np.float32)
    O.dense_backward(P, D, N, 0, bias, np.zeros(P * D + D, dtype=np.float32), x, np.zeros(D * N, dtype=np.float32),
                     err.copy(), None, dW)
    assert PC.relerr(g[:P * D], dW[:P * D]) < TOL
    assert PC.relerr(g[P * D:], dW[P * D:]) < TOL


def test_static_scratch_entry_point_two_calls_second_smaller():
    capi = PC.pkg().capi
    print("no-alloc dense weight gradient: 128 x 256 over 6000 slots, then 64 x 100 over 1501", flush=True)
    _one_call(capi, 128, 256, 6000, 0.5, seed=1)
    _one_call(capi, 64, 100, 1501, 2.0, seed=2)   # smaller: fewer splits, shorter stride, stale partials beyond it
    _one_call(capi, 33, 7, 90, 1.0, seed=3)       # a single split


def test_static_scratch_entry_point_takes_no_device_memory():
    """The device's free memory as the driver reports it is the same before and after calls of the entry point (a first
    call has been made, so the code object and its array are loaded); the allocating entry point beside it, called on a
    stream that has no scratch buffer yet, is seen to take its 16 MB, which shows that the probe can see an allocation."""
    import torch

    capi = PC.pkg().capi
    P, D, N = 128, 256, 6000
    rng = np.random.default_rng(5)
    xd = PC.dev(rng.standard_normal(P * N).astype(np.float32))
    ed = PC.dev(rng.standard_normal(D * N).astype(np.float32))
    dW = torch.zeros(P * D + D, dtype=torch.float32, device="cuda")
    capi.dense_backward_weights_static(P, D, N, 1.0, xd, ed, dW)
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        capi.dense_backward_weights_static(P, D, N, 1.0, xd, ed, dW)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0
    stream = torch.cuda.Stream()   # a stream the library has not seen: its first split product allocates the scratch
    capi.dense_backward_weights(P, D, N, 1.0, xd, ed, dW, stream=stream)
    torch.cuda.synchronize()
    free2, _ = torch.cuda.mem_get_info()
    capi.gemm_release(stream)
    assert free0 - free2 >= 16 << 20


def test_static_scratch_entry_point_rejects_oversized_layers():
    import torch

    capi = PC.pkg().capi
    a = torch.zeros(16, device="cuda")
    with pytest.raises(RuntimeError, match="exceed the static scratch"):
        capi.dense_backward_weights_static(2048, 2048, 4, 1.0, a, a, a)
