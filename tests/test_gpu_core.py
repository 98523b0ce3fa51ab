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


@pytest.mark.parametrize("P,D,N,act", [
    (382, 512, 600, 1), (512, 187, 600, 0), (33, 65, 130, 2), (64, 64, 256, 3),
    # small layers, long contraction (the shapes of a WaveNet-style stack's 1x1 layers): split-K weight gradients
    # with one, several and ragged tiles, sizes that are not multiples of the tile
    (64, 128, 3000, 0), (128, 1024, 777, 1), (80, 20, 1501, 2), (12, 8, 200, 0), (128, 132, 999, 3),
])
def test_dense(P, D, N, act):
    print("dense case", P, D, N, act, flush=True)
    assert PC.run_dense_case(P, D, N, act, 1.0, seed=P + D) < TOL


@pytest.mark.parametrize("P,D,N,bias", [
    # narrow layers over long inputs take the split-K path that sums partial products and carries the bias
    # gradient (row sums of the errors, times the layer's bias value) along; 300 x 300 is too large an output for it and
    # takes the atomic path with its separate column sum
    (64, 128, 3000, 0.5), (64, 64, 5000, 2.0), (100, 96, 2500, 0.25), (300, 300, 2500, 0.5),
])
def test_dense_bias_value_scales_the_bias_gradient(P, D, N, bias):
    print("dense bias case", P, D, N, bias, flush=True)
    assert PC.run_dense_case(P, D, N, 0, bias, seed=P + D + N) < TOL


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
    (24, 256, True, [7, 4, 7] * 6),        # 18 parallel sequences, bidirectional: the recursion that spans the XCDs
    (24, 128, False, [3, 9, 1, 9, 2]),     # very ragged, one sequence of a single step among longer ones
    # 2400 slots of which a third is valid: the layer lists the valid slots itself and its weight gradients sum over those
    (24, 128, True, [300, 50, 300, 20, 100, 300, 7, 1]),
    (20, 64, False, [1, 600, 1, 1]),       # the same for a forward-only layer: one long sequence beside three single frames
    # geometries without a persistent recursion kernel: step-by-step recursion
    (12, 64, True, [30, 23]),              # 32 cells per direction (the reference example's conditioning BLSTM)
    (7, 20, False, [9, 4, 9]),             # 20 cells, sizes that are no multiple of anything
    (25, 200, True, [11, 11, 6, 2]),       # 100 cells per direction
    (10, 64, False, [6] * 40),             # more than 32 parallel sequences
    (9, 6, True, [1, 1, 1]),               # a single time step
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


def test_weight_gradients_spread_between_runs():
    """The weight gradients are summed with fp32 atomics or per-split partial sums, so their bits may depend on the
    order in which workgroups finish.  Three passes over the same inputs: the layer's errors must be bit-identical
    (the recursion and the error products have a fixed summation order), the weight gradients within 1e-5
    L2-normalised of each other (the parity tolerance against the oracle is 1e-4)."""
    import numpy as np
    import torch

    print("lstm run-to-run spread", flush=True)
    capi = PC.pkg().capi
    P, L, S, T = 96, 512, 10, 160
    rng = np.random.default_rng(11)
    lengths = [int(v) for v in rng.integers(80, T + 1, size=S)]
    lengths[0] = T
    W, x, outerr = PC.lstm_inputs(P, L, True, S, T, lengths, 1)
    pat = PC.make_pat_types(lengths, T)
    Wd, xd, pd, ed = PC.dev(W), PC.dev(x), PC.dev(pat), PC.dev(outerr)
    out = torch.zeros(L * T * S, device="cuda")
    layer = capi.Lstm(P, L, True, S, T)
    runs = []
    for _ in range(3):
        ex = torch.zeros(P * T * S, device="cuda"); dW = torch.zeros_like(Wd)
        layer.load_sequences(pd, T, min(lengths))
        layer.forward(Wd, xd, out)
        layer.backward(Wd, xd, out, ed.clone(), ex, dW)
        layer.check()
        torch.cuda.synchronize()
        runs.append((ex.cpu().numpy().copy(), dW.cpu().numpy().copy()))
    layer.close()
    for ex, dW in runs[1:]:
        assert np.array_equal(ex, runs[0][0])
        assert PC.relerr(dW, runs[0][1]) < 1e-5


@pytest.mark.parametrize("L,bidir,S,T,cuts", [
    (512, True, 10, 60, [45]), (512, True, 10, 60, [1, 30, 59]), (256, False, 7, 50, [37]), (128, True, 3, 9, [2, 3]),
])
def test_lstm_recursion_in_several_launches_is_the_same_recursion(L, bidir, S, T, cuts):
    """The backward recursion run as ranges of its steps, and the error product for the preceding layer computed for
    the time steps that are final early and for the rest afterwards: every state array and every error is
    bit-identical to the single launch and the single product."""
    import numpy as np
    import torch

    print("lstm split recursion", L, bidir, S, T, cuts, flush=True)
    capi = PC.pkg().capi
    P = 40
    rng = np.random.default_rng(L + S)
    lengths = [int(v) for v in rng.integers(max(1, T // 2), T + 1, size=S)]
    lengths[0] = T
    W, x, outerr = PC.lstm_inputs(P, L, bidir, S, T, lengths, 3)
    pat = PC.make_pat_types(lengths, T)
    Wd, xd, pd, ed = PC.dev(W), PC.dev(x), PC.dev(pat), PC.dev(outerr)
    out = torch.zeros(L * T * S, device="cuda")
    layer = capi.Lstm(P, L, bidir, S, T)
    assert layer.backward_can_split()
    names = ["herr", "dni", "dig", "dfg", "dog", "cerr"]

    def snapshot(err, ex):
        torch.cuda.synchronize()
        got = {"outerr": err.cpu().numpy().copy(), "ex": ex.cpu().numpy().copy()}
        for d in range(2 if bidir else 1):
            for k in names:
                got["%s%d" % (k, d)] = layer.state(d, k).cpu().numpy().copy()
        return got

    layer.load_sequences(pd, T, min(lengths))
    layer.forward(Wd, xd, out)
    err, ex = ed.clone(), torch.full((P * T * S,), 7.0, device="cuda")
    layer.backward_errors(Wd, err, ex)
    layer.check()
    whole = snapshot(err, ex)

    layer.load_sequences(pd, T, min(lengths))
    layer.forward(Wd, xd, out)
    err, ex = ed.clone(), torch.full((P * T * S,), 7.0, device="cuda")
    edges = [0] + cuts + [T]
    done_lo, done_hi = T, T  # time steps whose columns of ex are written
    for a, b in zip(edges, edges[1:]):
        layer.backward_errors_range(Wd, err, a, b)
        lo, hi = layer.backward_steps_done(b)
        if hi > lo and done_lo == done_hi:
            layer.backward_prev_errors_range(Wd, ex, lo, hi)  # once, as soon as some time steps are final
            done_lo, done_hi = lo, hi
    if done_lo == done_hi:
        done_lo = done_hi = 0
    layer.backward_prev_errors_range(Wd, ex, 0, done_lo)
    layer.backward_prev_errors_range(Wd, ex, done_hi, T)
    layer.check()
    parts = snapshot(err, ex)
    layer.close()
    for k in whole:
        assert np.array_equal(whole[k], parts[k]), k


def test_lstm_abandoned_partial_recursion_does_not_leak_into_the_next_pass():
    """A range of the backward recursion that ends before T leaves its last partial errors in the mailbox for the range
    that continues it.  When the pass is abandoned instead -- the caller starts over at step 0, with or without a new
    fraction in between -- the next recursion must not consume them: every result equals that of a clean pass, a range
    that does not start where the last one ended is refused."""
    import numpy as np
    import torch

    print("lstm abandoned partial recursion", flush=True)
    capi = PC.pkg().capi
    P, L, S, T = 40, 512, 6, 30
    lengths = [T, 21, T, 17, 25, T]
    W, x, outerr = PC.lstm_inputs(P, L, True, S, T, lengths, 4)
    pat = PC.make_pat_types(lengths, T)
    Wd, xd, pd, ed = PC.dev(W), PC.dev(x), PC.dev(pat), PC.dev(outerr)
    out = torch.zeros(L * T * S, device="cuda")
    layer = capi.Lstm(P, L, True, S, T)

    def clean_pass():
        layer.load_sequences(pd, T, min(lengths))
        layer.forward(Wd, xd, out)
        err, ex = ed.clone(), torch.zeros(P * T * S, device="cuda")
        layer.backward_errors(Wd, err, ex)
        layer.check()
        torch.cuda.synchronize()
        return ex.cpu().numpy().copy(), [layer.state(d, k).cpu().numpy().copy() for d in range(2) for k in ("dni", "dog", "cerr")]

    ex0, st0 = clean_pass()
    # abandoned after 11 steps, new fraction loaded
    layer.load_sequences(pd, T, min(lengths))
    layer.forward(Wd, xd, out)
    layer.backward_errors_range(Wd, ed.clone(), 0, 11)
    with pytest.raises(RuntimeError, match="stands at step"):
        layer.backward_errors_range(Wd, ed.clone(), 14, T)   # not where the last range ended
    ex1, st1 = clean_pass()
    assert np.array_equal(ex0, ex1)
    for a, b in zip(st0, st1):
        assert np.array_equal(a, b)
    # abandoned, then a full recursion on the same fraction (no load_sequences: the stored output-gate deltas of the
    # eleven steps already done are added once more, as in the reference; every other array is that of a clean pass)
    layer.load_sequences(pd, T, min(lengths))
    layer.forward(Wd, xd, out)
    layer.backward_errors_range(Wd, ed.clone(), 0, 11)
    layer.load_sequences(pd, T, min(lengths))   # clears the stored output-gate deltas
    err, ex = ed.clone(), torch.zeros(P * T * S, device="cuda")
    layer.backward_errors(Wd, err, ex)
    layer.check()
    torch.cuda.synchronize()
    assert np.array_equal(ex0, ex.cpu().numpy())
    # a range after a forward pass has nothing to continue
    layer.load_sequences(pd, T, min(lengths))
    layer.forward(Wd, xd, out)
    layer.backward_errors_range(Wd, ed.clone(), 0, 7)
    layer.forward(Wd, xd, out)
    with pytest.raises(RuntimeError, match="stands at step"):
        layer.backward_errors_range(Wd, ed.clone(), 7, T)
    ex2, _ = clean_pass()
    assert np.array_equal(ex0, ex2)
    layer.close()


def test_hop_probes_measure_a_plausible_exchange():
    """The measurement hooks behind the benchmark's latency floor: a word between two workgroups of one XCD takes a
    fraction of a microsecond, across XCDs longer, and a 16 KB message longer than a 4 KB one (the reason the forward
    recursion exchanges outputs, 4 KB per workgroup and step, and not partial pre-activations, 16 KB)."""
    capi = PC.pkg().capi
    print("hop probes: word same XCD / across XCDs, message 4 KB / 16 KB", flush=True)
    near = capi.probe_hop_latency(True, False, 500)
    far = capi.probe_hop_latency(False, False, 500)
    m4 = capi.probe_hop_message(4, 500)
    m16 = capi.probe_hop_message(16, 500)
    assert 0.05 < near < 5.0 and near < far < 20.0
    assert near < m4 < m16 < 10.0
    with pytest.raises(RuntimeError, match="4, 8, 12 or 16 KB"):
        capi.probe_hop_message(5, 10)


def test_activation_functions_against_the_cpu_functions():
    """The scalar semantics of the path (Logistic.cuh / Tanh.cuh with the clamps at +-88.72) and the quick forms the
    forward recursion uses instead (hardware exp2 and reciprocal): swept over the whole unclamped range and across
    the clamps, against the CPU oracle's scalar functions.  Tolerances: the exact forms 2e-7 absolute (one rounding of
    exp and of the quotient) and 2e-5 relative, the quick forms 4e-6 (logistic) and 8e-6 (tanh) absolute and 1e-4 relative."""
    import numpy as np
    import torch

    import oracle_lib as O

    capi = PC.pkg().capi
    xs = np.concatenate([np.linspace(-89.5, 89.5, 40001), np.linspace(-12, 12, 40001), np.linspace(-1, 1, 4001),
                         np.array([-88.73, -88.72, -88.71, 88.71, 88.72, 88.73, 0.0, -0.0, 1e-30, -1e-30])]).astype(np.float32)
    L = O.lib()
    want_l = np.array([L.orc_logistic(float(v)) for v in xs], dtype=np.float32)
    want_t = np.array([L.orc_tanh(float(v)) for v in xs], dtype=np.float32)
    xd = PC.dev(xs)
    out = torch.empty_like(xd)
    got = []
    for which in range(4):
        capi.probe_activation(which, xd, out)
        torch.cuda.synchronize()
        got.append(out.cpu().numpy().copy())
    for g, w, quick, tol in ((got[0], want_l, False, 2e-7), (got[1], want_t, False, 4e-7), (got[2], want_l, True, 4e-6),
                             (got[3], want_t, True, 8e-6)):
        assert np.abs(g - w).max() <= tol
        big = np.abs(w) > 1e-30
        rel = np.abs(g[big] - w[big]) / np.abs(w[big])
        # tanh near 0 is a difference of nearly equal numbers in both forms: relative error only where |tanh| >= 0.01
        if w is want_t:
            rel = rel[np.abs(w[big]) >= 0.01]
        assert rel.max() <= (1e-4 if quick else 2e-5)   # the device's and the host's expf differ by an ulp or two
        # the clamps are exact in both forms
        assert np.all(g[xs <= -88.73] == (0.0 if w is want_l else -1.0))
        assert np.all(g[xs >= 88.73] == 1.0)


def test_lstm_config1_unidirectional():
    """benchmark config 1: P=382, H=256, T=200, S=4 with one sequence of 150 frames."""
    print("lstm config 1", flush=True)
    assert PC.run_lstm_case(382, 256, False, [200, 200, 200, 150], seed=1) < TOL


def test_lstm_gives_up_cleanly_and_recovers():
    """Failure handling, forced from the host: with a spin limit of zero and no pause before the first poll a
    workgroup gives up the moment a neighbour's data is not there yet; every workgroup then drains, the kernels
    end normally, cnt_lstm_check reports the failure, and the same handle works again afterwards."""
    import numpy as np
    import torch

    print("lstm give-up case", flush=True)
    capi = PC.pkg().capi
    P, L, S, T = 24, 512, 6, 40
    rng = np.random.default_rng(3)
    W = torch.from_numpy(rng.uniform(-0.1, 0.1, capi.lib().cnt_lstm_weight_count(P, L, 1)).astype(np.float32)).cuda()
    x = torch.from_numpy(rng.standard_normal(P * T * S).astype(np.float32)).cuda()
    pat = torch.full((T * S,), 2, dtype=torch.int8, device="cuda")
    out = torch.zeros(L * T * S, device="cuda"); err = torch.ones(L * T * S, device="cuda") * 0.01
    ex = torch.zeros(P * T * S, device="cuda"); dW = torch.zeros_like(W)
    layer = capi.Lstm(P, L, True, S, T)
    layer.load_sequences(pat, T, T)
    layer.forward(W, x, out)
    layer.backward(W, x, out, err.clone(), ex, dW)
    layer.check()
    good_out, good_ex, good_dW = out.clone(), ex.clone(), dW.clone()
    layer.set_wait_bounds(0, 0, 0)
    failures = 0
    for _ in range(3):  # an attempt only fails if some poll really comes back incomplete
        # a recursion that gave up is reported by cnt_lstm_check, or by whichever call into the handle comes
        # after the failed launch has ended -- a caller that never checks still gets the error
        try:
            layer.load_sequences(pat, T, T)
            layer.forward(W, x, out)
            layer.backward(W, x, out, err.clone(), ex, dW)
            layer.check()
        except RuntimeError as e:
            assert "gave up" in str(e)
            failures += 1
            torch.cuda.synchronize()
            try:
                layer.check()   # a second failed launch of the same attempt may have ended meanwhile
            except RuntimeError:
                pass
    assert failures >= 1
    layer.set_wait_bounds(1 << 22, 28, 34)
    layer.load_sequences(pat, T, T)
    layer.forward(W, x, out)
    layer.backward(W, x, out, err.clone(), ex, dW)
    layer.check()
    torch.cuda.synchronize()
    assert PC.relerr(out.cpu().numpy(), good_out.cpu().numpy()) < 1e-6
    assert PC.relerr(ex.cpu().numpy(), good_ex.cpu().numpy()) < 1e-6
    assert PC.relerr(dW.cpu().numpy(), good_dW.cpu().numpy()) < 1e-5   # atomic accumulation order differs
    layer.close()


def test_lstm_layers_on_two_streams_at_once():
    """Two layers of the benchmark's size driven from two non-blocking streams at the same time.  Each XCD-local
    recursion wants a compute unit per workgroup and all of them at once; the library orders recursion launches of
    different streams one behind the other, so both passes run to their end with the results each gives alone."""
    import numpy as np
    import torch

    print("two lstm layers on two streams", flush=True)
    capi = PC.pkg().capi
    P, L, S, T = 64, 512, 10, 200
    N = T * S
    rng = np.random.default_rng(9)
    pat = torch.full((N,), 2, dtype=torch.int8, device="cuda")
    layers, data, alone = [], [], []
    for k in range(2):
        W = torch.from_numpy(rng.uniform(-0.08, 0.08, capi.lib().cnt_lstm_weight_count(P, L, 1)).astype(np.float32)).cuda()
        x = torch.from_numpy(rng.standard_normal(P * N).astype(np.float32)).cuda()
        err = torch.from_numpy((0.1 * rng.standard_normal(L * N)).astype(np.float32)).cuda()
        layer = capi.Lstm(P, L, True, S, T)
        out = torch.zeros(L * N, device="cuda"); ex = torch.zeros(P * N, device="cuda"); dW = torch.zeros_like(W)
        layer.load_sequences(pat, T, T)
        layer.forward(W, x, out)
        layer.backward(W, x, out, err.clone(), ex, dW)
        layer.check()
        layers.append(layer); data.append((W, x, err)); alone.append((out.clone(), ex.clone(), dW.clone()))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    got = []
    for k in range(2):
        W, x, err = data[k]
        out = torch.zeros(L * N, device="cuda"); ex = torch.zeros(P * N, device="cuda"); dW = torch.zeros_like(W)
        got.append((out, ex, dW))
    torch.cuda.synchronize()
    for _ in range(3):   # forward and backward recursions of the two layers interleaved on the two streams
        for k in range(2):
            W, x, _ = data[k]
            layers[k].load_sequences(pat, T, T, stream=streams[k])
            layers[k].forward(W, x, got[k][0], stream=streams[k])
        for k in range(2):
            W, x, err = data[k]
            # a bidirectional layer leaves its output errors as they are: the same buffer serves every pass
            layers[k].backward(W, x, got[k][0], err, got[k][1], got[k][2], stream=streams[k])
    torch.cuda.synchronize()
    for k in range(2):
        layers[k].check()
        assert PC.relerr(got[k][0].cpu().numpy(), alone[k][0].cpu().numpy()) < 1e-6
        assert PC.relerr(got[k][1].cpu().numpy(), alone[k][1].cpu().numpy()) < 1e-6
        assert PC.relerr(got[k][2].cpu().numpy(), alone[k][2].cpu().numpy()) < 1e-5
        layers[k].close()


def test_lstm_step_by_step_recursion_equals_the_persistent_kernels(monkeypatch):
    """The two implementations of the recursion on a geometry both cover (clip active, ragged lengths): the handle
    created with CNT_LSTM_STEPWISE set runs step by step."""
    print("lstm stepwise vs persistent", flush=True)
    monkeypatch.setenv("CNT_LSTM_STEPWISE", "1")
    assert PC.run_lstm_case(24, 128, True, [10, 6, 10], seed=5, wscale=0.5, escale=20.0, repeat_backward=True) < TOL
    assert PC.run_lstm_case(30, 256, False, [12, 12, 7], seed=6) < TOL


def test_lstm_config2_layer_full_length_two_recursions():
    """A BLSTM layer of benchmark config 2 at its full size (512 inputs, 256 cells per direction, T=600, S=10,
    lengths drawn from 300..600): the persistent recursion kernels against the step-by-step schedule.  The CPU
    oracle needs two minutes for this fraction, so the full-length check is the agreement of two independent
    implementations, each of which the shorter cases above compare with the oracle."""
    print("lstm config 2 layer, full length, persistent vs stepwise", flush=True)
    import numpy as np

    rng = np.random.default_rng(2)
    lengths = [int(v) for v in rng.integers(300, 601, size=10)]
    lengths[3] = 600
    assert PC.run_lstm_two_recursions(512, 512, True, lengths, seed=12, wscale=0.08) < TOL


def test_lstm_config2_layer_full_length_against_oracle():
    """The same full-size BLSTM layer (512 inputs, 256 cells per direction, T=600, S=10, lengths drawn from
    300..600) against the CPU oracle: outputs, error to the preceding layer, every weight-gradient class and
    every state array, 1e-4 L2-normalised; exact zeros on padding slots.  The oracle shares its outputs out
    over the host's cores for this one (the sums themselves stay sequential)."""
    print("lstm config 2 layer, full length, against the oracle", flush=True)
    import numpy as np

    import oracle_lib as O

    O.use_all_cores()
    rng = np.random.default_rng(2)
    lengths = [int(v) for v in rng.integers(300, 601, size=10)]
    lengths[3] = 600
    assert PC.run_lstm_case(512, 512, True, lengths, seed=12, wscale=0.08) < TOL


def test_lstm_invalid_geometry_is_an_error():
    capi = PC.pkg().capi
    with pytest.raises(RuntimeError):
        capi.Lstm(10, 129, True, 4, 10)      # odd size of a bidirectional layer
    with pytest.raises(RuntimeError):
        capi.Lstm(10, 0, False, 4, 10)


def test_lstm_partial_recursion_rejects_what_it_cannot_do():
    import torch

    capi = PC.pkg().capi
    T, S = 12, 3
    pat = PC.dev(PC.make_pat_types([T] * S, T))
    # 20 cells: step-by-step recursion, which has no partial form
    small = capi.Lstm(8, 20, False, S, T)
    small.load_sequences(pat, T, T)
    assert not small.backward_can_split()
    W = torch.zeros(int(capi.lib().cnt_lstm_weight_count(8, 20, 0)), device="cuda")
    err = torch.zeros(20 * T * S, device="cuda")
    with pytest.raises(RuntimeError, match="cannot run a range"):
        small.backward_errors_range(W, err, 0, 6)
    small.close()
    layer = capi.Lstm(8, 128, True, S, T)
    layer.load_sequences(pat, T, T)
    assert layer.backward_can_split()
    W = torch.zeros(int(capi.lib().cnt_lstm_weight_count(8, 128, 1)), device="cuda")
    err = torch.zeros(128 * T * S, device="cuda")
    ex = torch.zeros(8 * T * S, device="cuda")
    for a, b in ((0, 0), (5, 4), (-1, 3), (0, T + 1)):
        with pytest.raises(RuntimeError, match="steps"):
            layer.backward_errors_range(W, err, a, b)
    with pytest.raises(RuntimeError, match="time steps"):
        layer.backward_prev_errors_range(W, ex, 3, T + 1)
    assert layer.backward_steps_done(0) == (T, T)
    assert layer.backward_steps_done(T) == (0, T)
    assert layer.backward_steps_done(9) == (3, 9)
    assert layer.backward_steps_done(4) == (8, 8)   # nothing final yet in a bidirectional layer
    layer.close()
