"""GPU tests of the C++ network sequencer (cnt_network_*): a network file in the reference's JSON structure is
turned into the layer list, and forward pass, error, backward pass and optimizer step of a fraction are compared
with the CPU oracle doing the same steps.  Tolerance 1e-4 on L2-normalised differences (fp32, different summation
orders), the tolerance of the layer kernels themselves."""
import json

import numpy as np
import pytest

import oracle_lib as O
import oracle_models as OM
import parity_cases as PC
import synth as WD
from torch_models import make_pat_types

pytestmark = pytest.mark.gpu
TOL = 1e-4


def _sections(doc_weights, name, w, n_in, n_bias):
    doc_weights[name] = {"input": w[:n_in].tolist(), "bias": w[n_in:n_in + n_bias].tolist(),
                         "internal": w[n_in + n_bias:].tolist()}


@pytest.mark.parametrize("option,momentum,overlap", [(0, 0.9, True), (5, 0.0, True), (0, 0.0, False)])
def test_stacked_network_trains_like_the_oracle(option, momentum, overlap):
    import torch

    print("network case", option, momentum, overlap, flush=True)
    pkg = PC.pkg()
    capi, networks = pkg.capi, PC.networks()
    P, Q, S = 20, 6, 4
    specs = [{"name": "ff1", "type": "feedforward_tanh", "size": 32, "bias": 1.0},
             {"name": "bl1", "type": "blstm", "size": 128, "bias": 1.0},
             {"name": "l2", "type": "lstm", "size": 64, "bias": 1.0},
             {"name": "out", "type": "feedforward_identity", "size": Q, "bias": 1.0},
             {"name": "postoutput", "type": "sse", "size": Q}]
    weights = OM.init_weights(P, specs, 4, 0.1)
    doc = {"layers": [{"size": P, "name": "input", "type": "input"}] + specs, "weights": {}}
    wi, prev = iter(weights), P
    for sp in specs:
        n_in, n_bias, _ = networks.weight_sections(sp, prev)
        if n_in:
            _sections(doc["weights"], sp["name"], next(wi), n_in, n_bias)
        prev = sp["size"]
    maxT = 30
    net = capi.Network(json.dumps(doc, indent=1), S, maxT, overlap=overlap)
    assert net.input_size == P and net.output_size == Q and net.n_weights == sum(w.size for w in weights)
    assert [L["type"] for L in net.layers] == ["input"] + [s["type"] for s in specs]
    for L, w in zip([L for L in net.layers if L["weight_count"]], weights):
        assert np.array_equal(L["weights"].cpu().numpy(), w)

    rng = np.random.default_rng(6)
    ow = [w.copy() for w in weights]
    deltas = [np.zeros_like(w) for w in ow]
    stats = [np.zeros(2 * w.size, np.float32) for w in ow]
    b1 = b2 = 1.0
    for step, lengths in enumerate(([30, 22, 13, 9], [17, 26, 28, 11], [19, 24, 8, 15])):
        T, Tmin = max(lengths), min(lengths)
        pat = make_pat_types(lengths, T)
        x = rng.standard_normal((T, S, P)).astype(np.float32)
        tgt = (0.3 * rng.standard_normal((T, S, Q))).astype(np.float32)
        valid = (pat != 0).reshape(T, S)
        x[~valid] = 0
        tgt[~valid] = 0
        net.load_sequences(PC.dev(pat), T, Tmin, PC.dev(x.reshape(-1)), PC.dev(tgt.reshape(-1)))
        net.forward()
        loss = float(net.calculate_error().item())
        net.backward()
        ref = OM.OracleNetwork(P, specs, S, T, Tmin, pat, ow)
        ref.forward(x.reshape(-1), tgt.reshape(-1))
        assert abs(loss - ref.error()) <= TOL * max(1.0, abs(ref.error()))
        ref.backward()
        grads = [L["updates"] for L in ref.layers if "updates" in L]
        torch.cuda.synchronize()
        for L, g in zip([L for L in net.layers if L["weight_count"]], grads):
            assert PC.relerr(L["updates"].cpu().numpy(), g) < TOL, (step, L["name"])
        frac = float(sum(lengths))
        net.update(option, 1e-3, momentum, frac)
        if option == 5:
            b1 = O.opt_next_beta_accum(b1, 1)
            b2 = O.opt_next_beta_accum(b2, 2)
        for w, g, d, st in zip(ow, grads, deltas, stats):
            cur = np.empty_like(g)
            O.opt_accumulate(g, cur, False)
            O.opt_adjust_gradient(option, cur, st, None, frac, b1, b2)
            O.opt_update_weights(w, cur, d, None, 1e-3, momentum)
    net.check()
    got = [L["weights"].cpu().numpy() for L in net.layers if L["weight_count"]]
    for g, w, w0 in zip(got, ow, weights):
        assert PC.relerr(g, w) < TOL
        assert PC.relerr(g, w0) > 1e-5  # the weights did move
    # export and re-import: same layers, bit-identical weights
    text = net.export_json()
    back = json.loads(text)
    assert [l["name"] for l in back["layers"]] == ["input"] + [s["name"] for s in specs]
    assert back["layers"][2] == specs[1]
    again = capi.Network(text, S, maxT)
    assert np.array_equal(again.weights.cpu().numpy(), net.weights.cpu().numpy())
    again.close()
    net.close()


def test_weight_gradients_of_a_fraction_that_is_mostly_padding():
    """One long sequence beside seven of a single frame: the weight gradients sum over the valid slots only (a list of them,
    made when the fraction is loaded), a recurrent layer's recurrent weights over the list without the first or the last
    time step, and most splits of the narrow layers' split-K products are left without a single slot."""
    import torch

    print("network case: mostly padding", flush=True)
    capi, networks = PC.pkg().capi, PC.networks()
    P, Q, S, T = 16, 8, 8, 600
    lengths = [T, 1, 1, 1, 1, 1, 1, 1]
    specs = [{"name": "ff1", "type": "feedforward_tanh", "size": 64, "bias": 1.0},
             {"name": "bl1", "type": "blstm", "size": 128, "bias": 1.0},
             {"name": "out", "type": "feedforward_identity", "size": Q, "bias": 1.0},
             {"name": "postoutput", "type": "sse", "size": Q}]
    weights = OM.init_weights(P, specs, 9, 0.1)
    doc = {"layers": [{"size": P, "name": "input", "type": "input"}] + specs, "weights": {}}
    wi, prev = iter(weights), P
    for sp in specs:
        n_in, n_bias, _ = networks.weight_sections(sp, prev)
        if n_in:
            _sections(doc["weights"], sp["name"], next(wi), n_in, n_bias)
        prev = sp["size"]
    net = capi.Network(json.dumps(doc), S, T)
    rng = np.random.default_rng(10)
    # a fraction without padding first: every split of the split-K products leaves its partial sums in the scratch buffer,
    # where a split of the next pass that wrote nothing would let them be counted again
    full = make_pat_types([T] * S, T)
    net.load_sequences(PC.dev(full), T, T, PC.dev(rng.standard_normal(T * S * P).astype(np.float32)),
                       PC.dev(rng.standard_normal(T * S * Q).astype(np.float32)))
    net.forward()
    net.backward()
    pat = make_pat_types(lengths, T)
    x = rng.standard_normal((T, S, P)).astype(np.float32)
    tgt = (0.3 * rng.standard_normal((T, S, Q))).astype(np.float32)
    valid = (pat != 0).reshape(T, S)
    x[~valid] = 0
    tgt[~valid] = 0
    net.load_sequences(PC.dev(pat), T, 1, PC.dev(x.reshape(-1)), PC.dev(tgt.reshape(-1)))
    net.forward()
    net.backward()
    net.check()
    ref = OM.OracleNetwork(P, specs, S, T, 1, pat, [w.copy() for w in weights])
    ref.forward(x.reshape(-1), tgt.reshape(-1))
    ref.backward()
    grads = [L["updates"] for L in ref.layers if "updates" in L]
    torch.cuda.synchronize()
    for L, g in zip([L for L in net.layers if L["weight_count"]], grads):
        assert PC.relerr(L["updates"].cpu().numpy(), g) < TOL, L["name"]
    net.close()


def test_network_reports_a_later_lstm_layer_that_gave_up_and_keeps_the_weights():
    """Failure handling at network level, forced from the host: the SECOND recurrent layer's recursions get a spin
    limit of zero, the first layer's stay as they are.  Every kernel still ends normally; the failure is reported by
    cnt_network_check (which looks at every recurrent layer) or by the call into the network that follows the failed
    launch, the optimizer step of that pass does not touch the weights, and with the bounds restored the same network
    handle trains on."""
    import torch

    print("network give-up case", flush=True)
    capi = PC.pkg().capi
    P, Q, S, T = 16, 5, 6, 40
    specs = [{"name": "bl1", "type": "blstm", "size": 128, "bias": 1.0},
             {"name": "bl2", "type": "blstm", "size": 512, "bias": 1.0},
             {"name": "out", "type": "feedforward_identity", "size": Q, "bias": 1.0},
             {"name": "postoutput", "type": "sse", "size": Q}]
    doc = {"layers": [{"size": P, "name": "input", "type": "input"}] + specs}
    net = capi.Network(json.dumps(doc), S, T)
    rng = np.random.default_rng(8)
    net.weights.copy_(torch.from_numpy(rng.uniform(-0.1, 0.1, net.n_weights).astype(np.float32)))
    pat = torch.full((T * S,), 2, dtype=torch.int8, device="cuda")
    x = PC.dev(rng.standard_normal(T * S * P).astype(np.float32))
    tgt = PC.dev(rng.standard_normal(T * S * Q).astype(np.float32))

    def one_pass():
        net.load_sequences(pat, T, T, x, tgt)
        net.forward()
        net.backward()
        net.update(0, 1e-3, 0.0, float(T * S))
        net.check()

    one_pass()
    torch.cuda.synchronize()
    before = net.weights.clone()
    second = [i for i, L in enumerate(net.layers) if L["type"] == "blstm"][1]
    with pytest.raises(RuntimeError):
        net.set_wait_bounds(0, 0, 0, 0)  # the input layer is not a recurrent layer
    net.set_wait_bounds(second, 0, 0, 0)
    failures = 0
    for _ in range(3):  # an attempt only fails if some poll really comes back incomplete
        try:
            one_pass()
        except RuntimeError as e:
            assert "gave up" in str(e)
            failures += 1
            torch.cuda.synchronize()
            try:
                net.check()  # a second failed launch of the same attempt may have ended meanwhile
            except RuntimeError:
                pass
            # the pass that failed did not reach the weights
            assert torch.equal(net.weights, before)
            break
        before = net.weights.clone()  # a pass in which every poll happened to succeed is an ordinary pass
    assert failures >= 1
    net.set_wait_bounds(second, 1 << 22, 28, 34)
    one_pass()
    torch.cuda.synchronize()
    assert not torch.equal(net.weights, before)
    assert bool(torch.isfinite(net.weights).all())
    net.close()


def test_network_give_up_on_a_nonblocking_stream_keeps_weights_and_adam_state():
    """The same failure, on a stream of the caller's own (non-blocking: nothing orders it against the legacy default
    stream) and without a check between the calls of a pass, with Adam: the failed pass's optimizer step is skipped on the
    device -- weights, moments and the bias-correction products stay where they were -- so that after two good passes
    around the failed one the weights equal those of a twin network that ran only the two good passes."""
    import torch

    print("network give-up on a non-blocking stream, Adam", flush=True)
    capi = PC.pkg().capi
    P, Q, S, T = 16, 5, 6, 40
    specs = [{"name": "bl1", "type": "blstm", "size": 512, "bias": 1.0},
             {"name": "out", "type": "feedforward_identity", "size": Q, "bias": 1.0},
             {"name": "postoutput", "type": "sse", "size": Q}]
    doc = json.dumps({"layers": [{"size": P, "name": "input", "type": "input"}] + specs})
    rng = np.random.default_rng(9)
    w0 = torch.from_numpy(rng.uniform(-0.1, 0.1, 10 ** 7).astype(np.float32))
    pat = torch.full((T * S,), 2, dtype=torch.int8, device="cuda")
    x = PC.dev(rng.standard_normal(T * S * P).astype(np.float32))
    tgt = PC.dev(rng.standard_normal(T * S * Q).astype(np.float32))
    stream = torch.cuda.Stream()

    def make():
        net = capi.Network(doc, S, T)
        net.weights.copy_(w0[:net.n_weights])
        torch.cuda.synchronize()
        return net

    def enqueue_pass(net):
        net.load_sequences(pat, T, T, x, tgt, stream=stream)
        net.forward(stream=stream)
        net.backward(stream=stream)
        net.update(5, 1e-3, 0.0, float(T * S), stream=stream)

    twin = make()
    enqueue_pass(twin); enqueue_pass(twin)
    twin.check(stream=stream)
    net = make()
    enqueue_pass(net)
    net.check(stream=stream)
    before = net.weights.clone()
    layer = [i for i, L in enumerate(net.layers) if L["type"] == "blstm"][0]
    net.set_wait_bounds(layer, 0, 0, 0)
    failed = False
    for _ in range(4):  # an attempt only fails if some poll really comes back incomplete
        try:
            enqueue_pass(net)       # no check in between: whichever call comes after the failed launch reports it
            net.check(stream=stream)
        except RuntimeError as e:
            assert "gave up" in str(e)
            failed = True
            stream.synchronize()
            try:
                net.check(stream=stream)  # the forward recursion of the same attempt may have given up as well
            except RuntimeError:
                pass
            break
        pytest.skip("every poll happened to succeed: nothing to check")
    assert failed
    torch.cuda.synchronize()
    assert torch.equal(net.weights, before)
    net.set_wait_bounds(layer, 1 << 22, 28, 34)
    enqueue_pass(net)
    net.check(stream=stream)
    torch.cuda.synchronize()
    a, b = (net.weights - w0[:net.n_weights].cuda()).cpu().numpy(), (twin.weights - w0[:twin.n_weights].cuda()).cpu().numpy()
    # Adam normalises every step to about the learning rate: a bias correction one step off would change the second
    # step by some 30 %; the sums inside the weight gradients are added in a different order from run to run
    assert PC.relerr(a, b) < 2e-2
    net.close(); twin.close()


# the last case has channel counts that are not multiples of four: no 16-byte accesses anywhere, and the skip layers'
# backward steps run as launches of their own instead of in the epilogue of the following layer's product
# The fifth case is a stack with benchmark config 4's layer sizes (64 residual / 128 skip channels, 80 conditioning
# dimensions up-sampled 80 times) and one full cycle of its dilations, 1 ... 512, over waveforms long enough that
# every dilation reaches valid history and the sequences' ragged ends, against the oracle's graph.
@pytest.mark.parametrize("nb,cnn_tanh,R,K,Q,C,lengths,cycle,upsample", [
    (4, 1, 32, 64, 64, 20, [120, 90], 3, 20), (11, 0, 32, 64, 64, 20, [120, 90], 3, 20),
    (3, 1, 30, 50, 64, 20, [120, 90], 3, 20),
    # the other widths the fused block launch is built for
    (3, 1, 64, 256, 64, 20, [70, 52], 3, 20), (3, 0, 64, 64, 64, 20, [70, 52], 3, 20),
    (3, 1, 32, 128, 64, 20, [70, 52], 3, 20), (3, 0, 32, 32, 64, 20, [70, 52], 3, 20),
    (10, 1, 64, 128, 256, 80, [4000, 3300], 10, 80),
])
def test_wavenet_network_file_against_oracle_graph(nb, cnn_tanh, R, K, Q, C, lengths, cycle, upsample):
    import torch

    print("wavenet network file", nb, cnn_tanh, R, K, Q, C, lengths, cycle, flush=True)
    pkg = PC.pkg()
    capi, networks = pkg.capi, PC.networks()
    O.use_all_cores()
    S, T = len(lengths), max(lengths)
    pat, onehot, ctx, target, N = WD.make(lengths, Q, C, upsample=upsample, seed=2)
    ref = networks.WaveNet(OM.OracleBackend(), nb, S, T, Q=Q, R=R, K=K, C=C, cnn_tanh=cnn_tanh, dilation_cycle=cycle)
    shapes = {k: len(ref.buf[k]["W"]) for k in ref.weight_names()}
    W = WD.init_weights(shapes, seed=3)
    for k, w in W.items():
        ref.buf[k]["W"][:] = w
    ref.set_inputs(pat, onehot, ctx, target)
    ref.forward()
    ref.calculate_error()
    ref.backward()

    doc = PC.pkg().specs.wavenet_network_doc(nb, Q, R, K, C, cnn_tanh, cycle)
    net = capi.Network(json.dumps(doc), S, T + 7, mdn_config=[1, 0, Q, 0, 1, -1])   # buffers longer than the fraction
    names = [L["name"] for L in net.layers if L["weight_count"]]
    assert sorted(names) == sorted(W)
    for L in net.layers:
        if L["weight_count"]:
            assert L["weight_count"] == W[L["name"]].size
            L["weights"].copy_(torch.from_numpy(W[L["name"]]))
    ctx_d = torch.zeros(C * S * (T + 7), dtype=torch.float32, device="cuda")
    ctx_d[: ctx.size].copy_(torch.from_numpy(ctx))
    net.set_context(ctx_d)
    dummy_in = torch.zeros(S * T, dtype=torch.float32, device="cuda")
    for _ in range(2):  # a second pass over the same fraction gives the same result (buffers cleared properly)
        net.load_sequences(PC.dev(pat), T, min(lengths), dummy_in, PC.dev(target))
        net.forward()
        loss = float(net.calculate_error().item())
        net.backward()
        torch.cuda.synchronize()
        ref_loss = float(ref.loss[0])
        assert abs(loss - ref_loss) <= TOL * abs(ref_loss)
        # teacher-forced one-hot input: equal on every valid slot (a padding slot right after a sequence's end holds
        # the one-hot of the last sample, as in the reference, where the oracle's input has zeros)
        fb = net.layer("feedbackBottom")["outputs"][: N * Q].cpu().numpy().reshape(N, Q)
        valid = pat != 0
        assert np.array_equal(fb[valid], onehot.reshape(N, Q)[valid])
        worst = 0.0
        for L in net.layers:
            if L["weight_count"]:
                e = PC.relerr(L["updates"].cpu().numpy(), ref.buf[L["name"]]["dW"])
                worst = max(worst, e)
                if e > TOL:
                    print("   ", L["name"], e, flush=True)
        assert worst < TOL
    # the comparison above was made on the path it is meant for: one launch per residual block where the library has
    # a block kernel for the widths (and layer by layer for the others), the block above folded in from the second on
    net.forward()
    capi.profile_enable(True)
    net.backward()
    torch.cuda.synchronize()
    launches = {k: n for k, (n, _) in capi.profile_read().items()}
    capi.profile_enable(False)
    if (R, K) in [(64, 128), (64, 256), (64, 64), (32, 128), (32, 64), (32, 32)]:
        assert launches.get("wavenet_block_errors") == 1 and launches.get("wavenet_block_errors+cnn") == nb - 1, launches
    else:
        assert "wavenet_block_errors" not in launches and "wavenet_block_errors+cnn" not in launches, launches
    net.update(0, 1e-4, 0.0, float(sum(lengths)))
    torch.cuda.synchronize()
    moved = net.layer("cnn0")["weights"].cpu().numpy()
    assert PC.relerr(moved, W["cnn0"] - 1e-4 * ref.buf["cnn0"]["dW"]) < TOL
    net.close()


def test_network_file_rejections():
    capi = PC.pkg().capi

    def make(layers, weights=None):
        doc = {"layers": layers}
        if weights is not None:
            doc["weights"] = weights
        return json.dumps(doc)

    inp = {"size": 3, "name": "input", "type": "input"}
    post = {"size": 4, "name": "post", "type": "sse"}
    with pytest.raises(RuntimeError, match="does not cover"):
        capi.Network(make([inp, {"size": 4, "name": "c", "type": "maxpooling", "bias": 1.0}, post]), 2, 10)
    with pytest.raises(RuntimeError, match="expected 12"):
        capi.Network(make([inp, {"size": 4, "name": "o", "type": "feedforward_identity", "bias": 1.0}, post],
                          {"o": {"input": [0.0] * 11, "bias": [0.0] * 4, "internal": []}}), 2, 10)
    with pytest.raises(RuntimeError, match="Missing value 'bias'|missing value 'bias'"):
        capi.Network(make([inp, {"size": 4, "name": "o", "type": "feedforward_identity"}, post]), 2, 10)
    with pytest.raises(RuntimeError, match="post-output"):
        capi.Network(make([inp, {"size": 4, "name": "o", "type": "feedforward_identity", "bias": 1.0},
                           {"size": 4, "name": "o2", "type": "feedforward_identity", "bias": 1.0}]), 2, 10)
    with pytest.raises(RuntimeError, match="linked to"):
        capi.Network(make([inp, {"size": 4, "name": "o", "type": "feedforward_identity", "bias": 1.0},
                           {"size": 5, "name": "s", "type": "skipini", "bias": 1.0}, post]), 2, 10)
    with pytest.raises(RuntimeError, match="resolution"):
        capi.Network(make([inp, {"size": 4, "name": "o", "type": "feedforward_identity", "bias": 1.0, "resolution": 80},
                           post]), 2, 10)
    net = capi.Network(make([inp, {"size": 4, "name": "o", "type": "feedforward_identity", "bias": 1.0}, post]), 2, 10)
    with pytest.raises(RuntimeError, match="no fraction"):
        net.forward()
    net.close()


def test_layer_specific_learning_rate():
    """A layer's own "learningRate" replaces the optimizer's for that layer (0 freezes it)."""
    import torch

    capi = PC.pkg().capi
    doc = {"layers": [{"size": 3, "name": "input", "type": "input"},
                      {"size": 5, "name": "frozen", "type": "feedforward_tanh", "bias": 1.0, "learningRate": 0.0},
                      {"size": 4, "name": "fast", "type": "feedforward_identity", "bias": 1.0, "learningRate": 0.5},
                      {"size": 4, "name": "plain", "type": "feedforward_identity", "bias": 1.0},
                      {"size": 4, "name": "post", "type": "sse"}]}
    S, T = 2, 6
    net = capi.Network(json.dumps(doc), S, T)
    net.randomize(3, 0.3)
    w0 = net.weights.clone()
    rng = np.random.default_rng(2)
    pat = make_pat_types([T, T], T)
    net.load_sequences(PC.dev(pat), T, T, PC.dev(rng.standard_normal(3 * S * T).astype(np.float32)),
                       PC.dev(rng.standard_normal(4 * S * T).astype(np.float32)))
    net.forward()
    net.backward()
    net.update(0, 0.01, 0.0, float(S * T))
    torch.cuda.synchronize()
    g = net.updates
    for name, lr in (("frozen", 0.0), ("fast", 0.5), ("plain", 0.01)):
        L = net.layer(name)
        a, b = L["weight_offset"], L["weight_offset"] + L["weight_count"]
        assert torch.allclose(net.weights[a:b], w0[a:b] - lr * g[a:b], rtol=1e-6, atol=1e-7), name
    net.close()


class _CondOracleBackend(OM.OracleBackend):
    """Oracle back end whose gated layers also accumulate the gradient with respect to the conditioning features."""
    ctx_grad = None

    def wavnetc_backward(self, D, C, N, pat, W, ctx, core, cth, err, prev_err, dW):
        O.wavnetc_backward(D, C, N, pat, W, ctx, core, cth, err, prev_err, dW, self.ctx_grad)


@pytest.mark.parametrize("context_mv", [False, True])
def test_wavenet_with_frame_rate_conditioning_network(context_mv, tmp_path):
    """The reference example's layout in full: externalloader -> skipini -> blstm -> cnn -> skipcat at one slot per
    R time steps, flagged as the wavnetc layers' input; the oracle side walks the same graph with the oracle's
    primitives (conditioning part spelled out here, sample-rate part by the shared graph walk).  With context_mv the
    wavnetc layers name a "contextMV" file (means and standard deviations of the conditioning features, one of them
    vanishing), which the first of them applies while it up-samples (layers/wavNetCore.cu:143-190, :322-351)."""
    import torch

    print("wavenet network file with conditioning sub-network, contextMV", context_mv, flush=True)
    pkg = PC.pkg()
    capi, networks = pkg.capi, PC.networks()
    nb, Q, R, K = 3, 64, 32, 64
    E, HB, DC, C, RES = 12, 128, 10, 11, 4
    lengths = [120, 90]
    S, T = len(lengths), max(lengths)
    Tr = -(-T // RES)
    lengths_r = [-(-n // RES) for n in lengths]
    pat, onehot, _, target, N = WD.make(lengths, Q, C, upsample=RES, seed=2)
    pat_r = make_pat_types(lengths_r, Tr)
    Nr = S * Tr
    rng = np.random.default_rng(11)
    frame_index = np.zeros((T, S), dtype=np.float32)
    for s, n in enumerate(lengths):
        frame_index[:n, s] = np.arange(n) // RES
    data = rng.standard_normal((Tr, S, E)).astype(np.float32)
    mean_std = np.concatenate([0.1 * rng.standard_normal(E), rng.uniform(0.5, 2.0, E)]).astype(np.float32)
    mean_std[E + 3] = 1e-7   # a vanishing deviation counts as 1

    # ---- oracle: conditioning part -----------------------------------------------------------------------------
    valid_r = (pat_r != 0)
    sd = np.where(mean_std[E:] < 1e-5, 1.0, mean_std[E:])
    ext = ((data - mean_std[:E]) / sd).astype(np.float32).reshape(Nr, E)
    ext[~valid_r] = 0
    ext = np.ascontiguousarray(ext.reshape(-1))
    w_lstm = rng.uniform(-0.1, 0.1, OM.weight_count({"type": "blstm", "size": HB}, E)).astype(np.float32)
    hw, it = np.ones(DC, dtype=np.int32), np.ones(DC, dtype=np.int32)
    w_cnn = rng.uniform(-0.1, 0.1, HB * 3 * DC + DC).astype(np.float32)
    desc = O.LstmDesc(E, HB, 1, S, Tr, min(lengths_r), 1.0)
    fw, bw = O.LstmState(HB // 2, Nr), O.LstmState(HB // 2, Nr)
    l2 = np.zeros(HB * Nr, dtype=np.float32)
    O.lstm_forward(desc, w_lstm, pat_r, ext, fw, bw, l2)
    l3 = np.zeros(DC * Nr, dtype=np.float32)
    con = np.zeros(3 * DC * Nr, dtype=np.float32)
    O.cnn_forward(HB, DC, S, Tr, 0, 0, 1.0, hw, it, pat_r, w_cnn, l2, con, l3)
    cat = np.concatenate([l3.reshape(Nr, DC), ext.reshape(Nr, E)[:, 11:12]], axis=1).astype(np.float32)
    ctx = np.zeros(C * N, dtype=np.float32)
    ctx_mv = None
    if context_mv:
        ctx_mv = np.concatenate([0.2 * rng.standard_normal(C), rng.uniform(0.4, 1.5, C)]).astype(np.float32)
        ctx_mv[C + 2] = 1e-6   # a vanishing deviation counts as 1
        ctx_mv.tofile(tmp_path / "context.mv")
    O.wavnetc_load_context(C, S, N, Tr, False, np.ascontiguousarray(cat.reshape(-1)), frame_index.reshape(-1), ctx_mv, pat, ctx)

    # ---- oracle: sample-rate part --------------------------------------------------------------------------------
    backend = _CondOracleBackend()
    backend.ctx_grad = np.zeros(C * N, dtype=np.float32)
    ref = networks.WaveNet(backend, nb, S, T, Q=Q, R=R, K=K, C=C, cnn_tanh=1, dilation_cycle=3)
    W = WD.init_weights({k: len(ref.buf[k]["W"]) for k in ref.weight_names()}, seed=3)
    for k, w in W.items():
        ref.buf[k]["W"][:] = w
    ref.set_inputs(pat, onehot, ctx, target)
    ref.forward()
    ref.calculate_error()
    ref.backward()
    cat_err = np.zeros(C * Nr, dtype=np.float32)
    O.wavnetc_sum_context_grad(C, S, RES, Nr, N, pat_r, pat, backend.ctx_grad, cat_err)
    cat_err = cat_err.reshape(Nr, C)
    l3_err = np.zeros((Nr, DC), dtype=np.float32)
    l3_err[valid_r] = cat_err[valid_r, :DC]
    l3_err = np.ascontiguousarray(l3_err.reshape(-1))
    l2_err = np.zeros(HB * Nr, dtype=np.float32)
    dw_cnn = np.zeros_like(w_cnn)
    O.cnn_backward(HB, DC, S, Tr, 0, 0, 1.0, hw, it, pat_r, w_cnn, l2, l3, l3_err, con, l2_err, dw_cnn)
    skip_err = np.zeros(E * Nr, dtype=np.float32)
    dw_lstm = np.zeros_like(w_lstm)
    O.lstm_backward(desc, w_lstm, pat_r, ext, l2_err, fw, bw, skip_err, dw_lstm)
    W["exL2"], W["exL3"] = w_lstm, w_cnn
    dW_ref = {k: ref.buf[k]["dW"] for k in ref.weight_names()}
    dW_ref["exL2"], dW_ref["exL3"] = dw_lstm, dw_cnn

    # ---- the library, from the network file ---------------------------------------------------------------------
    doc = PC.pkg().specs.wavenet_network_doc(nb, Q, R, K, C, 1, 3)
    cond = [{"size": E, "name": "exL1", "type": "externalloader", "bias": 1.0, "resolution": RES},
            {"size": E, "name": "exSkip", "bias": 1.0, "type": "skipini", "resolution": RES},
            {"size": HB, "name": "exL2", "bias": 1.0, "type": "blstm", "resolution": RES},
            {"size": DC, "name": "exL3", "bias": 1.0, "type": "cnn", "window_width": "%d*1" % DC,
             "window_tap_interval": "%d*1" % DC, "tanhoutput": 0, "resolution": RES},
            {"size": C, "name": "exAdd", "bias": 1.0, "type": "skipcat", "resolution": RES,
             "preSkipLayer": "exL3,exSkip", "preSkipLayerDim": "0_%d_11_12" % DC,
             "layerFlag": "wavenetConditionInputLayer"}]
    doc["layers"] = doc["layers"][:1] + cond + doc["layers"][1:]
    if context_mv:
        for layer in doc["layers"]:
            if layer["type"] == "wavnetc":
                layer["contextMV"] = str(tmp_path / "context.mv")
        bad = json.loads(json.dumps(doc))
        (tmp_path / "short.mv").write_bytes(ctx_mv[:-1].tobytes())
        [l for l in bad["layers"] if l["type"] == "wavnetc"][1]["contextMV"] = str(tmp_path / "short.mv")
        with pytest.raises(RuntimeError, match="mean variance dim unequal"):
            capi.Network(json.dumps(bad), S, T + 6, mdn_config=[1, 0, Q, 0, 1, -1])
    net = capi.Network(json.dumps(doc), S, T + 6, mdn_config=[1, 0, Q, 0, 1, -1])
    assert net.layer("exL2")["resolution"] == RES and net.layer("emb")["resolution"] == 1
    for L in net.layers:
        if L["weight_count"]:
            assert L["weight_count"] == W[L["name"]].size, L["name"]
            L["weights"].copy_(torch.from_numpy(W[L["name"]]))
    net.set_external_input("exL1", PC.dev(data.reshape(-1)), Tr, PC.dev(mean_std))
    with pytest.raises(RuntimeError, match="computes the conditioning features itself"):
        net.set_context(PC.dev(ctx))
    for _ in range(2):
        net.load_sequences(PC.dev(pat), T, min(lengths), PC.dev(frame_index.reshape(-1)), PC.dev(target))
        net.forward()
        loss = float(net.calculate_error().item())
        net.backward()
        net.check()
        torch.cuda.synchronize()
        assert PC.relerr(net.layer("exL1")["outputs"][: ext.size].cpu().numpy(), ext) < 1e-6
        assert PC.relerr(net.layer("exAdd")["outputs"][: cat.size].cpu().numpy(), cat.reshape(-1)) < TOL
        ref_loss = float(ref.loss[0])
        assert abs(loss - ref_loss) <= TOL * abs(ref_loss)
        assert PC.relerr(net.layer("exAdd")["errors"][: cat_err.size].cpu().numpy(), cat_err.reshape(-1)) < TOL
        worst = 0.0
        for L in net.layers:
            if L["weight_count"]:
                e = PC.relerr(L["updates"].cpu().numpy(), dW_ref[L["name"]])
                worst = max(worst, e)
                if e > TOL:
                    print("   ", L["name"], e, flush=True)
        assert worst < TOL
    net.close()


def test_full_size_acoustic_backward_is_affine_in_the_targets():
    """benchmark configs[1] at its real size (T = 600, S = 10, 382-512-512-blstm512-blstm512-187), where the oracle
    would take minutes: with the forward state fixed, the SSE error is y - target and every later step of the
    backward pass is linear in it as long as no LSTM delta reaches the clipping bound, so
    dW(t1) + dW(t2) = dW(t1 + t2) + dW(0) for every weight tensor.  A wrong accumulation, a stale buffer (the stored
    output-gate deltas are read-modify-write) or a race between the streams breaks it."""
    import torch

    print("full-size acoustic linearity", flush=True)
    pkg = PC.pkg()
    capi, networks = pkg.capi, PC.networks()
    S, Tmax = 10, 600
    input_size, specs = PC.pkg().specs.acoustic_model_spec()
    rng = np.random.default_rng(77)
    lengths = [int(v) for v in rng.integers(300, Tmax + 1, size=S)]
    T = max(lengths)
    pat = make_pat_types(lengths, T)
    valid = (pat != 0).reshape(T, S)
    x = rng.standard_normal((T, S, input_size)).astype(np.float32)
    x[~valid] = 0
    layers = [{"size": input_size, "name": "input", "type": "input"}]
    layers += [dict(sp, name="l%d" % i) for i, sp in enumerate(specs)]
    net = capi.Network(json.dumps({"layers": layers}), S, Tmax)
    net.randomize(5, 0.08)
    pat_d, x_d = PC.dev(pat), PC.dev(x.reshape(-1))

    def grads(target):
        tgt = target.copy()
        tgt[~valid] = 0
        net.load_sequences(pat_d, T, min(lengths), x_d, PC.dev(tgt.reshape(-1)))
        net.forward()
        net.backward()
        net.check()
        torch.cuda.synchronize()
        return net.updates.clone()

    t1 = (0.05 * rng.standard_normal((T, S, 187))).astype(np.float32)
    t2 = (0.05 * rng.standard_normal((T, S, 187))).astype(np.float32)
    g1, g2, g12, g0 = grads(t1), grads(t2), grads(t1 + t2), grads(np.zeros_like(t1))
    assert float(g1.abs().max()) > 0
    for L in net.layers:
        if not L["weight_count"]:
            continue
        a, b = L["weight_offset"], L["weight_offset"] + L["weight_count"]
        lhs = (g1[a:b] + g2[a:b]).cpu().numpy()
        rhs = (g12[a:b] + g0[a:b]).cpu().numpy()
        assert PC.relerr(lhs, rhs) < TOL, L["name"]
    net.close()


def test_full_size_wavenet_sequencer_matches_layer_by_layer_walk():
    """benchmark configs[3] at its real size (30 blocks, 2 x 16000 samples, 1024 classes): the sequencer (shared sums,
    aliased buffers, fan-in / fan-out tables, side streams, fused delta) against the plain layer-by-layer walk over
    the same kernels, which the shortened-stack tests tie to the oracle.  Loss equal to 1e-6, every weight gradient
    to the tolerance of the split-K atomics' summation order."""
    import torch

    print("full-size wavenet sequencer vs walk", flush=True)
    pkg = PC.pkg()
    capi, networks = pkg.capi, PC.networks()
    nb, Q, R, K, C = 30, 1024, 64, 128, 80
    lengths = [16000, 15000]
    S, T = 2, 16000
    pat, onehot, ctx, target, N = WD.make(lengths, Q, C, upsample=80, seed=4)
    walk = networks.WaveNet(networks.HipBackend(), nb, S, T, Q=Q, R=R, K=K, C=C, cnn_tanh=1)
    W = WD.init_weights({k: len(walk.buf[k]["W"]) for k in walk.weight_names()}, seed=5)
    for k, w in W.items():
        walk.buf[k]["W"].copy_(torch.from_numpy(w))
    pat_d, ctx_d, tgt_d = PC.dev(pat), PC.dev(ctx), PC.dev(target)
    walk.set_inputs(pat_d, PC.dev(onehot), ctx_d, tgt_d)
    walk.forward()
    walk.calculate_error()
    walk.backward()
    net = capi.Network(json.dumps(PC.pkg().specs.wavenet_network_doc(nb, Q, R, K, C, 1, 10)), S, T, mdn_config=[1, 0, Q, 0, 1, -1])
    for L in net.layers:
        if L["weight_count"]:
            L["weights"].copy_(torch.from_numpy(W[L["name"]]))
    net.set_context(ctx_d)
    net.load_sequences(pat_d, T, min(lengths), torch.zeros(N, dtype=torch.float32, device="cuda"), tgt_d)
    net.forward()
    loss = float(net.calculate_error().item())
    net.backward()
    torch.cuda.synchronize()
    ref_loss = float(walk.loss.item())
    assert abs(loss - ref_loss) <= 1e-6 * abs(ref_loss)
    for L in net.layers:
        if L["weight_count"]:
            assert PC.relerr(L["updates"].cpu().numpy(), walk.buf[L["name"]]["dW"].cpu().numpy()) < TOL, L["name"]
    walk.close()
    net.close()


def test_gatedact_layer_and_dft_post_output_in_a_network_file():
    """Two more layer types of the reference's registry through the sequencer: `gatedact` inside a small stack with
    an sse output, and a `dft` post-output layer (two resolutions, spectral distance type 1, phase term) after a
    stack that produces a waveform -- each against the oracle's primitives."""
    import torch

    print("gatedact and dft layers in network files", flush=True)
    capi = PC.pkg().capi
    rng = np.random.default_rng(21)

    # ---- gatedact ------------------------------------------------------------------------------------------------
    P, D, Q, lengths = 6, 8, 5, [20, 13, 17]
    S, T = len(lengths), max(lengths)
    N = S * T
    pat = make_pat_types(lengths, T)
    valid = pat != 0
    x = rng.standard_normal((N, P)).astype(np.float32); x[~valid] = 0
    tgt = rng.standard_normal((N, Q)).astype(np.float32); tgt[~valid] = 0
    w1 = rng.uniform(-0.5, 0.5, P * 2 * D + 2 * D).astype(np.float32)
    w2 = rng.uniform(-0.5, 0.5, D * Q + Q).astype(np.float32)
    h1, g, y = np.zeros(2 * D * N, np.float32), np.zeros(D * N, np.float32), np.zeros(Q * N, np.float32)
    O.dense_forward(P, 2 * D, N, 0, 1.0, w1, x.reshape(-1), h1)
    O.gated_forward(D, N, pat, h1, g)
    O.dense_forward(D, Q, N, 1, 1.0, w2, g, y)
    ref_loss = O.sse_error(Q, N, pat, y, tgt.reshape(-1))
    ey, eg, eh1 = np.zeros(Q * N, np.float32), np.zeros(D * N, np.float32), np.zeros(2 * D * N, np.float32)
    dw1, dw2 = np.zeros_like(w1), np.zeros_like(w2)
    O.sse_backward(Q, N, pat, y, tgt.reshape(-1), ey)
    O.dense_backward(D, Q, N, 1, 1.0, w2, g, y, ey, eg, dw2)
    O.gated_backward(D, N, pat, h1, eg, eh1)
    O.dense_backward(P, 2 * D, N, 0, 1.0, w1, x.reshape(-1), h1, eh1, None, dw1)
    doc = {"layers": [{"size": P, "name": "input", "type": "input"},
                      {"size": 2 * D, "name": "pre", "type": "feedforward_identity", "bias": 1.0},
                      {"size": D, "name": "gate", "type": "gatedact", "bias": 1.0},
                      {"size": Q, "name": "out", "type": "feedforward_tanh", "bias": 1.0},
                      {"size": Q, "name": "post", "type": "sse"}]}
    net = capi.Network(json.dumps(doc), S, T)
    net.layer("pre")["weights"].copy_(torch.from_numpy(w1))
    net.layer("out")["weights"].copy_(torch.from_numpy(w2))
    net.load_sequences(PC.dev(pat), T, min(lengths), PC.dev(x.reshape(-1)), PC.dev(tgt.reshape(-1)))
    net.forward()
    loss = float(net.calculate_error().item())
    net.backward()
    torch.cuda.synchronize()
    assert abs(loss - ref_loss) <= TOL * abs(ref_loss)
    assert PC.relerr(net.layer("gate")["outputs"][: g.size].cpu().numpy(), g) < TOL
    assert PC.relerr(net.layer("pre")["updates"].cpu().numpy(), dw1) < TOL
    assert PC.relerr(net.layer("out")["updates"].cpu().numpy(), dw2) < TOL
    net.close()

    # ---- dft -------------------------------------------------------------------------------------------------------
    P, Hd, T, maxT = 4, 16, 900, 1000
    pat = make_pat_types([T], T)
    x = rng.standard_normal((T, P)).astype(np.float32)
    tgt = (0.3 * rng.standard_normal(T)).astype(np.float32)
    w1 = rng.uniform(-0.5, 0.5, P * Hd + Hd).astype(np.float32)
    w2 = rng.uniform(-0.5, 0.5, Hd + 1).astype(np.float32)
    h1, y = np.zeros(Hd * T, np.float32), np.zeros(T, np.float32)
    O.dense_forward(P, Hd, T, 1, 1.0, w1, x.reshape(-1), h1)
    O.dense_forward(Hd, 1, T, 0, 1.0, w2, h1, y)
    res = [(128, 100, 25), (64, 64, 16)]
    gamma, zeta, dis, beta = 0.7, 0.4, 1, 0.3
    src = np.zeros(maxT, np.float32); src[:T] = y
    tg = np.zeros(maxT, np.float32); tg[:T] = tgt
    ey, ref_loss = np.zeros(maxT, np.float64), 0.0
    for (Nf, Nw, Hs) in res:
        gbuf = np.zeros(maxT, np.float32)
        ref_loss += O.dft_spectral_loss(dis, Nf, Nw, Hs, 0, maxT, T, gamma, 1e-5, src.copy(), tg.copy(), gbuf)
        gbuf[T:] = 0
        ey += gbuf
        ref_loss += O.dft_phase_loss(Nf, Nw, Hs, 0, maxT, T, zeta, src.copy(), tg.copy(), gbuf)
        gbuf[T:] = 0
        ey += gbuf
    ey = (ey[:T] + beta * (y.astype(np.float64) - tgt)).astype(np.float32)   # waveform MSE term: gradient only
    eh1, dw1, dw2 = np.zeros(Hd * T, np.float32), np.zeros_like(w1), np.zeros_like(w2)
    O.dense_backward(Hd, 1, T, 0, 1.0, w2, h1, y, ey, eh1, dw2)
    O.dense_backward(P, Hd, T, 1, 1.0, w1, x.reshape(-1), h1, eh1, None, dw1)
    doc = {"layers": [{"size": P, "name": "input", "type": "input"},
                      {"size": Hd, "name": "h", "type": "feedforward_tanh", "bias": 1.0},
                      {"size": 1, "name": "wave", "type": "feedforward_identity", "bias": 1.0},
                      {"size": 1, "name": "post", "type": "dft", "gamma": gamma, "zeta": zeta, "specDisType": dis, "beta": beta,
                       "fftLength": 128, "frameLength": 100, "frameShift": 25,
                       "fftLength2": 64, "frameLength2": 64, "frameShift2": 16}]}
    net = capi.Network(json.dumps(doc), 1, maxT)
    net.layer("h")["weights"].copy_(torch.from_numpy(w1))
    net.layer("wave")["weights"].copy_(torch.from_numpy(w2))
    for _ in range(2):
        net.load_sequences(PC.dev(pat), T, T, PC.dev(x.reshape(-1)), PC.dev(tgt))
        net.forward()
        loss = float(net.calculate_error().item())
        net.backward()
        torch.cuda.synchronize()
        assert abs(loss - ref_loss) <= TOL * abs(ref_loss)
        assert PC.relerr(net.layer("wave")["errors"][:T].cpu().numpy(), ey) < TOL
        assert PC.relerr(net.layer("h")["updates"].cpu().numpy(), dw1) < TOL
        assert PC.relerr(net.layer("wave")["updates"].cpu().numpy(), dw2) < TOL
    net.close()
    with pytest.raises(RuntimeError, match="parallel_sequences = 1"):
        capi.Network(json.dumps(doc), 2, maxT)
    doc["layers"][-1]["kappa"] = 1.0
    with pytest.raises(RuntimeError, match="'kappa' term"):
        capi.Network(json.dumps(doc), 1, maxT)


def test_mixture_density_network_file():
    """benchmark config 3's layout in small: ... -> feedforward_identity -> mdn with one untied-variance mixture unit
    (mdn config [1, 0, Lp, 0, D, M]); loss, the error handed to the output layer and the weight gradients against
    the oracle."""
    import torch

    print("mixture density network file", flush=True)
    capi = PC.pkg().capi
    rng = np.random.default_rng(31)
    P, Hd, M, D = 5, 8, 4, 3
    Lp = M + 2 * M * D
    lengths = [14, 9, 14, 11]
    S, T = len(lengths), max(lengths)
    N = S * T
    pat = make_pat_types(lengths, T)
    valid = pat != 0
    x = rng.standard_normal((N, P)).astype(np.float32); x[~valid] = 0
    tgt = rng.standard_normal((N, D)).astype(np.float32); tgt[~valid] = 0
    w1 = rng.uniform(-0.5, 0.5, P * Hd + Hd).astype(np.float32)
    w2 = rng.uniform(-0.5, 0.5, Hd * Lp + Lp).astype(np.float32)
    h1, y = np.zeros(Hd * N, np.float32), np.zeros(Lp * N, np.float32)
    O.dense_forward(P, Hd, N, 1, 1.0, w1, x.reshape(-1), h1)
    O.dense_forward(Hd, Lp, N, 0, 1.0, w2, h1, y)
    para, tmp = np.zeros(N * M * (1 + 2 * D), np.float32), np.zeros(N * M + N, np.float32)
    O.mdn_mixture_forward(N, Lp, 0, M, D, 0.0, pat, y, para)
    ref_loss = O.mdn_mixture_error(N, D, 0, M, D, pat, tgt.reshape(-1), para, tmp)
    ey = np.zeros(Lp * N, np.float32)
    O.mdn_mixture_backward(N, Lp, D, 0, 0, M, D, 0.0, pat, tgt.reshape(-1), para, tmp, ey)
    eh1, dw1, dw2 = np.zeros(Hd * N, np.float32), np.zeros_like(w1), np.zeros_like(w2)
    O.dense_backward(Hd, Lp, N, 0, 1.0, w2, h1, y, ey.copy(), eh1, dw2)
    O.dense_backward(P, Hd, N, 1, 1.0, w1, x.reshape(-1), h1, eh1, None, dw1)
    doc = {"layers": [{"size": P, "name": "input", "type": "input"},
                      {"size": Hd, "name": "h", "type": "feedforward_tanh", "bias": 1.0},
                      {"size": Lp, "name": "out", "type": "feedforward_identity", "bias": 1.0},
                      {"size": D, "name": "post", "type": "mdn"}]}
    net = capi.Network(json.dumps(doc), S, T + 3, mdn_config=[1, 0, Lp, 0, D, M])
    net.layer("h")["weights"].copy_(torch.from_numpy(w1))
    net.layer("out")["weights"].copy_(torch.from_numpy(w2))
    net.load_sequences(PC.dev(pat), T, min(lengths), PC.dev(x.reshape(-1)), PC.dev(tgt.reshape(-1)))
    net.forward()
    loss = float(net.calculate_error().item())
    net.backward()
    torch.cuda.synchronize()
    assert abs(loss - ref_loss) <= TOL * abs(ref_loss)
    assert PC.relerr(net.layer("out")["errors"][: ey.size].cpu().numpy(), ey) < TOL
    assert PC.relerr(net.layer("h")["updates"].cpu().numpy(), dw1) < TOL
    assert PC.relerr(net.layer("out")["updates"].cpu().numpy(), dw2) < TOL
    net.close()
    with pytest.raises(RuntimeError, match="mdn config"):
        capi.Network(json.dumps(doc), S, T)
