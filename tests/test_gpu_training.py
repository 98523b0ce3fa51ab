"""GPU test of the whole "train one fraction" path through the C ABI: network JSON -> layers, .nc file -> fractions,
forward / error / backward, fused optimizer step -- against the CPU oracle doing the same steps.
Tolerance: 1e-4 on the L2-normalised difference of every weight vector after three updates (fp32, different
summation order in the gradients), the tolerance of the backward pass itself."""
import json
import os

import numpy as np
import pytest
from scipy.io import netcdf_file

import oracle_lib as O
import oracle_models as OM
import parity_cases as PC

pytestmark = pytest.mark.gpu
TOL = 1e-4


def _write_data(path, lengths, P, Q, seed):
    rng = np.random.default_rng(seed)
    total = int(sum(lengths))
    f = netcdf_file(path, "w", version=2)
    for name, n in (("numSeqs", len(lengths)), ("numTimesteps", total), ("inputPattSize", P), ("targetPattSize", Q), ("maxSeqTagLength", 8)):
        f.createDimension(name, n)
    tags = f.createVariable("seqTags", "c", ("numSeqs", "maxSeqTagLength"))
    for i in range(len(lengths)):
        tags[i] = np.frombuffer(("s%02d" % i).encode().ljust(8, b"\0"), dtype="S1")
    f.createVariable("seqLengths", "i", ("numSeqs",))[:] = np.asarray(lengths, np.int32)
    f.createVariable("inputs", "f", ("numTimesteps", "inputPattSize"))[:] = rng.standard_normal((total, P)).astype(np.float32)
    f.createVariable("targetPatterns", "f", ("numTimesteps", "targetPattSize"))[:] = (0.3 * rng.standard_normal((total, Q))).astype(np.float32)
    f.close()


@pytest.mark.parametrize("option,momentum", [(0, 0.9), (5, 0.0)])
def test_train_fractions_from_json_and_nc(tmp_path, option, momentum):
    import torch

    print("training case", option, momentum, flush=True)
    pkg = PC.pkg()
    capi, networks = pkg.capi, PC.networks()
    P, Q, S = 20, 6, 4
    specs = [{"name": "ff1", "type": "feedforward_tanh", "size": 32, "bias": 1.0},
             {"name": "bl1", "type": "blstm", "size": 128, "bias": 1.0},
             {"name": "out", "type": "feedforward_identity", "size": Q, "bias": 1.0},
             {"name": "postoutput", "type": "sse", "size": Q}]
    weights = OM.init_weights(P, specs, 4, 0.1)
    # network file in the reference's structure
    jpath = str(tmp_path / "network.jsn")
    doc = {"layers": [{"size": P, "name": "input", "type": "input"}] + specs, "weights": {}}
    wi, prev = iter(weights), P
    for sp in specs:
        n_in, n_bias, n_int = networks.weight_sections(sp, prev)
        if n_in:
            w = next(wi)
            doc["weights"][sp["name"]] = {"input": w[:n_in].tolist(), "bias": w[n_in:n_in + n_bias].tolist(),
                                          "internal": w[n_in + n_bias:].tolist()}
        prev = sp["size"]
    json.dump(doc, open(jpath, "w"))
    dpath = str(tmp_path / "train.nc")
    lengths = [13, 30, 22, 9, 17, 26, 30, 11, 19, 24, 8, 15]
    _write_data(dpath, lengths, P, Q, 5)

    in_size, jspecs, jweights = networks.load_network_json(jpath)
    assert in_size == P and [s["type"] for s in jspecs] == [s["type"] for s in specs]
    for a, b in zip(jweights, weights):
        assert np.array_equal(a, b)
    ds = capi.Dataset(dpath, S, True, 0, 1.0)
    net = networks.StackedNetwork(in_size, jspecs, S, ds.max_len)
    net.set_weights(jweights)
    trainer = networks.Trainer(net, 1e-3, momentum, option)

    # the oracle does the same three steps
    ow = [w.copy() for w in weights]
    deltas = [np.zeros_like(w) for w in ow]
    stats = [np.zeros(2 * w.size, np.float32) for w in ow]
    b1 = b2 = 1.0
    losses, ref_losses = [], []
    for first in range(0, 3 * S, S):
        fr = ds.fraction(first)
        losses.append(float(trainer.train_fraction(fr).item()))
        ref = OM.OracleNetwork(P, specs, S, fr["max_len"], fr["min_len"], fr["patTypes"], ow)
        ref.forward(fr["inputs"], fr["targets"])
        ref_losses.append(ref.error())
        ref.backward()
        if option == 5:
            b1 = O.opt_next_beta_accum(b1, 1); b2 = O.opt_next_beta_accum(b2, 2)
        grads = [L["updates"] for L in ref.layers if "updates" in L]
        for w, g, d, st in zip(ow, grads, deltas, stats):
            cur = np.empty_like(g)
            O.opt_accumulate(g, cur, False)
            O.opt_adjust_gradient(option, cur, st, None, float(fr["total_length"]), b1, b2)
            O.opt_update_weights(w, cur, d, None, 1e-3, momentum)
    net.check()
    torch.cuda.synchronize()
    for a, b in zip(losses, ref_losses):
        assert abs(a - b) <= TOL * max(1.0, abs(b))
    got = [L["weights"].cpu().numpy() for L in net.layers if "weights" in L]
    for g, w, w0 in zip(got, ow, weights):
        assert PC.relerr(g, w) < TOL
        assert PC.relerr(g, w0) > 1e-5     # the weights did move
    # the network can be written back and read again unchanged
    out = str(tmp_path / "saved.jsn")
    networks.save_network_json(out, net)
    _, specs2, weights2 = networks.load_network_json(out)
    assert [s["name"] for s in specs2] == [s["name"] for s in specs]
    for a, b in zip(weights2, got):
        assert np.array_equal(a, b)
    net.close()
    ds.close()


def test_network_json_errors(tmp_path):
    networks = PC.networks()
    p = str(tmp_path / "n.jsn")
    json.dump({"layers": [{"size": 3, "name": "input", "type": "input"}, {"size": 4, "name": "c", "type": "cnn"},
                          {"size": 4, "name": "post", "type": "sse"}]}, open(p, "w"))
    with pytest.raises(ValueError, match="does not cover"):
        networks.load_network_json(p)
    json.dump({"layers": [{"size": 3, "name": "input", "type": "input"},
                          {"size": 4, "name": "o", "type": "feedforward_identity", "bias": 1.0},
                          {"size": 4, "name": "post", "type": "sse"}],
               "weights": {"o": {"input": [0.0] * 11, "bias": [0.0] * 4, "internal": []}}}, open(p, "w"))
    with pytest.raises(ValueError, match="expected 16"):
        networks.load_network_json(p)
