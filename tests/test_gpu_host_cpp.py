"""The C++ layer shells (project-currennt-public_amd/host/layers.hpp) driven end to end by the run_stack
executable on the GPU, compared with the CPU oracle network on the same job: loss, every layer's outputs and
every weight-update vector at 1e-4 L2-normalised."""
import os
import struct
import subprocess

import numpy as np
import pytest

import oracle_models as OM
import parity_cases as PC
from torch_models import make_pat_types

pytestmark = pytest.mark.gpu

KIND = {"feedforward_identity": 0, "feedforward_tanh": 1, "feedforward_logistic": 2, "feedforward_relu": 3,
        "lstm": 10, "blstm": 11}


def test_cpp_layer_stack_matches_oracle(tmp_path):
    print("c++ host stack", flush=True)
    capi = PC.pkg().capi
    driver = os.path.join(os.path.dirname(capi.LIB_PATH), "..", "bin", "run_stack")
    assert os.path.exists(driver), "host driver not built"
    input_size = 20
    specs = [{"type": "feedforward_tanh", "size": 32, "bias": 1.0}, {"type": "blstm", "size": 128, "bias": 1.0},
             {"type": "lstm", "size": 64, "bias": 0.5}, {"type": "feedforward_identity", "size": 7, "bias": 1.0},
             {"type": "sse", "size": 7}]
    lengths = [13, 9, 13, 4]
    S, T = len(lengths), max(lengths)
    rng = np.random.default_rng(12)
    x = rng.standard_normal((T, S, input_size)).astype(np.float32)
    tgt = rng.standard_normal((T, S, 7)).astype(np.float32)
    for s, n in enumerate(lengths):
        x[n:, s] = 0
        tgt[n:, s] = 0
    pat = make_pat_types(lengths, T)
    weights = OM.init_weights(input_size, specs, 3, 0.1)

    ref = OM.OracleNetwork(input_size, specs, S, T, min(lengths), pat, [w.copy() for w in weights])
    ref.forward(x.reshape(-1), tgt.reshape(-1))
    ref_loss = ref.error()
    ref.backward()

    job, res = tmp_path / "job.bin", tmp_path / "res.bin"
    with open(job, "wb") as f:
        f.write(struct.pack("<5i", input_size, len(specs) - 1, S, T, min(lengths)))
        for sp, w in zip(specs[:-1], weights):
            f.write(struct.pack("<iifq", KIND[sp["type"]], sp["size"], sp["bias"], len(w)))
            f.write(w.tobytes())
        f.write(pat.tobytes())
        f.write(x.tobytes())
        f.write(tgt.tobytes())
    r = subprocess.run([driver, str(job), str(res)], capture_output=True, text=True, timeout=100)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0
    data = open(res, "rb").read()
    loss = struct.unpack_from("<f", data, 0)[0]
    off = 4
    assert abs(loss - ref_loss) <= 1e-4 * abs(ref_loss)
    for L in ref.layers[:-1]:
        n = struct.unpack_from("<q", data, off)[0]; off += 8
        out = np.frombuffer(data, dtype=np.float32, count=n, offset=off); off += 4 * n
        nw = struct.unpack_from("<q", data, off)[0]; off += 8
        up = np.frombuffer(data, dtype=np.float32, count=nw, offset=off); off += 4 * nw
        assert PC.relerr(out[:len(L["outputs"])], L["outputs"]) < 1e-4
        assert PC.relerr(up, L["updates"]) < 1e-4


def test_cpp_driver_reports_errors_like_the_reference(tmp_path):
    capi = PC.pkg().capi
    driver = os.path.join(os.path.dirname(capi.LIB_PATH), "..", "bin", "run_stack")
    job = tmp_path / "bad.bin"
    with open(job, "wb") as f:
        # one blstm layer with an odd size: refused, as LstmLayer.cu:1091-1092 does
        f.write(struct.pack("<5i", 4, 1, 1, 2, 2))
        f.write(struct.pack("<iifq", 11, 33, 1.0, 0))
    r = subprocess.run([driver, str(job), str(tmp_path / "o.bin")], capture_output=True, text=True, timeout=100)
    assert r.returncode == 2
    assert "FAILED in running CURENNT" in r.stderr and "odd layer size" in r.stderr
