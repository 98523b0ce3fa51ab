"""GPU parity of a whole WaveNet-style stack (reference example topology, benchmark config 4 layer sizes, few
blocks, short waveforms) against the same graph on the CPU oracle: loss and every weight-update vector."""
import numpy as np
import pytest

import oracle_models as OM
import parity_cases as PC
import synth as WD

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("cnn_tanh", [1, 0])
def test_wavenet_stack(cnn_tanh):
    import torch

    print("wavenet stack", cnn_tanh, flush=True)
    networks = PC.networks()
    nb, Q, R, K, C = 4, 64, 64, 128, 80
    lengths = [120, 90]
    S, T = len(lengths), max(lengths)
    pat, onehot, ctx, target, N = WD.make(lengths, Q, C, upsample=20, seed=2)
    ref = networks.WaveNet(OM.OracleBackend(), nb, S, T, Q=Q, R=R, K=K, C=C, cnn_tanh=cnn_tanh, dilation_cycle=3)
    gpu = networks.WaveNet(networks.HipBackend(), nb, S, T, Q=Q, R=R, K=K, C=C, cnn_tanh=cnn_tanh, dilation_cycle=3)
    shapes = {k: len(ref.buf[k]["W"]) for k in ref.weight_names()}
    W = WD.init_weights(shapes, seed=3)
    for k, w in W.items():
        ref.buf[k]["W"][:] = w
        gpu.buf[k]["W"].copy_(torch.from_numpy(w))
    ref.set_inputs(pat, onehot, ctx, target)
    gpu.set_inputs(PC.dev(pat), PC.dev(onehot), PC.dev(ctx), PC.dev(target))
    for net in (ref, gpu):
        net.forward()
        net.calculate_error()
        net.backward()
    torch.cuda.synchronize()
    ref_loss, loss = float(ref.loss[0]), float(gpu.loss.item())
    assert abs(loss - ref_loss) <= 1e-4 * abs(ref_loss)
    worst = 0.0
    for k in ref.weight_names():
        e = PC.relerr(gpu.buf[k]["dW"].cpu().numpy(), ref.buf[k]["dW"])
        worst = max(worst, e)
        if e > 1e-4:
            print("   ", k, e, flush=True)
    gpu.close()
    assert worst < 1e-4
