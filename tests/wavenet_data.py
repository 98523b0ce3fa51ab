"""Seeded synthetic inputs of the WaveNet workload (benchmark config 4): mu-law quantised U(-1,1) waveforms, the
teacher-forced one-hot of the previous sample, frame-rate conditioning up-sampled by a frame index."""
import numpy as np

from torch_models import make_pat_types


def mulaw_classes(x, Q):
    y = np.sign(x) * np.log1p((Q - 1) * np.abs(x)) / np.log(Q)
    return np.floor((y + 1) / 2 * (Q - 1) + 0.5).astype(np.int64)


def make(lengths, Q, C, upsample, seed):
    S, T = len(lengths), max(lengths)
    N = S * T
    rng = np.random.default_rng(seed)
    wav = rng.uniform(-1, 1, size=(T, S))
    cls = mulaw_classes(wav, Q)
    pat = make_pat_types(lengths, T)
    valid = (pat != 0).reshape(T, S)
    onehot = np.zeros((T, S, Q), dtype=np.float32)
    for t in range(1, T):
        for s in range(S):
            if valid[t, s]:
                onehot[t, s, cls[t - 1, s]] = 1.0
    target = np.where(valid, cls, 0).astype(np.float32).reshape(-1)
    n_frames = -(-T // upsample)
    frames = rng.standard_normal((n_frames, S, C)).astype(np.float32)
    ctx = np.zeros((T, S, C), dtype=np.float32)
    for t in range(T):
        ctx[t] = frames[t // upsample]
    ctx[~valid] = 0
    return pat, onehot.reshape(-1), ctx.reshape(-1), target, N


def init_weights(net_weight_shapes, seed, scale=0.1):
    rng = np.random.default_rng(seed)
    return {k: rng.uniform(-scale, scale, n).astype(np.float32) for k, n in net_weight_shapes.items()}


def network_json(nb, Q, R, K, C, cnn_tanh, dilation_cycle):
    """Network file with the topology of the reference's example obsolete/scripts/EXAMPLE/MODEL_WAVENET/network.jsn
    (without its frame-rate conditioning sub-network: the conditioning features are handed to the library)."""
    def ff(name, size, kind="feedforward_identity"):
        return {"size": size, "name": name, "bias": 1.0, "type": kind}

    layers = [{"size": 1, "name": "input", "type": "input"},
              {"size": Q, "name": "feedbackBottom", "bias": 1.0, "type": "feedback", "previousDimEnd": 0,
               "previousDimStart": 0},
              ff("emb", R), {"size": R, "name": "causalSkip", "bias": 1.0, "type": "skipini"}]
    res = "causalSkip"
    for l in range(nb):
        dil = 2 ** (l % dilation_cycle)
        layers += [
            {"size": 2 * R, "name": "cnn%d" % l, "bias": 1.0, "type": "cnn", "window_width": "%d*1" % (2 * R),
             "window_tap_interval": "%d*%d" % (2 * R, dil), "causal": 1, "tanhoutput": cnn_tanh},
            {"size": R, "name": "wav%d" % l, "bias": 1.0, "type": "wavnetc", "contextDim": C},
            ff("out%d" % l, R),
            {"size": R, "name": "sadd%d" % l, "bias": 1.0, "type": "skipadd", "preSkipLayer": "%s,out%d" % (res, l)},
            {"size": R, "name": "temp%d" % l, "bias": 1.0, "type": "skipini"},
            ff("sot%d" % l, K),
            {"size": K, "name": "skip%d" % l, "bias": 1.0, "type": "skipini"},
            {"size": R, "name": "temp2_%d" % l, "bias": 1.0, "type": "skipadd", "preSkipLayer": "temp%d" % l}]
        res = "temp2_%d" % l
    layers += [{"size": K, "name": "postAdd", "bias": 1.0, "type": "skipadd",
                "preSkipLayer": ",".join("skip%d" % l for l in range(nb))},
               ff("postL1", K, "feedforward_tanh"), ff("output", Q), {"size": 1, "name": "postoutput", "type": "mdn"}]
    return {"layers": layers}
