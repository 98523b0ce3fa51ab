"""Descriptions of the benchmark networks in the reference's network-file vocabulary (layer dicts with the JSON keys
of a network file).  Pure data: nothing here touches the GPU or the oracle."""


def acoustic_model_spec():
    """benchmark config 2: 382 -> 2 x feedforward_tanh 512 -> 2 x blstm 512 -> feedforward_identity 187 -> sse."""
    return 382, [
        {"type": "feedforward_tanh", "size": 512, "bias": 1.0},
        {"type": "feedforward_tanh", "size": 512, "bias": 1.0},
        {"type": "blstm", "size": 512, "bias": 1.0},
        {"type": "blstm", "size": 512, "bias": 1.0},
        {"type": "feedforward_identity", "size": 187, "bias": 1.0},
        {"type": "sse", "size": 187},
    ]


def wavenet_network_doc(nb, Q, R, K, C, cnn_tanh, dilation_cycle):
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
