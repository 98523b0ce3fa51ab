"""Test harness: layer-by-layer sequencing of the HIP library for stacked networks (the role of
NeuralNetwork::__computeForward_LayerByLayer / __computeBackward_LayerByLayer,
NeuralNetwork.cpp:1419-1471 and :2743-2800 of the reference).  Buffers are torch CUDA tensors,
every computation is a C-ABI call; nothing here computes on the host.

Layer specs are dicts with the reference's JSON keys: {"type": "feedforward_tanh", "size": 512,
"bias": 1.0}.  Supported types: feedforward_tanh / feedforward_identity / feedforward_logistic /
feedforward_relu, lstm, blstm, and a final sse post-output layer.
"""
import torch

from __graft_entry__ import load_package

capi = load_package().capi

_FF_ACT = {"feedforward_identity": 0, "feedforward_tanh": 1, "feedforward_logistic": 2, "feedforward_relu": 3}


def layer_weight_count(spec, prev_size):
    t, D = spec["type"], spec["size"]
    if t in _FF_ACT:
        return prev_size * D + D
    if t in ("lstm", "blstm"):
        return int(capi.lib().cnt_lstm_weight_count(prev_size, D, int(t == "blstm")))
    return 0


class StackedNetwork:
    def __init__(self, input_size, layers, parallel_sequences, max_seq_length):
        self.S, self.maxT = parallel_sequences, max_seq_length
        self.input_size = input_size
        self.specs = layers
        assert layers[-1]["type"] == "sse"
        n = self.S * self.maxT
        dev = "cuda"
        self.layers = []
        prev = input_size
        for spec in layers:
            t, D = spec["type"], spec["size"]
            L = {"spec": spec, "type": t, "size": D, "prev": prev, "bias": float(spec.get("bias", 1.0))}
            L["outputs"] = torch.zeros(D * n, dtype=torch.float32, device=dev)
            L["errors"] = torch.zeros(D * n, dtype=torch.float32, device=dev)
            nW = layer_weight_count(spec, prev)
            if nW:
                L["weights"] = torch.zeros(nW, dtype=torch.float32, device=dev)
                L["updates"] = torch.zeros(nW, dtype=torch.float32, device=dev)
            if t in ("lstm", "blstm"):
                L["handle"] = capi.Lstm(prev, D, t == "blstm", self.S, self.maxT, L["bias"])
            self.layers.append(L)
            prev = D
        self.inputs = torch.zeros(input_size * n, dtype=torch.float32, device=dev)
        self.input_errors = None  # the input layer has no error buffer
        self.loss = torch.zeros(1, dtype=torch.float32, device=dev)
        self.T = 0

    def set_weights(self, flat_list):
        it = iter(flat_list)
        for L in self.layers:
            if "weights" in L:
                w = next(it)
                L["weights"].copy_(torch.as_tensor(w, dtype=torch.float32))

    def load_sequences(self, pat, T, Tmin, inputs=None, targets=None):
        """pat: int8 CUDA tensor of T*S pattern types.  inputs/targets are copied when given."""
        self.pat, self.T, self.Tmin = pat, T, Tmin
        if inputs is not None:
            self.inputs[: inputs.numel()].copy_(inputs)
        if targets is not None:
            # a post-output layer keeps the targets in its own outputs() (PostOutputLayer.cu:108-124)
            self.layers[-1]["outputs"][: targets.numel()].copy_(targets)
        for L in self.layers:
            if "handle" in L:
                L["handle"].load_sequences(pat, T, Tmin)

    def forward(self):
        N = self.T * self.S
        x = self.inputs
        for L in self.layers:
            t = L["type"]
            if t in _FF_ACT:
                capi.dense_forward(L["prev"], L["size"], N, _FF_ACT[t], L["bias"], L["weights"], x, L["outputs"])
            elif t in ("lstm", "blstm"):
                L["handle"].forward(L["weights"], x, L["outputs"])
            elif t == "sse":
                break
            x = L["outputs"]

    def calculate_error(self):
        N = self.T * self.S
        post, last = self.layers[-1], self.layers[-2]
        capi.sse_error(post["size"], N, self.pat, last["outputs"], post["outputs"], self.loss)
        return self.loss

    def backward(self):
        N = self.T * self.S
        for i in range(len(self.layers) - 1, -1, -1):
            L = self.layers[i]
            t = L["type"]
            x = self.layers[i - 1]["outputs"] if i > 0 else self.inputs
            prev_err = self.layers[i - 1]["errors"] if i > 0 else self.input_errors
            if t == "sse":
                # writes the preceding layer's error buffer
                capi.sse_backward(L["size"], N, self.pat, self.layers[i - 1]["outputs"], L["outputs"], prev_err)
            elif t in _FF_ACT:
                capi.dense_backward(L["prev"], L["size"], N, _FF_ACT[t], L["bias"], L["weights"], x, L["outputs"],
                                    L["errors"], prev_err, L["updates"])
            else:
                L["handle"].backward(L["weights"], x, L["outputs"], L["errors"], prev_err, L["updates"])

    def backward_overlapped(self, side_stream):
        """Same result as backward(); the weight-gradient halves run on `side_stream` while the main stream goes
        on with the next layer's error recursion (nothing reads weight updates before the optimizer).  The caller
        joins the two streams (torch.cuda.synchronize() or an event) before reading `updates`."""
        N = self.T * self.S
        main = torch.cuda.current_stream()
        for i in range(len(self.layers) - 1, -1, -1):
            L = self.layers[i]
            t = L["type"]
            x = self.layers[i - 1]["outputs"] if i > 0 else self.inputs
            prev_err = self.layers[i - 1]["errors"] if i > 0 else self.input_errors
            if t == "sse":
                capi.sse_backward(L["size"], N, self.pat, self.layers[i - 1]["outputs"], L["outputs"], prev_err)
                continue
            if t in _FF_ACT:
                capi.dense_backward_errors(L["prev"], L["size"], N, _FF_ACT[t], L["weights"], L["outputs"], L["errors"],
                                           prev_err)
            else:
                L["handle"].backward_errors(L["weights"], L["errors"], prev_err)
            # The weight gradients wait for the error product above as well: started right after the recursion
            # (cnt_lstm_backward_prev_errors allows that) the two products share the machine and the one on the
            # critical path takes 1.5x as long -- measured slower overall.
            ev = torch.cuda.Event()
            ev.record(main)
            side_stream.wait_event(ev)
            if t in _FF_ACT:
                capi.dense_backward_weights(L["prev"], L["size"], N, L["bias"], x, L["errors"], L["updates"],
                                            stream=side_stream)
            else:
                L["handle"].backward_weights(x, L["updates"], stream=side_stream)

    def check(self):
        for L in self.layers:
            if "handle" in L:
                L["handle"].check()

    def close(self):
        for L in self.layers:
            if "handle" in L:
                L["handle"].close()


# ---------------------------------------------------------------------------------------------------------
# Network files.  The reference keeps a network as JSON: "layers" is the ordered list of
# {"name", "type", "size", "bias", ...} objects (Layer::exportLayer, layers/Layer.cu:308-329, and
# TrainableLayer::exportLayer, layers/TrainableLayer.cu:483-492); "weights" maps a layer name to its
# "input" / "bias" / "internal" arrays, which are consecutive sections of the layer's flat weight vector
# (TrainableLayer::exportWeights, layers/TrainableLayer.cu:441-480; read back in the constructor, :100-170).
# ---------------------------------------------------------------------------------------------------------
def load_network_json(path):
    """Returns (input_size, layer specs without the input layer, per-layer flat weight arrays or None)."""
    import json

    import numpy as np

    with open(path) as f:
        doc = json.load(f)
    layers = doc.get("layers")
    if not isinstance(layers, list) or len(layers) < 3:
        raise ValueError("%s: a network needs an input layer, a hidden or output layer and a post-output layer" % path)
    if layers[0].get("type") != "input":
        raise ValueError("%s: the first layer must be of type 'input'" % path)
    input_size = int(layers[0]["size"])
    specs, weights = [], []
    have_weights = isinstance(doc.get("weights"), dict)
    prev = input_size
    for obj in layers[1:]:
        t = obj.get("type")
        if t not in _FF_ACT and t not in ("lstm", "blstm", "sse"):
            raise ValueError("%s: layer '%s' has type '%s', which this path does not cover" % (path, obj.get("name"), t))
        spec = {"name": obj.get("name", t), "type": t, "size": int(obj["size"])}
        if "bias" in obj:
            spec["bias"] = float(obj["bias"])
        specs.append(spec)
        nW = layer_weight_count(spec, prev)
        if nW and have_weights:
            sec = doc["weights"].get(spec["name"])
            if sec is None:
                raise ValueError("%s: no weights for layer '%s'" % (path, spec["name"]))
            w = np.concatenate([np.asarray(sec.get(k, []), dtype=np.float32) for k in ("input", "bias", "internal")])
            if w.size != nW:
                raise ValueError("%s: layer '%s' has %d weights, expected %d" % (path, spec["name"], w.size, nW))
            weights.append(w)
        prev = spec["size"]
    if specs[-1]["type"] != "sse":
        raise ValueError("%s: the last layer must be the sse post-output layer" % path)
    return input_size, specs, (weights if have_weights else None)


def weight_sections(spec, prev_size):
    """Lengths of the "input", "bias" and "internal" sections of a layer's weight vector."""
    D = spec["size"]
    if spec["type"] in _FF_ACT:
        return prev_size * D, D, 0
    if spec["type"] in ("lstm", "blstm"):
        H = D // (2 if spec["type"] == "blstm" else 1)
        return 4 * prev_size * D, 4 * D, 4 * D * H + 3 * D
    return 0, 0, 0


def save_network_json(path, net):
    """Writes layers and weights of a StackedNetwork in the reference's structure (the autosave's network part)."""
    import json

    layers = [{"size": net.input_size, "name": "input", "type": "input"}]
    weights = {}
    for i, L in enumerate(net.layers):
        spec = L["spec"]
        obj = {"size": L["size"], "name": spec.get("name", "%s_%d" % (L["type"], i)), "type": L["type"]}
        if "weights" in L:
            obj["bias"] = L["bias"]
            w = L["weights"].detach().cpu().numpy()
            n_in, n_bias, n_int = weight_sections(spec, L["prev"])
            weights[obj["name"]] = {"input": [float(v) for v in w[:n_in]],
                                    "bias": [float(v) for v in w[n_in:n_in + n_bias]],
                                    "internal": [float(v) for v in w[n_in + n_bias:]]}
        layers.append(obj)
    with open(path, "w") as f:
        json.dump({"layers": layers, "weights": weights}, f)


class Trainer:
    """One training step per fraction, as Optimizer::_processDataSet does in hybrid online/batch mode
    (optimizers/Optimizer.cu:95-237): load the fraction, forward, error, backward, then for every trainable layer
    the copy / gradient adjustment / momentum update of SteepestDescentOptimizer::_updateWeights in one fused
    pass.  `option` is the reference's optimizer option number (0 SGD, 1 AdaGrad, 2 averaged gradient, 5 Adam)."""

    def __init__(self, net, learning_rate, momentum=0.0, option=0):
        self.net, self.lr, self.momentum, self.option = net, learning_rate, momentum, option
        self.beta1 = self.beta2 = 1.0
        self.side = torch.cuda.Stream()
        for L in net.layers:
            if "weights" in L:
                n = L["weights"].numel()
                L["cur_updates"] = torch.zeros(n, dtype=torch.float32, device="cuda")
                L["deltas"] = torch.zeros(n, dtype=torch.float32, device="cuda")
                if option in (capi.OPT_ADAGRAD, capi.OPT_STOCHASTIC_ADAGRAD):
                    L["stats"] = torch.full((n,), 1e-6, dtype=torch.float32, device="cuda")
                elif option == capi.OPT_ADAM:
                    L["stats"] = torch.zeros(2 * n, dtype=torch.float32, device="cuda")
                else:
                    L["stats"] = None

    def train_fraction(self, fraction):
        """`fraction`: dict from capi.Dataset.fraction().  Returns the fraction's training error (a device tensor)."""
        net = self.net
        T = fraction["max_len"]
        pat = torch.from_numpy(fraction["patTypes"]).cuda()
        net.load_sequences(pat, T, fraction["min_len"], torch.from_numpy(fraction["inputs"]).cuda(),
                           torch.from_numpy(fraction["targets"]).cuda())
        net.forward()
        loss = net.calculate_error().clone()
        net.backward_overlapped(self.side)
        torch.cuda.current_stream().wait_stream(self.side)
        if self.option == capi.OPT_ADAM:
            self.beta1 = capi.opt_next_beta_accum(self.beta1, 1)
            self.beta2 = capi.opt_next_beta_accum(self.beta2, 2)
        for L in net.layers:
            if "weights" in L:
                capi.opt_step(self.option, L["weights"], L["updates"], L["cur_updates"], L["stats"], L["deltas"], None,
                              float(fraction["total_length"]), self.beta1, self.beta2, self.lr, self.momentum)
        return loss


class HipBackend:
    """Layer primitives on the HIP library; buffers are torch CUDA tensors."""

    def __init__(self):
        self.cnn_handles = {}

    def zeros(self, n):
        return torch.zeros(n, dtype=torch.float32, device="cuda")

    def upload(self, a):
        return torch.as_tensor(a).cuda()

    def dense_forward(self, P, D, N, act, W, x, y):
        capi.dense_forward(P, D, N, act, 1.0, W, x, y)

    def dense_backward(self, P, D, N, act, W, x, y, err, prev_err, dW):
        capi.dense_backward(P, D, N, act, 1.0, W, x, y, err, prev_err, dW)

    def _cnn(self, key, P, D, S, T, dil, out_tanh):
        if key not in self.cnn_handles:
            self.cnn_handles[key] = capi.Cnn(P, [1] * D, [dil] * D, S, T, 1, out_tanh, 1.0)
        return self.cnn_handles[key]

    def cnn_forward(self, key, P, D, S, T, dil, out_tanh, pat, W, x, out):
        self._cnn(key, P, D, S, T, dil, out_tanh).forward(pat, T, W, x, out)

    def cnn_backward(self, key, P, D, S, T, dil, out_tanh, pat, W, x, out, err, prev_err, dW):
        self._cnn(key, P, D, S, T, dil, out_tanh).backward(pat, T, W, x, out, err, prev_err, dW)

    def wavnetc_forward(self, D, C, N, pat, W, ctx, conv, core, cth, out):
        capi.wavnetc_forward(D, C, N, pat, W, ctx, conv, core, cth, out)

    def wavnetc_backward(self, D, C, N, pat, W, ctx, core, cth, err, prev_err, dW):
        capi.wavnetc_backward(D, C, N, pat, W, ctx, core, cth, err, prev_err, dW, None)

    def skipadd_forward(self, inputs, out, errors, errors_from_skip):
        capi.skipadd_forward(inputs[:8], out, errors, errors_from_skip)
        for i in range(8, len(inputs), 7):  # more than 8 inputs: keep summing into the output
            capi.skipadd_forward([out] + inputs[i:i + 7], out, None, None)

    def skipadd_backward(self, errors, errors_from_skip, targets, is_skip, zero):
        capi.skipadd_backward(errors, errors_from_skip, targets[-8:], is_skip[-8:])
        for hi in range(len(targets) - 8, 0, -8):  # remaining predecessors: fan-out only (the side buffer is spent)
            lo = max(0, hi - 8)
            capi.skipadd_backward(errors, zero, targets[lo:hi], is_skip[lo:hi])

    def softmax_make(self, Lp, S, T):
        return capi.Mdn(Lp, 1, S, T, [1, 0, Lp, 0, 1, -1])

    def close(self):
        for h in self.cnn_handles.values():
            h.close()


from oracle_models import WaveNet  # noqa: E402,F401  (the graph walk itself is backend-neutral and lives beside the oracle)
