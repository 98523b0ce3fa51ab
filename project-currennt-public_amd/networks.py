"""Layer-by-layer sequencing of the HIP library for stacked networks (the role of
NeuralNetwork::__computeForward_LayerByLayer / __computeBackward_LayerByLayer,
NeuralNetwork.cpp:1419-1471 and :2743-2800 of the reference).  Buffers are torch CUDA tensors,
every computation is a C-ABI call; nothing here computes on the host.

Layer specs are dicts with the reference's JSON keys: {"type": "feedforward_tanh", "size": 512,
"bias": 1.0}.  Supported types: feedforward_tanh / feedforward_identity / feedforward_logistic /
feedforward_relu, lstm, blstm, and a final sse post-output layer.
"""
import torch

from . import capi

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


def acoustic_model_spec():
    """BASELINE config 2: 382 -> 2 x feedforward_tanh 512 -> 2 x blstm 512 -> feedforward_identity 187 -> sse."""
    return 382, [
        {"type": "feedforward_tanh", "size": 512, "bias": 1.0},
        {"type": "feedforward_tanh", "size": 512, "bias": 1.0},
        {"type": "blstm", "size": 512, "bias": 1.0},
        {"type": "blstm", "size": 512, "bias": 1.0},
        {"type": "feedforward_identity", "size": 187, "bias": 1.0},
        {"type": "sse", "size": 187},
    ]
