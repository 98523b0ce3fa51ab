"""The acoustic model's backward pass the way a maintainer of the reference would bind it: one C-ABI call per layer
and pass (cnt_sse_backward, cnt_dense_backward, cnt_lstm_backward), all on ONE stream, every buffer owned by the
caller -- what `Layer::computeBackwardPass` of each layer shell does.  No side streams, no batching across layers:
the figure shows what the per-layer boundary costs against the library's own sequencer."""
import numpy as np

_FF_ACT = {"feedforward_identity": 0, "feedforward_tanh": 1, "feedforward_logistic": 2, "feedforward_relu": 3}


class LayerCallModel:
    def __init__(self, capi, input_size, specs, S, T, rng, scale):
        import torch

        self.capi, self.S, self.T = capi, S, T
        n = S * T
        self.layers = []
        prev = input_size
        for sp in specs:
            t, D = sp["type"], sp["size"]
            L = {"type": t, "size": D, "prev": prev, "bias": float(sp.get("bias", 1.0)),
                 "outputs": torch.zeros(D * n, dtype=torch.float32, device="cuda"),
                 "errors": torch.zeros(D * n, dtype=torch.float32, device="cuda")}
            if t in _FF_ACT:
                nW = prev * D + D
            elif t in ("lstm", "blstm"):
                nW = int(capi.lib().cnt_lstm_weight_count(prev, D, int(t == "blstm")))
                L["handle"] = capi.Lstm(prev, D, t == "blstm", S, T, L["bias"])
            else:
                nW = 0
            if nW:
                L["weights"] = torch.from_numpy(rng.uniform(-scale, scale, nW).astype(np.float32)).cuda()
                L["updates"] = torch.zeros(nW, dtype=torch.float32, device="cuda")
            self.layers.append(L)
            prev = D

    def load_sequences(self, pat, T, Tmin, inputs=None, targets=None):
        self.pat, self.T = pat, T
        if inputs is not None:
            self.inputs = inputs
        if targets is not None:
            self.layers[-1]["outputs"][: targets.numel()].copy_(targets)  # a post-output layer keeps the targets
        for L in self.layers:
            if "handle" in L:
                L["handle"].load_sequences(pat, T, Tmin)

    def forward(self):
        N, x = self.T * self.S, self.inputs
        for L in self.layers:
            t = L["type"]
            if t in _FF_ACT:
                self.capi.dense_forward(L["prev"], L["size"], N, _FF_ACT[t], L["bias"], L["weights"], x, L["outputs"])
            elif "handle" in L:
                L["handle"].forward(L["weights"], x, L["outputs"])
            else:
                break
            x = L["outputs"]

    def backward(self):
        N, capi = self.T * self.S, self.capi
        for i in range(len(self.layers) - 1, -1, -1):
            L = self.layers[i]
            t = L["type"]
            x = self.layers[i - 1]["outputs"] if i > 0 else self.inputs
            prev_err = self.layers[i - 1]["errors"] if i > 0 else None
            if t == "sse":
                capi.sse_backward(L["size"], N, self.pat, x, L["outputs"], prev_err)
            elif t in _FF_ACT:
                capi.dense_backward(L["prev"], L["size"], N, _FF_ACT[t], L["bias"], L["weights"], x, L["outputs"],
                                    L["errors"], prev_err, L["updates"])
            else:
                L["handle"].backward(L["weights"], x, L["outputs"], L["errors"], prev_err, L["updates"])

    def check(self):
        for L in self.layers:
            if "handle" in L:
                L["handle"].check()

    def close(self):
        for L in self.layers:
            if "handle" in L:
                L["handle"].close()
