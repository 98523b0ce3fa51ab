"""Stacked networks on the CPU oracle (the checker's side of parity tests and the CPU-baseline leg of the
benchmark).  Same layer specs as the HIP-side sequencer; numpy buffers."""
import numpy as np

import oracle_lib as O

_FF_ACT = {"feedforward_identity": 0, "feedforward_tanh": 1, "feedforward_logistic": 2, "feedforward_relu": 3}


def weight_count(spec, prev):
    t, D = spec["type"], spec["size"]
    if t in _FF_ACT:
        return prev * D + D
    if t in ("lstm", "blstm"):
        return int(O.lib().orc_lstm_weight_count(prev, D, int(t == "blstm")))
    return 0


def init_weights(input_size, specs, seed, scale):
    rng = np.random.default_rng(seed)
    out, prev = [], input_size
    for sp in specs:
        n = weight_count(sp, prev)
        if n:
            out.append(rng.uniform(-scale, scale, n).astype(np.float32))
        prev = sp["size"]
    return out


class OracleNetwork:
    def __init__(self, input_size, specs, S, T, Tmin, pat, weights):
        self.S, self.T, self.Tmin, self.pat = S, T, Tmin, pat
        N = S * T
        self.layers = []
        prev = input_size
        wi = iter(weights)
        for sp in specs:
            t, D = sp["type"], sp["size"]
            L = {"type": t, "size": D, "prev": prev, "bias": float(sp.get("bias", 1.0)),
                 "outputs": np.zeros(D * N, dtype=np.float32), "errors": np.zeros(D * N, dtype=np.float32)}
            if weight_count(sp, prev):
                L["weights"] = next(wi)
                L["updates"] = np.zeros_like(L["weights"])
            if t in ("lstm", "blstm"):
                nd = 2 if t == "blstm" else 1
                L["fw"] = O.LstmState(D // nd, N)
                L["bw"] = O.LstmState(D // nd, N) if nd == 2 else None
                L["desc"] = O.LstmDesc(prev, D, int(nd == 2), S, T, Tmin, L["bias"])
            self.layers.append(L)
            prev = D

    def forward(self, inputs, targets):
        N = self.S * self.T
        self.inputs = inputs
        x = inputs
        for L in self.layers:
            t = L["type"]
            if t in _FF_ACT:
                O.dense_forward(L["prev"], L["size"], N, _FF_ACT[t], L["bias"], L["weights"], x, L["outputs"])
            elif t in ("lstm", "blstm"):
                O.lstm_forward(L["desc"], L["weights"], self.pat, x, L["fw"], L["bw"], L["outputs"])
            else:
                L["outputs"][:] = targets
                break
            x = L["outputs"]

    def error(self):
        post, last = self.layers[-1], self.layers[-2]
        return O.sse_error(post["size"], self.S * self.T, self.pat, last["outputs"], post["outputs"])

    def backward(self):
        N = self.S * self.T
        for i in range(len(self.layers) - 1, -1, -1):
            L = self.layers[i]
            t = L["type"]
            x = self.layers[i - 1]["outputs"] if i > 0 else self.inputs
            prev_err = self.layers[i - 1]["errors"] if i > 0 else None
            if t == "sse":
                O.sse_backward(L["size"], N, self.pat, self.layers[i - 1]["outputs"], L["outputs"], prev_err)
            elif t in _FF_ACT:
                O.dense_backward(L["prev"], L["size"], N, _FF_ACT[t], L["bias"], L["weights"], x, L["outputs"],
                                 L["errors"], prev_err, L["updates"])
            else:
                O.lstm_backward(L["desc"], L["weights"], self.pat, x, L["errors"], L["fw"], L["bw"], prev_err,
                                L["updates"])
