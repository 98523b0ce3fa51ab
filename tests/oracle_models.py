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


class OracleSoftmax:
    """Softmax MDN unit on the oracle with the interface the WaveNet graph walk expects."""

    def __init__(self, Lp, S, T):
        self.Lp, self.S, self.T = Lp, S, T
        self.prob = np.zeros(Lp * S * T, dtype=np.float32)

    def load_sequences(self, pat, T):
        self.pat = pat

    def forward(self, x):
        O.softmax_forward(self.S * self.T, self.Lp, 0, self.Lp, 1.0, self.pat, x, self.prob)

    def calculate_error(self, target, loss):
        loss[0] = O.softmax_error(self.S * self.T, 1, 0, self.Lp, len(self.prob), self.pat, target, self.prob)

    def backward(self, target, err):
        err[:] = 0
        O.softmax_backward(self.S * self.T, self.Lp, 1, 0, 0, self.Lp, self.pat, target, self.prob, err)

    def close(self):
        pass


class OracleBackend:
    """Layer primitives on the CPU oracle; buffers are numpy arrays."""

    def zeros(self, n):
        return np.zeros(n, dtype=np.float32)

    def upload(self, a):
        return np.ascontiguousarray(a)

    def dense_forward(self, P, D, N, act, W, x, y):
        O.dense_forward(P, D, N, act, 1.0, W, x, y)

    def dense_backward(self, P, D, N, act, W, x, y, err, prev_err, dW):
        O.dense_backward(P, D, N, act, 1.0, W, x, y, err, prev_err, dW)

    def cnn_forward(self, key, P, D, S, T, dil, out_tanh, pat, W, x, out):
        hw, it = np.ones(D, dtype=np.int32), np.full(D, dil, dtype=np.int32)
        con = np.zeros(3 * D * S * T, dtype=np.float32)
        O.cnn_forward(P, D, S, T, 1, out_tanh, 1.0, hw, it, pat, W, x, con, out)

    def cnn_backward(self, key, P, D, S, T, dil, out_tanh, pat, W, x, out, err, prev_err, dW):
        hw, it = np.ones(D, dtype=np.int32), np.full(D, dil, dtype=np.int32)
        con = np.zeros(3 * D * S * T, dtype=np.float32)
        O.cnn_backward(P, D, S, T, 1, out_tanh, 1.0, hw, it, pat, W, x, out, err, con, prev_err, dW)

    def wavnetc_forward(self, D, C, N, pat, W, ctx, conv, core, cth, out):
        O.wavnetc_forward(D, C, N, pat, W, ctx, conv, core, cth, out)

    def wavnetc_backward(self, D, C, N, pat, W, ctx, core, cth, err, prev_err, dW):
        O.wavnetc_backward(D, C, N, pat, W, ctx, core, cth, err, prev_err, dW, None)

    def skipadd_forward(self, inputs, out, errors, errors_from_skip):
        O.skipadd_forward(inputs, out, errors, errors_from_skip)

    def skipadd_backward(self, errors, errors_from_skip, targets, is_skip, zero):
        O.skipadd_backward(errors, errors_from_skip, targets, is_skip)

    def softmax_make(self, Lp, S, T):
        return OracleSoftmax(Lp, S, T)

    def close(self):
        pass
