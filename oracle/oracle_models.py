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


# ---------------------------------------------------------------------------------------------------------
# WaveNet-style stack (benchmark config 4), topology of the reference's example network
# obsolete/scripts/EXAMPLE/MODEL_WAVENET/network.jsn: embedding of the fed-back one-hot sample, then per block
#   cnn (causal, dilated, 2R filters) -> wavnetc (gate, conditioned) -> out (R->R) -> skipadd(residual, out)
#   -> temp (skipini) -> skipouttrans (R->K) -> skip (skipini) ; temp2 = skipadd(temp) feeds the next block,
# then skipadd over all skip layers -> feedforward_tanh -> feedforward_identity (Q classes) -> mdn softmax.
# The graph walk below is shared by the CPU-oracle backend above and the tests' HIP backend; a backend
# supplies buffers and the layer primitives.  Error routing follows SkipAddLayer.cu:305-346: a skip
# layer adds its side buffer to its error buffer, accumulates into skip predecessors' side buffers and
# overwrites plain predecessors' error buffers.
# ---------------------------------------------------------------------------------------------------------
class WaveNet:
    def __init__(self, backend, n_blocks, S, T, Q=1024, R=64, K=128, C=80, cnn_tanh=1, dilation_cycle=10):
        self.b, self.nb, self.S, self.T = backend, n_blocks, S, T
        self.Q, self.R, self.K, self.C, self.cnn_tanh = Q, R, K, C, cnn_tanh
        self.N = S * T
        self.dils = [2 ** (l % dilation_cycle) for l in range(n_blocks)]
        N, z = self.N, backend.zeros
        self.buf = {}

        def layer(name, size, nW=0, skip=False):
            d = {"out": z(size * N), "err": z(size * N), "size": size}
            if nW:
                d["W"], d["dW"] = z(nW), z(nW)
            if skip:
                d["eskip"] = z(size * N)
            self.buf[name] = d
            return d

        layer("emb", R, Q * R + R)
        layer("causalSkip", R, skip=True)
        for l in range(n_blocks):
            layer("cnn%d" % l, 2 * R, R * 3 * 2 * R + 2 * R)
            w = layer("wav%d" % l, R, C * 2 * R)
            w["core"], w["cth"] = z(2 * R * N), z(2 * R * N)
            layer("out%d" % l, R, R * R + R)
            layer("sadd%d" % l, R, skip=True)
            layer("temp%d" % l, R, skip=True)
            layer("sot%d" % l, K, R * K + K)
            layer("skip%d" % l, K, skip=True)
            layer("temp2_%d" % l, R, skip=True)
        layer("postAdd", K, skip=True)
        layer("postL1", K, K * K + K)
        layer("output", Q, K * Q + Q)
        self.zeroK = z(K * N)
        self.softmax = backend.softmax_make(Q, S, T)
        self.loss = z(1)

    def weight_names(self):
        return [k for k, v in self.buf.items() if "W" in v]

    def set_inputs(self, pat, onehot, ctx, target):
        self.pat, self.x0, self.ctx, self.target = pat, onehot, ctx, target
        self.softmax.load_sequences(pat, self.T)

    def _res(self, l):
        return self.buf["causalSkip"] if l == 0 else self.buf["temp2_%d" % (l - 1)]

    def forward(self):
        B, b, N, R, K, Q, C = self.buf, self.b, self.N, self.R, self.K, self.Q, self.C
        b.dense_forward(Q, R, N, 0, B["emb"]["W"], self.x0, B["emb"]["out"])
        cs = B["causalSkip"]
        b.skipadd_forward([B["emb"]["out"]], cs["out"], cs["err"], cs["eskip"])
        for l in range(self.nb):
            res, cnn, wav, out = self._res(l), B["cnn%d" % l], B["wav%d" % l], B["out%d" % l]
            sadd, temp, sot, skip, temp2 = B["sadd%d" % l], B["temp%d" % l], B["sot%d" % l], B["skip%d" % l], B["temp2_%d" % l]
            b.cnn_forward(l, R, 2 * R, self.S, self.T, self.dils[l], self.cnn_tanh, self.pat, cnn["W"], res["out"], cnn["out"])
            b.wavnetc_forward(R, C, N, self.pat, wav["W"], self.ctx, cnn["out"], wav["core"], wav["cth"], wav["out"])
            b.dense_forward(R, R, N, 0, out["W"], wav["out"], out["out"])
            b.skipadd_forward([res["out"], out["out"]], sadd["out"], sadd["err"], sadd["eskip"])
            b.skipadd_forward([sadd["out"]], temp["out"], temp["err"], temp["eskip"])
            b.dense_forward(R, K, N, 0, sot["W"], temp["out"], sot["out"])
            b.skipadd_forward([sot["out"]], skip["out"], skip["err"], skip["eskip"])
            b.skipadd_forward([temp["out"]], temp2["out"], temp2["err"], temp2["eskip"])
        pa = B["postAdd"]
        b.skipadd_forward([B["skip%d" % l]["out"] for l in range(self.nb)], pa["out"], pa["err"], pa["eskip"])
        b.dense_forward(K, K, N, 1, B["postL1"]["W"], pa["out"], B["postL1"]["out"])
        b.dense_forward(K, Q, N, 0, B["output"]["W"], B["postL1"]["out"], B["output"]["out"])
        self.softmax.forward(B["output"]["out"])

    def calculate_error(self):
        self.softmax.calculate_error(self.target, self.loss)
        return self.loss

    def reset_skip_errors(self):
        """What the skip layers' forward pass clears (SkipAddLayer.cu:195-205); needed before a backward pass is
        repeated without a forward pass in between."""
        for v in self.buf.values():
            if "eskip" in v:
                v["err"].zero_()
                v["eskip"].zero_()

    def backward(self):
        B, b, N, R, K, Q, C = self.buf, self.b, self.N, self.R, self.K, self.Q, self.C
        self.softmax.backward(self.target, B["output"]["err"])
        b.dense_backward(K, Q, N, 0, B["output"]["W"], B["postL1"]["out"], B["output"]["out"], B["output"]["err"],
                         B["postL1"]["err"], B["output"]["dW"])
        pa = B["postAdd"]
        b.dense_backward(K, K, N, 1, B["postL1"]["W"], pa["out"], B["postL1"]["out"], B["postL1"]["err"], pa["err"],
                         B["postL1"]["dW"])
        b.skipadd_backward(pa["err"], pa["eskip"], [B["skip%d" % l]["eskip"] for l in range(self.nb)], [1] * self.nb,
                           self.zeroK)
        for l in range(self.nb - 1, -1, -1):
            res, cnn, wav, out = self._res(l), B["cnn%d" % l], B["wav%d" % l], B["out%d" % l]
            sadd, temp, sot, skip, temp2 = B["sadd%d" % l], B["temp%d" % l], B["sot%d" % l], B["skip%d" % l], B["temp2_%d" % l]
            b.skipadd_backward(temp2["err"], temp2["eskip"], [temp["eskip"]], [1], None)
            b.skipadd_backward(skip["err"], skip["eskip"], [sot["err"]], [0], None)
            b.dense_backward(R, K, N, 0, sot["W"], temp["out"], sot["out"], sot["err"], temp["err"], sot["dW"])
            b.skipadd_backward(temp["err"], temp["eskip"], [sadd["eskip"]], [1], None)
            b.skipadd_backward(sadd["err"], sadd["eskip"], [res["eskip"], out["err"]], [1, 0], None)
            b.dense_backward(R, R, N, 0, out["W"], wav["out"], out["out"], out["err"], wav["err"], out["dW"])
            b.wavnetc_backward(R, C, N, self.pat, wav["W"], self.ctx, wav["core"], wav["cth"], wav["err"], cnn["err"], wav["dW"])
            b.cnn_backward(l, R, 2 * R, self.S, self.T, self.dils[l], self.cnn_tanh, self.pat, cnn["W"], res["out"], cnn["out"],
                           cnn["err"], res["err"], cnn["dW"])
        cs = B["causalSkip"]
        b.skipadd_backward(cs["err"], cs["eskip"], [B["emb"]["err"]], [0], None)
        b.dense_backward(Q, R, N, 0, B["emb"]["W"], self.x0, B["emb"]["out"], B["emb"]["err"], None, B["emb"]["dW"])

    def close(self):
        self.softmax.close()
        self.b.close()
