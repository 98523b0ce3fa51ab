"""Independent float64 PyTorch statements of the forward maths; autograd of these pins the oracle's
gradients.  Nothing here shares code with the oracle or with the HIP library."""
import numpy as np
import torch


from synth import make_pat_types  # noqa: E402,F401  (one definition, shared with the benchmark)


def split_lstm_weights(W, P, L, bidir):
    """Views into the reference's flat LSTM weight vector (torch tensor, float64)."""
    nd = 2 if bidir else 1
    H = L // nd
    o_b = 4 * P * L
    o_i = o_b + 4 * L
    o_p = o_i + 4 * L * H
    out = []
    for d in range(nd):
        w_in = [W[g * P * L + d * P * H: g * P * L + (d + 1) * P * H].reshape(H, P) for g in range(4)]  # [unit][p]
        b = [W[o_b + g * L + d * H: o_b + g * L + (d + 1) * H] for g in range(4)]
        # stored [from + to*H] -> reshape gives [to][from]
        w_int = [W[o_i + g * L * H + d * H * H: o_i + g * L * H + (d + 1) * H * H].reshape(H, H) for g in range(4)]
        peep = [W[o_p + k * L + d * H: o_p + k * L + (d + 1) * H] for k in range(3)]
        out.append((w_in, b, w_int, peep))
    return out


def lstm_forward_torch(W, x, lengths, P, L, bidir, S, T, bias):
    """x: (T,S,P) float64 -> out (T,S,L). Dummy slots give 0 output and carry no state."""
    nd = 2 if bidir else 1
    H = L // nd
    parts = split_lstm_weights(W, P, L, bidir)
    valid = torch.zeros(T, S, dtype=torch.bool)
    for s, n in enumerate(lengths):
        valid[:n, s] = True
    outs = []
    for d in range(nd):
        w_in, b, w_int, peep = parts[d]
        hs = [None] * T
        h_prev = torch.zeros(S, H, dtype=W.dtype)
        c_prev = torch.zeros(S, H, dtype=W.dtype)
        order = range(T) if d == 0 else range(T - 1, -1, -1)
        for t in order:
            a = [x[t] @ w_in[g].T + bias * b[g] + h_prev @ w_int[g].T for g in range(4)]
            ni = torch.tanh(a[0])
            ig = torch.sigmoid(a[1] + c_prev * peep[0])
            fg = torch.sigmoid(a[2] + c_prev * peep[1])
            c = ni * ig + c_prev * fg
            og = torch.sigmoid(a[3] + c * peep[2])
            h = torch.tanh(c) * og
            m = valid[t].unsqueeze(1).to(W.dtype)
            h = h * m
            c = c * m
            hs[t] = h
            h_prev, c_prev = h, c
        outs.append(torch.stack(hs, 0))
    return torch.cat(outs, dim=2)
