"""Seeded synthetic inputs of the benchmark workloads: pattern types of ragged fractions, and for the WaveNet workload (benchmark config 4): mu-law quantised U(-1,1) waveforms, the
teacher-forced one-hot of the previous sample, frame-rate conditioning up-sampled by a frame index."""
import numpy as np



def make_pat_types(lengths, T):
    """patTypes[t*S+s]: 0 none, 1 first, 2 normal, 3 last (sequences left-aligned)."""
    S = len(lengths)
    pat = np.zeros((T, S), dtype=np.int8)
    for s, n in enumerate(lengths):
        pat[:n, s] = 2
        pat[0, s] = 1
        pat[n - 1, s] = 3
    return pat.reshape(-1)


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
