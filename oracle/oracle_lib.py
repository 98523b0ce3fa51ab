"""ctypes binding of the CPU oracle (oracle/_build/liboracle.so).

Only tests, the smoke check and the CPU-baseline leg of the benchmark import this module;
the oracle is the checker, never the thing that is measured or shipped.
"""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
LIB_PATH = os.path.join(ORACLE_DIR, "_build", "liboracle.so")

FP = C.POINTER(C.c_float)


def build(force=False):
    if force or not os.path.exists(LIB_PATH):
        subprocess.check_call(["make", "-C", ORACLE_DIR] + (["-B"] if force else []))
    return LIB_PATH


class LstmDesc(C.Structure):
    _fields_ = [("P", C.c_int), ("L", C.c_int), ("bidir", C.c_int), ("S", C.c_int), ("T", C.c_int),
                ("Tmin", C.c_int), ("bias", C.c_float)]


LSTM_FIELDS = ["ni", "ig", "fg", "og", "c", "h", "herr", "dni", "dig", "dfg", "dog", "cerr"]


class LstmDir(C.Structure):
    _fields_ = [(n, FP) for n in LSTM_FIELDS]


def fptr(a):
    if a is None:
        return None
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(FP)


def cptr(a):
    assert a.dtype == np.int8 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.c_char_p)


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(LIB_PATH)
        L.orc_logistic.restype = C.c_float
        L.orc_logistic.argtypes = [C.c_float]
        L.orc_tanh.restype = C.c_float
        L.orc_tanh.argtypes = [C.c_float]
        L.orc_safe_exp.restype = C.c_float
        L.orc_safe_exp.argtypes = [C.c_float]
        L.orc_safe_log.restype = C.c_float
        L.orc_safe_log.argtypes = [C.c_float]
        L.orc_log_add.restype = C.c_float
        L.orc_log_add.argtypes = [C.c_float, C.c_float]
        L.orc_lstm_weight_count.restype = C.c_long
        L.orc_sse_error.restype = C.c_float
        L.orc_mdn_mixture_error.restype = C.c_float
        L.orc_softmax_error.restype = C.c_float
        L.orc_sigmoid_error.restype = C.c_float
        L.orc_dft_logamp_loss.restype = C.c_float
        L.orc_dft_spectral_loss.restype = C.c_float
        L.orc_dft_phase_loss.restype = C.c_float
        L.orc_opt_next_beta_accum.restype = C.c_float
        L.orc_opt_next_beta_accum.argtypes = [C.c_float, C.c_int]
        _lib = L
    return _lib


def set_threads(n):
    """Worker threads of the oracle's large loops; results do not depend on it (whole outputs are shared out)."""
    lib().orc_set_threads(int(n))


def use_all_cores(limit=16):
    """For the full-size parity cases: as many threads as this process may run on, at most `limit`."""
    try:
        n = len(os.sched_getaffinity(0))
    except AttributeError:
        n = os.cpu_count() or 1
    set_threads(max(1, min(limit, n)))


class LstmState:
    """Host buffers of one direction: every field is an H x (T*S) column-major matrix."""

    def __init__(self, H, N):
        self.arr = {n: np.zeros(H * N, dtype=np.float32) for n in LSTM_FIELDS}
        self.c = LstmDir(**{n: fptr(a) for n, a in self.arr.items()})

    def __getitem__(self, k):
        return self.arr[k]


def lstm_forward(desc, W, pat, x, fw, bw, out):
    lib().orc_lstm_forward(C.byref(desc), fptr(W), cptr(pat), fptr(x), C.byref(fw.c),
                           C.byref(bw.c) if bw is not None else None, fptr(out))


def lstm_backward(desc, W, pat, x, outerr, fw, bw, ex, dW):
    lib().orc_lstm_backward(C.byref(desc), fptr(W), cptr(pat), fptr(x), fptr(outerr), C.byref(fw.c),
                            C.byref(bw.c) if bw is not None else None, fptr(ex), fptr(dW))


def mat_product(Cm, m, n, k, A, tA, B, tB, acc):
    lib().orc_mat_product(fptr(Cm), m, n, k, fptr(A), int(tA), fptr(B), int(tB), int(acc))


def dense_forward(P, D, N, act, bias, W, x, y):
    lib().orc_dense_forward(P, D, N, act, C.c_float(bias), fptr(W), fptr(x), fptr(y))


def dense_backward(P, D, N, act, bias, W, x, y, err, ex, dW):
    lib().orc_dense_backward(P, D, N, act, C.c_float(bias), fptr(W), fptr(x), fptr(y), fptr(err), fptr(ex),
                             fptr(dW))


def sse_error(D, N, pat, y, tgt):
    return float(lib().orc_sse_error(D, N, cptr(pat), fptr(y), fptr(tgt)))


def sse_backward(D, N, pat, y, tgt, err):
    lib().orc_sse_backward(D, N, cptr(pat), fptr(y), fptr(tgt), fptr(err))


def mdn_mixture_forward(F, Lp, startD, M, D, var_floor, pat, x, para):
    lib().orc_mdn_mixture_forward(F, Lp, startD, M, D, C.c_float(var_floor), cptr(pat), fptr(x), fptr(para))


def mdn_mixture_error(F, Lt, startDOut, M, D, pat, target, para, tmp):
    return float(lib().orc_mdn_mixture_error(F, Lt, startDOut, M, D, cptr(pat), fptr(target), fptr(para), fptr(tmp)))


def mdn_mixture_backward(F, Lp, Lt, startD, startDOut, M, D, var_floor, pat, target, para, tmp, errors):
    lib().orc_mdn_mixture_backward(F, Lp, Lt, startD, startDOut, M, D, C.c_float(var_floor), cptr(pat),
                                   fptr(target), fptr(para), fptr(tmp), fptr(errors))


def softmax_forward(F, Lp, startD, K, temperature, pat, x, prob):
    lib().orc_softmax_forward(F, Lp, startD, K, C.c_float(temperature), cptr(pat), fptr(x), fptr(prob))


def softmax_error(F, Lt, startDOut, K, cap, pat, target, prob):
    return float(lib().orc_softmax_error(F, Lt, startDOut, K, C.c_long(cap), cptr(pat), fptr(target), fptr(prob)))


def softmax_backward(F, Lp, Lt, startD, startDOut, K, pat, target, prob, errors):
    lib().orc_softmax_backward(F, Lp, Lt, startD, startDOut, K, cptr(pat), fptr(target), fptr(prob), fptr(errors))


IP = C.POINTER(C.c_int)


def iptr(a):
    assert a.dtype == np.int32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(IP)


def cnn_total_width(hw):
    return int(lib().orc_cnn_total_width(len(hw), iptr(hw)))


def cnn_forward(P, D, S, T, causal, out_tanh, bias, hw, inter, pat, W, x, conbuf, out):
    lib().orc_cnn_forward(P, D, S, T, causal, out_tanh, C.c_float(bias), iptr(hw), iptr(inter), cptr(pat), fptr(W),
                          fptr(x), fptr(conbuf), fptr(out))


def cnn_backward(P, D, S, T, causal, out_tanh, bias, hw, inter, pat, W, x, out, err, conbuf, ex, dW):
    lib().orc_cnn_backward(P, D, S, T, causal, out_tanh, C.c_float(bias), iptr(hw), iptr(inter), cptr(pat), fptr(W),
                           fptr(x), fptr(out), fptr(err), fptr(conbuf), fptr(ex), fptr(dW))


def wavnetc_load_context(Cdim, S, N, max_len, res_one, source, frame_index, mean_std, pat, ctx):
    lib().orc_wavnetc_load_context(Cdim, S, N, max_len, int(res_one), fptr(source), fptr(frame_index),
                                   fptr(mean_std), cptr(pat), fptr(ctx))


def wavnetc_forward(D, Cdim, N, pat, W, ctx, conv, core, ctx_tanh, out):
    lib().orc_wavnetc_forward(D, Cdim, N, cptr(pat), fptr(W), fptr(ctx), fptr(conv), fptr(core), fptr(ctx_tanh),
                              fptr(out))


def wavnetc_backward(D, Cdim, N, pat, W, ctx, core, ctx_tanh, err, prev_err, dW, ctx_grad):
    lib().orc_wavnetc_backward(D, Cdim, N, cptr(pat), fptr(W), fptr(ctx), fptr(core), fptr(ctx_tanh), fptr(err),
                               fptr(prev_err), fptr(dW), fptr(ctx_grad))


def wavnetc_sum_context_grad(Cdim, S, resolution, n_frame_slots, N, pat_frames, pat, ctx_grad, frame_grad):
    lib().orc_wavnetc_sum_context_grad(Cdim, S, resolution, n_frame_slots, N, cptr(pat_frames), cptr(pat),
                                       fptr(ctx_grad), fptr(frame_grad))


def gated_forward(D, N, pat, pre, out):
    lib().orc_gated_forward(D, N, cptr(pat), fptr(pre), fptr(out))


def gated_backward(D, N, pat, pre, err, prev_err):
    lib().orc_gated_backward(D, N, cptr(pat), fptr(pre), fptr(err), fptr(prev_err))


def _fpp(arrs):
    return (FP * len(arrs))(*[fptr(a) for a in arrs])


def skipadd_forward(inputs, out, errors, errors_from_skip):
    lib().orc_skipadd_forward(C.c_long(out.size), len(inputs), _fpp(inputs), fptr(out), fptr(errors),
                              fptr(errors_from_skip))


def skipadd_backward(errors, errors_from_skip, targets, is_skip):
    flags = (C.c_int * len(is_skip))(*[int(v) for v in is_skip])
    lib().orc_skipadd_backward(C.c_long(errors.size), fptr(errors), fptr(errors_from_skip), len(targets),
                               _fpp(targets), flags)


def dft_frame_count(n, frame_length, frame_shift):
    return int(lib().orc_dft_frame_count(n, frame_length, frame_shift))


def dft_r2c(x):
    n = len(x)
    out = np.zeros(2 * (n // 2 + 1), dtype=np.float32)
    lib().orc_dft_r2c(n, fptr(x), fptr(out))
    return out[0::2] + 1j * out[1::2]


def dft_c2r(X, n):
    buf = np.zeros(2 * (n // 2 + 1), dtype=np.float32)
    buf[0::2] = X.real
    buf[1::2] = X.imag
    out = np.zeros(n, dtype=np.float32)
    lib().orc_dft_c2r(n, fptr(buf), fptr(out))
    return out


def dft_logamp_loss(N, Nw, Hs, window_type, max_len, length, gamma, floor, src, tgt, grad):
    return float(lib().orc_dft_logamp_loss(N, Nw, Hs, window_type, max_len, length, C.c_float(gamma), C.c_float(floor),
                                           fptr(src), fptr(tgt), fptr(grad)))


def dft_spectral_loss(dis_type, N, Nw, Hs, window_type, max_len, length, gamma, floor, src, tgt, grad):
    return float(lib().orc_dft_spectral_loss(int(dis_type), N, Nw, Hs, window_type, max_len, length, C.c_float(gamma),
                                             C.c_float(floor), fptr(src), fptr(tgt), fptr(grad)))


def dft_phase_loss(N, Nw, Hs, window_type, max_len, length, zeta, src, tgt, grad):
    return float(lib().orc_dft_phase_loss(N, Nw, Hs, window_type, max_len, length, C.c_float(zeta), fptr(src),
                                          fptr(tgt), fptr(grad)))


def opt_accumulate(layer_updates, cur_updates, add):
    lib().orc_opt_accumulate(C.c_long(cur_updates.size), fptr(layer_updates), fptr(cur_updates), int(add))


def opt_adjust_gradient(option, g, stats, mask, frac_length, beta1_accum=0.0, beta2_accum=0.0):
    lib().orc_opt_adjust_gradient(int(option), C.c_long(g.size), fptr(g), fptr(stats) if stats is not None else None,
                                  fptr(mask) if mask is not None else None, C.c_float(frac_length),
                                  C.c_float(beta1_accum), C.c_float(beta2_accum))


def opt_update_weights(weights, g, deltas, mask, learning_rate, momentum):
    lib().orc_opt_update_weights(C.c_long(g.size), fptr(weights), fptr(g), fptr(deltas),
                                 fptr(mask) if mask is not None else None, C.c_float(learning_rate),
                                 C.c_float(momentum))


def opt_next_beta_accum(accum, which):
    return float(lib().orc_opt_next_beta_accum(accum, which))


def sigmoid_forward(F, Lp, startD, K, pat, x, prob):
    lib().orc_sigmoid_forward(F, Lp, startD, K, cptr(pat), fptr(x), fptr(prob))


def sigmoid_error(F, Lt, startDOut, K, continuous, pat, target, prob):
    return float(lib().orc_sigmoid_error(F, Lt, startDOut, K, int(continuous), cptr(pat), fptr(target), fptr(prob)))


def sigmoid_backward(F, Lp, Lt, startD, startDOut, K, continuous, pat, target, prob, errors):
    lib().orc_sigmoid_backward(F, Lp, Lt, startD, startDOut, K, int(continuous), cptr(pat), fptr(target), fptr(prob),
                               fptr(errors))
