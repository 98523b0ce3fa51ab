"""ctypes binding of libcurrennt_hip.so.  Device buffers are passed as raw pointers (torch tensors'
data_ptr()); every call checks the returned status and raises RuntimeError with cnt_last_error()."""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libcurrennt_hip.so")

CNT_OK = 0
ACT = {"identity": 0, "tanh": 1, "logistic": 2, "relu": 3}

LSTM_STATE = {"ni": 0, "ig": 1, "fg": 2, "og": 3, "c": 4, "h": 5, "herr": 6, "dni": 7, "dig": 8, "dfg": 9,
              "dog": 10, "cerr": 11}


class MdnDesc(C.Structure):
    _fields_ = [("Lp", C.c_int), ("Lt", C.c_int), ("S", C.c_int), ("maxT", C.c_int), ("tie_variance", C.c_int),
                ("sigmoid_continuous", C.c_int)]


class CnnDesc(C.Structure):
    _fields_ = [("P", C.c_int), ("D", C.c_int), ("S", C.c_int), ("maxT", C.c_int), ("causal", C.c_int),
                ("output_tanh", C.c_int), ("bias", C.c_float)]


class DftDesc(C.Structure):
    _fields_ = [("n_res", C.c_int), ("fft_length", C.c_int * 3), ("frame_length", C.c_int * 3),
                ("frame_shift", C.c_int * 3), ("window_type", C.c_int * 3), ("gamma", C.c_float),
                ("log_floor", C.c_float), ("spec_dis_type", C.c_int), ("max_length", C.c_int), ("max_waves", C.c_int),
                ("zeta", C.c_float), ("phase_dis_type", C.c_int)]


class DatasetDesc(C.Structure):
    _fields_ = [("parallel_sequences", C.c_int), ("training_mode", C.c_int), ("truncate_seq", C.c_int),
                ("fraction", C.c_float)]


class NetworkOptions(C.Structure):
    _fields_ = [("mdn_config", C.POINTER(C.c_float)), ("mdn_config_len", C.c_int), ("tie_variance", C.c_int),
                ("no_overlap", C.c_int)]


class LayerInfo(C.Structure):
    _fields_ = [("name", C.c_char * 64), ("type", C.c_char * 32), ("size", C.c_int), ("weight_offset", C.c_long),
                ("n_input", C.c_long), ("n_bias", C.c_long), ("n_internal", C.c_long), ("outputs", C.c_void_p),
                ("output_errors", C.c_void_p), ("resolution", C.c_int)]


class LstmDesc(C.Structure):
    _fields_ = [("P", C.c_int), ("L", C.c_int), ("bidir", C.c_int), ("S", C.c_int), ("maxT", C.c_int),
                ("bias", C.c_float)]


_lib = None

VP = C.c_void_p
I = C.c_int
F = C.c_float

_SIGNATURES = {
    "cnt_version": (I, []),
    "cnt_last_error": (C.c_char_p, []),
    "cnt_profile_enable": (I, [I]),
    "cnt_profile_get": (I, [I, C.c_char_p, I, C.POINTER(I), C.POINTER(F)]),
    "cnt_matrix_product": (I, [VP, VP, I, I, I, VP, I, VP, I, I]),
    "cnt_dense_forward": (I, [VP, I, I, I, I, F, VP, VP, VP]),
    "cnt_dense_backward": (I, [VP, I, I, I, I, F, VP, VP, VP, VP, VP, VP]),
    "cnt_dense_backward_errors": (I, [VP, I, I, I, I, VP, VP, VP, VP]),
    "cnt_dense_backward_weights": (I, [VP, I, I, I, F, VP, VP, VP]),
    "cnt_dense_backward_weights_static": (I, [VP, I, I, I, F, VP, VP, VP]),
    "cnt_probe_hop_latency": (I, [VP, I, I, I, C.POINTER(F)]),
    "cnt_probe_hop_message": (I, [VP, I, I, C.POINTER(F)]),
    "cnt_probe_activation": (I, [VP, I, C.c_long, VP, VP]),
    "cnt_gemm_reserve": (I, [VP]),
    "cnt_gemm_release": (I, [VP]),
    "cnt_gemm_scratch_buffers": (I, []),
    "cnt_sse_backward": (I, [VP, I, I, VP, VP, VP, VP]),
    "cnt_sse_error": (I, [VP, I, I, VP, VP, VP, VP]),
    "cnt_dataset_open": (I, [C.c_char_p, C.POINTER(DatasetDesc), C.POINTER(VP)]),
    "cnt_dataset_close": (I, [VP]),
    "cnt_dataset_shuffle": (I, [VP, I, I, C.c_uint]),
    "cnt_dataset_info": (I, [VP, C.POINTER(I), C.POINTER(I), C.POINTER(I), C.POINTER(I), C.POINTER(C.c_long),
                             C.POINTER(I), C.POINTER(I)]),
    "cnt_dataset_sequence": (I, [VP, I, C.POINTER(I), C.POINTER(I), C.c_char_p, I]),
    "cnt_dataset_fraction_shape": (I, [VP, I, C.POINTER(I), C.POINTER(I), C.POINTER(I), C.POINTER(I)]),
    "cnt_dataset_fraction_fill": (I, [VP, I, VP, VP, VP, VP]),
    "cnt_opt_accumulate": (I, [VP, C.c_long, VP, VP, I]),
    "cnt_opt_adjust_gradient": (I, [VP, I, C.c_long, VP, VP, VP, F, F, F]),
    "cnt_opt_update_weights": (I, [VP, C.c_long, VP, VP, VP, VP, F, F]),
    "cnt_opt_step": (I, [VP, I, C.c_long, VP, VP, VP, VP, VP, VP, F, F, F, F, F]),
    "cnt_opt_next_beta_accum": (F, [F, I]),
    "cnt_lstm_create": (I, [C.POINTER(LstmDesc), C.POINTER(VP)]),
    "cnt_lstm_destroy": (I, [VP]),
    "cnt_lstm_load_sequences": (I, [VP, VP, VP, I, I]),
    "cnt_lstm_forward": (I, [VP, VP, VP, VP, VP]),
    "cnt_lstm_backward": (I, [VP, VP, VP, VP, VP, VP, VP, VP]),
    "cnt_lstm_backward_errors": (I, [VP, VP, VP, VP, VP]),
    "cnt_lstm_backward_weights": (I, [VP, VP, VP, VP]),
    "cnt_lstm_backward_prev_errors": (I, [VP, VP, VP, VP]),
    "cnt_lstm_backward_can_split": (I, [VP]),
    "cnt_lstm_backward_errors_range": (I, [VP, VP, VP, VP, I, I]),
    "cnt_lstm_backward_steps_done": (I, [VP, I, C.POINTER(I), C.POINTER(I)]),
    "cnt_lstm_backward_prev_errors_range": (I, [VP, VP, VP, VP, I, I]),
    "cnt_lstm_set_wait_bounds": (I, [VP, C.c_uint, I, I]),
    "cnt_network_set_wait_bounds": (I, [VP, I, C.c_uint, I, I]),
    "cnt_lstm_state": (VP, [VP, I, I]),
    "cnt_lstm_weight_count": (C.c_long, [I, I, I]),
    "cnt_lstm_check": (I, [VP, VP]),
    "cnt_mdn_create": (I, [C.POINTER(MdnDesc), C.POINTER(F), I, C.POINTER(VP)]),
    "cnt_mdn_destroy": (I, [VP]),
    "cnt_mdn_set_var_floor": (I, [VP, I, F]),
    "cnt_mdn_load_sequences": (I, [VP, VP, VP, I]),
    "cnt_mdn_forward": (I, [VP, VP, VP]),
    "cnt_mdn_calculate_error": (I, [VP, VP, VP, VP]),
    "cnt_mdn_backward": (I, [VP, VP, VP, VP]),
    "cnt_mdn_error_backward": (I, [VP, VP, VP, VP, VP]),
    "cnt_mdn_unit_buffer": (VP, [VP, I, I, C.POINTER(C.c_long)]),
    "cnt_dft_create": (I, [C.POINTER(DftDesc), C.POINTER(VP)]),
    "cnt_dft_destroy": (I, [VP]),
    "cnt_dft_forward": (I, [VP, VP, I, C.POINTER(I), VP, VP, VP]),
    "cnt_dft_backward": (I, [VP, VP, VP]),
    "cnt_cnn_create": (I, [C.POINTER(CnnDesc), C.POINTER(I), C.POINTER(I), C.POINTER(VP)]),
    "cnt_cnn_destroy": (I, [VP]),
    "cnt_cnn_weight_count": (C.c_long, [VP]),
    "cnt_cnn_forward": (I, [VP, VP, VP, I, VP, VP, VP]),
    "cnt_cnn_backward": (I, [VP, VP, VP, I, VP, VP, VP, VP, VP, VP]),
    "cnt_cnn_backward_errors": (I, [VP, VP, VP, I, VP, VP, VP, VP, I]),
    "cnt_cnn_backward_weights": (I, [VP, VP, VP, I, VP, VP, VP]),
    "cnt_wavnetc_backward_errors": (I, [VP, I, I, I, VP, VP, VP, VP, VP, VP, VP, VP]),
    "cnt_wavnetc_backward_weights": (I, [VP, I, I, I, VP, VP, VP]),
    "cnt_wavnetc_load_context": (I, [VP, I, I, I, I, I, VP, VP, VP, VP, VP]),
    "cnt_wavnetc_forward": (I, [VP, I, I, I, VP, VP, VP, VP, VP, VP, VP]),
    "cnt_wavnetc_backward": (I, [VP, I, I, I, VP, VP, VP, VP, VP, VP, VP, VP, VP]),
    "cnt_wavnetc_sum_context_grad": (I, [VP, I, I, I, I, I, VP, VP, VP, VP]),
    "cnt_gatedact_forward": (I, [VP, I, I, VP, VP, VP]),
    "cnt_gatedact_backward": (I, [VP, I, I, VP, VP, VP, VP]),
    "cnt_network_create": (I, [C.c_char_p, I, I, C.POINTER(NetworkOptions), C.POINTER(VP)]),
    "cnt_network_destroy": (I, [VP]),
    "cnt_network_info": (I, [VP, C.POINTER(I), C.POINTER(I), C.POINTER(I), C.POINTER(C.c_long)]),
    "cnt_network_layer_info": (I, [VP, I, C.POINTER(LayerInfo)]),
    "cnt_network_weights": (VP, [VP]),
    "cnt_network_weight_updates": (VP, [VP]),
    "cnt_network_randomize": (I, [VP, C.c_uint, F]),
    "cnt_network_set_context": (I, [VP, VP]),
    "cnt_network_set_external_input": (I, [VP, I, VP, I, VP]),
    "cnt_network_load_sequences": (I, [VP, VP, I, I, VP, VP, VP]),
    "cnt_network_forward": (I, [VP, VP]),
    "cnt_network_calculate_error": (I, [VP, VP, VP]),
    "cnt_network_backward": (I, [VP, VP]),
    "cnt_network_check": (I, [VP, VP]),
    "cnt_network_update": (I, [VP, VP, I, F, F, F]),
    "cnt_network_export_json": (I, [VP, C.c_char_p, C.c_size_t, C.POINTER(C.c_size_t)]),
    "cnt_skipadd_forward": (I, [VP, C.c_long, I, C.POINTER(VP), VP, VP, VP]),
    "cnt_skipadd_backward": (I, [VP, C.c_long, VP, VP, I, C.POINTER(VP), C.POINTER(I)]),
}


def exported_symbols():
    return sorted(_SIGNATURES)


def lib():
    """Loads the library; raises if it has not been built (there is no fallback path)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libcurrennt_hip.so is not built (%s); run __graft_entry__.build()" % LIB_PATH)
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(status):
    if status != CNT_OK:
        raise RuntimeError("currennt_hip error %d: %s" % (status, lib().cnt_last_error().decode(errors="replace")))


def ptr(t):
    """Raw device pointer of a torch tensor (or None)."""
    if t is None:
        return None
    return C.c_void_p(t.data_ptr())


def stream_ptr(stream=None):
    import torch

    s = stream if stream is not None else torch.cuda.current_stream()
    return C.c_void_p(s.cuda_stream)


def profile_enable(on):
    check(lib().cnt_profile_enable(int(on)))


def profile_read():
    """{label: (launches, total_ms)} of everything recorded since profile_enable(True)."""
    out = {}
    i = 0
    while True:
        buf = C.create_string_buffer(128)
        n, ms = I(0), F(0.0)
        if lib().cnt_profile_get(i, buf, 128, C.byref(n), C.byref(ms)) != CNT_OK:
            break
        out[buf.value.decode()] = (n.value, ms.value)
        i += 1
    return out


def matrix_product(Cm, m, n, k, A, tA, B, tB, accumulate, stream=None):
    check(lib().cnt_matrix_product(stream_ptr(stream), ptr(Cm), m, n, k, ptr(A), int(tA), ptr(B), int(tB),
                                   int(accumulate)))


def dense_forward(P, D, N, act, bias, W, x, y, stream=None):
    check(lib().cnt_dense_forward(stream_ptr(stream), P, D, N, act, bias, ptr(W), ptr(x), ptr(y)))


def dense_backward(P, D, N, act, bias, W, x, y, err, prev_err, dW, stream=None):
    check(lib().cnt_dense_backward(stream_ptr(stream), P, D, N, act, bias, ptr(W), ptr(x), ptr(y), ptr(err),
                                   ptr(prev_err), ptr(dW)))


def dense_backward_errors(P, D, N, act, W, y, err, prev_err, stream=None):
    check(lib().cnt_dense_backward_errors(stream_ptr(stream), P, D, N, act, ptr(W), ptr(y), ptr(err), ptr(prev_err)))


def dense_backward_weights(P, D, N, bias, x, err, dW, stream=None):
    check(lib().cnt_dense_backward_weights(stream_ptr(stream), P, D, N, bias, ptr(x), ptr(err), ptr(dW)))


def dense_backward_weights_static(P, D, N, bias, x, err, dW, stream=None):
    check(lib().cnt_dense_backward_weights_static(stream_ptr(stream), P, D, N, bias, ptr(x), ptr(err), ptr(dW)))


def probe_hop_latency(same_xcd=True, with_compute=True, rounds=2000, stream=None):
    """Microseconds per hop of a word between two workgroups (see cnt_probe_hop_latency)."""
    out = F(0.0)
    check(lib().cnt_probe_hop_latency(stream_ptr(stream), int(same_xcd), int(with_compute), int(rounds), C.byref(out)))
    return float(out.value)


def probe_hop_message(kilobytes=4, rounds=2000, stream=None):
    """Microseconds per hop of a message of 4..16 KB between two four-wave workgroups on one XCD."""
    out = F(0.0)
    check(lib().cnt_probe_hop_message(stream_ptr(stream), int(kilobytes), int(rounds), C.byref(out)))
    return float(out.value)


def probe_activation(which, x, out, stream=None):
    check(lib().cnt_probe_activation(stream_ptr(stream), int(which), x.numel(), ptr(x), ptr(out)))


def gemm_reserve(stream=None):
    check(lib().cnt_gemm_reserve(stream_ptr(stream)))


def gemm_release(stream=None):
    check(lib().cnt_gemm_release(stream_ptr(stream)))


def sse_backward(D, N, pat, y, tgt, err, stream=None):
    check(lib().cnt_sse_backward(stream_ptr(stream), D, N, ptr(pat), ptr(y), ptr(tgt), ptr(err)))


def sse_error(D, N, pat, y, tgt, result, stream=None):
    check(lib().cnt_sse_error(stream_ptr(stream), D, N, ptr(pat), ptr(y), ptr(tgt), ptr(result)))


class Dataset:
    """One .nc file as the reference's data_sets::DataSet sees it; fractions come back as numpy arrays."""

    def __init__(self, path, parallel_sequences, training_mode=True, truncate_seq=0, fraction=1.0):
        self.handle = VP()
        self.S = parallel_sequences
        desc = DatasetDesc(parallel_sequences, int(training_mode), truncate_seq, fraction)
        check(lib().cnt_dataset_open(path.encode(), C.byref(desc), C.byref(self.handle)))
        n, p, q, cls, mn, mx = I(), I(), I(), I(), I(), I()
        tot = C.c_long()
        check(lib().cnt_dataset_info(self.handle, C.byref(n), C.byref(p), C.byref(q), C.byref(cls), C.byref(tot),
                                     C.byref(mn), C.byref(mx)))
        self.num_sequences, self.input_size, self.output_size = n.value, p.value, q.value
        self.is_classification, self.total_timesteps = bool(cls.value), tot.value
        self.min_len, self.max_len = mn.value, mx.value

    def shuffle(self, sequences, fractions, seed=0):
        """What the reference does at the start of an epoch with --shuffle_sequences / --shuffle_fractions."""
        check(lib().cnt_dataset_shuffle(self.handle, int(sequences), int(fractions), seed))

    def sequence(self, index):
        length, orig = I(), I()
        tag = C.create_string_buffer(512)
        check(lib().cnt_dataset_sequence(self.handle, index, C.byref(length), C.byref(orig), tag, 512))
        return length.value, orig.value, tag.value.decode()

    def fraction(self, first_seq):
        import numpy as np

        n, mx, mn, tot = I(), I(), I(), I()
        check(lib().cnt_dataset_fraction_shape(self.handle, first_seq, C.byref(n), C.byref(mx), C.byref(mn), C.byref(tot)))
        slots = mx.value * self.S
        pat = np.zeros(slots, np.int8)
        x = np.zeros(slots * self.input_size, np.float32)
        tgt = np.zeros(slots * self.output_size, np.float32) if not self.is_classification else None
        cls = np.zeros(slots, np.int32) if self.is_classification else None
        as_ptr = lambda a: a.ctypes.data_as(VP) if a is not None else None
        check(lib().cnt_dataset_fraction_fill(self.handle, first_seq, as_ptr(pat), as_ptr(x), as_ptr(tgt), as_ptr(cls)))
        return {"num_seqs": n.value, "max_len": mx.value, "min_len": mn.value, "total_length": tot.value,
                "patTypes": pat, "inputs": x, "targets": tgt, "target_classes": cls}

    def close(self):
        if self.handle:
            lib().cnt_dataset_close(self.handle)
            self.handle = VP()


OPT_SGD, OPT_ADAGRAD, OPT_AVEGRAD, OPT_STOCHASTIC_ADAGRAD, OPT_SGD_DECAY, OPT_ADAM = 0, 1, 2, 3, 4, 5


def opt_accumulate(layer_updates, cur_updates, add, stream=None):
    check(lib().cnt_opt_accumulate(stream_ptr(stream), layer_updates.numel(), ptr(layer_updates), ptr(cur_updates), int(add)))


def opt_adjust_gradient(option, cur_updates, stats, mask, frac_length, beta1_accum=0.0, beta2_accum=0.0, stream=None):
    check(lib().cnt_opt_adjust_gradient(stream_ptr(stream), option, cur_updates.numel(), ptr(cur_updates), ptr(stats),
                                        ptr(mask), frac_length, beta1_accum, beta2_accum))


def opt_update_weights(weights, cur_updates, deltas, mask, learning_rate, momentum, stream=None):
    check(lib().cnt_opt_update_weights(stream_ptr(stream), weights.numel(), ptr(weights), ptr(cur_updates), ptr(deltas),
                                       ptr(mask), learning_rate, momentum))


def opt_step(option, weights, layer_updates, cur_updates, stats, deltas, mask, frac_length, beta1_accum, beta2_accum,
             learning_rate, momentum, stream=None):
    check(lib().cnt_opt_step(stream_ptr(stream), option, weights.numel(), ptr(weights), ptr(layer_updates),
                             ptr(cur_updates), ptr(stats), ptr(deltas), ptr(mask), frac_length, beta1_accum,
                             beta2_accum, learning_rate, momentum))


def opt_next_beta_accum(accum, which):
    return float(lib().cnt_opt_next_beta_accum(accum, which))


class Lstm:
    """Thin owner of a cnt_lstm handle."""

    def __init__(self, P, L, bidir, S, maxT, bias=1.0):
        self.P, self.L, self.bidir, self.S, self.maxT = P, L, bool(bidir), S, maxT
        self.H = L // (2 if bidir else 1)
        self.handle = VP()
        desc = LstmDesc(P, L, int(bidir), S, maxT, bias)
        check(lib().cnt_lstm_create(C.byref(desc), C.byref(self.handle)))
        self.T = 0

    def close(self):
        if self.handle:
            lib().cnt_lstm_destroy(self.handle)
            self.handle = VP()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def load_sequences(self, pat, T, Tmin, stream=None):
        self._pat = pat  # keep the device buffer alive
        self.T = T
        check(lib().cnt_lstm_load_sequences(self.handle, stream_ptr(stream), ptr(pat), T, Tmin))

    def forward(self, W, x, out, stream=None):
        check(lib().cnt_lstm_forward(self.handle, stream_ptr(stream), ptr(W), ptr(x), ptr(out)))

    def backward(self, W, x, out, outerr, prev_err, dW, stream=None):
        check(lib().cnt_lstm_backward(self.handle, stream_ptr(stream), ptr(W), ptr(x), ptr(out), ptr(outerr),
                                      ptr(prev_err), ptr(dW)))

    def backward_errors(self, W, outerr, prev_err, stream=None):
        check(lib().cnt_lstm_backward_errors(self.handle, stream_ptr(stream), ptr(W), ptr(outerr), ptr(prev_err)))

    def backward_weights(self, x, dW, stream=None):
        check(lib().cnt_lstm_backward_weights(self.handle, stream_ptr(stream), ptr(x), ptr(dW)))

    def set_wait_bounds(self, spin_limit, poll_delay_backward, poll_delay_forward):
        check(lib().cnt_lstm_set_wait_bounds(self.handle, spin_limit, poll_delay_backward, poll_delay_forward))

    def backward_prev_errors(self, W, prev_err, stream=None):
        check(lib().cnt_lstm_backward_prev_errors(self.handle, stream_ptr(stream), ptr(W), ptr(prev_err)))

    def backward_can_split(self):
        return bool(lib().cnt_lstm_backward_can_split(self.handle))

    def backward_errors_range(self, W, outerr, step_begin, step_end, stream=None):
        check(lib().cnt_lstm_backward_errors_range(self.handle, stream_ptr(stream), ptr(W), ptr(outerr), step_begin, step_end))

    def backward_steps_done(self, steps):
        a, b = I(0), I(0)
        check(lib().cnt_lstm_backward_steps_done(self.handle, steps, C.byref(a), C.byref(b)))
        return a.value, b.value

    def backward_prev_errors_range(self, W, prev_err, t_begin, t_end, stream=None):
        check(lib().cnt_lstm_backward_prev_errors_range(self.handle, stream_ptr(stream), ptr(W), ptr(prev_err), t_begin, t_end))

    def check(self, stream=None):
        check(lib().cnt_lstm_check(self.handle, stream_ptr(stream)))

    def state(self, direction, name):
        """Copy of one internal H x (T*S) buffer as a torch tensor."""
        import torch

        p = lib().cnt_lstm_state(self.handle, direction, LSTM_STATE[name])
        if not p:
            raise RuntimeError("no such LSTM state buffer: %r direction %d" % (name, direction))
        n = self.H * self.T * self.S
        torch.cuda.synchronize()
        return torch.as_tensor(_DeviceArray(p, n), device="cuda").clone()


class Cnn:
    """Thin owner of a cnt_cnn handle (1-D convolution layer)."""

    def __init__(self, P, half_width, interval, S, maxT, causal, output_tanh, bias=1.0):
        D = len(half_width)
        self.P, self.D, self.S, self.maxT = P, D, S, maxT
        self.handle = VP()
        desc = CnnDesc(P, D, S, maxT, int(causal), int(output_tanh), bias)
        hw = (I * D)(*[int(v) for v in half_width])
        it = (I * D)(*[int(v) for v in interval])
        check(lib().cnt_cnn_create(C.byref(desc), hw, it, C.byref(self.handle)))
        self.weight_count = int(lib().cnt_cnn_weight_count(self.handle))

    def close(self):
        if self.handle:
            lib().cnt_cnn_destroy(self.handle)
            self.handle = VP()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def forward(self, pat, T, W, x, out, stream=None):
        check(lib().cnt_cnn_forward(self.handle, stream_ptr(stream), ptr(pat), T, ptr(W), ptr(x), ptr(out)))

    def backward(self, pat, T, W, x, out, err, prev_err, dW, stream=None):
        check(lib().cnt_cnn_backward(self.handle, stream_ptr(stream), ptr(pat), T, ptr(W), ptr(x), ptr(out), ptr(err),
                                     ptr(prev_err), ptr(dW)))


def wavnetc_load_context(Cdim, S, N, max_len, res_one, source, frame_index, mean_std, pat, ctx, stream=None):
    check(lib().cnt_wavnetc_load_context(stream_ptr(stream), Cdim, S, N, max_len, int(res_one), ptr(source),
                                         ptr(frame_index), ptr(mean_std), ptr(pat), ptr(ctx)))


def wavnetc_forward(D, Cdim, N, pat, W, ctx, conv, core, ctx_tanh, out, stream=None):
    check(lib().cnt_wavnetc_forward(stream_ptr(stream), D, Cdim, N, ptr(pat), ptr(W), ptr(ctx), ptr(conv), ptr(core),
                                    ptr(ctx_tanh), ptr(out)))


def wavnetc_backward(D, Cdim, N, pat, W, ctx, core, ctx_tanh, err, prev_err, dW, ctx_grad, stream=None):
    check(lib().cnt_wavnetc_backward(stream_ptr(stream), D, Cdim, N, ptr(pat), ptr(W), ptr(ctx), ptr(core),
                                     ptr(ctx_tanh), ptr(err), ptr(prev_err), ptr(dW), ptr(ctx_grad)))


def wavnetc_sum_context_grad(Cdim, S, resolution, n_frame_slots, N, pat_frames, pat, ctx_grad, frame_grad, stream=None):
    check(lib().cnt_wavnetc_sum_context_grad(stream_ptr(stream), Cdim, S, resolution, n_frame_slots, N,
                                             ptr(pat_frames), ptr(pat), ptr(ctx_grad), ptr(frame_grad)))


def gatedact_forward(D, N, pat, pre, out, stream=None):
    check(lib().cnt_gatedact_forward(stream_ptr(stream), D, N, ptr(pat), ptr(pre), ptr(out)))


def gatedact_backward(D, N, pat, pre, err, prev_err, stream=None):
    check(lib().cnt_gatedact_backward(stream_ptr(stream), D, N, ptr(pat), ptr(pre), ptr(err), ptr(prev_err)))


def _ptr_array(tensors):
    return (VP * len(tensors))(*[t.data_ptr() for t in tensors])


def skipadd_forward(inputs, out, errors, errors_from_skip, stream=None):
    check(lib().cnt_skipadd_forward(stream_ptr(stream), out.numel(), len(inputs), _ptr_array(inputs), ptr(out),
                                    ptr(errors), ptr(errors_from_skip)))


def skipadd_backward(errors, errors_from_skip, targets, is_skip, stream=None):
    flags = (I * len(is_skip))(*[int(v) for v in is_skip])
    check(lib().cnt_skipadd_backward(stream_ptr(stream), errors.numel(), ptr(errors), ptr(errors_from_skip),
                                     len(targets), _ptr_array(targets), flags))


class Network:
    """Thin owner of a cnt_network handle (the C++ sequencer).  Device memory belongs to the handle; `weights`,
    `updates`, and a layer's `outputs` / `errors` are torch views of it (no copies)."""

    def __init__(self, json_text, parallel_sequences, max_seq_length, mdn_config=None, overlap=True):
        import torch

        self.S, self.maxT = parallel_sequences, max_seq_length
        opt = NetworkOptions()
        self._cfg = None
        if mdn_config is not None:
            self._cfg = (F * len(mdn_config))(*[float(v) for v in mdn_config])
            opt.mdn_config, opt.mdn_config_len = self._cfg, len(mdn_config)
        opt.no_overlap = 0 if overlap else 1
        self.handle = VP()
        check(lib().cnt_network_create(json_text.encode(), parallel_sequences, max_seq_length, C.byref(opt),
                                       C.byref(self.handle)))
        n_layers, n_in, n_out, n_w = I(), I(), I(), C.c_long()
        check(lib().cnt_network_info(self.handle, C.byref(n_layers), C.byref(n_in), C.byref(n_out), C.byref(n_w)))
        self.n_layers, self.input_size, self.output_size, self.n_weights = n_layers.value, n_in.value, n_out.value, n_w.value
        self.weights = _device_view(lib().cnt_network_weights(self.handle), self.n_weights, self)
        self.updates = _device_view(lib().cnt_network_weight_updates(self.handle), self.n_weights, self)
        self.layers = []
        for i in range(self.n_layers):
            info = LayerInfo()
            check(lib().cnt_network_layer_info(self.handle, i, C.byref(info)))
            n = info.n_input + info.n_bias + info.n_internal
            slots = parallel_sequences * (-(-max_seq_length // info.resolution))
            self.layers.append({
                "name": info.name.decode(), "type": info.type.decode(), "size": info.size,
                "weight_offset": info.weight_offset, "weight_count": n,
                "sections": (info.n_input, info.n_bias, info.n_internal), "resolution": info.resolution,
                "outputs": _device_view(info.outputs, info.size * slots, self),
                "errors": _device_view(info.output_errors, info.size * slots, self),
                "weights": self.weights[info.weight_offset:info.weight_offset + n] if n else None,
                "updates": self.updates[info.weight_offset:info.weight_offset + n] if n else None,
            })
        self.loss = torch.zeros(1, dtype=torch.float32, device="cuda")

    def layer(self, name):
        for L in self.layers:
            if L["name"] == name:
                return L
        raise KeyError(name)

    def close(self):
        if self.handle:
            lib().cnt_network_destroy(self.handle)
            self.handle = VP()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def randomize(self, seed, weight_range):
        check(lib().cnt_network_randomize(self.handle, seed, weight_range))

    def set_context(self, ctx):
        self._ctx = ctx  # the library keeps the pointer only
        check(lib().cnt_network_set_context(self.handle, ptr(ctx)))

    def set_external_input(self, layer_name, data, max_frames, mean_std=None):
        index = [L["name"] for L in self.layers].index(layer_name)
        self._ext = getattr(self, "_ext", {})
        self._ext[layer_name] = (data, mean_std)  # the library keeps the pointers only
        check(lib().cnt_network_set_external_input(self.handle, index, ptr(data), max_frames, ptr(mean_std)))

    def load_sequences(self, pat, T, Tmin, inputs=None, targets=None, stream=None):
        self._pat = pat
        check(lib().cnt_network_load_sequences(self.handle, stream_ptr(stream), T, Tmin, ptr(pat), ptr(inputs),
                                               ptr(targets)))

    def forward(self, stream=None):
        check(lib().cnt_network_forward(self.handle, stream_ptr(stream)))

    def calculate_error(self, stream=None):
        check(lib().cnt_network_calculate_error(self.handle, stream_ptr(stream), ptr(self.loss)))
        return self.loss

    def backward(self, stream=None):
        check(lib().cnt_network_backward(self.handle, stream_ptr(stream)))

    def check(self, stream=None):
        check(lib().cnt_network_check(self.handle, stream_ptr(stream)))

    def set_wait_bounds(self, layer_index, spin_limit, poll_delay_backward, poll_delay_forward):
        check(lib().cnt_network_set_wait_bounds(self.handle, layer_index, spin_limit, poll_delay_backward,
                                                poll_delay_forward))

    def update(self, option, learning_rate, momentum, frac_length, stream=None):
        check(lib().cnt_network_update(self.handle, stream_ptr(stream), option, learning_rate, momentum, frac_length))

    def export_json(self):
        need = C.c_size_t()
        check(lib().cnt_network_export_json(self.handle, None, 0, C.byref(need)))
        buf = C.create_string_buffer(need.value)
        check(lib().cnt_network_export_json(self.handle, buf, need.value, C.byref(need)))
        return buf.value.decode()


def _device_view(address, count, owner):
    """float32 torch tensor over `count` floats of device memory that `owner` keeps alive (None for a null pointer)."""
    import torch

    if not address or count == 0:
        return None

    class _Span:
        pass

    span = _Span()
    span.__cuda_array_interface__ = {"shape": (count,), "typestr": "<f4", "data": (int(address), False), "version": 3}
    span.owner = owner
    return torch.as_tensor(span, device="cuda")


class Dft:
    """Thin owner of a cnt_dft handle.  resolutions: list of (fftLength, frameLength, frameShift)."""

    def __init__(self, resolutions, max_length, max_waves, gamma=1.0, log_floor=1e-5, window_type=0, spec_dis_type=0,
                 zeta=0.0, phase_dis_type=0):
        d = DftDesc()
        d.n_res = len(resolutions)
        for r, (n, nw, hs) in enumerate(resolutions[:3]):
            d.fft_length[r], d.frame_length[r], d.frame_shift[r], d.window_type[r] = n, nw, hs, window_type
        d.gamma, d.log_floor, d.spec_dis_type = gamma, log_floor, spec_dis_type
        d.max_length, d.max_waves = max_length, max_waves
        d.zeta, d.phase_dis_type = zeta, phase_dis_type
        self.n_res = d.n_res
        self.handle = VP()
        check(lib().cnt_dft_create(C.byref(d), C.byref(self.handle)))

    def close(self):
        if self.handle:
            lib().cnt_dft_destroy(self.handle)
            self.handle = VP()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def forward(self, lengths, source, target, errors, stream=None):
        arr = (I * len(lengths))(*[int(v) for v in lengths])
        check(lib().cnt_dft_forward(self.handle, stream_ptr(stream), len(lengths), arr, ptr(source), ptr(target),
                                    ptr(errors)))

    def backward(self, prev_errors, stream=None):
        check(lib().cnt_dft_backward(self.handle, stream_ptr(stream), ptr(prev_errors)))


class Mdn:
    """Thin owner of a cnt_mdn handle.  config: flat list [n, (startD, endD, startDOut, endDOut, type) * n]."""

    def __init__(self, Lp, Lt, S, maxT, config, tie_variance=False, sigmoid_continuous=False):
        self.handle = VP()
        desc = MdnDesc(Lp, Lt, S, maxT, int(tie_variance), int(sigmoid_continuous))
        arr = (F * len(config))(*[float(v) for v in config])
        check(lib().cnt_mdn_create(C.byref(desc), arr, len(config), C.byref(self.handle)))

    def close(self):
        if self.handle:
            lib().cnt_mdn_destroy(self.handle)
            self.handle = VP()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def set_var_floor(self, unit, v):
        check(lib().cnt_mdn_set_var_floor(self.handle, unit, v))

    def load_sequences(self, pat, T, stream=None):
        self._pat = pat
        check(lib().cnt_mdn_load_sequences(self.handle, stream_ptr(stream), ptr(pat), T))

    def forward(self, x, stream=None):
        check(lib().cnt_mdn_forward(self.handle, stream_ptr(stream), ptr(x)))

    def calculate_error(self, targets, result, stream=None):
        check(lib().cnt_mdn_calculate_error(self.handle, stream_ptr(stream), ptr(targets), ptr(result)))

    def backward(self, targets, prev_errors, stream=None):
        check(lib().cnt_mdn_backward(self.handle, stream_ptr(stream), ptr(targets), ptr(prev_errors)))

    def error_backward(self, targets, result, prev_errors, stream=None):
        check(lib().cnt_mdn_error_backward(self.handle, stream_ptr(stream), ptr(targets), ptr(result), ptr(prev_errors)))

    def unit_buffer(self, unit, which):
        import torch

        n = C.c_long(0)
        p = lib().cnt_mdn_unit_buffer(self.handle, unit, which, C.byref(n))
        if not p:
            raise RuntimeError("no such MDN unit buffer")
        torch.cuda.synchronize()
        return torch.as_tensor(_DeviceArray(p, n.value), device="cuda").clone()


class _DeviceArray:
    """Exposes a raw device pointer of n floats through __cuda_array_interface__."""

    def __init__(self, pointer, n):
        self.__cuda_array_interface__ = {"shape": (n,), "typestr": "<f4", "data": (int(pointer), False),
                                         "version": 2}
