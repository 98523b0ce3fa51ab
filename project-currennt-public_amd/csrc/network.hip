// Network sequencer: builds the layer list of a network file and runs forward pass, error, backward pass and
// weight update of one fraction through the layer entry points of this library.
//
// Reference behaviour: NeuralNetwork.cpp (:374-609 constructor with the skip-layer and wavnetc wiring, :805-812
// feedback link, :1367-1417 loadSequences, :1419-1471 layer-by-layer forward pass, :2744-2800 backward pass in
// reverse order, :2897-2990 calculateError, :2993-3040 exportLayers / exportWeights), layers/TrainableLayer.cu
// (:93-220 weight sections of a network file, :441-492 export), layers/SkipAddLayer.cu (:77-170 preSkipLayer, :186-240, :305-346),
// layers/FeedBackLayer.cu (:60-130, :607-650, :841-865), layers/MDNUnit.cu (:753-783 one-hot of the target).
//
// Differences by design: all weights (and all weight updates) of a network are ONE device allocation, layers in
// file order, so the optimizer step is a single launch; error buffers of the skip layers are one allocation
// cleared by one launch per forward pass; a skip layer with a single source (every skipini, and a skipadd with one
// preSkipLayer) aliases that source's outputs instead of copying them; fan-in and fan-out of a skip layer are one
// launch each, whatever the number of linked layers (pointer tables live in device memory); the weight-gradient
// halves of dense and LSTM layers run on a second stream of the same priority.
#include "common.hpp"

#include <algorithm>
#include <cerrno>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <new>
#include <random>
#include <string>
#include <utility>
#include <vector>

namespace cnt {
namespace json {

// A small JSON reader: objects, arrays of objects, arrays of numbers (kept as floats), strings, numbers, literals.
struct Value {
    enum Type { NUL, BOOL, NUM, STR, ARR, NUMS, OBJ } type = NUL;
    double num = 0.0;
    bool flag = false;
    std::string str;
    std::vector<Value> arr;
    std::vector<float> nums;
    std::vector<std::pair<std::string, Value>> obj;
    size_t begin = 0, end = 0;  // extent in the source text

    const Value *get(const char *key) const {
        if (type != OBJ) return nullptr;
        for (const auto &kv : obj)
            if (kv.first == key) return &kv.second;
        return nullptr;
    }
    bool has(const char *key) const { return get(key) != nullptr; }
};

struct Parser {
    const char *s;
    size_t n, i = 0;
    std::string error;

    bool fail(const char *what) {
        if (error.empty()) {
            char buf[160];
            snprintf(buf, sizeof(buf), "%s at offset %zu", what, i);
            error = buf;
        }
        return false;
    }
    void ws() {
        while (i < n && (s[i] == ' ' || s[i] == '\t' || s[i] == '\n' || s[i] == '\r')) ++i;
    }
    bool string(std::string &out) {
        if (i >= n || s[i] != '"') return fail("expected a string");
        ++i;
        out.clear();
        while (i < n && s[i] != '"') {
            char c = s[i++];
            if (c == '\\') {
                if (i >= n) return fail("unfinished escape");
                const char e = s[i++];
                switch (e) {
                    case 'n': c = '\n'; break;
                    case 't': c = '\t'; break;
                    case 'r': c = '\r'; break;
                    case 'b': c = '\b'; break;
                    case 'f': c = '\f'; break;
                    case 'u': {  // names and options of a network file are ASCII; keep the low byte
                        if (i + 4 > n) return fail("unfinished \\u escape");
                        c = (char)strtol(std::string(s + i, 4).c_str(), nullptr, 16);
                        i += 4;
                        break;
                    }
                    default: c = e;
                }
            }
            out.push_back(c);
        }
        if (i >= n) return fail("unterminated string");
        ++i;
        return true;
    }
    bool number(double &out) {
        char *endp = nullptr;
        errno = 0;
        out = strtod(s + i, &endp);
        if (endp == s + i) return fail("expected a number");
        i = (size_t)(endp - s);
        return true;
    }
    bool value(Value &v, int depth) {
        if (depth > 16) return fail("nesting too deep");
        ws();
        if (i >= n) return fail("unexpected end of text");
        v.begin = i;
        const char c = s[i];
        if (c == '{') {
            v.type = Value::OBJ;
            ++i;
            ws();
            if (i < n && s[i] == '}') {
                ++i;
            } else {
                for (;;) {
                    ws();
                    std::string key;
                    if (!string(key)) return false;
                    ws();
                    if (i >= n || s[i] != ':') return fail("expected ':'");
                    ++i;
                    v.obj.emplace_back(std::move(key), Value());
                    if (!value(v.obj.back().second, depth + 1)) return false;
                    ws();
                    if (i < n && s[i] == ',') { ++i; continue; }
                    if (i < n && s[i] == '}') { ++i; break; }
                    return fail("expected ',' or '}'");
                }
            }
        } else if (c == '[') {
            ++i;
            ws();
            v.type = Value::ARR;
            if (i < n && s[i] == ']') {
                ++i;
            } else {
                const bool numeric = (s[i] == '-' || s[i] == '+' || (s[i] >= '0' && s[i] <= '9'));
                if (numeric) v.type = Value::NUMS;
                for (;;) {
                    ws();
                    if (numeric) {
                        double d;
                        if (!number(d)) return false;
                        v.nums.push_back((float)d);
                    } else {
                        v.arr.emplace_back();
                        if (!value(v.arr.back(), depth + 1)) return false;
                    }
                    ws();
                    if (i < n && s[i] == ',') { ++i; continue; }
                    if (i < n && s[i] == ']') { ++i; break; }
                    return fail("expected ',' or ']'");
                }
            }
        } else if (c == '"') {
            v.type = Value::STR;
            if (!string(v.str)) return false;
        } else if (!strncmp(s + i, "true", 4)) {
            v.type = Value::BOOL; v.flag = true; i += 4;
        } else if (!strncmp(s + i, "false", 5)) {
            v.type = Value::BOOL; v.flag = false; i += 5;
        } else if (!strncmp(s + i, "null", 4)) {
            v.type = Value::NUL; i += 4;
        } else {
            v.type = Value::NUM;
            if (!number(v.num)) return false;
        }
        v.end = i;
        return true;
    }
};

}  // namespace json

namespace {

enum Kind { K_INPUT, K_DENSE, K_LSTM, K_SKIPINI, K_SKIPADD, K_SKIPCAT, K_CNN, K_WAVNETC, K_GATED, K_FEEDBACK, K_EXTERNAL,
            K_SSE, K_MDN, K_DFT };

inline bool is_post_kind(int k) { return k == K_SSE || k == K_MDN || k == K_DFT; }

inline bool is_sum_skip(int k) { return k == K_SKIPINI || k == K_SKIPADD; }
inline bool is_skip_kind(int k) { return is_sum_skip(k) || k == K_SKIPCAT; }

struct NetLayer {
    std::string name, type, text;  // text: the layer's object as it stands in the network file
    int kind = K_INPUT;
    int size = 0, prev = -1;
    float bias = 0.0f;
    float learning_rate = -1.0f;  // "learningRate" of a trainable layer; below -0.5: the optimizer's
    int act = 0, bidir = 0;
    std::vector<int> pre;  // skip layers: linked source layers
    long w_off = 0, n_in = 0, n_bias = 0, n_int = 0;
    float *out = nullptr, *err = nullptr, *eskip = nullptr;
    cnt_lstm *lstm = nullptr;
    cnt_cnn *cnn = nullptr;
    cnt_mdn *mdn = nullptr;
    cnt_dft *dft = nullptr;
    float *dft_errors = nullptr;             // dft: per-resolution distances written by the forward pass
    int dft_error_count = 0;
    float dft_beta = 0.0f;                   // dft: weight of the waveform MSE gradient
    float *core = nullptr, *cth = nullptr;  // wavnetc
    int ctx_dim = 0;
    int fb_start = 0, fb_end = 0;            // feedback: dimensions taken from the preceding layer
    // time base: a layer with "resolution" r has one slot per r time steps (layers/Layer.cu:254-305)
    int res = 1, maxTr = 0;
    int T = 0, Tmin = 0, N = 0;              // of the current fraction, at this layer's resolution
    const char *pat = nullptr;               // pattern types at this layer's resolution
    SlotOrder order = {nullptr, nullptr};    // the fraction's slots at this layer's resolution, valid ones first (or none)
    std::string flag;                        // "layerFlag"
    std::vector<int> cat_lo, cat_hi;         // skipcat: dimension range taken from each source
    const float *ext_data = nullptr;         // externalloader: [frame][sequence][dimension], set by the caller
    const float *ext_mean_std = nullptr;
    bool mdn_errors_done = false;            // mdn: calculate_error has already written the preceding layer's errors
    int ext_frames = 0, index_load_method = 0;
    int cnn_tanh = 0;                        // cnn: "tanhoutput"
    bool delta_fused = false;                // cnn followed by a wavnetc layer: that layer writes this layer's delta
    bool fold_ok = false;                    // cnn whose error product can ride in the launch of the block below it
    bool direct_ok = false;                  // ... and the block above hands its sum to nothing but that launch
    float *colsum = nullptr;                 // cnn in front of a wavnetc layer: per-workgroup sums of its deltas ([rows][size])
    int colsum_rows = 0;                     // rows written by this pass's block launch (0: none)
    const float *total = nullptr;            // skip layers: where the summed error stands after the layer's step
    bool needs_sum = false;                  // skip layers: errors += side buffer is not a no-op
    int live_targets = 0;                    // skip layers: sources that receive the sum through a launch
    const float **in_ptrs = nullptr;         // skip layers: device tables
    float **tgt_ptrs = nullptr;
    int *tgt_is_skip = nullptr;
    bool ptrs_aligned = false;               // every buffer the skip kernels touch for this layer is 16-byte aligned
    long weight_count() const { return n_in + n_bias + n_int; }
};

inline int blocks_for(size_t count) {
    size_t b = (count + 255) / 256;
    if (b > 4096) b = 4096;
    return (int)(b < 1 ? 1 : b);
}

// The skip kernels move V = float or float4 (16-byte accesses: count % 4 == 0 and every buffer 16-byte aligned);
// `count` is in units of V.
__device__ __forceinline__ float vadd(float a, float b) { return a + b; }
__device__ __forceinline__ float4 vadd(float4 a, float4 b) { return make_float4(a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w); }

template <typename V>
__global__ void skip_sum_kernel(size_t count, int n, const float *const *__restrict__ in, float *__restrict__ out) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) {
        V acc = reinterpret_cast<const V *>(in[0])[i];
        for (int k = 1; k < n; ++k) acc = vadd(acc, reinterpret_cast<const V *>(in[k])[i]);
        reinterpret_cast<V *>(out)[i] = acc;
    }
}

// errors += errors_from_skip, then to every linked source in reverse order: added to a skip layer's side buffer,
// written over any other layer's error buffer (layers/SkipAddLayer.cu:305-346)
// errors_from_skip == NULL: nothing to add, `errors` is only read
template <typename V>
__global__ void skip_fan_kernel(size_t count, int n, float *const *__restrict__ target, const int *__restrict__ is_skip,
                                float *errors, const float *__restrict__ errors_from_skip) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) {
        V e = reinterpret_cast<const V *>(errors)[i];
        if (errors_from_skip) {
            e = vadd(reinterpret_cast<const V *>(errors_from_skip)[i], e);
            reinterpret_cast<V *>(errors)[i] = e;
        }
        for (int k = 0; k < n; ++k) {
            V *t = reinterpret_cast<V *>(target[k]);
            t[i] = is_skip[k] ? vadd(e, t[i]) : e;
        }
    }
}

// FeedBackLayer::computeForwardPass in training (layers/FeedBackLayer.cu:60-130, :607-650) with look-back of one
// step, fed by a softmax unit's ground-truth one-hot vector (layers/MDNUnit.cu:753-783): dimensions
// [0, d1) = preceding layer's [start, start+d1); the rest = one-hot of the previous step's target class, all zero
// for the first step and where the previous slot is padding.
__global__ void feedback_kernel(size_t count, int dim_out, int d1, int prev_total, int prev_start, int S, int target_dim,
                                int target_start, const char *__restrict__ pat, const float *__restrict__ prev_out,
                                const float *__restrict__ targets, float *__restrict__ out) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) {
        const long slot = (long)(i / dim_out);
        const int d = (int)(i % dim_out);
        float v = 0.0f;
        if (d < d1) {
            v = prev_out[slot * prev_total + prev_start + d];
        } else if (slot >= S && pat[slot - S] != 0) {
            const int cls = (int)targets[(slot - S) * target_dim + target_start];
            v = (cls == d - d1) ? 1.0f : 0.0f;
        }
        out[i] = v;
    }
}

// FeedBackLayer::computeBackwardPass (layers/FeedBackLayer.cu:338-360, :841-865)
__global__ void feedback_backward_kernel(size_t count, int prev_total, int prev_start, int prev_end, int dim_out,
                                         const float *__restrict__ errors, float *__restrict__ prev_errors) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) {
        const long slot = (long)(i / prev_total);
        const int d = (int)(i % prev_total);
        prev_errors[i] = (d >= prev_start && d < prev_end) ? errors[slot * dim_out + d - prev_start] : 0.0f;
    }
}

// Pattern types at a lower time resolution, as data_sets/DataSet.cpp:993-1012 leaves them: slot t' covers the time
// steps [t'*res, (t'+1)*res); none if the sequence has ended before it, first for t' = 0, otherwise the type of the
// last time step of the sequence inside the block (normal, or last if the sequence ends there).
__global__ void lowres_pat_kernel(int S, int T, int Tr, int res, const char *__restrict__ pat, char *__restrict__ out) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= Tr * S) return;
    const int tr = i / S, s = i % S;
    const int t0 = tr * res;
    char v = 0;
    if (pat[(size_t)t0 * S + s] != 0) {
        if (tr == 0) {
            v = 1;
        } else {
            const int tl = min(t0 + res - 1, T - 1);
            const char p = pat[(size_t)tl * S + s];
            v = p == 0 ? 3 : p;
        }
    }
    out[i] = v;
}

// ExternalLoader::loadSequences (layers/ExternalLoader.cu:58-110, :205-250): slot (t', s) takes frame
// frame_index[(t'*res)*S + s] (divided by res for indexLoadMethod 1) of sequence s from the external data,
// optionally (x - mean) / std with std < 1e-5 taken as 1; 0 on padding slots and beyond the data.
__global__ void external_load_kernel(size_t count, int dim, int S, int res, int method, int max_frames,
                                     const float *__restrict__ data, const float *__restrict__ frame_index,
                                     const float *__restrict__ mean_std, const char *__restrict__ pat,
                                     float *__restrict__ out) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) {
        const int d = (int)(i % dim);
        const long slot = (long)(i / dim);
        const long tr = slot / S;
        const int s = (int)(slot % S);
        float v = 0.0f;
        if (pat[slot] != 0) {
            int frame = (int)frame_index[(size_t)tr * res * S + s];
            if (method == 1) frame /= res;
            if (frame < max_frames) {
                v = data[((size_t)frame * S + s) * dim + d];
                if (mean_std) {
                    const float sd = mean_std[dim + d];
                    v = (v - mean_std[d]) / (sd < 1e-5f ? 1.0f : sd);
                }
            }
        }
        out[i] = v;
    }
}

// SkipCatLayer (layers/SkipCatLayer.cu:52-91): dimensions [lo, lo+n) of the source into [at, at+n) of this layer
// (forward), and the errors back (backward: added to a skip layer's side buffer on non-padding slots, written to
// any other layer's error buffer, which the caller has zero-filled, on non-padding slots).
__global__ void skipcat_forward_kernel(size_t count, int n, int src_dim, int lo, int dst_dim, int at,
                                       const float *__restrict__ src, float *__restrict__ dst) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) {
        const size_t slot = i / n;
        const int j = (int)(i % n);
        dst[slot * dst_dim + at + j] = src[slot * src_dim + lo + j];
    }
}
__global__ void skipcat_backward_kernel(size_t count, int n, int src_dim, int lo, int dst_dim, int at, int accumulate,
                                        const char *__restrict__ pat, const float *__restrict__ errors,
                                        float *__restrict__ target) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) {
        const size_t slot = i / n;
        const int j = (int)(i % n);
        float *t = target + slot * src_dim + lo + j;
        if (pat[slot] == 0) {
            if (!accumulate) *t = 0.0f;
            continue;
        }
        const float e = errors[slot * dst_dim + at + j];
        *t = accumulate ? *t + e : e;
    }
}
__global__ void sum_few_kernel(int n, const float *__restrict__ v, float *__restrict__ out) {
    if (blockIdx.x == 0 && threadIdx.x == 0) {
        float acc = 0.0f;
        for (int i = 0; i < n; ++i) acc += v[i];
        *out = acc;
    }
}
// gradient of the dft layer's waveform MSE term, added to the spectral gradients (ComputeMseWaveformGrad,
// layers/DFTErrorPostoutputLayer.cu:87-120, :1157-1183)
__global__ void waveform_mse_grad_kernel(size_t count, int dim, float beta, const char *__restrict__ pat,
                                         const float *__restrict__ y, const float *__restrict__ target,
                                         float *__restrict__ err) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride)
        if (pat[i / dim] != 0) err[i] += (y[i] - target[i]) * beta;
}
__global__ void add_inplace_kernel(size_t count, float *__restrict__ a, const float *__restrict__ b) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) a[i] += b[i];
}

// "64*1_64*2": <count>*<value> runs joined by '_' (the reference's CNN option strings); one value per filter
bool parse_runs(const std::string &opt, int D, std::vector<int> &out) {
    out.clear();
    size_t i = 0;
    while (i < opt.size()) {
        char *endp = nullptr;
        const long a = strtol(opt.c_str() + i, &endp, 10);
        if (endp == opt.c_str() + i) return false;
        i = (size_t)(endp - opt.c_str());
        if (i < opt.size() && opt[i] == '*') {
            ++i;
            const long b = strtol(opt.c_str() + i, &endp, 10);
            if (endp == opt.c_str() + i || a < 0) return false;
            i = (size_t)(endp - opt.c_str());
            for (long k = 0; k < a; ++k) out.push_back((int)b);
        } else {
            out.push_back((int)a);
        }
        if (i < opt.size()) {
            if (opt[i] != '_') return false;
            ++i;
        }
    }
    return (int)out.size() == D;
}

int get_int(const json::Value &o, const char *key, int def) {
    const json::Value *v = o.get(key);
    return (v && v->type == json::Value::NUM) ? (int)v->num : def;
}
std::string get_str(const json::Value &o, const char *key) {
    const json::Value *v = o.get(key);
    return (v && v->type == json::Value::STR) ? v->str : std::string();
}

}  // namespace
}  // namespace cnt

struct cnt_network {
    std::vector<cnt::NetLayer> layers;
    int S = 0, maxT = 0, T = 0, Tmin = 0;
    const char *pat = nullptr;
    long n_weights = 0;
    float *weights = nullptr, *updates = nullptr;
    float *skip_errors = nullptr;  // err and eskip of every skip layer, one allocation
    size_t skip_error_count = 0;
    const float *ctx = nullptr;    // conditioning features of the wavnetc layers, C x (maxT*S)
    // conditioning sub-network: the layer flagged "wavenetConditionInputLayer" feeds the wavnetc layers
    int flagged = -1, first_wavnetc = -1;
    float *ctx_own = nullptr, *ctx_grad = nullptr;
    float *ctx_mv = nullptr;  // the first wavnetc layer's "contextMV": [means | standard deviations] (device), or NULL
    struct LowRes { int res; char *pat; int *order; int *order_count; bool order_built; };
    int *order = nullptr, *order_count = nullptr;  // the fraction's slots at resolution 1, valid ones first (slot_order_build)
    bool skip_padding = true;
    std::vector<LowRes> low_res;
    std::vector<void *> allocations;
    // weight gradients go round-robin to these streams (default priority); CNT_NET_SIDE_STREAMS overrides the count
    static constexpr int kMaxSide = 4;
    hipStream_t side[kMaxSide] = {};
    hipEvent_t ev_main = nullptr, ev_side[kMaxSide] = {};
    int n_side = 3;
    int overlap = 1;
    // optimizer state (allocated by the first update)
    float *cur_updates = nullptr, *deltas = nullptr, *stats = nullptr;
    int stats_option = -1;
    float *adam_accum = nullptr;  // beta1^t, beta2^t of Adam's bias correction (device)
    int mdn_target_start = 0, mdn_classes = 0;
    // set on the device by an LSTM recursion that gives up; the optimizer step looks at it and leaves the weights alone
    int *veto = nullptr;
};

namespace cnt {
namespace {

int device_alloc(cnt_network *n, void **p, size_t bytes, bool zero) {
    CNT_HIP(hipMalloc(p, bytes ? bytes : 4));
    n->allocations.push_back(*p);
    if (zero) CNT_HIP(hipMemset(*p, 0, bytes ? bytes : 4));
    return CNT_OK;
}

// TrainableLayer's three sections of a layer's weight vector (layers/TrainableLayer.cu:160-220)
void weight_sections(NetLayer &L, int P) {
    const long D = L.size;
    L.n_in = L.n_bias = L.n_int = 0;
    if (L.kind == K_DENSE) {
        L.n_in = (long)P * D;
        L.n_bias = D;
    } else if (L.kind == K_LSTM) {
        const long H = L.bidir ? D / 2 : D;
        L.n_in = 4L * P * D;
        L.n_bias = 4L * D;
        L.n_int = 4L * D * H + 3L * D;
    } else if (L.kind == K_CNN) {
        L.n_int = cnt_cnn_weight_count(L.cnn);
    } else if (L.kind == K_WAVNETC) {
        L.n_int = 2L * L.ctx_dim * D;
    }
}

int build_layer_into(cnt_network *net, NetLayer &L, const json::Value &obj, const char *text,
                     const cnt_network_options *opt);

// a layer that fails half way must not leave its handles behind
int build_layer(cnt_network *net, const json::Value &obj, const char *text, const cnt_network_options *opt) {
    NetLayer L;
    const int status = build_layer_into(net, L, obj, text, opt);
    if (status != CNT_OK) {
        if (L.lstm) cnt_lstm_destroy(L.lstm);
        if (L.cnn) cnt_cnn_destroy(L.cnn);
        if (L.mdn) cnt_mdn_destroy(L.mdn);
        if (L.dft) cnt_dft_destroy(L.dft);
        return status;
    }
    net->layers.push_back(std::move(L));
    return CNT_OK;
}

int build_layer_into(cnt_network *net, NetLayer &L, const json::Value &obj, const char *text,
                     const cnt_network_options *opt) {
    const int index = (int)net->layers.size();
    L.text.assign(text + obj.begin, obj.end - obj.begin);
    L.name = get_str(obj, "name");
    L.type = get_str(obj, "type");
    L.size = get_int(obj, "size", 0);
    const json::Value *bias = obj.get("bias");
    L.bias = (bias && bias->type == json::Value::NUM) ? (float)bias->num : 0.0f;
    L.prev = index - 1;
    if (const json::Value *lr = obj.get("learningRate"))
        if (lr->type == json::Value::NUM) L.learning_rate = (float)lr->num;
    CNT_REQUIRE(L.size > 0, "network: layer %d ('%s') has no positive size", index, L.name.c_str());
    L.res = get_int(obj, "resolution", 1);
    CNT_REQUIRE(L.res >= 1, "network: layer '%s' has resolution %d", L.name.c_str(), L.res);
    L.maxTr = (net->maxT + L.res - 1) / L.res;
    L.flag = get_str(obj, "layerFlag");
    const int P = index > 0 ? net->layers[(size_t)index - 1].size : 0;
    const int prev_res = index > 0 ? net->layers[(size_t)index - 1].res : 1;
    const size_t slots = (size_t)net->S * L.maxTr;
    const std::string &t = L.type;
    static const char *ff[] = {"feedforward_identity", "feedforward_tanh", "feedforward_logistic", "feedforward_relu"};
    bool trainable = true;
    if (index == 0) {
        CNT_REQUIRE(t == "input", "network: the first layer must be of type 'input'");
        L.kind = K_INPUT;
        trainable = false;
    } else if (t == ff[0] || t == ff[1] || t == ff[2] || t == ff[3]) {
        L.kind = K_DENSE;
        for (int a = 0; a < 4; ++a)
            if (t == ff[a]) L.act = a;
    } else if (t == "lstm" || t == "blstm") {
        L.kind = K_LSTM;
        L.bidir = t == "blstm";
        cnt_lstm_desc d = {P, L.size, L.bidir, net->S, L.maxTr, L.bias};
        CNT_TRY(cnt_lstm_create(&d, &L.lstm));
        if (!net->veto) CNT_TRY(device_alloc(net, (void **)&net->veto, sizeof(int), true));
        cnt::lstm_set_veto(L.lstm, net->veto);
        cnt::lstm_set_slot_order(L.lstm, nullptr);  // the sequencer lists a fraction's valid slots once for all layers
    } else if (t == "skipini" || t == "skipadd") {
        // NeuralNetwork.cpp:470-530 offers every earlier skip layer plus the layer right before; SkipAddLayer.cu:
        // 96-138 keeps those named by preSkipLayer, or by default the last two of the offer (a skipini, and the
        // first skip layer of a network, is offered the layer right before only)
        L.kind = t == "skipini" ? K_SKIPINI : K_SKIPADD;
        std::vector<int> offer;
        if (L.kind == K_SKIPADD)
            for (int j = 0; j < index; ++j)
                if (is_skip_kind(net->layers[(size_t)j].kind)) offer.push_back(j);
        offer.push_back(index - 1);
        const std::string names = L.kind == K_SKIPADD ? get_str(obj, "preSkipLayer") : std::string();
        if (!names.empty()) {
            size_t b = 0;
            while (b <= names.size()) {
                size_t e = names.find(',', b);
                if (e == std::string::npos) e = names.size();
                const std::string one = names.substr(b, e - b);
                for (int j : offer)
                    if (net->layers[(size_t)j].name == one) {
                        L.pre.push_back(j);
                        break;
                    }
                b = e + 1;
            }
        } else if (offer.size() < 2) {
            L.pre = offer;
        } else {
            L.pre.assign(offer.end() - 2, offer.end());
        }
        CNT_REQUIRE(!L.pre.empty(), "network: skip layer '%s' is linked to no layer", L.name.c_str());
        for (int j : L.pre) {
            CNT_REQUIRE(net->layers[(size_t)j].size == L.size, "network: skip layer '%s' (size %d) is linked to '%s' of "
                        "size %d", L.name.c_str(), L.size, net->layers[(size_t)j].name.c_str(), net->layers[(size_t)j].size);
            CNT_REQUIRE(net->layers[(size_t)j].res == L.res, "network: skip layer '%s' is linked to '%s' of another "
                        "resolution", L.name.c_str(), net->layers[(size_t)j].name.c_str());
        }
    } else if (t == "skipcat") {
        // SkipCatLayer::SkipCatLayer (layers/SkipCatLayer.cu:100-200): the layers named by preSkipLayer, of each the
        // dimension range [a, b) given by preSkipLayerDim "a_b_a_b..." (default: all of it)
        L.kind = K_SKIPCAT;
        std::vector<int> offer;
        for (int j = 0; j < index; ++j)
            if (is_skip_kind(net->layers[(size_t)j].kind)) offer.push_back(j);
        offer.push_back(index - 1);
        const std::string names = get_str(obj, "preSkipLayer");
        CNT_REQUIRE(!names.empty(), "network: no preSkipLayer configuration in skipcat layer '%s'", L.name.c_str());
        size_t b = 0;
        while (b <= names.size()) {
            size_t e = names.find(',', b);
            if (e == std::string::npos) e = names.size();
            const std::string one = names.substr(b, e - b);
            for (int j : offer)
                if (net->layers[(size_t)j].name == one) {
                    L.pre.push_back(j);
                    break;
                }
            b = e + 1;
        }
        CNT_REQUIRE(!L.pre.empty(), "network: skipcat layer '%s' is linked to no layer", L.name.c_str());
        std::vector<int> dims;
        const std::string ds = get_str(obj, "preSkipLayerDim");
        if (!ds.empty()) {
            size_t i = 0;
            while (i < ds.size()) {
                char *endp = nullptr;
                const long v = strtol(ds.c_str() + i, &endp, 10);
                CNT_REQUIRE(endp != ds.c_str() + i, "network: skipcat layer '%s': bad preSkipLayerDim", L.name.c_str());
                dims.push_back((int)v);
                i = (size_t)(endp - ds.c_str());
                if (i < ds.size() && ds[i] == '_') ++i;
            }
        } else {
            for (int j : L.pre) {
                dims.push_back(0);
                dims.push_back(net->layers[(size_t)j].size);
            }
        }
        CNT_REQUIRE(dims.size() == 2 * L.pre.size(), "network: skipcat layer '%s': preSkipLayerDim needs two numbers per "
                    "layer of preSkipLayer", L.name.c_str());
        int total = 0;
        for (size_t k = 0; k < L.pre.size(); ++k) {
            const NetLayer &src = net->layers[(size_t)L.pre[k]];
            const int lo = dims[2 * k], hi = dims[2 * k + 1];
            CNT_REQUIRE(lo >= 0 && hi >= lo && hi <= src.size, "network: skipcat layer '%s': range %d..%d outside layer "
                        "'%s'", L.name.c_str(), lo, hi, src.name.c_str());
            CNT_REQUIRE(src.res == L.res, "network: skipcat layer '%s' needs layers of its own resolution", L.name.c_str());
            L.cat_lo.push_back(lo);
            L.cat_hi.push_back(hi);
            total += hi - lo;
        }
        CNT_REQUIRE(total == L.size, "network: skipcat layer '%s' has size %d, its sources give %d", L.name.c_str(), L.size,
                    total);
    } else if (t == "externalloader") {
        L.kind = K_EXTERNAL;
        L.index_load_method = get_int(obj, "indexLoadMethod", 0);
        CNT_REQUIRE(net->layers.front().size == 1, "network: externalloader layer '%s' reads the frame index from an input "
                    "layer of size 1", L.name.c_str());
    } else if (t == "cnn") {
        L.kind = K_CNN;
        CNT_REQUIRE(!obj.has("window_height") && get_int(obj, "repeat_padding", 0) == 0,
                    "network: cnn layer '%s' uses the 2-D path or repeat_padding, which are not built", L.name.c_str());
        std::vector<int> hw, dil;
        CNT_REQUIRE(parse_runs(get_str(obj, "window_width"), L.size, hw), "network: cnn layer '%s': window_width does "
                    "not give one value per filter", L.name.c_str());
        CNT_REQUIRE(parse_runs(get_str(obj, "window_tap_interval"), L.size, dil), "network: cnn layer '%s': "
                    "window_tap_interval does not give one value per filter", L.name.c_str());
        L.cnn_tanh = get_int(obj, "tanhoutput", 1);
        cnt_cnn_desc d = {P, L.size, net->S, L.maxTr, get_int(obj, "causal", 0), L.cnn_tanh, L.bias};
        CNT_TRY(cnt_cnn_create(&d, hw.data(), dil.data(), &L.cnn));
    } else if (t == "wavnetc") {
        L.kind = K_WAVNETC;
        L.ctx_dim = get_int(obj, "contextDim", 0);
        CNT_REQUIRE(P == 2 * L.size, "network: wavnetc layer '%s' of size %d needs a preceding layer of size %d",
                    L.name.c_str(), L.size, 2 * L.size);
        CNT_REQUIRE(L.res == 1, "network: wavnetc layer '%s' must have resolution 1", L.name.c_str());
        // "contextMV": a file of contextDim means followed by contextDim standard deviations, raw float32
        // (layers/wavNetCore.cu:322-332, :343-351); every such layer reads its file, the first one's is the one in use
        // (:455-492: only the initial core fills the shared conditioning buffer)
        const std::string mv_path = get_str(obj, "contextMV");
        if (!mv_path.empty() && L.ctx_dim > 0) {
            std::vector<float> mv;
            if (FILE *f = std::fopen(mv_path.c_str(), "rb")) {
                float v;
                while (mv.size() <= 2 * (size_t)L.ctx_dim && std::fread(&v, sizeof(v), 1, f) == 1) mv.push_back(v);
                std::fclose(f);
            } else {
                set_error("network: wavnetc layer '%s': cannot open contextMV file %s", L.name.c_str(), mv_path.c_str());
                return CNT_ERR_ARG;
            }
            CNT_REQUIRE(mv.size() == 2 * (size_t)L.ctx_dim, "network: wavnetc layer '%s': context mean variance dim unequal "
                        "(%s does not hold 2 x %d floats)", L.name.c_str(), mv_path.c_str(), L.ctx_dim);
            if (net->first_wavnetc < 0) {
                CNT_TRY(device_alloc(net, (void **)&net->ctx_mv, mv.size() * sizeof(float), false));
                CNT_HIP(hipMemcpy(net->ctx_mv, mv.data(), mv.size() * sizeof(float), hipMemcpyHostToDevice));
            }
        }
        if (net->first_wavnetc < 0) net->first_wavnetc = index;
        NetLayer &before = net->layers[(size_t)index - 1];
        if (before.kind == K_CNN && before.cnn_tanh) before.delta_fused = true;
        CNT_TRY(device_alloc(net, (void **)&L.core, 2 * (size_t)L.size * slots * sizeof(float), true));
        CNT_TRY(device_alloc(net, (void **)&L.cth, 2 * (size_t)L.size * slots * sizeof(float), true));
    } else if (t == "gatedact") {
        // GatedActLayer::GatedActLayer (layers/GatedActLayer.cu:131-143)
        L.kind = K_GATED;
        CNT_REQUIRE(P == 2 * L.size, "network: gatedact layer '%s' of size %d needs a preceding layer of size %d",
                    L.name.c_str(), L.size, 2 * L.size);
    } else if (t == "dft") {
        // DFTPostoutputLayer::DFTPostoutputLayer (layers/DFTErrorPostoutputLayer.cu:599-849)
        L.kind = K_DFT;
        trainable = false;
        CNT_REQUIRE(L.size == 1 && P == 1, "network: the dft layer evaluates one waveform (size 1), found size %d after "
                    "a layer of size %d", L.size, P);
        CNT_REQUIRE(net->S == 1, "network: the dft layer needs parallel_sequences = 1 (one waveform per fraction)");
        const char *off[] = {"eta", "kappa", "tau", "iota"};
        for (const char *key : off) {
            const json::Value *v = obj.get(key);
            CNT_REQUIRE(!v || v->type != json::Value::NUM || v->num <= 0.0, "network: dft layer '%s': the '%s' term is not "
                        "built", L.name.c_str(), key);
        }
        const char *flags[] = {"preEmphasisNaturalWav", "hnmMode", "multiDimSignalMode", "lpcOrder", "lpcOrder2", "lpcOrder3"};
        for (const char *key : flags)
            CNT_REQUIRE(get_int(obj, key, 0) == 0, "network: dft layer '%s': '%s' is not built", L.name.c_str(), key);
        CNT_REQUIRE(get_str(obj, "specWeightVec").empty() && get_str(obj, "specWeightVec2").empty() &&
                    get_str(obj, "specWeightVec3").empty(), "network: dft layer '%s': spectral weight vectors are not "
                    "built", L.name.c_str());
        auto real = [&](const char *key, double def) {
            const json::Value *v = obj.get(key);
            return (v && v->type == json::Value::NUM) ? v->num : def;
        };
        cnt_dft_desc d = {};
        const char *suffix[3] = {"", "2", "3"};
        const int def_len[3] = {320, 80, 80}, def_shift[3] = {80, 40, 40};
        for (int r = 0; r < 3; ++r) {
            const std::string sx = suffix[r];
            const int fft = get_int(obj, ("fftLength" + sx).c_str(), r == 0 ? 512 : 0);
            if (fft <= 0) continue;
            d.fft_length[d.n_res] = fft;
            d.frame_length[d.n_res] = get_int(obj, ("frameLength" + sx).c_str(), def_len[r]);
            d.frame_shift[d.n_res] = get_int(obj, ("frameShift" + sx).c_str(), def_shift[r]);
            d.window_type[d.n_res] = get_int(obj, ("windowType" + sx).c_str(), 0);
            ++d.n_res;
        }
        L.dft_beta = (float)real("beta", 0.0);
        d.gamma = (float)real("gamma", 0.0);
        d.zeta = (float)real("zeta", 0.0);
        d.log_floor = (float)real("logSpecAmpFloor", 0.00001);
        d.spec_dis_type = get_int(obj, "specDisType", 0);
        d.phase_dis_type = get_int(obj, "phaseDisType", 0);
        d.max_length = net->maxT;
        d.max_waves = 1;
        CNT_TRY(cnt_dft_create(&d, &L.dft));
        L.dft_error_count = d.n_res * (d.zeta > 0.0f ? 2 : 1);
        CNT_TRY(device_alloc(net, (void **)&L.dft_errors, 8 * sizeof(float), true));
    } else if (t == "feedback") {
        L.kind = K_FEEDBACK;
        L.fb_start = get_int(obj, "previousDimStart", 0);
        L.fb_end = get_int(obj, "previousDimEnd", P);
        CNT_REQUIRE(L.fb_start >= 0 && L.fb_end >= L.fb_start && L.fb_end <= P, "network: feedback layer '%s': "
                    "previousDimStart/End outside the preceding layer", L.name.c_str());
        CNT_REQUIRE(!obj.has("lookBack") && !obj.has("aggregate") && !obj.has("lookbackStep"),
                    "network: feedback layer '%s': look-back other than one step and aggregation are not built",
                    L.name.c_str());
        trainable = false;
    } else if (t == "sse") {
        L.kind = K_SSE;
        CNT_REQUIRE(L.size == P, "network: sse layer of size %d after a layer of size %d", L.size, P);
        trainable = false;
    } else if (t == "mdn") {
        L.kind = K_MDN;
        CNT_REQUIRE(opt && opt->mdn_config && opt->mdn_config_len >= 6, "network: an mdn layer needs the mdn config "
                    "(options.mdn_config)");
        cnt_mdn_desc d = {P, L.size, net->S, net->maxT, opt->tie_variance, 0};
        CNT_TRY(cnt_mdn_create(&d, opt->mdn_config, opt->mdn_config_len, &L.mdn));
        if ((int)opt->mdn_config[0] == 1 && (int)opt->mdn_config[5] == -1) {
            net->mdn_target_start = (int)opt->mdn_config[3];
            net->mdn_classes = (int)opt->mdn_config[2] - (int)opt->mdn_config[1];
        }
        trainable = false;
    } else {
        set_error("network: layer '%s' has type '%s', which this path does not cover", L.name.c_str(), t.c_str());
        return CNT_ERR_ARG;
    }
    // a layer runs on the time base of the layer before it; an externalloader starts one, a feedback layer that takes
    // nothing from the layer before it is independent of that layer's
    if (index > 0 && L.kind != K_EXTERNAL && !(L.kind == K_FEEDBACK && L.fb_end == L.fb_start))
        CNT_REQUIRE(prev_res == L.res, "network: layer '%s' has resolution %d, the layer before it %d", L.name.c_str(),
                    L.res, prev_res);
    // every trainable layer of a network file carries "bias" (layers/TrainableLayer.cu:118-120)
    if (trainable) CNT_REQUIRE(bias != nullptr, "network: missing value 'bias' in layer '%s'", L.name.c_str());
    weight_sections(L, P);
    const size_t count = (size_t)L.size * slots;
    const bool alias = is_sum_skip(L.kind) && L.pre.size() == 1;
    if (alias) L.out = net->layers[(size_t)L.pre[0]].out;
    else CNT_TRY(device_alloc(net, (void **)&L.out, count * sizeof(float), true));
    if (L.kind != K_INPUT && L.kind != K_EXTERNAL && !is_post_kind(L.kind) && !is_skip_kind(L.kind))
        CNT_TRY(device_alloc(net, (void **)&L.err, count * sizeof(float), true));
    return CNT_OK;
}

int finish_build(cnt_network *net, const json::Value *weights) {
    const size_t slots = (size_t)net->S * net->maxT;
    // flat weights
    long total = 0;
    for (auto &L : net->layers) {
        L.w_off = total;
        total += L.weight_count();
    }
    net->n_weights = total;
    CNT_TRY(device_alloc(net, (void **)&net->weights, (size_t)total * sizeof(float), true));
    CNT_TRY(device_alloc(net, (void **)&net->updates, (size_t)total * sizeof(float), true));
    if (weights && weights->type == json::Value::OBJ) {
        std::vector<float> host((size_t)total, 0.0f);
        for (auto &L : net->layers) {
            if (L.weight_count() == 0) continue;
            const json::Value *sec = weights->get(L.name.c_str());
            CNT_REQUIRE(sec && sec->type == json::Value::OBJ, "network: missing weights section for layer '%s'",
                        L.name.c_str());
            const char *keys[3] = {"input", "bias", "internal"};
            const long want[3] = {L.n_in, L.n_bias, L.n_int};
            long at = L.w_off;
            for (int k = 0; k < 3; ++k) {
                const json::Value *a = sec->get(keys[k]);
                CNT_REQUIRE(a && (a->type == json::Value::NUMS || a->type == json::Value::ARR),
                            "network: missing array 'weights/%s/%s'", L.name.c_str(), keys[k]);
                CNT_REQUIRE((long)a->nums.size() == want[k], "network: layer '%s' has %zu %s weights, expected %ld",
                            L.name.c_str(), a->nums.size(), keys[k], want[k]);
                std::memcpy(host.data() + at, a->nums.data(), (size_t)want[k] * sizeof(float));
                at += want[k];
            }
        }
        CNT_HIP(hipMemcpy(net->weights, host.data(), (size_t)total * sizeof(float), hipMemcpyHostToDevice));
    }
    // ---- routing of the skip layers' errors -------------------------------------------------------------------
    // The reference gives every skip layer an error buffer and a side buffer, adds the two in the layer's backward
    // step and hands the sum to every linked source (layers/SkipAddLayer.cu:305-346).  Which of these buffers ever
    // differ is known once the layer list stands:
    //   * a skip layer that no ordinary layer follows (nothing writes its error buffer) and that exactly one later
    //     skip layer links to only forwards that layer's sum: it shares the sum by pointer and owns no buffers;
    //   * a skip layer that no later skip layer links to has an all-zero side buffer: no addition, no side buffer;
    //   * a source that is a feedforward_identity layer (its backward step only reads its errors) and that receives
    //     its errors from this link alone shares the sum by pointer instead of receiving a copy.
    // What remains is one launch per skip layer that still has something to add or to hand on.
    const int n_layers = (int)net->layers.size();
    std::vector<int> links(n_layers, 0), linker(n_layers, -1), link_slot(n_layers, -1);
    for (int y = 0; y < n_layers; ++y)
        if (is_skip_kind(net->layers[(size_t)y].kind))
            for (size_t k = 0; k < net->layers[(size_t)y].pre.size(); ++k) {
                const int x = net->layers[(size_t)y].pre[k];
                // a skipcat hands on parts of its sum: whatever it links to keeps buffers of its own
                links[x] += net->layers[(size_t)y].kind == K_SKIPCAT ? 2 : 1;
                linker[x] = y;
                link_slot[x] = (int)k;
            }
    // the layer that feeds the wavnetc layers receives its errors from them
    if (net->first_wavnetc >= 0 && net->layers[(size_t)net->first_wavnetc].ctx_dim > 0)
        for (int j = 0; j < net->first_wavnetc; ++j)
            if (net->layers[(size_t)j].flag == "wavenetConditionInputLayer") {
                net->flagged = j;
                break;
            }
    auto followed_by_writer = [&](int i) {
        if (i + 1 >= n_layers) return false;
        const NetLayer &nx = net->layers[(size_t)i + 1];
        if (i == net->flagged) return true;
        if (is_skip_kind(nx.kind) || nx.kind == K_EXTERNAL) return false;
        return !(nx.kind == K_FEEDBACK && nx.fb_end == nx.fb_start);
    };
    std::vector<char> shares(n_layers, 0);  // skip layer that shares its linker's sum
    size_t skip_total = 0;
    for (int i = 0; i < n_layers; ++i) {
        NetLayer &L = net->layers[(size_t)i];
        if (!is_skip_kind(L.kind)) continue;
        const size_t lslots = (size_t)net->S * L.maxTr;
        if (L.kind == K_SKIPCAT) links[i] = std::max(links[i], 2);  // always keeps both buffers
        shares[i] = (is_sum_skip(L.kind) && !followed_by_writer(i) && links[i] == 1) ? 1 : 0;
        L.needs_sum = !shares[i] && links[i] > 0;
        if (!shares[i]) skip_total += (size_t)L.size * lslots * (links[i] > 0 ? 2 : 1);
    }
    net->skip_error_count = skip_total;
    if (skip_total) {
        CNT_TRY(device_alloc(net, (void **)&net->skip_errors, skip_total * sizeof(float), true));
        size_t at = 0;
        for (int i = 0; i < n_layers; ++i) {
            NetLayer &L = net->layers[(size_t)i];
            if (!is_skip_kind(L.kind) || shares[i]) continue;
            const size_t lslots = (size_t)net->S * L.maxTr;
            L.err = net->skip_errors + at;
            at += (size_t)L.size * lslots;
            if (links[i] > 0) {
                L.eskip = net->skip_errors + at;
                at += (size_t)L.size * lslots;
            }
        }
    }
    // sums, from the last layer to the first (a linker comes after the layers it links to)
    for (int i = n_layers - 1; i >= 0; --i) {
        NetLayer &L = net->layers[(size_t)i];
        if (!is_skip_kind(L.kind)) continue;
        L.total = shares[i] ? net->layers[(size_t)linker[i]].total : L.err;
        if (shares[i]) L.err = const_cast<float *>(L.total);  // what cnt_network_layer_info reports as this layer's errors
    }
    // pointer tables.  A source that shares the sum needs no write; what a sharing skip layer hands on is handed on
    // by the layer that owns the sum, in that layer's launch (sums into side buffers commute, and a source whose
    // error buffer an ordinary layer writes later is overwritten then either way).
    std::vector<int> owner(n_layers, -1);
    for (int i = n_layers - 1; i >= 0; --i)
        if (is_skip_kind(net->layers[(size_t)i].kind)) owner[i] = shares[i] ? owner[linker[i]] : i;
    std::vector<std::vector<float *>> tgt(n_layers);
    std::vector<std::vector<int>> flag(n_layers);
    for (int i = n_layers - 1; i >= 0; --i) {
        NetLayer &L = net->layers[(size_t)i];
        if (!is_sum_skip(L.kind)) continue;
        for (size_t k = L.pre.size(); k-- > 0;) {  // last source first, as the reference walks them
            const int x = L.pre[k];
            NetLayer &src = net->layers[(size_t)x];
            float *t = nullptr;
            const int skip = is_skip_kind(src.kind) ? 1 : 0;
            if (skip) {
                t = shares[x] ? nullptr : src.eskip;
            } else if (src.kind == K_DENSE && src.act == ACT_IDENTITY && links[x] == 1 && !followed_by_writer(x)) {
                src.err = const_cast<float *>(L.total);  // the buffer allocated for it stays unused
            } else {
                t = src.err;
            }
            if (t) {
                tgt[(size_t)owner[i]].push_back(t);
                flag[(size_t)owner[i]].push_back(skip);
            }
        }
    }
    for (int i = 0; i < n_layers; ++i) {
        NetLayer &L = net->layers[(size_t)i];
        if (!is_sum_skip(L.kind)) continue;
        const size_t n = L.pre.size();
        std::vector<const float *> in(n);
        for (size_t k = 0; k < n; ++k) in[k] = net->layers[(size_t)L.pre[k]].out;
        CNT_TRY(device_alloc(net, (void **)&L.in_ptrs, n * sizeof(float *), false));
        CNT_HIP(hipMemcpy(L.in_ptrs, in.data(), n * sizeof(float *), hipMemcpyHostToDevice));
        std::vector<float *> &t = tgt[(size_t)i];
        L.live_targets = (int)t.size();
        {
            auto aligned = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
            bool ok = aligned(L.out) && aligned(L.total) && aligned(L.eskip);
            for (const float *p : in) ok = ok && aligned(p);
            for (const float *p : t) ok = ok && aligned(p);
            L.ptrs_aligned = ok;
        }
        if (t.empty()) continue;
        CNT_TRY(device_alloc(net, (void **)&L.tgt_ptrs, t.size() * sizeof(float *), false));
        CNT_TRY(device_alloc(net, (void **)&L.tgt_is_skip, t.size() * sizeof(int), false));
        CNT_HIP(hipMemcpy(L.tgt_ptrs, t.data(), t.size() * sizeof(float *), hipMemcpyHostToDevice));
        CNT_HIP(hipMemcpy(L.tgt_is_skip, flag[(size_t)i].data(), t.size() * sizeof(int), hipMemcpyHostToDevice));
    }
    // A convolution layer i that sits on a block's closing skipadd layer [i-1], behind that block's skip collector
    // [i-2], skip 1x1 layer [i-3] and skipini layer [i-4]: when the closing layer does nothing but add what the later
    // block handed to it and hand the sum to the skipini layer, and nothing else writes that layer's side buffer, the
    // convolution's error product can be added to the block's sum inside the block's own launch (the buffers in between
    // are then never written).  Checked here on the pointer tables; sizes and alignment when the launch is made.
    for (int i = 8; i < n_layers; ++i) {
        NetLayer &C = net->layers[(size_t)i];
        if (C.kind != K_CNN) continue;
        const NetLayer &closing = net->layers[(size_t)i - 1], &collector = net->layers[(size_t)i - 2];
        const NetLayer &ini = net->layers[(size_t)i - 4];
        if (closing.kind != K_SKIPADD || closing.pre.size() != 1 || closing.pre[0] != i - 4) continue;
        if (!closing.err || closing.err != closing.total || !closing.needs_sum || !closing.eskip) continue;
        if (ini.kind != K_SKIPINI || !ini.needs_sum || !ini.eskip) continue;
        if (tgt[(size_t)i - 1].size() != 1 || tgt[(size_t)i - 1][0] != ini.eskip || !flag[(size_t)i - 1][0]) continue;
        if (!is_sum_skip(collector.kind) || collector.needs_sum || !tgt[(size_t)i - 2].empty()) continue;
        int writers = 0;
        for (int y = 0; y < n_layers; ++y)
            for (float *t : tgt[(size_t)y]) writers += t == ini.eskip ? 1 : 0;
        C.fold_ok = writers == 1;
        // The closing layer's side buffer has one writer too, the skipini layer of the block above (layer i+4), which
        // hands its sum to nothing else: the block below can then read that sum where it stands, and the copy into the
        // side buffer is left out.
        if (!C.fold_ok || i + 4 >= n_layers) continue;
        const NetLayer &above = net->layers[(size_t)i + 4];
        if (above.kind != K_SKIPINI || !above.total || above.total != above.err) continue;
        if (tgt[(size_t)i + 4].size() != 1 || tgt[(size_t)i + 4][0] != closing.eskip || !flag[(size_t)i + 4][0]) continue;
        writers = 0;
        for (int y = 0; y < n_layers; ++y)
            for (float *t : tgt[(size_t)y]) writers += t == closing.eskip ? 1 : 0;
        C.direct_ok = writers == 1;
    }
    // a block launch leaves the sums of the convolution layer's deltas per workgroup (bias gradient without another
    // pass over the deltas)
    for (int i = 1; i + 1 < n_layers; ++i) {
        NetLayer &C = net->layers[(size_t)i];
        if (C.kind != K_CNN || net->layers[(size_t)i + 1].kind != K_WAVNETC || C.size != 2 * net->layers[(size_t)i + 1].size) continue;
        const size_t rows = ((size_t)net->S * C.maxTr + 63) / 64;
        CNT_TRY(device_alloc(net, (void **)&C.colsum, rows * C.size * sizeof(float), false));
    }
    // the slots of a fraction with the valid ones first: the weight gradients of the dense and recurrent layers sum over
    // those only (CNT_NET_SKIP_PADDING=0: over all slots)
    {
        const char *e = std::getenv("CNT_NET_SKIP_PADDING");
        net->skip_padding = !e || std::atoi(e) != 0;
        CNT_TRY(device_alloc(net, (void **)&net->order, ((size_t)net->S * net->maxT + 4) * sizeof(int), true));
        net->order_count = net->order + (size_t)net->S * net->maxT;
    }
    // pattern types of the lower time resolutions, one buffer per resolution
    for (auto &L : net->layers) {
        if (L.res == 1) continue;
        bool have = false;
        for (auto &lr : net->low_res) have = have || lr.res == L.res;
        if (have) continue;
        cnt_network::LowRes lr = {L.res, nullptr, nullptr, nullptr, false};
        CNT_TRY(device_alloc(net, (void **)&lr.pat, (size_t)net->S * L.maxTr, true));
        CNT_TRY(device_alloc(net, (void **)&lr.order, ((size_t)net->S * L.maxTr + 4) * sizeof(int), true));
        lr.order_count = lr.order + (size_t)net->S * L.maxTr;
        net->low_res.push_back(lr);
    }
    // conditioning sub-network (NeuralNetwork.cpp:544-561, layers/wavNetCore.cu:455-492, :895-913): the wavnetc
    // layers read the flagged layer's outputs through the frame index in the input layer and send their summed
    // gradient back to it
    if (net->flagged >= 0) {
        const NetLayer &f = net->layers[(size_t)net->flagged];
        const int C = net->layers[(size_t)net->first_wavnetc].ctx_dim;
        CNT_REQUIRE(f.kind != K_WAVNETC && f.size == C, "network: layer '%s' feeds the wavnetc layers but has size %d, "
                    "contextDim is %d", f.name.c_str(), f.size, C);
        CNT_REQUIRE(net->layers.front().size == 1, "network: the conditioning sub-network reads the frame index from an "
                    "input layer of size 1");
        CNT_REQUIRE(f.err != nullptr, "network: layer '%s' feeds the wavnetc layers but has no error buffer",
                    f.name.c_str());
        CNT_TRY(device_alloc(net, (void **)&net->ctx_own, (size_t)C * slots * sizeof(float), true));
        CNT_TRY(device_alloc(net, (void **)&net->ctx_grad, (size_t)C * slots * sizeof(float), true));
        net->ctx = net->ctx_own;
    }
    for (auto &L : net->layers)
        if (L.kind == K_WAVNETC)
            CNT_REQUIRE(L.ctx_dim == net->layers[(size_t)net->first_wavnetc].ctx_dim, "network: wavnetc layer '%s' has "
                        "another contextDim than the first one", L.name.c_str());
    // checks that need the whole list
    const NetLayer &post = net->layers.back();
    CNT_REQUIRE(is_post_kind(post.kind), "network: the last layer must be a post-output layer (sse, mdn or dft), found "
                "'%s'", post.type.c_str());
    for (size_t i = 0; i + 1 < net->layers.size(); ++i)
        CNT_REQUIRE(!is_post_kind(net->layers[i].kind), "network: post-output layer '%s' is not the last layer",
                    net->layers[i].name.c_str());
    for (auto &L : net->layers)
        if (L.kind == K_FEEDBACK) {
            // NeuralNetwork.cpp:805-812 links every feedback layer to the post-output layer
            CNT_REQUIRE(post.kind == K_MDN && net->mdn_classes > 0, "network: a feedback layer needs an mdn post-output "
                        "layer with one softmax unit");
            CNT_REQUIRE(L.size == (L.fb_end - L.fb_start) + net->mdn_classes, "network: feedback layer '%s' has size "
                        "%d, expected %d + %d classes", L.name.c_str(), L.size, L.fb_end - L.fb_start, net->mdn_classes);
        }
    if (const char *e = std::getenv("CNT_NET_SIDE_STREAMS"))
        net->n_side = std::max(1, std::min((int)cnt_network::kMaxSide, std::atoi(e)));
    CNT_HIP(hipEventCreateWithFlags(&net->ev_main, hipEventDisableTiming));
    for (int k = 0; k < net->n_side; ++k) {
        CNT_HIP(hipStreamCreateWithFlags(&net->side[k], hipStreamNonBlocking));
        CNT_HIP(hipEventCreateWithFlags(&net->ev_side[k], hipEventDisableTiming));
        CNT_TRY(cnt::gemm_reserve_stream(net->side[k]));  // the weight halves' split-K scratch, not inside a pass
    }
    return CNT_OK;
}

}  // namespace
}  // namespace cnt

extern "C" {

int cnt_network_destroy(cnt_network *net) {
    if (!net) return CNT_OK;
    for (auto &L : net->layers) {
        if (L.lstm) cnt_lstm_destroy(L.lstm);
        if (L.cnn) cnt_cnn_destroy(L.cnn);
        if (L.mdn) cnt_mdn_destroy(L.mdn);
        if (L.dft) cnt_dft_destroy(L.dft);
    }
    for (void *p : net->allocations) (void)hipFree(p);
    for (int k = 0; k < cnt_network::kMaxSide; ++k) {
        if (net->side[k]) {
            // the product launcher keeps a scratch buffer per stream it has seen
            (void)hipStreamSynchronize(net->side[k]);
            cnt::gemm_release_stream(net->side[k]);
            (void)hipStreamDestroy(net->side[k]);
        }
        if (net->ev_side[k]) (void)hipEventDestroy(net->ev_side[k]);
    }
    if (net->ev_main) (void)hipEventDestroy(net->ev_main);
    delete net;
    return CNT_OK;
}

int cnt_network_create(const char *json_text, int parallel_sequences, int max_seq_length,
                       const cnt_network_options *options, cnt_network **out) {
    using namespace cnt;
    CNT_REQUIRE(json_text && out, "network_create: null argument");
    CNT_REQUIRE(parallel_sequences >= 1 && max_seq_length >= 1, "network_create: non-positive geometry");
    json::Parser parser{json_text, std::strlen(json_text)};
    json::Value doc;
    if (!parser.value(doc, 0)) {
        set_error("network_create: JSON error: %s", parser.error.c_str());
        return CNT_ERR_ARG;
    }
    CNT_REQUIRE(doc.type == json::Value::OBJ, "network_create: the network file is not a JSON object");
    const json::Value *layers = doc.get("layers");
    CNT_REQUIRE(layers && layers->type == json::Value::ARR, "network_create: missing section 'layers'");
    CNT_REQUIRE(layers->arr.size() >= 3, "network_create: a network needs an input layer, a hidden or output layer and "
                "a post-output layer");
    cnt_network *net = new (std::nothrow) cnt_network();
    CNT_REQUIRE(net != nullptr, "network_create: out of host memory");
    net->S = parallel_sequences;
    net->maxT = max_seq_length;
    if (options) net->overlap = options->no_overlap ? 0 : 1;
    if (const char *e = std::getenv("CNT_NET_OVERLAP")) net->overlap = std::atoi(e) != 0 ? 1 : 0;  // measurements
    int status = CNT_OK;
    for (const auto &obj : layers->arr) {
        if (obj.type != json::Value::OBJ) {
            set_error("network_create: an entry of 'layers' is not an object");
            status = CNT_ERR_ARG;
        } else {
            status = build_layer(net, obj, json_text, options);
        }
        if (status != CNT_OK) break;
    }
    if (status == CNT_OK) status = finish_build(net, doc.get("weights"));
    if (status != CNT_OK) {
        cnt_network_destroy(net);
        return status;
    }
    *out = net;
    return CNT_OK;
}

int cnt_network_info(cnt_network *net, int *n_layers, int *input_size, int *output_size, long *n_weights) {
    using namespace cnt;
    CNT_REQUIRE(net, "network_info: null handle");
    if (n_layers) *n_layers = (int)net->layers.size();
    if (input_size) *input_size = net->layers.front().size;
    if (output_size) *output_size = net->layers.back().size;
    if (n_weights) *n_weights = net->n_weights;
    return CNT_OK;
}

int cnt_network_layer_info(cnt_network *net, int index, cnt_layer_info *info) {
    using namespace cnt;
    CNT_REQUIRE(net && info, "network_layer_info: null argument");
    CNT_REQUIRE(index >= 0 && index < (int)net->layers.size(), "network_layer_info: no layer %d", index);
    const NetLayer &L = net->layers[(size_t)index];
    std::memset(info, 0, sizeof(*info));
    std::strncpy(info->name, L.name.c_str(), sizeof(info->name) - 1);
    std::strncpy(info->type, L.type.c_str(), sizeof(info->type) - 1);
    info->size = L.size;
    info->weight_offset = L.w_off;
    info->n_input = L.n_in;
    info->n_bias = L.n_bias;
    info->n_internal = L.n_int;
    info->outputs = L.out;
    info->output_errors = L.err;
    info->resolution = L.res;
    return CNT_OK;
}

float *cnt_network_weights(cnt_network *net) { return net ? net->weights : nullptr; }
float *cnt_network_weight_updates(cnt_network *net) { return net ? net->updates : nullptr; }

int cnt_network_randomize(cnt_network *net, unsigned seed, float range) {
    using namespace cnt;
    CNT_REQUIRE(net, "network_randomize: null handle");
    std::mt19937 gen(seed);
    std::uniform_real_distribution<float> dist(-range, range);
    std::vector<float> host((size_t)net->n_weights);
    for (auto &v : host) v = dist(gen);
    CNT_HIP(hipMemcpy(net->weights, host.data(), host.size() * sizeof(float), hipMemcpyHostToDevice));
    return CNT_OK;
}

int cnt_network_set_context(cnt_network *net, const float *ctx) {
    using namespace cnt;
    CNT_REQUIRE(net, "network_set_context: null handle");
    CNT_REQUIRE(net->flagged < 0, "network_set_context: this network computes the conditioning features itself (layer "
                "'%s')", net->layers[(size_t)net->flagged].name.c_str());
    // features handed over one column per slot are used where they stand; mean and deviation of a "contextMV" file
    // are applied where the library up-samples frame-rate features itself
    CNT_REQUIRE(!net->ctx_mv, "network_set_context: the wavnetc layers name a contextMV file; hand over normalised features "
                "and drop the key, or let the network up-sample them (layerFlag wavenetConditionInputLayer)");
    net->ctx = ctx;
    return CNT_OK;
}

int cnt_network_set_external_input(cnt_network *net, int layer_index, const float *data, int max_frames,
                                   const float *mean_std) {
    using namespace cnt;
    CNT_REQUIRE(net && data, "network_set_external_input: null argument");
    CNT_REQUIRE(layer_index >= 0 && layer_index < (int)net->layers.size() &&
                net->layers[(size_t)layer_index].kind == K_EXTERNAL,
                "network_set_external_input: layer %d is not an externalloader layer", layer_index);
    CNT_REQUIRE(max_frames >= 1, "network_set_external_input: no frames");
    NetLayer &L = net->layers[(size_t)layer_index];
    L.ext_data = data;
    L.ext_frames = max_frames;
    L.ext_mean_std = mean_std;
    return CNT_OK;
}

int cnt_network_load_sequences(cnt_network *net, void *stream_, int T, int Tmin, const char *patTypes,
                               const float *inputs, const float *targets) {
    using namespace cnt;
    CNT_REQUIRE(net && patTypes, "network_load_sequences: null argument");
    CNT_TRY(report_failure(net, static_cast<hipStream_t>(stream_)));
    CNT_REQUIRE(T >= 1 && T <= net->maxT && Tmin >= 1 && Tmin <= T, "network_load_sequences: lengths %d / %d outside "
                "1..%d", T, Tmin, net->maxT);
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    net->T = T;
    net->Tmin = Tmin;
    net->pat = patTypes;
    const size_t slots = (size_t)T * net->S;
    NetLayer &in = net->layers.front(), &post = net->layers.back();
    if (inputs)
        CNT_HIP(hipMemcpyAsync(in.out, inputs, slots * in.size * sizeof(float), hipMemcpyDeviceToDevice, stream));
    // a post-output layer keeps the targets in its own outputs() (layers/PostOutputLayer.cu:108-124)
    if (targets)
        CNT_HIP(hipMemcpyAsync(post.out, targets, slots * post.size * sizeof(float), hipMemcpyDeviceToDevice, stream));
    // Layer::loadSequences (layers/Layer.cu:254-305): lengths and pattern types at each layer's resolution
    for (auto &lr : net->low_res) {
        const int Tr = (T + lr.res - 1) / lr.res;
        const int n = Tr * net->S;
        hipLaunchKernelGGL(lowres_pat_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, net->S, T, Tr, lr.res,
                           patTypes, lr.pat);
        CNT_HIP(hipGetLastError());
    }
    // which time bases have a layer whose weight gradient can use the slot order; a fraction whose sequences all have the
    // full length has no padding slots
    bool wanted_main = false;
    for (size_t i = 1; i < net->layers.size(); ++i) {
        const NetLayer &L = net->layers[i];
        if (net->skip_padding && Tmin < T && (L.kind == K_DENSE || L.kind == K_LSTM) && L.res == 1) wanted_main = true;
    }
    LoadClears clears = {};  // the recurrent layers' per-fraction clears, done with the slot order in one launch below
    for (auto &lr : net->low_res) {
        bool wanted = false;
        for (size_t i = 1; i < net->layers.size(); ++i) {
            const NetLayer &L = net->layers[i];
            if (net->skip_padding && Tmin < T && (L.kind == K_DENSE || L.kind == K_LSTM) && L.res == lr.res) wanted = true;
        }
        lr.order_built = wanted;
        if (wanted) CNT_TRY(slot_order_build(stream, lr.pat, ((T + lr.res - 1) / lr.res) * net->S, net->S, lr.order, lr.order_count));
    }
    for (auto &L : net->layers) {
        L.T = (T + L.res - 1) / L.res;
        L.Tmin = (Tmin + L.res - 1) / L.res;
        L.N = L.T * net->S;
        L.pat = patTypes;
        L.order = wanted_main && L.res == 1 ? SlotOrder{net->order, net->order_count} : SlotOrder{nullptr, nullptr};
        for (auto &lr : net->low_res)
            if (lr.res == L.res) {
                L.pat = lr.pat;
                L.order = lr.order_built ? SlotOrder{lr.order, lr.order_count} : SlotOrder{nullptr, nullptr};
            }
        if (L.lstm) {
            CNT_TRY(lstm_load_sequences_collect(L.lstm, stream, L.pat, L.T, L.Tmin, clears));
            lstm_set_slot_order(L.lstm, &L.order);
        }
        if (L.mdn) CNT_TRY(cnt_mdn_load_sequences(L.mdn, stream, L.pat, L.T));
    }
    CNT_TRY(load_clear_and_order(stream, clears, patTypes, (int)slots, net->S, wanted_main ? net->order : nullptr,
                                 net->order_count));
    return CNT_OK;
}

int cnt_network_forward(cnt_network *net, void *stream_) {
    using namespace cnt;
    CNT_REQUIRE(net && net->T > 0, "network_forward: no fraction loaded");
    CNT_TRY(report_failure(net, static_cast<hipStream_t>(stream_)));
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    // what the skip layers' forward passes clear (layers/SkipAddLayer.cu:195-205)
    if (net->skip_error_count) CNT_TRY(fill_zero(stream, net->skip_errors, net->skip_error_count));
    for (size_t i = 1; i < net->layers.size(); ++i) {
        NetLayer &L = net->layers[i];
        const NetLayer &prev = net->layers[i - 1];
        const float *W = net->weights + L.w_off;
        const int N = L.N;
        const size_t count = (size_t)L.size * N;
        switch (L.kind) {
            case K_DENSE:
                CNT_TRY(cnt_dense_forward(stream, prev.size, L.size, N, L.act, L.bias, W, prev.out, L.out));
                break;
            case K_LSTM:
                CNT_TRY(cnt_lstm_forward(L.lstm, stream, W, prev.out, L.out));
                break;
            case K_SKIPINI:
            case K_SKIPADD:
                if (L.pre.size() > 1) {
                    ProfileScope prof(stream, "skip_sum");
                    if (L.ptrs_aligned && count % 4 == 0)
                        hipLaunchKernelGGL(skip_sum_kernel<float4>, dim3(blocks_for(count / 4)), dim3(256), 0, stream,
                                           count / 4, (int)L.pre.size(), L.in_ptrs, L.out);
                    else
                        hipLaunchKernelGGL(skip_sum_kernel<float>, dim3(blocks_for(count)), dim3(256), 0, stream, count,
                                           (int)L.pre.size(), L.in_ptrs, L.out);
                    CNT_HIP(hipGetLastError());
                }
                break;
            case K_SKIPCAT: {
                int at = 0;
                for (size_t k = 0; k < L.pre.size(); ++k) {
                    const NetLayer &src = net->layers[(size_t)L.pre[k]];
                    const int n = L.cat_hi[k] - L.cat_lo[k];
                    if (n == 0) continue;
                    const size_t c = (size_t)n * N;
                    hipLaunchKernelGGL(skipcat_forward_kernel, dim3(blocks_for(c)), dim3(256), 0, stream, c, n, src.size,
                                       L.cat_lo[k], L.size, at, src.out, L.out);
                    CNT_HIP(hipGetLastError());
                    at += n;
                }
                break;
            }
            case K_EXTERNAL:
                CNT_REQUIRE(L.ext_data, "network_forward: externalloader layer '%s' has no data "
                            "(cnt_network_set_external_input)", L.name.c_str());
                hipLaunchKernelGGL(external_load_kernel, dim3(blocks_for(count)), dim3(256), 0, stream, count, L.size,
                                   net->S, L.res, L.index_load_method, L.ext_frames, L.ext_data, net->layers.front().out,
                                   L.ext_mean_std, L.pat, L.out);
                CNT_HIP(hipGetLastError());
                break;
            case K_CNN:
                CNT_TRY(cnt_cnn_forward(L.cnn, stream, L.pat, L.T, W, prev.out, L.out));
                break;
            case K_WAVNETC:
                CNT_REQUIRE(L.ctx_dim == 0 || net->ctx, "network_forward: wavnetc layer '%s' has no conditioning features "
                            "(cnt_network_set_context)", L.name.c_str());
                if ((int)i == net->first_wavnetc && net->flagged >= 0) {
                    // WavNetCore::__loadContextBuff (layers/wavNetCore.cu:455-492) and the clearing of the gradient
                    // buffer for the conditioning sub-network (:645-647)
                    const NetLayer &f = net->layers[(size_t)net->flagged];
                    CNT_TRY(fill_zero(stream, net->ctx_grad, (size_t)L.ctx_dim * N));
                    CNT_TRY(cnt_wavnetc_load_context(stream, L.ctx_dim, net->S, N, f.T, f.res == 1 ? 1 : 0, f.out,
                                                     net->layers.front().out, net->ctx_mv, L.pat, net->ctx_own));
                }
                CNT_TRY(cnt_wavnetc_forward(stream, L.size, L.ctx_dim, N, L.pat, W, net->ctx, prev.out, L.core, L.cth,
                                            L.out));
                break;
            case K_FEEDBACK: {
                const NetLayer &post = net->layers.back();
                ProfileScope prof(stream, "feedback");
                hipLaunchKernelGGL(feedback_kernel, dim3(blocks_for(count)), dim3(256), 0, stream, count, L.size,
                                   L.fb_end - L.fb_start, prev.size, L.fb_start, net->S, post.size, net->mdn_target_start,
                                   L.pat, prev.out, post.out, L.out);
                CNT_HIP(hipGetLastError());
                break;
            }
            case K_MDN:
                CNT_TRY(cnt_mdn_forward(L.mdn, stream, prev.out));
                L.mdn_errors_done = false;  // new parameters: errors written for the old ones do not count
                break;
            case K_GATED:
                CNT_TRY(cnt_gatedact_forward(stream, L.size, N, L.pat, prev.out, L.out));
                break;
            case K_DFT: {
                // distances and gradient are both computed here (layers/DFTErrorPostoutputLayer.cu:1782-1839)
                const int len = L.T;
                CNT_TRY(cnt_dft_forward(L.dft, stream, 1, &len, prev.out, L.out, L.dft_errors));
                break;
            }
            default:
                break;
        }
    }
    return CNT_OK;
}

int cnt_network_calculate_error(cnt_network *net, void *stream_, float *loss_dev) {
    using namespace cnt;
    CNT_REQUIRE(net && loss_dev && net->T > 0, "network_calculate_error: null argument or no fraction loaded");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    NetLayer &post = net->layers.back();
    const NetLayer &last = net->layers[net->layers.size() - 2];
    if (post.kind == K_SSE) return cnt_sse_error(stream, post.size, post.N, post.pat, last.out, post.out, loss_dev);
    if (post.kind == K_DFT) {
        // DFTPostoutputLayer::calculateError (layers/DFTErrorPostoutputLayer.cu:2105-2150): the plain sum of the
        // distances of every resolution
        hipLaunchKernelGGL(sum_few_kernel, dim3(1), dim3(64), 0, stream, post.dft_error_count, post.dft_errors, loss_dev);
        CNT_HIP(hipGetLastError());
        return CNT_OK;
    }
    // The error pass and the gradient pass of a mixture layer read the same parameters: with an error buffer to write
    // to, both happen here, in one pass (cnt_mdn_error_backward), and the backward pass finds the layer's step done.
    // The preceding layer's error buffer has no other writer between the forward pass and the backward pass.
    if (last.err) {
        CNT_TRY(cnt_mdn_error_backward(post.mdn, stream, post.out, loss_dev, last.err));
        post.mdn_errors_done = true;
        return CNT_OK;
    }
    return cnt_mdn_calculate_error(post.mdn, stream, post.out, loss_dev);
}

int cnt_network_backward(cnt_network *net, void *stream_) {
    using namespace cnt;
    CNT_REQUIRE(net && net->T > 0, "network_backward: no fraction loaded");
    CNT_TRY(report_failure(net, static_cast<hipStream_t>(stream_)));
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    int next_side = 0;
    bool side_used[cnt_network::kMaxSide] = {};

    // The weight half of a layer's backward pass has no consumer before the optimizer, so it runs on a side stream
    // after the layer's error half.  Handing work to another stream costs the host two event calls; a network of
    // many small layers cannot afford them per layer (the host's enqueue rate then bounds its backward pass), so the
    // weight halves of small layers are collected and handed over a few at a time, those of large layers at once.
    std::vector<char> fan_done(net->layers.size(), 0);
    std::vector<char> errors_done(net->layers.size(), 0);  // error step done by the block launch of a later layer
    // A dense layer whose output errors are written by the one product of the layer above it (no skip layer links to
    // it): that product's epilogue multiplies with the derivative of the dense layer's activation, so the errors
    // arrive as deltas and the layer's own delta launch is left out.
    std::vector<char> delta_done(net->layers.size(), 0);
    std::vector<char> feeds_skip(net->layers.size(), 0);
    for (const NetLayer &S : net->layers)
        for (int x : S.pre)
            if (x >= 0 && (size_t)x < feeds_skip.size()) feeds_skip[(size_t)x] = 1;
    static const bool fuse_delta = [] { const char *e = std::getenv("CNT_NET_FUSE_DELTA"); return !e || std::atoi(e) != 0; }();
    auto delta_target = [&](size_t below) {
        const NetLayer &B = net->layers[below];
        // (the layer that feeds the conditioning of wavnetc layers gets their share of the gradient added later)
        return fuse_delta && below >= 1 && B.kind == K_DENSE && B.act != ACT_IDENTITY && B.err && !feeds_skip[below] &&
               (int)below != net->flagged && !is_skip_kind(net->layers[below + 1].kind);
    };
    for (auto &L : net->layers) L.colsum_rows = 0;
    static const bool fuse_blocks = [] { const char *e = std::getenv("CNT_NET_FUSE_BLOCKS"); return !e || std::atoi(e) != 0; }();
    // WaveNet residual block seen from its skip 1x1 layer i: [cnn 2R][wavnetc R][dense R, identity][skipadd, shares
    // the following sum][skipini][dense K, identity (i)]
    std::vector<int> fold_from(net->layers.size(), -1);  // skip 1x1 layer -> convolution layer folded into its launch
    std::vector<const float *> direct_from(net->layers.size(), nullptr);  // skip 1x1 layer -> the block above's sum
    static const bool direct_sums = [] { const char *e = std::getenv("CNT_NET_DIRECT_SUMS"); return !e || std::atoi(e) != 0; }();
    auto block_at = [&](size_t i) {
        if (!fuse_blocks || i < 5) return false;
        const NetLayer &sk = net->layers[i], &ini = net->layers[i - 1], &add = net->layers[i - 2], &out = net->layers[i - 3];
        const NetLayer &wav = net->layers[i - 4], &cnn = net->layers[i - 5];
        const int R = ini.size;
        auto aligned = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
        return sk.kind == K_DENSE && sk.act == ACT_IDENTITY && ini.kind == K_SKIPINI && ini.err && ini.err == ini.total &&
               is_sum_skip(add.kind) && add.total == ini.total && !add.needs_sum && add.live_targets == 0 && add.size == R &&
               out.kind == K_DENSE && out.act == ACT_IDENTITY && out.err == ini.total && out.size == R &&
               wav.kind == K_WAVNETC && wav.size == R && wav.core && (wav.ctx_dim == 0 || wav.cth) &&
               cnn.kind == K_CNN && cnn.size == 2 * R && cnn.err &&
               sk.N == ini.N && sk.N == out.N && sk.N == wav.N && sk.N == cnn.N &&
               wavenet_block_errors_supported(R, sk.size) && aligned(sk.err) && aligned(ini.total) && aligned(ini.eskip) &&
               aligned(wav.core) && aligned(wav.cth) && aligned(cnn.out) && aligned(cnn.err) &&
               aligned(net->weights + sk.w_off) && aligned(net->weights + out.w_off);
    };
    auto fold_at = [&](size_t i) {
        if (i < 8) return false;
        const NetLayer &C = net->layers[i], &closing = net->layers[i - 1], &sk = net->layers[i - 3];
        auto aligned = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
        return C.fold_ok && block_at(i - 3) && C.N == sk.N && closing.N == sk.N && cnn_foldable(C.cnn, closing.size) &&
               (C.delta_fused || !C.cnn_tanh) && aligned(net->weights + C.w_off) && aligned(C.err) && aligned(closing.eskip);
    };
    std::vector<size_t> pending;
    auto weight_half = [&](size_t i, hipStream_t ws) -> int {
        NetLayer &L = net->layers[i];
        NetLayer &prev = net->layers[i - 1];
        float *dW = net->updates + L.w_off;
        if (L.kind == K_DENSE) {
            const float *x = prev.out, *e = L.err;
            return dense_backward_weights_batch(ws, prev.size, L.size, L.N, 1, &L.bias, &x, &e, &dW, &L.order);
        }
        if (L.kind == K_LSTM) return cnt_lstm_backward_weights(L.lstm, ws, prev.out, dW);
        if (L.kind == K_CNN) return cnt_cnn_backward_weights(L.cnn, ws, L.pat, L.T, prev.out, L.err, dW);
        return cnt_wavnetc_backward_weights(ws, L.size, L.ctx_dim, L.N, net->ctx, L.cth, dW);
    };
    // Large layers' weight halves go round-robin over all side streams, the collected small ones over the first two:
    // measured on MI355X, a third stream gains 1% on the acoustic model (its last recurrent layer's and the dense
    // layers' weight gradients end the pass side by side) and loses 2% on the WaveNet stack (three batched products
    // at once crowd the error chain on the main stream).
    int next_small = 0;
    cnt_lstm *after_recursion = nullptr;  // set: the side stream waits for this layer's recursion, just launched
    auto next_side_stream = [&](hipStream_t *ws, bool large) -> int {
        int &cursor = large ? next_side : next_small;
        const int span = large ? net->n_side : std::min(net->n_side, 2);
        cursor %= span;
        *ws = net->side[cursor];
        if (after_recursion) {
            CNT_TRY(lstm_wait_recursion(after_recursion, *ws));
        } else {
            CNT_HIP(hipEventRecord(net->ev_main, stream));
            CNT_HIP(hipStreamWaitEvent(*ws, net->ev_main, 0));
        }
        side_used[cursor] = true;
        cursor = (cursor + 1) % span;
        return CNT_OK;
    };
    auto hand_over = [&](bool large) -> int {
        if (pending.empty()) return CNT_OK;
        hipStream_t ws;
        CNT_TRY(next_side_stream(&ws, large));
        static const bool split_lstm = [] { const char *e = std::getenv("CNT_NET_SPLIT_LSTM_WEIGHTS"); return e && std::atoi(e) != 0; }();
        for (size_t i : pending) {
            NetLayer &L = net->layers[i];
            if (L.kind == K_LSTM && split_lstm && net->n_side >= 2) {
                // CNT_NET_SPLIT_LSTM_WEIGHTS=1: the input-weight product and the recurrent-weight product (with the bias /
                // peephole sums) of a recurrent layer, which write disjoint ranges, side by side on two streams.  Off by
                // default: one after the other on one stream they take less from the recursion of the layer below and from
                // the error product beside them (acoustic model 2.51 -> 2.44 ms on MI355X).
                CNT_TRY(lstm_backward_weights_parts(L.lstm, ws, net->layers[i - 1].out, net->updates + L.w_off, 1));
                hipStream_t ws2;
                CNT_TRY(next_side_stream(&ws2, large));
                CNT_TRY(lstm_backward_weights_parts(L.lstm, ws2, net->layers[i - 1].out, net->updates + L.w_off, 2));
            } else {
                CNT_TRY(weight_half(i, ws));
            }
        }
        pending.clear();
        return CNT_OK;
    };
    // Small dense and wavnetc layers of one shape (the 1x1 layers and the conditioning projections of a stack of
    // identical blocks) wait for each other: eight of them are the problems of ONE product launch, which gives each
    // workgroup a k range eight times as long as a launch per layer would.  A layer's deltas, its input and its
    // tanh(context) buffer are final once its error half has run and stay untouched until the next pass, so the
    // weight half can wait for as long as the pass lasts.
    struct ShapeGroup {
        int kind, a, b, n, cap;
        std::vector<size_t> layers;
    };
    std::vector<ShapeGroup> groups;
    auto hand_over_group = [&](ShapeGroup &g) -> int {
        if (g.layers.empty()) return CNT_OK;
        hipStream_t ws;
        CNT_TRY(next_side_stream(&ws, false));
        const int count = (int)g.layers.size();
        const float *in0[kGemmMaxProb], *in1[kGemmMaxProb];
        float *dW[kGemmMaxProb], bias[kGemmMaxProb];
        cnt_cnn *cnn[kGemmMaxProb];
        const float *colsum[kGemmMaxProb];
        int colsum_rows[kGemmMaxProb];
        const NetLayer &first = net->layers[g.layers[0]];
        for (int z = 0; z < count; ++z) {
            NetLayer &L = net->layers[g.layers[(size_t)z]];
            NetLayer &prev = net->layers[g.layers[(size_t)z] - 1];
            dW[z] = net->updates + L.w_off;
            bias[z] = L.bias;
            in0[z] = g.kind == K_WAVNETC ? L.cth : prev.out;
            in1[z] = L.err;
            cnn[z] = L.cnn;
            colsum[z] = L.colsum; colsum_rows[z] = L.colsum_rows;
        }
        g.layers.clear();
        if (g.kind == K_DENSE) return dense_backward_weights_batch(ws, g.a, g.b, g.n, count, bias, in0, in1, dW, &first.order);
        if (g.kind == K_CNN) return cnn_backward_weights_batch(cnn, count, ws, first.pat, first.T, in0, in1, dW, colsum, colsum_rows);
        return wavnetc_backward_weights_batch(ws, g.a, g.b, g.n, count, net->ctx, in0, dW);
    };
    auto join_group = [&](size_t i) -> int {
        NetLayer &L = net->layers[i];
        const int a = L.kind == K_DENSE ? net->layers[i - 1].size : L.size;
        const int b = L.kind == K_DENSE ? L.size : L.ctx_dim;
        ShapeGroup *g = nullptr;
        for (ShapeGroup &c : groups) {
            if (c.kind != L.kind || c.a != a || c.b != b || c.n != L.N) continue;
            if (L.kind == K_CNN && !c.layers.empty()) {
                // same time base and pattern types, same window: only the dilation may differ
                const NetLayer &o = net->layers[c.layers[0]];
                if (o.pat != L.pat || o.T != L.T || !cnn_batch_compatible(o.cnn, L.cnn)) continue;
            }
            g = &c;
        }
        if (!g) {
            const int cap = L.kind == K_CNN ? kGemmMaxProb / cnn_batch_taps(L.cnn) : kGemmMaxProb;
            groups.push_back({L.kind, a, b, L.N, cap, {}});
            g = &groups.back();
        }
        g->layers.push_back(i);
        if ((int)g->layers.size() >= g->cap) CNT_TRY(hand_over_group(*g));
        // a network of many small layers that do not share shapes: do not let all of them wait for the pass's end
        size_t waiting = 0;
        for (const ShapeGroup &c : groups) waiting += c.layers.size();
        if (waiting >= 32)
            for (ShapeGroup &c : groups) CNT_TRY(hand_over_group(c));
        return CNT_OK;
    };
    for (size_t i = net->layers.size() - 1; i >= 1; --i) {
        NetLayer &L = net->layers[i];
        NetLayer &prev = net->layers[i - 1];
        const float *W = net->weights + L.w_off;
        const int N = L.N;
        // the input layer has no error buffer; a feedback layer that takes nothing from its preceding layer passes
        // nothing on, and neither does anything that feeds such a feedback layer's one-hot part
        float *prev_err = prev.err;
        if (prev.kind == K_FEEDBACK && prev.fb_end == prev.fb_start) prev_err = nullptr;
        const size_t count = (size_t)L.size * N;
        switch (L.kind) {
            case K_SSE:
                CNT_TRY(cnt_sse_backward(stream, L.size, N, L.pat, prev.out, L.out, prev.err));
                break;
            case K_MDN:
                // already written by cnt_network_calculate_error of this fraction's forward pass
                if (L.mdn_errors_done) L.mdn_errors_done = false;
                else CNT_TRY(cnt_mdn_backward(L.mdn, stream, L.out, prev.err));
                break;
            case K_DFT:
                // writes the whole preceding error buffer: gradients up to the waveform's length, zeros beyond
                // (the reference clears the buffer first, :1855-1856)
                CNT_TRY(cnt_dft_backward(L.dft, stream, prev.err));
                if (L.dft_beta > 0.0f) {
                    hipLaunchKernelGGL(waveform_mse_grad_kernel, dim3(blocks_for(count)), dim3(256), 0, stream, count,
                                       L.size, L.dft_beta, L.pat, prev.out, L.out, prev.err);
                    CNT_HIP(hipGetLastError());
                }
                break;
            case K_GATED:
                CNT_TRY(cnt_gatedact_backward(stream, L.size, N, L.pat, prev.out, L.err, prev.err));
                break;
            case K_DENSE:
            case K_LSTM:
            case K_CNN:
            case K_WAVNETC:
                if (L.kind == K_DENSE || L.kind == K_CNN) {
                    // a skip layer in front, whose errors this layer's product writes: its backward step (add the side
                    // buffer, hand the sum on) rides in the product's epilogue, and its own launch below is left out
                    FanOut fan = {};
                    const bool wanted = is_sum_skip(prev.kind) && prev_err && prev_err == prev.total && prev.N == N &&
                                        (prev.needs_sum || prev.live_targets > 0);
                    if (wanted) {
                        fan.n = prev.live_targets;
                        fan.targets = prev.tgt_ptrs;
                        fan.is_skip = prev.tgt_is_skip;
                        fan.from_skip = prev.needs_sum ? prev.eskip : nullptr;
                    }
                    bool fused = false;
                    if (errors_done[i]) {
                        // its errors went on inside the block launch of the skip 1x1 layer
                    } else if (L.kind == K_CNN && fold_at(i)) {
                        // the block below adds this layer's error product to its own sum
                        fold_from[i - 3] = (int)i;
                        fan_done[i - 1] = 1;
                        goto weight_half_of_layer;
                    } else if (block_at(i)) {
                        const NetLayer &out = net->layers[i - 3], &wav = net->layers[i - 4], &cnn = net->layers[i - 5];
                        const NetLayer *fold = fold_from[i] >= 0 ? &net->layers[(size_t)fold_from[i]] : nullptr;
                        FanOut block_fan = fan;
                        // with a folded convolution, what the later block handed to the closing skipadd layer comes in
                        // directly (that layer would have added it to the convolution's product and handed the sum on)
                        if (fold)
                            block_fan.from_skip = direct_from[i] ? direct_from[i] : net->layers[(size_t)fold_from[i] - 1].eskip;
                        // the block below folds this block's convolution in and is this sum's only reader: it reads
                        // the sum where this launch leaves it, nothing is handed on
                        if (direct_sums && wanted && cnn.direct_ok && fold_at(i - 5)) {
                            block_fan.n = 0;
                            block_fan.targets = nullptr;
                            block_fan.is_skip = nullptr;
                            direct_from[i - 8] = prev_err;
                        }
                        const bool fan_live = block_fan.n > 0 || block_fan.from_skip;
                        CNT_TRY(wavenet_block_errors(stream, prev.size, L.size, N, L.pat, W, net->weights + out.w_off, L.err,
                                                     prev_err, fan_live ? &block_fan : nullptr, wav.core,
                                                     wav.ctx_dim > 0 ? wav.cth : nullptr, cnn.delta_fused ? cnn.out : nullptr,
                                                     cnn.err, fold ? fold->cnn : nullptr,
                                                     fold ? net->weights + fold->w_off : nullptr, fold ? fold->err : nullptr,
                                                     cnn.colsum));
                        if (cnn.colsum) net->layers[i - 5].colsum_rows = wavenet_block_rows(N, fold != nullptr);
                        fan_done[i - 1] = 1;
                        errors_done[i - 3] = errors_done[i - 4] = 1;
                        goto weight_half_of_layer;
                    }
                    static const bool early = [] { const char *e = std::getenv("CNT_NET_EARLY_WEIGHTS"); return !e || std::atoi(e) != 0; }();
                    if (errors_done[i]) goto weight_half_of_layer;
                    if (L.kind == K_DENSE && early && net->overlap && prev_err && (double)prev.size * L.size * N >= 4e8) {
                        // a large dense layer: deltas first, then its weight half starts on a side stream next to the
                        // product for the preceding layer's errors instead of after it
                        CNT_TRY(dense_backward_errors_fan(stream, prev.size, L.size, N, delta_done[i] ? ACT_IDENTITY : L.act, W,
                                                          L.out, L.err, nullptr, nullptr, nullptr));
                        pending.push_back(i);
                        CNT_TRY(hand_over(true));
                        const bool below = !wanted && prev_err == prev.err && prev.N == N && delta_target(i - 1);
                        CNT_TRY(dense_backward_errors_fan(stream, prev.size, L.size, N, ACT_IDENTITY, W, L.out, L.err, prev_err,
                                                          wanted ? &fan : nullptr, &fused, below ? prev.act : ACT_IDENTITY,
                                                          below ? prev.out : nullptr));
                        if (below) delta_done[i - 1] = 1;
                        fan_done[i - 1] = fused ? 1 : 0;
                        break;
                    }
                    if (L.kind == K_DENSE) {
                        const bool below = !wanted && prev_err && prev_err == prev.err && prev.N == N && delta_target(i - 1);
                        CNT_TRY(dense_backward_errors_fan(stream, prev.size, L.size, N, delta_done[i] ? ACT_IDENTITY : L.act, W,
                                                          L.out, L.err, prev_err, wanted ? &fan : nullptr, &fused,
                                                          below ? prev.act : ACT_IDENTITY, below ? prev.out : nullptr));
                        if (below) delta_done[i - 1] = 1;
                    } else
                        CNT_TRY(cnn_backward_errors_fan(L.cnn, stream, L.pat, L.T, W, L.out, L.err, prev_err,
                                                        L.delta_fused ? 1 : 0, wanted ? &fan : nullptr, &fused));
                    fan_done[i - 1] = fused ? 1 : 0;
                } else if (L.kind == K_LSTM) {
                    static const bool early = [] { const char *e = std::getenv("CNT_NET_EARLY_WEIGHTS"); return !e || std::atoi(e) != 0; }();
                    if (early && net->overlap && prev_err) {
                        // The weight half starts right after the recursion, next to the product for the preceding
                        // layer's errors, instead of after it.  Each of these products alone keeps the matrix pipes about
                        // half busy (it waits on memory); two at once fill more of the machine, and the weight half is
                        // further along when the next layer's recursion starts: acoustic model 2.88 -> 2.78 ms.
                        CNT_TRY(cnt_lstm_backward_errors(L.lstm, stream, W, L.err, nullptr));
                        pending.push_back(i);
                        after_recursion = lstm_is_persistent(L.lstm) ? L.lstm : nullptr;
                        const int handed = hand_over(true);
                        after_recursion = nullptr;
                        CNT_TRY(handed);
                        if (prev_err == prev.err && prev.N == N && delta_target(i - 1)) {
                            CNT_TRY(lstm_prev_errors_delta(L.lstm, stream, W, prev_err, prev.act, prev.out));
                            delta_done[i - 1] = 1;
                        } else {
                            CNT_TRY(cnt_lstm_backward_prev_errors(L.lstm, stream, W, prev_err));
                        }
                        break;
                    }
                    CNT_TRY(cnt_lstm_backward_errors(L.lstm, stream, W, L.err, prev_err));
                } else {
                    if (errors_done[i]) {
                        if (L.ctx_dim > 0 && net->flagged >= 0)
                            CNT_TRY(wavnetc_context_grad(stream, L.size, L.ctx_dim, N, W, L.cth, net->ctx_grad));
                    } else {
                        CNT_TRY(cnt_wavnetc_backward_errors(stream, L.size, L.ctx_dim, N, L.pat, W, L.core, L.cth, L.err,
                                                            prev.err, net->flagged >= 0 ? net->ctx_grad : nullptr,
                                                            prev.delta_fused ? prev.out : nullptr));
                    }
                    if ((int)i == net->first_wavnetc && net->flagged >= 0) {
                        // every wavnetc layer has added its share; hand the sum per frame to the layer that feeds them
                        // (layers/wavNetCore.cu:895-913)
                        NetLayer &f = net->layers[(size_t)net->flagged];
                        CNT_TRY(cnt_wavnetc_sum_context_grad(stream, L.ctx_dim, net->S, f.res, f.N, N, f.pat, L.pat,
                                                             net->ctx_grad, f.err));
                    }
                }
            weight_half_of_layer:
                if (L.kind == K_WAVNETC && L.ctx_dim == 0) break;
                if (!net->overlap) {
                    CNT_TRY(weight_half(i, stream));
                    break;
                }
                if ((L.kind == K_DENSE || L.kind == K_WAVNETC ||
                     (L.kind == K_CNN && cnn_batch_taps(L.cnn) > 0 && cnn_batch_taps(L.cnn) <= kGemmMaxProb / 2)) &&
                    (double)prev.size * L.size * N < 4e8) {
                    CNT_TRY(join_group(i));
                    break;
                }
                pending.push_back(i);
                {
                    // small: below 4e8 multiply-adds (a WaveNet block's 64..128-wide layers over 32 000 samples are
                    // 1.6-2.6e8, the acoustic model's dense layers over 5 880 frames 5.6e8 and more); four at a time
                    // measured best on the 30-block WaveNet stack (5.36 -> 5.23 ms; two: no gain, eight: 5.31 ms)
                    const double macs = (double)prev.size * L.size * N;
                    const bool large = L.kind == K_LSTM || macs >= 4e8;
                    if (large || pending.size() >= 4) CNT_TRY(hand_over(large));
                }
                break;
            case K_SKIPINI:
            case K_SKIPADD: {
                if (!L.needs_sum && L.live_targets == 0) break;
                if (fan_done[i]) break;  // done in the epilogue of the following layer's product
                ProfileScope prof(stream, "skip_fan");
                const float *from_skip = L.needs_sum ? L.eskip : static_cast<const float *>(nullptr);
                if (L.ptrs_aligned && count % 4 == 0)
                    hipLaunchKernelGGL(skip_fan_kernel<float4>, dim3(blocks_for(count / 4)), dim3(256), 0, stream, count / 4,
                                       L.live_targets, L.tgt_ptrs, L.tgt_is_skip, const_cast<float *>(L.total), from_skip);
                else
                    hipLaunchKernelGGL(skip_fan_kernel<float>, dim3(blocks_for(count)), dim3(256), 0, stream, count,
                                       L.live_targets, L.tgt_ptrs, L.tgt_is_skip, const_cast<float *>(L.total), from_skip);
                CNT_HIP(hipGetLastError());
                break;
            }
            case K_SKIPCAT: {
                // SkipCatLayer::computeBackwardPass (layers/SkipCatLayer.cu:340-397)
                hipLaunchKernelGGL(add_inplace_kernel, dim3(blocks_for(count)), dim3(256), 0, stream, count, L.err, L.eskip);
                CNT_HIP(hipGetLastError());
                int at = 0;
                for (size_t k = 0; k < L.pre.size(); ++k) {
                    NetLayer &src = net->layers[(size_t)L.pre[k]];
                    const int n = L.cat_hi[k] - L.cat_lo[k];
                    const int skip = is_skip_kind(src.kind) ? 1 : 0;
                    float *target = skip ? src.eskip : src.err;
                    if (target != nullptr) {
                        if (!skip) CNT_TRY(fill_zero(stream, src.err, (size_t)src.size * net->S * src.maxTr));
                        if (n > 0) {
                            const size_t c = (size_t)n * N;
                            hipLaunchKernelGGL(skipcat_backward_kernel, dim3(blocks_for(c)), dim3(256), 0, stream, c, n,
                                               src.size, L.cat_lo[k], L.size, at, skip, L.pat, L.err, target);
                            CNT_HIP(hipGetLastError());
                        }
                    }
                    at += n;
                }
                break;
            }
            case K_FEEDBACK:
                if (L.fb_end > L.fb_start && prev.err) {
                    const size_t pc = (size_t)prev.size * N;
                    hipLaunchKernelGGL(feedback_backward_kernel, dim3(blocks_for(pc)), dim3(256), 0, stream, pc,
                                       prev.size, L.fb_start, L.fb_end, L.size, L.err, prev.err);
                    CNT_HIP(hipGetLastError());
                }
                break;
            default:
                break;
        }
    }
    CNT_TRY(hand_over(false));
    for (ShapeGroup &g : groups) CNT_TRY(hand_over_group(g));
    for (int k = 0; k < net->n_side; ++k) {
        if (!side_used[k]) continue;
        CNT_HIP(hipEventRecord(net->ev_side[k], net->side[k]));
        CNT_HIP(hipStreamWaitEvent(stream, net->ev_side[k], 0));
    }
    return CNT_OK;
}

// CNT_ERR_DEVICE if a recursion of one of the network's LSTM layers has given up (and ended) since the last report;
// clears every layer's mark and the device flag that holds the optimizer step back.
extern "C++" int cnt::report_failure(cnt_network *net, hipStream_t stream) {
    bool failed = false;
    for (auto &L : net->layers)
        if (L.lstm && cnt::lstm_take_failure(L.lstm)) failed = true;
    if (!failed) return CNT_OK;
    // The launch that gave up has ended (lstm_take_failure reports nothing earlier), so nothing sets the flag again.
    // The flag is cleared IN STREAM ORDER: an optimizer step of the failed pass that is already enqueued on this
    // stream still finds it set, whatever kind of stream this is.
    if (net->veto) CNT_TRY(fill_words(stream, reinterpret_cast<unsigned *>(net->veto), 1, 0u));

    set_error("network: an LSTM recursion gave up waiting for a neighbouring workgroup; the results of that pass are "
              "invalid and a weight update that followed it was skipped");
    return CNT_ERR_DEVICE;
}

int cnt_network_check(cnt_network *net, void *stream) {
    using namespace cnt;
    CNT_REQUIRE(net, "network_check: null handle");
    // every recurrent layer is looked at (each report clears that layer's mark), the first failure is returned
    int status = CNT_OK;
    for (auto &L : net->layers)
        if (L.lstm) {
            const int s = cnt_lstm_check(L.lstm, stream);
            if (s != CNT_OK && status == CNT_OK) status = s;
        }
    if (status != CNT_OK) {
        // every stream of the network has been waited for: the flag is cleared on this stream and the clear awaited
        if (net->veto) {
            CNT_TRY(fill_words(static_cast<hipStream_t>(stream), reinterpret_cast<unsigned *>(net->veto), 1, 0u));
            CNT_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
        }
    }
    if (status == CNT_OK) status = report_failure(net, static_cast<hipStream_t>(stream));  // a launch that ended on another stream
    return status;
}

int cnt_network_set_wait_bounds(cnt_network *net, int layer_index, unsigned spin_limit, int poll_delay_backward,
                                int poll_delay_forward) {
    using namespace cnt;
    CNT_REQUIRE(net, "network_set_wait_bounds: null handle");
    CNT_REQUIRE(layer_index >= 0 && (size_t)layer_index < net->layers.size() && net->layers[(size_t)layer_index].lstm,
                "network_set_wait_bounds: layer %d is not an LSTM layer", layer_index);
    return cnt_lstm_set_wait_bounds(net->layers[(size_t)layer_index].lstm, spin_limit, poll_delay_backward, poll_delay_forward);
}

int cnt_network_update(cnt_network *net, void *stream_, int option, float learning_rate, float momentum,
                       float frac_length) {
    using namespace cnt;
    CNT_REQUIRE(net, "network_update: null handle");
    // A pass whose recursion gave up must not reach the weights.  Two nets: launches that have already ended are
    // seen here, on the host; one that ends later sets the device flag the optimizer kernel looks at, and the next
    // call into the network reports it.
    CNT_TRY(report_failure(net, static_cast<hipStream_t>(stream_)));
    const size_t n = (size_t)net->n_weights;
    if (!net->cur_updates) {
        CNT_TRY(device_alloc(net, (void **)&net->cur_updates, n * sizeof(float), true));
        CNT_TRY(device_alloc(net, (void **)&net->deltas, n * sizeof(float), true));
    }
    const bool adagrad = option == 1 || option == 3, adam = option == 5;
    if ((adagrad || adam) && net->stats_option != option) {
        CNT_REQUIRE(net->stats_option < 0, "network_update: the optimizer option changed from %d to %d", net->stats_option,
                    option);
        // optimizers/Optimizer.cu:427-447: AdaGrad statistics start at 1e-6, Adam's (m, v) pairs at 0
        std::vector<float> init(adam ? 2 * n : n, adam ? 0.0f : 1e-6f);
        CNT_TRY(device_alloc(net, (void **)&net->stats, init.size() * sizeof(float), false));
        CNT_HIP(hipMemcpy(net->stats, init.data(), init.size() * sizeof(float), hipMemcpyHostToDevice));
        net->stats_option = option;
    }
    if (adam) {
        // beta1^t and beta2^t live in device memory and advance under the same flag as the step itself, so that a step
        // the device-side veto skips leaves them untouched as well
        if (!net->adam_accum) {
            const float ones[2] = {1.0f, 1.0f};
            CNT_TRY(device_alloc(net, (void **)&net->adam_accum, sizeof(ones), false));
            CNT_HIP(hipMemcpy(net->adam_accum, ones, sizeof(ones), hipMemcpyHostToDevice));
        }
        CNT_TRY(opt_adam_advance(static_cast<hipStream_t>(stream_), net->adam_accum, net->veto));
    }
    const float *accum_dev = adam ? net->adam_accum : nullptr;
    bool own_rates = false;
    for (const auto &L : net->layers) own_rates = own_rates || (L.weight_count() > 0 && L.learning_rate > -0.5f);
    if (!own_rates)
        return opt_step_guarded(static_cast<hipStream_t>(stream_), option, (long)n, net->weights, net->updates, net->cur_updates,
                                net->stats, net->deltas, nullptr, frac_length, 0.0f, 0.0f, learning_rate, momentum, net->veto,
                                accum_dev);
    // a layer's own "learningRate" replaces the optimizer's (optimizers/SteepestDescentOptimizer.cu:402-403, :425-426): one
    // launch per trainable layer
    for (const auto &L : net->layers) {
        const long c = L.weight_count();
        if (c == 0) continue;
        const long o = L.w_off;
        float *st = net->stats ? net->stats + (adam ? 2 * o : o) : nullptr;
        CNT_TRY(opt_step_guarded(static_cast<hipStream_t>(stream_), option, c, net->weights + o, net->updates + o,
                                 net->cur_updates + o, st, net->deltas + o, nullptr, frac_length, 0.0f, 0.0f,
                                 L.learning_rate > -0.5f ? L.learning_rate : learning_rate, momentum, net->veto, accum_dev));
    }
    return CNT_OK;
}

int cnt_network_export_json(cnt_network *net, char *buf, size_t cap, size_t *needed) {
    using namespace cnt;
    CNT_REQUIRE(net && needed, "network_export_json: null argument");
    std::vector<float> host((size_t)net->n_weights);
    CNT_HIP(hipDeviceSynchronize());
    if (!host.empty())
        CNT_HIP(hipMemcpy(host.data(), net->weights, host.size() * sizeof(float), hipMemcpyDeviceToHost));
    std::string s = "{\"layers\":[";
    for (size_t i = 0; i < net->layers.size(); ++i) {
        if (i) s += ",";
        s += net->layers[i].text;
    }
    s += "],\"weights\":{";
    bool first = true;
    char num[32];
    for (const auto &L : net->layers) {
        if (L.weight_count() == 0) continue;
        if (!first) s += ",";
        first = false;
        s += "\"" + L.name + "\":{";
        const char *keys[3] = {"input", "bias", "internal"};
        const long len[3] = {L.n_in, L.n_bias, L.n_int};
        long at = L.w_off;
        for (int k = 0; k < 3; ++k) {
            s += std::string(k ? "," : "") + "\"" + keys[k] + "\":[";
            for (long j = 0; j < len[k]; ++j) {
                snprintf(num, sizeof(num), j ? ",%.9g" : "%.9g", (double)host[(size_t)(at + j)]);
                s += num;
            }
            s += "]";
            at += len[k];
        }
        s += "}";
    }
    s += "}}";
    *needed = s.size() + 1;
    if (buf && cap >= s.size() + 1) std::memcpy(buf, s.c_str(), s.size() + 1);
    return CNT_OK;
}

}  // extern "C"
