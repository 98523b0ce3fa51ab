// C++ layer shells over the C ABI (include/currennt_hip.h).
//
// These classes mirror the part of the reference's layer interface that the backward hot path uses
// (CURRENNT_codes/currennt_lib/src/layers/Layer.hpp:41-415, TrainableLayer.hpp:36-212,
// PostOutputLayer.cu:108-124): a layer owns outputs(), outputErrors() and patTypes(), a trainable
// layer owns weights() and weightUpdates(), a layer writes its predecessor's outputErrors(), and the
// call order per fraction is loadSequences -> computeForwardPass -> calculateError ->
// computeBackwardPass.  Method names and argument meaning follow the reference; the bodies only
// forward to the C ABI, and a non-zero status becomes std::runtime_error as in the reference
// (currennt/src/main.cpp:692-695 catches it).  Device memory is plain hipMalloc.
#pragma once

#include <cstdlib>
#include <hip/hip_runtime.h>

#include <cstddef>
#include <memory>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/currennt_hip.h"

namespace currennt_amd {

inline void check(int status, const char *what) {
    if (status != CNT_OK) throw std::runtime_error(std::string(what) + ": " + cnt_last_error());
}
inline void hip_check(hipError_t e, const char *what) {
    if (e != hipSuccess) throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
}

// Minimal device vector (the role thrust::device_vector plays in the reference).
template <typename T>
class DeviceVector {
public:
    DeviceVector() : ptr_(nullptr), n_(0) {}
    explicit DeviceVector(size_t n) : ptr_(nullptr), n_(0) { resize(n); }
    DeviceVector(const DeviceVector &) = delete;
    DeviceVector &operator=(const DeviceVector &) = delete;
    ~DeviceVector() { if (ptr_) (void)hipFree(ptr_); }
    void resize(size_t n) {
        if (ptr_) (void)hipFree(ptr_);
        ptr_ = nullptr; n_ = n;
        if (n) {
            hip_check(hipMalloc(reinterpret_cast<void **>(&ptr_), n * sizeof(T)), "hipMalloc");
            hip_check(hipMemset(ptr_, 0, n * sizeof(T)), "hipMemset");
        }
    }
    void assign(const std::vector<T> &h) {
        if (h.size() > n_) resize(h.size());
        if (!h.empty()) hip_check(hipMemcpy(ptr_, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice), "hipMemcpy");
    }
    std::vector<T> to_host() const {
        std::vector<T> h(n_);
        if (n_) hip_check(hipMemcpy(h.data(), ptr_, n_ * sizeof(T), hipMemcpyDeviceToHost), "hipMemcpy");
        return h;
    }
    T *data() { return ptr_; }
    const T *data() const { return ptr_; }
    size_t size() const { return n_; }

private:
    T *ptr_;
    size_t n_;
};

typedef DeviceVector<float> real_vector;
typedef DeviceVector<char> pattype_vector;

// What Layer::loadSequences needs from a DataSetFraction (data_sets/DataSetFraction.hpp).
struct Fraction {
    int maxSeqLength;  // curMaxSeqLength
    int minSeqLength;  // curMinSeqLength
    std::vector<char> patTypes;  // T*S
    std::vector<float> inputs;   // inputSize x T*S
    std::vector<float> targets;  // targetSize x T*S
};

class Layer {
public:
    Layer(const std::string &name, int size, int parallelSequences, int maxSeqLength, Layer *preceding, hipStream_t stream)
        : m_name(name), m_size(size), m_parallel(parallelSequences), m_maxSeqLength(maxSeqLength),
          m_curMaxSeqLength(0), m_curMinSeqLength(0), m_preceding(preceding), m_stream(stream),
          m_outputs((size_t)size * parallelSequences * maxSeqLength),
          m_outputErrors((size_t)size * parallelSequences * maxSeqLength),
          m_patTypes((size_t)parallelSequences * maxSeqLength) {}
    virtual ~Layer() {}

    virtual const std::string &type() const = 0;
    virtual void loadSequences(const Fraction &fraction) {
        m_curMaxSeqLength = fraction.maxSeqLength;
        m_curMinSeqLength = fraction.minSeqLength;
        m_patTypes.assign(fraction.patTypes);
    }
    virtual void computeForwardPass(int nnState) = 0;
    virtual void computeBackwardPass(int nnState) = 0;

    const std::string &name() const { return m_name; }
    int size() const { return m_size; }
    int parallelSequences() const { return m_parallel; }
    int maxSeqLength() const { return m_maxSeqLength; }
    int curMaxSeqLength() const { return m_curMaxSeqLength; }
    int curMinSeqLength() const { return m_curMinSeqLength; }
    int curSlots() const { return m_curMaxSeqLength * m_parallel; }
    real_vector &outputs() { return m_outputs; }
    real_vector &outputErrors() { return m_outputErrors; }
    pattype_vector &patTypes() { return m_patTypes; }
    Layer &precedingLayer() { return *m_preceding; }
    bool hasPrecedingLayer() const { return m_preceding != nullptr; }
    hipStream_t stream() const { return m_stream; }

protected:
    std::string m_name;
    int m_size, m_parallel, m_maxSeqLength, m_curMaxSeqLength, m_curMinSeqLength;
    Layer *m_preceding;
    hipStream_t m_stream;
    real_vector m_outputs, m_outputErrors;
    pattype_vector m_patTypes;
};

class InputLayer : public Layer {
public:
    InputLayer(int size, int parallelSequences, int maxSeqLength, hipStream_t stream)
        : Layer("input", size, parallelSequences, maxSeqLength, nullptr, stream) {}
    const std::string &type() const override { static const std::string s("input"); return s; }
    void loadSequences(const Fraction &fraction) override {
        Layer::loadSequences(fraction);
        m_outputs.assign(fraction.inputs);
    }
    void computeForwardPass(int) override {}
    void computeBackwardPass(int) override {}
};

class TrainableLayer : public Layer {
public:
    TrainableLayer(const std::string &name, int size, int parallelSequences, int maxSeqLength, Layer *preceding,
                   hipStream_t stream, size_t weightCount, float bias)
        : Layer(name, size, parallelSequences, maxSeqLength, preceding, stream), m_bias(bias), m_weights(weightCount),
          m_weightUpdates(weightCount) {
        // a weight gradient may go through split partial products: the stream's scratch buffer for them is allocated
        // here, at construction (once per stream, later calls find it), so that no computeBackwardPass allocates
        // (CNT_HOST_NO_RESERVE leaves it to the first product that needs it: how the test sees the difference)
        if (!std::getenv("CNT_HOST_NO_RESERVE")) check(cnt_gemm_reserve(stream), "gemm reserve");
    }
    real_vector &weights() { return m_weights; }
    real_vector &weightUpdates() { return m_weightUpdates; }
    float bias() const { return m_bias; }

protected:
    float m_bias;
    real_vector m_weights, m_weightUpdates;
};

// FeedForwardLayer<TDevice, TActFn> (layers/FeedForwardLayer.cu); act is one of CNT_ACT_*.
class FeedForwardLayer : public TrainableLayer {
public:
    FeedForwardLayer(const std::string &name, int act, int size, Layer *preceding, float bias = 1.0f)
        : TrainableLayer(name, size, preceding->parallelSequences(), preceding->maxSeqLength(), preceding,
                         preceding->stream(), (size_t)preceding->size() * size + size, bias),
          m_act(act) {}
    const std::string &type() const override {
        static const std::string names[4] = {"feedforward_identity", "feedforward_tanh", "feedforward_logistic",
                                             "feedforward_relu"};
        return names[m_act];
    }
    void computeForwardPass(int) override {
        check(cnt_dense_forward(m_stream, m_preceding->size(), m_size, curSlots(), m_act, m_bias, m_weights.data(),
                                m_preceding->outputs().data(), m_outputs.data()), "feedforward forward");
    }
    void computeBackwardPass(int) override {
        float *prev = m_preceding->hasPrecedingLayer() ? m_preceding->outputErrors().data() : nullptr;
        check(cnt_dense_backward(m_stream, m_preceding->size(), m_size, curSlots(), m_act, m_bias, m_weights.data(),
                                 m_preceding->outputs().data(), m_outputs.data(), m_outputErrors.data(), prev,
                                 m_weightUpdates.data()), "feedforward backward");
    }

private:
    int m_act;
};

// LstmLayer<TDevice> (layers/LstmLayer.cu), "lstm" and "blstm".
class LstmLayer : public TrainableLayer {
public:
    LstmLayer(const std::string &name, int size, bool bidirectional, Layer *preceding, float bias = 1.0f)
        : TrainableLayer(name, size, preceding->parallelSequences(), preceding->maxSeqLength(), preceding,
                         preceding->stream(), (size_t)cnt_lstm_weight_count(preceding->size(), size, bidirectional), bias),
          m_bidirectional(bidirectional), m_handle(nullptr) {
        cnt_lstm_desc d = {preceding->size(), size, bidirectional ? 1 : 0, m_parallel, m_maxSeqLength, bias};
        check(cnt_lstm_create(&d, &m_handle), "lstm create");
    }
    ~LstmLayer() override { cnt_lstm_destroy(m_handle); }
    const std::string &type() const override {
        static const std::string u("lstm"), b("blstm");
        return m_bidirectional ? b : u;
    }
    void loadSequences(const Fraction &fraction) override {
        Layer::loadSequences(fraction);
        check(cnt_lstm_load_sequences(m_handle, m_stream, m_patTypes.data(), m_curMaxSeqLength, m_curMinSeqLength),
              "lstm loadSequences");
    }
    void computeForwardPass(int) override {
        check(cnt_lstm_forward(m_handle, m_stream, m_weights.data(), m_preceding->outputs().data(), m_outputs.data()),
              "lstm forward");
    }
    void computeBackwardPass(int) override {
        float *prev = m_preceding->hasPrecedingLayer() ? m_preceding->outputErrors().data() : nullptr;
        check(cnt_lstm_backward(m_handle, m_stream, m_weights.data(), m_preceding->outputs().data(), m_outputs.data(),
                                m_outputErrors.data(), prev, m_weightUpdates.data()), "lstm backward");
    }
    // waits for the stream; throws if a recursion kernel reported a stalled neighbour
    void synchronizeAndCheck() { check(cnt_lstm_check(m_handle, m_stream), "lstm check"); }

private:
    bool m_bidirectional;
    cnt_lstm *m_handle;
};

// SkipLayer (layers/SkipLayer.hpp:40-75): a layer that sums several earlier layers and, in the backward pass, receives
// errors both from the layer that follows it (outputErrors()) and from later skip layers that read it
// (outputErrorsFromSkipLayer()).
class SkipLayer : public Layer {
public:
    SkipLayer(const std::string &name, int size, const std::vector<Layer *> &precedingLayers)
        : Layer(name, size, precedingLayers.back()->parallelSequences(), precedingLayers.back()->maxSeqLength(),
                precedingLayers.back(), precedingLayers.back()->stream()),
          m_preLayers(precedingLayers), m_outputErrorsFromSkipLayer(m_outputs.size()) {}
    real_vector &outputErrorsFromSkipLayer() { return m_outputErrorsFromSkipLayer; }
    std::vector<Layer *> &PreLayers() { return m_preLayers; }

protected:
    std::vector<Layer *> m_preLayers;
    real_vector m_outputErrorsFromSkipLayer;
};

// SkipAddLayer<TDevice> (layers/SkipAddLayer.cu:77-170, 186-240, 305-346), "skipini" and "skipadd": outputs = sum of
// the preceding layers' outputs; backward: errors += errors from later skip layers, then every predecessor gets the
// sum -- added to its outputErrorsFromSkipLayer() if it is a skip layer, assigned to its outputErrors() otherwise.
class SkipAddLayer : public SkipLayer {
public:
    SkipAddLayer(const std::string &name, const std::string &type, int size, const std::vector<Layer *> &precedingLayers)
        : SkipLayer(name, size, precedingLayers), m_type(type) {
        if (precedingLayers.empty() || precedingLayers.size() > 8)
            throw std::runtime_error("SkipAddLayer: 1..8 preceding layers");
        for (Layer *l : precedingLayers)
            if (l->size() != size) throw std::runtime_error("Error in skipadd/skipini: layer size mismatch in " + name);
    }
    const std::string &type() const override { return m_type; }
    void computeForwardPass(int) override {
        std::vector<const float *> in;
        for (Layer *l : m_preLayers) in.push_back(l->outputs().data());
        check(cnt_skipadd_forward(m_stream, (long)m_size * curSlots(), (int)in.size(), in.data(), m_outputs.data(),
                                  m_outputErrors.data(), m_outputErrorsFromSkipLayer.data()), "skipadd forward");
    }
    void computeBackwardPass(int) override {
        std::vector<float *> targets;
        std::vector<int> is_skip;
        for (Layer *l : m_preLayers) {
            SkipLayer *sk = dynamic_cast<SkipLayer *>(l);
            targets.push_back(sk ? sk->outputErrorsFromSkipLayer().data() : l->outputErrors().data());
            is_skip.push_back(sk ? 1 : 0);
        }
        check(cnt_skipadd_backward(m_stream, (long)m_size * curSlots(), m_outputErrors.data(),
                                   m_outputErrorsFromSkipLayer.data(), (int)targets.size(), targets.data(),
                                   is_skip.data()), "skipadd backward");
    }

private:
    std::string m_type;
};

// CNNLayer<TDevice>, 1-D path (layers/CNNLayer.cu:880-1097 constructor, :1099-1224, :1409-1597): one half width and one
// tap interval per filter ("window_width", "window_tap_interval"), "causal", "tanhoutput".
class CNNLayer : public TrainableLayer {
public:
    CNNLayer(const std::string &name, int size, Layer *preceding, const std::vector<int> &halfWidth,
             const std::vector<int> &tapInterval, bool causal, bool tanhOutput, float bias = 1.0f)
        : TrainableLayer(name, size, preceding->parallelSequences(), preceding->maxSeqLength(), preceding,
                         preceding->stream(), 0, bias), m_handle(nullptr) {
        if ((int)halfWidth.size() != size || (int)tapInterval.size() != size)
            throw std::runtime_error("CNNLayer: one window width and one tap interval per filter");
        cnt_cnn_desc d = {preceding->size(), size, m_parallel, m_maxSeqLength, causal ? 1 : 0, tanhOutput ? 1 : 0, bias};
        check(cnt_cnn_create(&d, halfWidth.data(), tapInterval.data(), &m_handle), "cnn create");
        m_weights.resize((size_t)cnt_cnn_weight_count(m_handle));
        m_weightUpdates.resize((size_t)cnt_cnn_weight_count(m_handle));
    }
    ~CNNLayer() override { cnt_cnn_destroy(m_handle); }
    const std::string &type() const override { static const std::string s("cnn"); return s; }
    void computeForwardPass(int) override {
        check(cnt_cnn_forward(m_handle, m_stream, m_patTypes.data(), m_curMaxSeqLength, m_weights.data(),
                              m_preceding->outputs().data(), m_outputs.data()), "cnn forward");
    }
    void computeBackwardPass(int) override {
        float *prev = m_preceding->hasPrecedingLayer() ? m_preceding->outputErrors().data() : nullptr;
        check(cnt_cnn_backward(m_handle, m_stream, m_patTypes.data(), m_curMaxSeqLength, m_weights.data(),
                               m_preceding->outputs().data(), m_outputs.data(), m_outputErrors.data(), prev,
                               m_weightUpdates.data()), "cnn backward");
    }

private:
    cnt_cnn *m_handle;
};

// WavNetCore<TDevice> (layers/wavNetCore.cu:455-492, 629-711, 801-916), "wavnetc": tanh(a + W^T c) * sigmoid(b + V^T c)
// over the two halves of the preceding layer, c = conditioning features.  The first such layer of a network owns the
// conditioning buffer and its gradient; later ones link to it (layers/wavNetCore.cu:300-360).
class WavNetCore : public TrainableLayer {
public:
    WavNetCore(const std::string &name, int size, Layer *preceding, int contextDim, WavNetCore *firstCore)
        : TrainableLayer(name, size, preceding->parallelSequences(), preceding->maxSeqLength(), preceding,
                         preceding->stream(), (size_t)contextDim * 2 * size, 1.0f),
          m_contextDim(contextDim), m_first(firstCore ? firstCore : this),
          m_coreBuf((size_t)2 * size * m_parallel * m_maxSeqLength),
          m_contextTanhBuf((size_t)2 * size * m_parallel * m_maxSeqLength) {
        if (preceding->size() != 2 * size) throw std::runtime_error("wavnetc: the preceding layer must be twice as wide");
        if (!firstCore) {
            m_contextBuf.resize((size_t)contextDim * m_parallel * m_maxSeqLength);
            m_contextGraBuf.resize((size_t)contextDim * m_parallel * m_maxSeqLength);
        }
    }
    const std::string &type() const override { static const std::string s("wavnetc"); return s; }
    // conditioning features of the fraction at the layer's time resolution, contextDim x T*S (the reference reads and
    // up-samples them from the fraction's auxiliary data: cnt_wavnetc_load_context does that part)
    void loadContext(const std::vector<float> &context) { m_first->m_contextBuf.assign(context); }
    real_vector &contextGradients() { return m_first->m_contextGraBuf; }
    void computeForwardPass(int) override {
        check(cnt_wavnetc_forward(m_stream, m_size, m_contextDim, curSlots(), m_patTypes.data(), m_weights.data(),
                                  m_first->m_contextBuf.data(), m_preceding->outputs().data(), m_coreBuf.data(),
                                  m_contextTanhBuf.data(), m_outputs.data()), "wavnetc forward");
    }
    void computeBackwardPass(int) override {
        check(cnt_wavnetc_backward(m_stream, m_size, m_contextDim, curSlots(), m_patTypes.data(), m_weights.data(),
                                   m_first->m_contextBuf.data(), m_coreBuf.data(), m_contextTanhBuf.data(),
                                   m_outputErrors.data(), m_preceding->outputErrors().data(), m_weightUpdates.data(),
                                   nullptr), "wavnetc backward");
    }

private:
    int m_contextDim;
    WavNetCore *m_first;
    real_vector m_coreBuf, m_contextTanhBuf, m_contextBuf, m_contextGraBuf;
};

// GatedActLayer<TDevice> (layers/GatedActLayer.cu:177-263), "gatedact": tanh(first half) * sigmoid(second half).
class GatedActLayer : public Layer {
public:
    GatedActLayer(const std::string &name, int size, Layer *preceding)
        : Layer(name, size, preceding->parallelSequences(), preceding->maxSeqLength(), preceding, preceding->stream()) {
        if (preceding->size() != 2 * size) throw std::runtime_error("gatedact: the preceding layer must be twice as wide");
    }
    const std::string &type() const override { static const std::string s("gatedact"); return s; }
    void computeForwardPass(int) override {
        check(cnt_gatedact_forward(m_stream, m_size, curSlots(), m_patTypes.data(), m_preceding->outputs().data(),
                                   m_outputs.data()), "gatedact forward");
    }
    void computeBackwardPass(int) override {
        check(cnt_gatedact_backward(m_stream, m_size, curSlots(), m_patTypes.data(), m_preceding->outputs().data(),
                                    m_outputErrors.data(), m_preceding->outputErrors().data()), "gatedact backward");
    }
};

// Post-output layers keep the targets in their own outputs() and write the preceding layer's errors
// (layers/PostOutputLayer.cu:108-124); calculateError() returns the fraction's error.
class PostOutputLayer : public Layer {
public:
    PostOutputLayer(const std::string &name, int size, Layer *preceding)
        : Layer(name, size, preceding->parallelSequences(), preceding->maxSeqLength(), preceding, preceding->stream()),
          m_error(8) {}
    void loadSequences(const Fraction &fraction) override {
        Layer::loadSequences(fraction);
        m_outputs.assign(fraction.targets);
    }
    virtual float calculateError() = 0;

protected:
    real_vector m_error;
};

// SsePostOutputLayer<TDevice> (layers/SsePostOutputLayer.cu:94-136, 166-267), "sse".
class SsePostOutputLayer : public PostOutputLayer {
public:
    explicit SsePostOutputLayer(Layer *preceding) : PostOutputLayer("postoutput", preceding->size(), preceding) {}
    const std::string &type() const override { static const std::string s("sse"); return s; }
    void computeForwardPass(int) override {}
    float calculateError() override {
        check(cnt_sse_error(m_stream, m_size, curSlots(), m_patTypes.data(), m_preceding->outputs().data(),
                            m_outputs.data(), m_error.data()), "sse calculateError");
        hip_check(hipStreamSynchronize(m_stream), "hipStreamSynchronize");
        return m_error.to_host()[0];
    }
    void computeBackwardPass(int) override {
        check(cnt_sse_backward(m_stream, m_size, curSlots(), m_patTypes.data(), m_preceding->outputs().data(),
                               m_outputs.data(), m_preceding->outputErrors().data()), "sse backward");
    }
};

// MDNLayer<TDevice> (layers/MDNLayer.cu:280-324, 457-545, 797-917), "mdn": `config` is the mixture configuration the
// reference reads from its --mdn_config file, [nUnits | 5 numbers per unit].
class MDNLayer : public PostOutputLayer {
public:
    MDNLayer(int size, Layer *preceding, const std::vector<float> &config)
        : PostOutputLayer("postoutput", size, preceding), m_handle(nullptr) {
        cnt_mdn_desc d = {preceding->size(), size, m_parallel, m_maxSeqLength, 0, 0};
        check(cnt_mdn_create(&d, config.data(), (int)config.size(), &m_handle), "mdn create");
    }
    ~MDNLayer() override { cnt_mdn_destroy(m_handle); }
    const std::string &type() const override { static const std::string s("mdn"); return s; }
    void loadSequences(const Fraction &fraction) override {
        PostOutputLayer::loadSequences(fraction);
        check(cnt_mdn_load_sequences(m_handle, m_stream, m_patTypes.data(), m_curMaxSeqLength), "mdn loadSequences");
    }
    void computeForwardPass(int) override {
        check(cnt_mdn_forward(m_handle, m_stream, m_preceding->outputs().data()), "mdn forward");
    }
    float calculateError() override {
        check(cnt_mdn_calculate_error(m_handle, m_stream, m_outputs.data(), m_error.data()), "mdn calculateError");
        hip_check(hipStreamSynchronize(m_stream), "hipStreamSynchronize");
        return m_error.to_host()[0];
    }
    void computeBackwardPass(int) override {
        check(cnt_mdn_backward(m_handle, m_stream, m_outputs.data(), m_preceding->outputErrors().data()), "mdn backward");
    }

private:
    cnt_mdn *m_handle;
};

// DFTPostoutputLayer<TDevice> (layers/DFTErrorPostoutputLayer.cu:752-845 options, :1782-1885), "dft": size 1, one
// waveform per fraction; the forward pass computes the spectral distances and keeps their gradient, the backward
// pass hands the gradient to the preceding layer.
class DFTPostoutputLayer : public PostOutputLayer {
public:
    struct Resolution { int fftLength, frameLength, frameShift; };
    DFTPostoutputLayer(Layer *preceding, const std::vector<Resolution> &resolutions, float gamma, int specDisType = 0,
                       float zeta = 0.0f)
        : PostOutputLayer("postoutput", 1, preceding), m_handle(nullptr), m_nres((int)resolutions.size()),
          m_phase(zeta > 0.0f) {
        if (preceding->size() != 1 || m_parallel != 1)
            throw std::runtime_error("dft: the layer takes one waveform per fraction (size 1, parallel_sequences = 1)");
        if (resolutions.empty() || resolutions.size() > 3) throw std::runtime_error("dft: one to three resolutions");
        cnt_dft_desc d = {};
        d.n_res = m_nres;
        for (int r = 0; r < m_nres; ++r) {
            d.fft_length[r] = resolutions[(size_t)r].fftLength;
            d.frame_length[r] = resolutions[(size_t)r].frameLength;
            d.frame_shift[r] = resolutions[(size_t)r].frameShift;
        }
        d.gamma = gamma; d.log_floor = 1e-5f; d.spec_dis_type = specDisType;
        d.max_length = m_maxSeqLength; d.max_waves = 1; d.zeta = zeta;
        check(cnt_dft_create(&d, &m_handle), "dft create");
    }
    ~DFTPostoutputLayer() override { cnt_dft_destroy(m_handle); }
    const std::string &type() const override { static const std::string s("dft"); return s; }
    void computeForwardPass(int) override {
        const int length = m_curMaxSeqLength;
        check(cnt_dft_forward(m_handle, m_stream, 1, &length, m_preceding->outputs().data(), m_outputs.data(),
                              m_error.data()), "dft forward");
    }
    float calculateError() override {
        hip_check(hipStreamSynchronize(m_stream), "hipStreamSynchronize");
        const std::vector<float> e = m_error.to_host();
        float sum = 0.0f;
        for (int r = 0; r < m_nres * (m_phase ? 2 : 1); ++r) sum += e[(size_t)r];
        return sum;
    }
    void computeBackwardPass(int) override {
        check(cnt_dft_backward(m_handle, m_stream, m_preceding->outputErrors().data()), "dft backward");
    }

private:
    cnt_dft *m_handle;
    int m_nres;
    bool m_phase;
};

// NeuralNetwork's layer-by-layer passes (NeuralNetwork.cpp:1419-1471, 2743-2800) for a plain stack.
class LayerStack {
public:
    void add(std::unique_ptr<Layer> layer) { m_layers.push_back(std::move(layer)); }
    Layer &layer(size_t i) { return *m_layers[i]; }
    size_t size() const { return m_layers.size(); }
    void loadSequences(const Fraction &fraction) {
        for (auto &l : m_layers) l->loadSequences(fraction);
    }
    void computeForwardPass() {
        for (auto &l : m_layers) l->computeForwardPass(0);
    }
    void computeBackwardPass() {
        for (size_t i = m_layers.size(); i-- > 0;) m_layers[i]->computeBackwardPass(0);
    }

private:
    std::vector<std::unique_ptr<Layer>> m_layers;
};

}  // namespace currennt_amd
