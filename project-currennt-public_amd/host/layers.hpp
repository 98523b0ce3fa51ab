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
          m_weightUpdates(weightCount) {}
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

// PostOutputLayer: targets live in the layer's own outputs(), errors go to the preceding layer
// (layers/PostOutputLayer.cu:108-124).
class SsePostOutputLayer : public Layer {
public:
    explicit SsePostOutputLayer(Layer *preceding)
        : Layer("postoutput", preceding->size(), preceding->parallelSequences(), preceding->maxSeqLength(), preceding,
                preceding->stream()), m_error(1) {}
    const std::string &type() const override { static const std::string s("sse"); return s; }
    void loadSequences(const Fraction &fraction) override {
        Layer::loadSequences(fraction);
        m_outputs.assign(fraction.targets);
    }
    void computeForwardPass(int) override {}
    float calculateError() {
        check(cnt_sse_error(m_stream, m_size, curSlots(), m_patTypes.data(), m_preceding->outputs().data(),
                            m_outputs.data(), m_error.data()), "sse calculateError");
        hip_check(hipStreamSynchronize(m_stream), "hipStreamSynchronize");
        return m_error.to_host()[0];
    }
    void computeBackwardPass(int) override {
        check(cnt_sse_backward(m_stream, m_size, curSlots(), m_patTypes.data(), m_preceding->outputs().data(),
                               m_outputs.data(), m_preceding->outputErrors().data()), "sse backward");
    }

private:
    real_vector m_error;
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
