// Drives a plain layer stack (feed-forward / LSTM / BLSTM layers + SSE) through the C++ layer shells:
// loadSequences -> computeForwardPass -> calculateError -> computeBackwardPass for one fraction read from a
// job file, results written to a result file.  Used by the test-suite to exercise the C++ host side
// end to end; the reference's counterpart is one iteration of Optimizer::_processDataSet
// (optimizers/Optimizer.cu:85-197) without the weight update.
//
// Job file (little endian): int32 inputSize, nLayers, S, T, Tmin; per layer int32 kind (0..3 feed-forward
// identity/tanh/logistic/relu, 10 lstm, 11 blstm), int32 size, float bias, int64 nW, float W[nW];
// char patTypes[T*S]; float inputs[inputSize*T*S]; float targets[lastSize*T*S].
// Result file: float loss; per layer: int64 n, float outputs[n], int64 nW, float weightUpdates[nW].
#include <cstdint>
#include <cstdio>
#include <fstream>
#include <iostream>

#include "layers.hpp"

using namespace currennt_amd;

template <typename T>
static T rd(std::ifstream &f) {
    T v;
    f.read(reinterpret_cast<char *>(&v), sizeof(T));
    if (!f) throw std::runtime_error("job file truncated");
    return v;
}
template <typename T>
static std::vector<T> rdv(std::ifstream &f, size_t n) {
    std::vector<T> v(n);
    f.read(reinterpret_cast<char *>(v.data()), (std::streamsize)(n * sizeof(T)));
    if (!f) throw std::runtime_error("job file truncated");
    return v;
}

int main(int argc, char **argv) {
    if (argc != 3) {
        std::fprintf(stderr, "usage: run_stack <job> <result>\n");
        return 2;
    }
    try {
        std::ifstream f(argv[1], std::ios::binary);
        if (!f) throw std::runtime_error("cannot open job file");
        const int inputSize = rd<int32_t>(f), nLayers = rd<int32_t>(f), S = rd<int32_t>(f), T = rd<int32_t>(f),
                  Tmin = rd<int32_t>(f);
        hipStream_t stream = nullptr;
        hip_check(hipStreamCreate(&stream), "hipStreamCreate");
        LayerStack net;
        net.add(std::unique_ptr<Layer>(new InputLayer(inputSize, S, T, stream)));
        std::vector<TrainableLayer *> trainable;
        std::vector<LstmLayer *> lstms;
        for (int i = 0; i < nLayers; ++i) {
            const int kind = rd<int32_t>(f), size = rd<int32_t>(f);
            const float bias = rd<float>(f);
            const int64_t nW = rd<int64_t>(f);
            std::vector<float> W = rdv<float>(f, (size_t)nW);
            Layer *prev = &net.layer(net.size() - 1);
            TrainableLayer *l = nullptr;
            const std::string name = "layer" + std::to_string(i);
            if (kind >= 0 && kind <= 3) {
                l = new FeedForwardLayer(name, kind, size, prev, bias);
            } else if (kind == 10 || kind == 11) {
                LstmLayer *ls = new LstmLayer(name, size, kind == 11, prev, bias);
                lstms.push_back(ls);
                l = ls;
            } else {
                throw std::runtime_error("unknown layer kind");
            }
            if ((int64_t)l->weights().size() != nW) throw std::runtime_error("weight count mismatch in " + name);
            l->weights().assign(W);
            trainable.push_back(l);
            net.add(std::unique_ptr<Layer>(l));
        }
        SsePostOutputLayer *post = new SsePostOutputLayer(&net.layer(net.size() - 1));
        net.add(std::unique_ptr<Layer>(post));

        Fraction fr;
        fr.maxSeqLength = T;
        fr.minSeqLength = Tmin;
        fr.patTypes = rdv<char>(f, (size_t)T * S);
        fr.inputs = rdv<float>(f, (size_t)inputSize * T * S);
        fr.targets = rdv<float>(f, (size_t)post->size() * T * S);

        net.loadSequences(fr);
        net.computeForwardPass();
        const float loss = post->calculateError();
        net.computeBackwardPass();
        for (LstmLayer *l : lstms) l->synchronizeAndCheck();
        hip_check(hipStreamSynchronize(stream), "hipStreamSynchronize");

        std::ofstream o(argv[2], std::ios::binary);
        o.write(reinterpret_cast<const char *>(&loss), sizeof(float));
        for (TrainableLayer *l : trainable) {
            std::vector<float> out = l->outputs().to_host(), up = l->weightUpdates().to_host();
            const int64_t n = (int64_t)out.size(), nw = (int64_t)up.size();
            o.write(reinterpret_cast<const char *>(&n), sizeof(n));
            o.write(reinterpret_cast<const char *>(out.data()), (std::streamsize)(out.size() * sizeof(float)));
            o.write(reinterpret_cast<const char *>(&nw), sizeof(nw));
            o.write(reinterpret_cast<const char *>(up.data()), (std::streamsize)(up.size() * sizeof(float)));
        }
        std::printf("run_stack ok: loss %.6f\n", loss);
        return 0;
    } catch (const std::exception &e) {
        // same wording as the reference's top-level handler (currennt/src/main.cpp:692-695)
        std::fprintf(stderr, "FAILED in running CURENNT: %s\n", e.what());
        return 2;
    }
}
