// Drives a network of C++ layer shells (host/layers.hpp) for one fraction: loadSequences -> computeForwardPass ->
// calculateError -> computeBackwardPass, the order of one iteration of Optimizer::_processDataSet
// (optimizers/Optimizer.cu:85-197) without the weight update.  Unlike run_stack it covers every layer type of the
// path: feed-forward, LSTM / BLSTM, cnn, wavnetc, gatedact, skipini / skipadd, and the sse / mdn / dft post-output
// layers.  The test-suite uses it to exercise the C++ host side end to end.
//
// usage: run_graph <directory>.  The directory holds `job.txt` and raw little-endian float32 files:
//   job.txt   one statement per line, tokens separated by blanks; every layer follows the one before it, as in the
//             reference's network file:
//               geometry <S> <T> <Tmin>
//               input <size>
//               ff <name> <act 0..3> <size> <bias>
//               lstm <name> <size> <bidirectional 0|1> <bias>
//               cnn <name> <size> <bias> <causal> <tanhoutput> <half width> <tap interval>
//               wavnetc <name> <size> <contextDim>
//               gatedact <name> <size>
//               skipini <name> <size>
//               skipadd <name> <size> <source>[,<source>...]        (names of earlier layers)
//               post sse | post mdn <targetDim> <n> <config...> | post dft <gamma> <specDisType> <zeta> <nres> <N Nw Hs>...
//   pat.bin (char), input.bin, targets.bin, context.bin (only with wavnetc layers), <name>.W.bin per trainable layer.
// It writes loss.txt and, per trainable layer, <name>.dW.bin; per layer <name>.out.bin and <name>.err.bin.
#include <cstdio>
#include <fstream>
#include <iostream>
#include <map>
#include <sstream>

#include "layers.hpp"

using namespace currennt_amd;

template <typename T>
static std::vector<T> read_file(const std::string &path, size_t expect) {
    std::ifstream f(path, std::ios::binary);
    if (!f) throw std::runtime_error("cannot open " + path);
    f.seekg(0, std::ios::end);
    const size_t n = (size_t)f.tellg() / sizeof(T);
    f.seekg(0);
    if (expect && n != expect) throw std::runtime_error(path + ": expected " + std::to_string(expect) + " values, found " + std::to_string(n));
    std::vector<T> v(n);
    f.read(reinterpret_cast<char *>(v.data()), (std::streamsize)(n * sizeof(T)));
    return v;
}
static void write_file(const std::string &path, const std::vector<float> &v, size_t n) {
    std::ofstream o(path, std::ios::binary);
    o.write(reinterpret_cast<const char *>(v.data()), (std::streamsize)(std::min(n, v.size()) * sizeof(float)));
}

int main(int argc, char **argv) {
    if (argc != 2) {
        std::fprintf(stderr, "usage: run_graph <directory>\n");
        return 2;
    }
    try {
        const std::string dir = std::string(argv[1]) + "/";
        std::ifstream job(dir + "job.txt");
        if (!job) throw std::runtime_error("cannot open job.txt");
        hipStream_t stream = nullptr;
        hip_check(hipStreamCreate(&stream), "hipStreamCreate");
        int S = 0, T = 0, Tmin = 0;
        LayerStack net;
        std::map<std::string, Layer *> by_name;
        std::vector<TrainableLayer *> trainable;
        std::vector<LstmLayer *> lstms;
        WavNetCore *first_core = nullptr;
        PostOutputLayer *post = nullptr;
        int context_dim = 0;
        std::string line;
        while (std::getline(job, line)) {
            std::istringstream in(line);
            std::string kind, name;
            if (!(in >> kind) || kind[0] == '#') continue;
            Layer *prev = net.size() ? &net.layer(net.size() - 1) : nullptr;
            Layer *made = nullptr;
            if (kind == "geometry") {
                in >> S >> T >> Tmin;
                continue;
            }
            if (S <= 0 || T <= 0) throw std::runtime_error("job.txt: geometry comes first");
            if (kind == "input") {
                int size;
                in >> size;
                name = "input";
                made = new InputLayer(size, S, T, stream);
            } else if (!prev) {
                throw std::runtime_error("job.txt: the input layer comes first");
            } else if (kind == "ff") {
                int act, size; float bias;
                in >> name >> act >> size >> bias;
                made = new FeedForwardLayer(name, act, size, prev, bias);
            } else if (kind == "lstm") {
                int size, bidir; float bias;
                in >> name >> size >> bidir >> bias;
                LstmLayer *l = new LstmLayer(name, size, bidir != 0, prev, bias);
                lstms.push_back(l);
                made = l;
            } else if (kind == "cnn") {
                int size, causal, tanhout, hw, dil; float bias;
                in >> name >> size >> bias >> causal >> tanhout >> hw >> dil;
                made = new CNNLayer(name, size, prev, std::vector<int>((size_t)size, hw), std::vector<int>((size_t)size, dil),
                                    causal != 0, tanhout != 0, bias);
            } else if (kind == "wavnetc") {
                int size, cdim;
                in >> name >> size >> cdim;
                WavNetCore *l = new WavNetCore(name, size, prev, cdim, first_core);
                if (!first_core) first_core = l;
                context_dim = cdim;
                made = l;
            } else if (kind == "gatedact") {
                int size;
                in >> name >> size;
                made = new GatedActLayer(name, size, prev);
            } else if (kind == "skipini") {
                int size;
                in >> name >> size;
                made = new SkipAddLayer(name, "skipini", size, std::vector<Layer *>(1, prev));
            } else if (kind == "skipadd") {
                int size; std::string sources;
                in >> name >> size >> sources;
                std::vector<Layer *> pre;
                std::istringstream ss(sources);
                std::string one;
                while (std::getline(ss, one, ',')) {
                    if (!by_name.count(one)) throw std::runtime_error("skipadd " + name + ": unknown source " + one);
                    pre.push_back(by_name[one]);
                }
                made = new SkipAddLayer(name, "skipadd", size, pre);
            } else if (kind == "post") {
                std::string what;
                in >> what;
                name = "postoutput";
                if (what == "sse") {
                    post = new SsePostOutputLayer(prev);
                } else if (what == "mdn") {
                    int target_dim, n;
                    in >> target_dim >> n;
                    std::vector<float> cfg((size_t)n);
                    for (float &v : cfg) in >> v;
                    post = new MDNLayer(target_dim, prev, cfg);
                } else if (what == "dft") {
                    float gamma, zeta; int dis, nres;
                    in >> gamma >> dis >> zeta >> nres;
                    std::vector<DFTPostoutputLayer::Resolution> res((size_t)nres);
                    for (auto &r : res) in >> r.fftLength >> r.frameLength >> r.frameShift;
                    post = new DFTPostoutputLayer(prev, res, gamma, dis, zeta);
                } else {
                    throw std::runtime_error("job.txt: unknown post-output layer " + what);
                }
                made = post;
            } else {
                throw std::runtime_error("job.txt: unknown statement " + kind);
            }
            if (!in) throw std::runtime_error("job.txt: malformed line: " + line);
            if (TrainableLayer *t = dynamic_cast<TrainableLayer *>(made)) {
                t->weights().assign(read_file<float>(dir + name + ".W.bin", t->weights().size()));
                trainable.push_back(t);
            }
            by_name[name] = made;
            net.add(std::unique_ptr<Layer>(made));
        }
        if (!post) throw std::runtime_error("job.txt: no post-output layer");

        Fraction fr;
        fr.maxSeqLength = T;
        fr.minSeqLength = Tmin;
        fr.patTypes = read_file<char>(dir + "pat.bin", (size_t)T * S);
        fr.inputs = read_file<float>(dir + "input.bin", (size_t)net.layer(0).size() * T * S);
        fr.targets = read_file<float>(dir + "targets.bin", (size_t)post->size() * T * S);
        net.loadSequences(fr);
        if (first_core) first_core->loadContext(read_file<float>(dir + "context.bin", (size_t)context_dim * T * S));
        // Everything is allocated at construction: the library's only allocation on the path of a pass is a stream's
        // scratch buffer for split products, and the number of those it holds is the same before and after the passes.
        // (The device's free memory still drops over a first pass: the runtime loads each code object of the library at
        // the first launch of one of its kernels.)
        hip_check(hipDeviceSynchronize(), "hipDeviceSynchronize");
        size_t free_before = 0, free_after = 0, total = 0;
        hip_check(hipMemGetInfo(&free_before, &total), "hipMemGetInfo");
        const int scratch_before = cnt_gemm_scratch_buffers();
        net.computeForwardPass();
        const float loss = post->calculateError();
        net.computeBackwardPass();
        for (LstmLayer *l : lstms) l->synchronizeAndCheck();
        hip_check(hipStreamSynchronize(stream), "hipStreamSynchronize");
        hip_check(hipMemGetInfo(&free_after, &total), "hipMemGetInfo");

        {
            std::ofstream o(dir + "loss.txt");
            o.precision(9);
            o << loss << "\n";
        }
        for (size_t i = 1; i < net.size(); ++i) {
            Layer &l = net.layer(i);
            const size_t n = (size_t)l.size() * T * S;
            write_file(dir + l.name() + ".out.bin", l.outputs().to_host(), n);
            write_file(dir + l.name() + ".err.bin", l.outputErrors().to_host(), n);
        }
        for (TrainableLayer *t : trainable) write_file(dir + t->name() + ".dW.bin", t->weightUpdates().to_host(), t->weightUpdates().size());
        std::printf("run_graph ok: %zu layers, loss %.6f, scratch buffers allocated during the passes: %d, device memory taken "
                    "(code objects included): %lld bytes\n", net.size(), loss, cnt_gemm_scratch_buffers() - scratch_before,
                    (long long)free_before - (long long)free_after);
        return 0;
    } catch (const std::exception &e) {
        // same wording as the reference's top-level handler (currennt/src/main.cpp:692-695)
        std::fprintf(stderr, "FAILED in running CURENNT: %s\n", e.what());
        return 2;
    }
}
