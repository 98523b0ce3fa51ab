// Weight update of the training loop, as streaming kernels.
//
// Reference behaviour: optimizers/Optimizer.cu:186-198 (copy / accumulation of a layer's weight updates
// per fraction), optimizers/SteepestDescentOptimizer.cu:119-203 (AdaGrad / Adam / averaging functors),
// :312-405 (which of them runs for which optimizer option), :41-98 and :408-436 (the momentum update, with
// and without weight mask), MacroDefine.hpp:32-42 (option numbers, constants).
//
// The reference runs up to three passes over every weight vector (copy, adjust, update).  cnt_opt_step does
// the same arithmetic in one pass: per weight it reads the layer's gradient, the optimizer state and the
// weight and writes them back once (Adam: 20 B read + 20 B written).  The three separate entry points exist
// for callers that keep the reference's call structure.  The Adam moment updates use the reference's double
// constants (0.9, 0.999, 1e-8 are double literals there), so they are evaluated in double and rounded once.
// This file is compiled with -ffp-contract=off: every product and sum is rounded on its own, as in the
// reference, which makes the results bit-identical to a sequential host evaluation.
#include "common.hpp"

namespace cnt {
namespace {

constexpr double kBeta1 = 0.9, kBeta2 = 0.999, kEps = 0.00000001;

struct OptArgs {
    size_t n;
    const float *layer_updates;  // gradient of this fraction (step / accumulate)
    float *cur;                  // the optimizer's current weight updates
    float *stats;                // AdaGrad: n floats, Adam: n (m, v) pairs
    float *deltas;               // momentum state
    float *weights;
    const float *mask;           // optional weight mask
    int option;                  // 0 plain, 1 AdaGrad, 2 averaged, 3 stochastic AdaGrad, 5 Adam
    int add;                     // accumulate: add to cur instead of overwriting it
    float frac_length, beta1_accum, beta2_accum, learning_rate, momentum;
    const int *veto;             // optional device flag: non-zero means the gradients are invalid, nothing is touched
    const float *accum_dev;      // optional: Adam's two bias-correction products in device memory (replace the two floats)
};

__device__ __forceinline__ bool bad(float g) { return isnan(g) || isinf(g); }

__device__ __forceinline__ float adjust_one(const OptArgs &a, size_t i, float g) {
    if (a.option == 2) return g / a.frac_length;
    if (a.option != 1 && a.option != 3 && a.option != 5) return g;
    if (bad(g)) g = 0.0f;
    if (a.mask && a.mask[i] < 1.0f) return g;
    const float ave = g / a.frac_length;
    if (a.option == 5) {
        const float m = (float)(a.stats[2 * i] * kBeta1 + ave * (1 - kBeta1));
        const float v = (float)(a.stats[2 * i + 1] * kBeta2 + (double)(ave * ave) * (1 - kBeta2));
        a.stats[2 * i] = m;
        a.stats[2 * i + 1] = v;
        const float b1 = a.accum_dev ? a.accum_dev[0] : a.beta1_accum, b2 = a.accum_dev ? a.accum_dev[1] : a.beta2_accum;
        const float mh = m / (1 - b1);
        const float vh = v / (1 - b2);
        return (float)(mh / (sqrtf(vh) + kEps));
    }
    const float acc = a.stats[i] + (ave * ave);
    a.stats[i] = acc;
    return a.option == 1 ? ave / sqrtf(acc) : g;
}

__device__ __forceinline__ float update_one(const OptArgs &a, size_t i, float g) {
    if (bad(g)) g = 0.0f;
    const float delta = a.momentum * a.deltas[i] - a.learning_rate * g;
    a.deltas[i] = delta;
    const float w = a.weights[i] + delta;
    a.weights[i] = a.mask ? w * a.mask[i] : w;
    return g;
}

// MODE 0 accumulate, 1 adjust, 2 update, 3 all three in one pass
template <int MODE>
__global__ __launch_bounds__(256) void optimizer_kernel(const OptArgs a) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    if (a.veto && *a.veto != 0) return;
    for (; i < a.n; i += stride) {
        float g;
        if (MODE == 0 || MODE == 3) g = a.add ? a.layer_updates[i] + a.cur[i] : a.layer_updates[i];
        else g = a.cur[i];
        if (MODE == 1 || MODE == 3) g = adjust_one(a, i, g);
        if (MODE == 2 || MODE == 3) g = update_one(a, i, g);
        a.cur[i] = g;
    }
}

// Adam's bias-correction products beta1^t, beta2^t kept in device memory, advanced in stream order in front of a step
// and under the same veto flag as the step: a step that the flag skips leaves them where they stood.
__global__ void adam_advance_kernel(float *accum, const int *veto) {
    if (veto && *veto != 0) return;
    accum[0] = (float)(accum[0] * kBeta1);
    accum[1] = (float)(accum[1] * kBeta2);
}

int blocks_for(size_t n) {
    size_t b = (n + 255) / 256;
    if (b > 8192) b = 8192;
    return (int)(b < 1 ? 1 : b);
}

bool known_option(int o) { return o == 0 || o == 1 || o == 2 || o == 3 || o == 4 || o == 5; }

}  // namespace
}  // namespace cnt

extern "C" {

int cnt_opt_accumulate(void *stream, long n, const float *layer_updates, float *cur_updates, int add) {
    using namespace cnt;
    CNT_REQUIRE(n >= 0 && (n == 0 || (layer_updates && cur_updates)), "opt_accumulate: bad argument");
    if (n == 0) return CNT_OK;
    OptArgs a = {};
    a.n = (size_t)n; a.layer_updates = layer_updates; a.cur = cur_updates; a.add = add;
    ProfileScope prof(static_cast<hipStream_t>(stream), "opt_accumulate");
    hipLaunchKernelGGL(optimizer_kernel<0>, dim3(blocks_for(a.n)), dim3(256), 0, static_cast<hipStream_t>(stream), a);
    CNT_HIP(hipGetLastError());
    return CNT_OK;
}

int cnt_opt_adjust_gradient(void *stream, int option, long n, float *cur_updates, float *stats, const float *mask,
                            float frac_length, float beta1_accum, float beta2_accum) {
    using namespace cnt;
    CNT_REQUIRE(n >= 0 && (n == 0 || cur_updates), "opt_adjust_gradient: bad argument");
    CNT_REQUIRE(known_option(option), "opt_adjust_gradient: unknown optimizer option %d", option);
    CNT_REQUIRE(!(option == 1 || option == 3 || option == 5) || stats, "opt_adjust_gradient: option %d needs a statistics buffer",
                option);
    if (n == 0 || option == 0 || option == 4) return CNT_OK;
    OptArgs a = {};
    a.n = (size_t)n; a.cur = cur_updates; a.stats = stats; a.mask = mask; a.option = option;
    a.frac_length = frac_length; a.beta1_accum = beta1_accum; a.beta2_accum = beta2_accum;
    ProfileScope prof(static_cast<hipStream_t>(stream), "opt_adjust_gradient");
    hipLaunchKernelGGL(optimizer_kernel<1>, dim3(blocks_for(a.n)), dim3(256), 0, static_cast<hipStream_t>(stream), a);
    CNT_HIP(hipGetLastError());
    return CNT_OK;
}

int cnt_opt_update_weights(void *stream, long n, float *weights, float *cur_updates, float *weight_deltas,
                           const float *mask, float learning_rate, float momentum) {
    using namespace cnt;
    CNT_REQUIRE(n >= 0 && (n == 0 || (weights && cur_updates && weight_deltas)), "opt_update_weights: bad argument");
    // the reference skips the update altogether for a negative learning rate (SteepestDescentOptimizer.cu:283-285)
    if (n == 0 || learning_rate < 0) return CNT_OK;
    OptArgs a = {};
    a.n = (size_t)n; a.cur = cur_updates; a.deltas = weight_deltas; a.weights = weights; a.mask = mask;
    a.learning_rate = learning_rate; a.momentum = momentum;
    ProfileScope prof(static_cast<hipStream_t>(stream), "opt_update_weights");
    hipLaunchKernelGGL(optimizer_kernel<2>, dim3(blocks_for(a.n)), dim3(256), 0, static_cast<hipStream_t>(stream), a);
    CNT_HIP(hipGetLastError());
    return CNT_OK;
}

int cnt_opt_step(void *stream, int option, long n, float *weights, const float *layer_updates, float *cur_updates,
                 float *stats, float *weight_deltas, const float *mask, float frac_length, float beta1_accum,
                 float beta2_accum, float learning_rate, float momentum) {
    return cnt::opt_step_guarded(static_cast<hipStream_t>(stream), option, n, weights, layer_updates, cur_updates, stats,
                                 weight_deltas, mask, frac_length, beta1_accum, beta2_accum, learning_rate, momentum, nullptr,
                                 nullptr);
}

extern "C++" int cnt::opt_adam_advance(hipStream_t stream, float *accum_dev, const int *veto) {
    hipLaunchKernelGGL(adam_advance_kernel, dim3(1), dim3(1), 0, stream, accum_dev, veto);
    CNT_HIP(hipGetLastError());
    return CNT_OK;
}

extern "C++" int cnt::opt_step_guarded(hipStream_t stream, int option, long n, float *weights, const float *layer_updates,
                                       float *cur_updates, float *stats, float *weight_deltas, const float *mask,
                                       float frac_length, float beta1_accum, float beta2_accum, float learning_rate,
                                       float momentum, const int *veto, const float *accum_dev) {
    using namespace cnt;
    CNT_REQUIRE(n >= 0 && (n == 0 || (weights && layer_updates && cur_updates && weight_deltas)), "opt_step: bad argument");
    CNT_REQUIRE(known_option(option), "opt_step: unknown optimizer option %d", option);
    CNT_REQUIRE(!(option == 1 || option == 3 || option == 5) || stats, "opt_step: option %d needs a statistics buffer", option);
    CNT_REQUIRE(learning_rate >= 0, "opt_step: negative learning rate (the reference skips the update; call cnt_opt_accumulate)");
    if (n == 0) return CNT_OK;
    OptArgs a = {};
    a.n = (size_t)n; a.layer_updates = layer_updates; a.cur = cur_updates; a.stats = stats; a.deltas = weight_deltas;
    a.weights = weights; a.mask = mask; a.option = option == 4 ? 0 : option;
    a.frac_length = frac_length; a.beta1_accum = beta1_accum; a.beta2_accum = beta2_accum;
    a.learning_rate = learning_rate; a.momentum = momentum;
    a.veto = veto;
    a.accum_dev = accum_dev;
    ProfileScope prof(stream, "opt_step");
    hipLaunchKernelGGL(optimizer_kernel<3>, dim3(blocks_for(a.n)), dim3(256), 0, stream, a);
    CNT_HIP(hipGetLastError());
    return CNT_OK;
}

float cnt_opt_next_beta_accum(float accum, int which) { return (float)(accum * (which == 1 ? cnt::kBeta1 : cnt::kBeta2)); }

}  // extern "C"
