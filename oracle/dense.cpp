// CPU oracle, feed-forward layer and SSE post-output layer -- TEST INFRASTRUCTURE ONLY
// (see oracle_common.h).
//
// Restates /root/reference/CURRENNT_codes/currennt_lib/src/layers:
//   FeedForwardLayer.cu:52-74      output = act(W^T x + bias * b)
//   FeedForwardLayer.cu:1060-1101  forward driver
//   FeedForwardLayer.cu:105-116    delta = act'(y) * err, every slot including dummies
//   FeedForwardLayer.cu:118-138, 1516-1533  bias update = sum over patterns of bias * delta
//   FeedForwardLayer.cu:1633-1738  backward driver (ex = W delta, dW = x delta^T)
//   SsePostOutputLayer.cu:94-136, 166-267   0.5 * sum (t-y)^2 and err = y - t, zero on dummy slots
#include "currennt_oracle.h"
#include "oracle_common.h"

namespace {
inline float act_fn(int act, float a) {
    switch (act) {
        case 1: return orc::tanh_act(a);
        case 2: return orc::logistic(a);
        case 3: return orc::relu_act(a);
        default: return a;
    }
}
inline float act_deriv(int act, float y) {
    switch (act) {
        case 1: return orc::tanh_deriv(y);
        case 2: return orc::logistic_deriv(y);
        case 3: return orc::relu_deriv(y);
        default: return 1.0f;
    }
}
}  // namespace

extern "C" {

void orc_dense_forward(int P, int D, int N, int act, float bias, const float *weights, const float *x,
                       float *y) {
    orc::mat_product(y, D, N, P, weights, true, x, false, false);
    const float *b = weights + (size_t)P * D;
    for (size_t i = 0; i < (size_t)D * N; ++i) y[i] = act_fn(act, y[i] + bias * b[i % D]);
}

void orc_dense_backward(int P, int D, int N, int act, float bias, const float *weights, const float *x,
                        const float *y, float *err, float *ex, float *dW) {
    for (size_t i = 0; i < (size_t)D * N; ++i) err[i] = act_deriv(act, y[i]) * err[i];
    if (ex) orc::mat_product(ex, P, N, D, weights, false, err, false, false);
    orc::mat_product(dW, P, D, N, x, false, err, true, false);
    for (int d = 0; d < D; ++d) {
        float wu = 0.0f;
        for (int i = 0; i < N; ++i) wu += bias * err[d + (size_t)i * D];
        dW[(size_t)P * D + d] = wu;
    }
}

float orc_sse_error(int D, int N, const char *patTypes, const float *y, const float *target) {
    float acc = 0.0f;
    for (size_t i = 0; i < (size_t)D * N; ++i) {
        if (patTypes[i / D] == orc::PAT_NONE) continue;
        const float diff = target[i] - y[i];
        acc += diff * diff;
    }
    return 0.5f * acc;
}

void orc_sse_backward(int D, int N, const char *patTypes, const float *y, const float *target, float *err) {
    for (size_t i = 0; i < (size_t)D * N; ++i)
        err[i] = (patTypes[i / D] == orc::PAT_NONE) ? 0.0f : (y[i] - target[i]);
}

}  // extern "C"
