// CPU oracle, weight update of the training loop -- TEST INFRASTRUCTURE ONLY (see oracle_common.h).
//
// Restates /root/reference/CURRENNT_codes/currennt_lib/src:
//   optimizers/Optimizer.cu:186-198                 per-fraction copy / accumulation of a layer's weight updates
//   optimizers/SteepestDescentOptimizer.cu:119-190  AdaGradAccumulate, AdaGradAccumulateUpdate, AdamAccumulateUpdate
//   optimizers/SteepestDescentOptimizer.cu:192-203  divideOpe (gradient averaged over the fraction)
//   optimizers/SteepestDescentOptimizer.cu:312-405  which adjustment runs for which optimizer option
//   optimizers/SteepestDescentOptimizer.cu:41-98, 408-436   UpdateWeightFn (with and without weight mask)
//   MacroDefine.hpp:32-42                           option numbers and the Adam / AdaGrad constants
// The constants are double literals in the reference, so the Adam moment updates and the final quotient are
// evaluated in double and rounded to float once; the restatement keeps that.
#include "currennt_oracle.h"

#include <cmath>

namespace {
const double kBeta1 = 0.9, kBeta2 = 0.999, kEps = 0.00000001;
inline bool bad(float g) { return std::isnan(g) || std::isinf(g); }
}  // namespace

extern "C" {

void orc_opt_accumulate(long n, const float *layer_updates, float *cur_updates, int add) {
    for (long i = 0; i < n; ++i) cur_updates[i] = add ? layer_updates[i] + cur_updates[i] : layer_updates[i];
}

// option: 1 AdaGrad, 2 averaged gradient, 3 stochastic AdaGrad (accumulate only), 5 Adam; anything else: nothing.
// stats: one float per weight (AdaGrad) or interleaved (m, v) pairs (Adam).  mask may be NULL.
void orc_opt_adjust_gradient(int option, long n, float *g, float *stats, const float *mask, float frac_length,
                             float beta1_accum, float beta2_accum) {
    for (long i = 0; i < n; ++i) {
        if (option == 2) {
            g[i] = g[i] / frac_length;
            continue;
        }
        if (option != 1 && option != 3 && option != 5) continue;
        if (bad(g[i])) g[i] = 0.0f;
        if (mask && mask[i] < 1.0) continue;
        const float ave = g[i] / frac_length;
        if (option == 1 || option == 3) {
            stats[i] = stats[i] + (ave * ave);
            if (option == 1) g[i] = ave / std::sqrt(stats[i]);
        } else {
            stats[2 * i] = (float)(stats[2 * i] * kBeta1 + ave * (1 - kBeta1));
            stats[2 * i + 1] = (float)(stats[2 * i + 1] * kBeta2 + ave * ave * (1 - kBeta2));
            const float m = stats[2 * i] / (1 - beta1_accum);
            const float v = stats[2 * i + 1] / (1 - beta2_accum);
            g[i] = (float)(m / (std::sqrt(v) + kEps));
        }
    }
}

void orc_opt_update_weights(long n, float *weights, float *g, float *deltas, const float *mask, float learning_rate,
                            float momentum) {
    for (long i = 0; i < n; ++i) {
        if (bad(g[i])) g[i] = 0.0f;
        const float delta = momentum * deltas[i] - learning_rate * g[i];
        deltas[i] = delta;
        weights[i] = mask ? ((weights[i] + delta) * mask[i]) : (weights[i] + delta);
    }
}

// m_adamBeta?Accum *= OP_ADAMBETA? (float times double literal, stored as float), once per update call
float orc_opt_next_beta_accum(float accum, int which) { return (float)(accum * (which == 1 ? kBeta1 : kBeta2)); }

}  // extern "C"
