// CPU oracle for the CURRENNT backward hot path -- TEST INFRASTRUCTURE ONLY.
//
// This directory restates, in plain sequential C++, the arithmetic of the
// reference's host ("Cpu", Thrust sequential backend) code path.  It exists to
// check the HIP library and to time a CPU baseline.  Nothing in the product
// library links, loads or calls it.
//
// Scalar semantics restated here (paths below /root/reference/CURRENNT_codes/currennt_lib/src):
//   activation_functions/Logistic.cuh:33-48   clamped logistic, derivative from the output
//   activation_functions/Maxmin1.cuh:33-36    2*logistic(x)-1
//   activation_functions/Tanh.cuh:33-41       tanh(x) := maxmin1(2x), derivative 1-y^2
//   helpers/boundRange.cuh, limitedError.cuh  clip to [-1, 1]
//   helpers/NumericLimits.cuh:34-49           float limits used by the safe exp/log family
//   helpers/safeExp.cuh:31-87                 safeExp / logAdd / safeLog
//   helpers/Matrix.cu:41-183, 353-377         column-major products, sequential k-order sums
#ifndef CURRENNT_ORACLE_COMMON_H
#define CURRENNT_ORACLE_COMMON_H

#include <cmath>
#include <cstddef>
#include <cstdint>

namespace orc {

// pattern types, Types.hpp:35-38
enum { PAT_NONE = 0, PAT_FIRST = 1, PAT_NORMAL = 2, PAT_LAST = 3 };

struct Lim {
    static constexpr float kMin      = 1.1754944e-038f;
    static constexpr float kMax      = 3.4028235e+038f;
    static constexpr float kExpLimit = 88.722839f;
    static constexpr float kLogZero  = -1e30f;
    static constexpr float kLSmall   = -0.5e10f;
    static constexpr float kMinLarg  = 1.1754944e-038f;
    static constexpr float kMinLogExp = -69.0776f;
};

static inline float logistic(float x) {
    if (x < Lim::kExpLimit) {
        if (x > -Lim::kExpLimit) return 1.0f / (1.0f + std::exp(-x));
        return 0.0f;
    }
    return 1.0f;
}
static inline float logistic_deriv(float y) { return y * (1.0f - y); }
static inline float maxmin1(float x) { return 2.0f * logistic(x) - 1.0f; }
static inline float tanh_act(float x) { return maxmin1(2.0f * x); }
static inline float tanh_deriv(float y) { return 1.0f - y * y; }
static inline float relu_act(float x) { return x > 0.0f ? x : 0.0f; }
static inline float relu_deriv(float y) { return y > 0.0f ? 1.0f : 0.0f; }
static inline float clip1(float e) { return e < -1.0f ? -1.0f : (e > 1.0f ? 1.0f : e); }

static inline float safe_exp(float x) {
    if (x <= Lim::kLogZero) return 0.0f;
    if (x >= Lim::kExpLimit) return Lim::kMax;
    return std::exp(x);
}
static inline float safe_log(float x) {
    if (x < Lim::kMinLarg) return Lim::kLogZero;
    return std::log(x);
}
// The reference mixes a double literal into the sum, so the inner part is
// evaluated in double and rounded once on return.
static inline float log_add(float x, float y) {
    float hi = (x > y) ? x : y;
    float lo = (x > y) ? y : x;
    if ((lo - hi) < Lim::kMinLogExp) return (hi < Lim::kLSmall) ? Lim::kLogZero : hi;
    return (float)((double)hi + std::log(1.0 + (double)std::exp(lo - hi)));
}

// Worker threads the oracle may use (orc_set_threads; 1 unless a caller asks for more).  Threads only ever
// share out whole output elements: every output is still one sequential, k-ordered sum formed by one thread,
// so results do not depend on the thread count.
int threads();

// Column-major products with the reference's summation order: every output is a
// k-ordered dot product formed from zero, then (optionally) added to the old value.
//   C (m x n, ldc=m);  tA=false: A is m x k (lda=m)  tA=true: A is k x m (lda=k)
//                      tB=false: B is k x n (ldb=k)  tB=true: B is n x k (ldb=n)
static inline void mat_product(float *C, int m, int n, int k, const float *A, bool tA, const float *B,
                               bool tB, bool accumulate) {
    const int nthr = ((long long)m * n * k >= 200000) ? threads() : 1;
#pragma omp parallel for collapse(2) schedule(static) num_threads(nthr) if (nthr > 1)
    for (int j = 0; j < n; ++j) {
        for (int i = 0; i < m; ++i) {
            float x = 0.0f;
            if (!tA && !tB) {
                for (int q = 0; q < k; ++q) x += A[i + (size_t)q * m] * B[q + (size_t)j * k];
            } else if (tA && !tB) {
                for (int q = 0; q < k; ++q) x += A[q + (size_t)i * k] * B[q + (size_t)j * k];
            } else {  // !tA && tB
                for (int q = 0; q < k; ++q) x += A[i + (size_t)q * m] * B[j + (size_t)q * n];
            }
            float *c = &C[i + (size_t)j * m];
            *c = accumulate ? (*c + x) : x;
        }
    }
}

}  // namespace orc

#endif
