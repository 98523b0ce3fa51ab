// CPU oracle, mixture-density post-output layer -- TEST INFRASTRUCTURE ONLY (see oracle_common.h).
//
// Restates /root/reference/CURRENNT_codes/currennt_lib/src/layers/MDNUnit.cu and MDNLayer.cu:
//   offset / exp / sum / normalise (softmax and mixture weights)   MDNUnit.cu:227-296, 372-405, 437-470
//   mean copy, std = max(exp(x), floor)                            MDNUnit.cu:503-530, 333-369
//   mixture unit forward driver                                    MDNUnit.cu:5249-5420
//   mixture distance, per-mixture log-likelihood, logAdd           MDNUnit.cu:1003-1063, 2096-2169
//   mixture unit calculateError / computeBackward drivers          MDNUnit.cu:6036-6193, 6195-6416
//   mixture-weight, mean and std gradients                         MDNUnit.cu:2172-2212, 2215-2325
//   softmax unit forward / cross entropy / gradient                MDNUnit.cu:4170-4339, 683-750,
//                                                                  4685-4754, 921-1000
//   layer: zero the preceding error buffer, run the units in order MDNLayer.cu:797-827, 841-852, 875-917
// Only the flat softmax (no voiced/unvoiced split) and the untied-variance mixture unit are restated.
// The statements run in the order of the reference's sequential host backend, including the write
// of a padding frame's mixture-weight zero to index t*M+m instead of t*L+startD+m.
#include "currennt_oracle.h"
#include "oracle_common.h"

#include <cmath>

namespace {

constexpr float kSkipMarker = orc::Lim::kMax;
constexpr double kPiAsWritten = 3.141215;  // the reference's own constant

// offset, exp, sum, normalise over columns [startD, endD) of every frame; para is F x K
void softmax_rows(int F, int Lp, int startD, int endD, float temperature, const char *pat, const float *x,
                  float *para) {
    const int K = endD - startD;
    for (int f = 0; f < F; ++f) {
        float *row = para + (size_t)f * K;
        if (pat[f] == orc::PAT_NONE) {
            for (int k = 0; k < K; ++k) row[k] = kSkipMarker;
            continue;
        }
        const float *in = x + (size_t)f * Lp + startD;
        float mx = orc::Lim::kMin, mn = orc::Lim::kMax;
        for (int k = 0; k < K; ++k) {
            mn = in[k] < mn ? in[k] : mn;
            mx = in[k] > mx ? in[k] : mx;
        }
        const float offset = 0.5f * (mn + mx);
        for (int k = 0; k < K; ++k) row[k] = orc::safe_exp((in[k] - offset) / temperature);
        float sum = 0.0f;
        for (int k = 0; k < K; ++k) sum += row[k];
        if (sum == kSkipMarker) continue;
        for (int k = 0; k < K; ++k) row[k] = row[k] / sum;
    }
}

}  // namespace

extern "C" {

void orc_mdn_mixture_forward(int F, int Lp, int startD, int M, int D, float var_floor, const char *pat,
                             const float *x, float *para) {
    softmax_rows(F, Lp, startD, startD + M, 1.0f, pat, x, para);
    float *mean = para + (size_t)F * M;
    float *sd = para + (size_t)F * M * (1 + D);
    for (int f = 0; f < F; ++f) {
        const float *in = x + (size_t)f * Lp + startD + M;
        for (int i = 0; i < M * D; ++i) {
            if (pat[f] == orc::PAT_NONE) {
                sd[(size_t)f * M * D + i] = kSkipMarker;  // the mean slot is left as it was
                continue;
            }
            mean[(size_t)f * M * D + i] = in[i];
            float b = orc::safe_exp(in[M * D + i]);
            sd[(size_t)f * M * D + i] = b < var_floor ? var_floor : b;
        }
    }
}

// tmp holds F*M per-mixture log-likelihoods followed by F per-frame log-sums
float orc_mdn_mixture_error(int F, int Lt, int startDOut, int M, int D, const char *pat, const float *target,
                            const float *para, float *tmp) {
    const float *mean = para + (size_t)F * M;
    const float *sd = para + (size_t)F * M * (1 + D);
    for (int f = 0; f < F; ++f)
        for (int m = 0; m < M; ++m) {
            float acc = 0.0f;
            if (pat[f] != orc::PAT_NONE) {
                const float *t = target + (size_t)f * Lt + startDOut;
                const float *mu = mean + ((size_t)f * M + m) * D;
                const float *s = sd + ((size_t)f * M + m) * D;
                // the division by the double literal 2.0 promotes the running sum to double
                for (int d = 0; d < D; ++d) acc = (float)((double)acc + (double)((t[d] - mu[d]) * (t[d] - mu[d]) / (s[d] * s[d])) / 2.0);
            }
            tmp[(size_t)f * M + m] = acc;
        }
    float total = 0.0f;
    for (int f = 0; f < F; ++f) {
        if (pat[f] == orc::PAT_NONE) continue;
        float lsum = orc::Lim::kLogZero;
        for (int m = 0; m < M; ++m) {
            const float *s = sd + ((size_t)f * M + m) * D;
            float lp = (float)((double)(std::log(para[(size_t)f * M + m]) - tmp[(size_t)f * M + m]) -
                               D * std::log(2 * kPiAsWritten) / 2.0);
            for (int d = 0; d < D; ++d) lp = lp - orc::safe_log(s[d]);
            if (lp < orc::Lim::kLSmall) lp = orc::Lim::kLSmall;
            lsum = orc::log_add(lsum, lp);
            tmp[(size_t)f * M + m] = lp;
        }
        tmp[(size_t)F * M + f] = lsum;
        total += -1 * lsum;
    }
    return total;
}

// errors is the preceding layer's error buffer (Lp per frame); the layer zero-fills it beforehand
void orc_mdn_mixture_backward(int F, int Lp, int Lt, int startD, int startDOut, int M, int D, float var_floor,
                              const char *pat, const float *target, const float *para, const float *tmp,
                              float *errors) {
    const float *mean = para + (size_t)F * M;
    const float *sd = para + (size_t)F * M * (1 + D);
    // pass 1: mixture weights, in index order
    for (int f = 0; f < F; ++f)
        for (int m = 0; m < M; ++m) {
            if (pat[f] == orc::PAT_NONE) {
                errors[(size_t)f * M + m] = 0.0f;  // (sic) not f*Lp + startD + m
            } else {
                const float post = orc::safe_exp(tmp[(size_t)f * M + m] - tmp[(size_t)F * M + f]);
                errors[(size_t)f * Lp + startD + m] = para[(size_t)f * M + m] - post;
            }
        }
    // pass 2: means and standard deviations
    for (int f = 0; f < F; ++f)
        for (int m = 0; m < M; ++m)
            for (int d = 0; d < D; ++d) {
                float *e_mu = errors + (size_t)f * Lp + startD + M + m * D + d;
                float *e_sd = e_mu + M * D;
                if (pat[f] == orc::PAT_NONE) {
                    *e_mu = 0.0f;
                    *e_sd = 0.0f;
                    continue;
                }
                const float t = target[(size_t)f * Lt + startDOut + d];
                const float mu = mean[((size_t)f * M + m) * D + d];
                const float s = sd[((size_t)f * M + m) * D + d];
                const float post = orc::safe_exp(tmp[(size_t)f * M + m] - tmp[(size_t)F * M + f]);
                *e_mu = post * (mu - t) / s / s;
                *e_sd = (s > var_floor) ? post - (*e_mu) * (mu - t) : 0.0f;
            }
}

void orc_softmax_forward(int F, int Lp, int startD, int K, float temperature, const char *pat, const float *x,
                         float *prob) {
    softmax_rows(F, Lp, startD, startD + K, temperature, pat, x, prob);
}

// prob_capacity is the allocated size of the probability buffer (the reference bounds the lookup by it)
float orc_softmax_error(int F, int Lt, int startDOut, int K, long prob_capacity, const char *pat,
                        const float *target, const float *prob) {
    float total = 0.0f;
    for (int f = 0; f < F; ++f) {
        float v = 0.0f;
        if (pat[f] != orc::PAT_NONE) {
            const int ti = (int)target[(size_t)f * Lt + startDOut];
            const long idx = (long)f * K + ti;
            float p = 1.0f;
            if (idx < prob_capacity && idx >= 0) p = prob[idx] > orc::Lim::kMin ? prob[idx] : orc::Lim::kMin;
            v = (float)(-1.0 * std::log(p));
        }
        total += v;
    }
    return total;
}

void orc_softmax_backward(int F, int Lp, int Lt, int startD, int startDOut, int K, const char *pat,
                          const float *target, const float *prob, float *errors) {
    for (int f = 0; f < F; ++f) {
        if (pat[f] == orc::PAT_NONE) continue;  // stays at the layer's zero fill
        const float t = target[(size_t)f * Lt + startDOut];
        for (int k = 0; k < K; ++k) {
            const bool hit = (double)((t - k) * (t - k)) < 0.0001;
            const float p = prob[(size_t)f * K + k];
            errors[(size_t)f * Lp + startD + k] = hit ? (-1 + p) : p;
        }
    }
}

// ---- sigmoid unit (layers/MDNUnit.cu:198-225 ComputeSigmoid, :563-596 ComputeSigmoidError, :539-551 FrameNum,
// :634-676 ComputeSigmoidBP, drivers :3553-3588, :3729-3823, :3825-3856).  K = endD - startD columns, one target
// per column.  The error is the summed binary cross entropy divided by the number of non-padding frames (the
// gradient is not divided); continuous = the unit's conValSig flag.
void orc_sigmoid_forward(int F, int Lp, int startD, int K, const char *pat, const float *x, float *prob) {
    for (int f = 0; f < F; ++f)
        for (int k = 0; k < K; ++k)
            prob[(size_t)f * K + k] = pat[f] == orc::PAT_NONE ? 0.0f : orc::logistic(x[(size_t)f * Lp + startD + k]);
}

float orc_sigmoid_error(int F, int Lt, int startDOut, int K, int continuous, const char *pat, const float *target,
                        const float *prob) {
    float likelihood = 0.0f, num = 0.0f;
    for (int f = 0; f < F; ++f) {
        if (pat[f] == orc::PAT_NONE) continue;
        num += 1.0f;
        for (int k = 0; k < K; ++k) {
            const float p = prob[(size_t)f * K + k], pr = (float)(1.0 - p);
            const float d = target[(size_t)f * Lt + startDOut + k];
            float v;
            if (continuous) {
                const float p1 = std::log(p > orc::Lim::kMin ? p : orc::Lim::kMin);
                const float p2 = std::log(pr > orc::Lim::kMin ? pr : orc::Lim::kMin);
                v = (float)(-1.0 * d * p1 - (1 - d) * p2);
            } else {
                const float b = d > 0 ? p : 1 - p;
                v = (float)(-1.0 * std::log(b > orc::Lim::kMin ? b : orc::Lim::kMin));
            }
            likelihood += v;
        }
    }
    return likelihood / num;
}

void orc_sigmoid_backward(int F, int Lp, int Lt, int startD, int startDOut, int K, int continuous, const char *pat,
                          const float *target, const float *prob, float *errors) {
    for (int f = 0; f < F; ++f)
        for (int k = 0; k < K; ++k) {
            float &e = errors[(size_t)f * Lp + startD + k];
            if (pat[f] == orc::PAT_NONE) { e = 0.0f; continue; }
            const float p = prob[(size_t)f * K + k], d = target[(size_t)f * Lt + startDOut + k];
            e = continuous ? p - d : (d > 0 ? -1 + p : p);
        }
}

}  // extern "C"
