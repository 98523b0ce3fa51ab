// CPU oracle, WaveNet building blocks -- TEST INFRASTRUCTURE ONLY (see oracle_common.h).
//
// Restates, from /root/reference/CURRENNT_codes/currennt_lib/src/layers:
//   CNNLayer.cu:78-179     ConvolutionCore      (sum of shifted columns of W^T x, bias, optional tanh)
//   CNNLayer.cu:182-237    ConvolutionCoreGra   (scatter of the deltas into the column buffer)
//   CNNLayer.cu:1099-1224  forward driver;  CNNLayer.cu:1409-1597  backward driver (1-D path only,
//                          zero padding; repeat_padding and the 2-D window_height path are not restated)
//   wavNetCore.cu:69-138   tanhSigMerge / tanhSigMergeGradient
//   wavNetCore.cu:143-190  loadLinguisticFeature (up-sampling by frame index, optional mean/std)
//   wavNetCore.cu:193-232  AddLinguisticFeature / AddLinguisticFeatureGrad
//   wavNetCore.cu:237-270  SumGradientsForExternalInput
//   wavNetCore.cu:629-711  forward driver;  wavNetCore.cu:801-916  backward driver
//   GatedActLayer.cu:64-121, 177-263            the unconditioned twin
//   SkipAddLayer.cu:186-240, 305-346            sum of inputs / fan-out of the errors
#include "currennt_oracle.h"
#include "oracle_common.h"

#include <cstring>
#include <vector>

namespace {

// column of filter d, tap shift (-hw..hw): cum[d] + hw[d] + shift
struct ConvGeom {
    int P, D, S, T, causal;
    const int *hw;     // half width per filter
    const int *inter;  // tap interval (dilation) per filter
    std::vector<int> cum;
    int Lw;
    ConvGeom(int P_, int D_, int S_, int T_, int causal_, const int *hw_, const int *inter_)
        : P(P_), D(D_), S(S_), T(T_), causal(causal_), hw(hw_), inter(inter_), cum((size_t)D_ + 1, 0) {
        for (int d = 0; d < D; ++d) cum[(size_t)d + 1] = cum[(size_t)d] + 2 * hw[d] + 1;
        Lw = cum[(size_t)D];
    }
};

}  // namespace

extern "C" {

int orc_cnn_total_width(int D, const int *half_width) {
    int w = 0;
    for (int d = 0; d < D; ++d) w += 2 * half_width[d] + 1;
    return w;
}

// weights = [P x Lw column-major | D bias]; conbuf is Lw x (T*S) scratch; out is D x (T*S)
void orc_cnn_forward(int P, int D, int S, int T, int causal, int output_tanh, float bias, const int *half_width,
                     const int *interval, const char *pat, const float *weights, const float *x, float *conbuf,
                     float *out) {
    const ConvGeom G(P, D, S, T, causal, half_width, interval);
    const int N = T * S;
    orc::mat_product(conbuf, G.Lw, N, P, weights, true, x, false, false);
    const float *b = weights + (size_t)P * G.Lw;
    for (int t = 0; t < N; ++t) {
        if (pat[t] == orc::PAT_NONE) continue;  // the output slot keeps its old content
        for (int d = 0; d < D; ++d) {
            const int hw = G.hw[d];
            float acc = 0.0f;
            for (int shift = -hw; shift <= (causal > 0 ? 0 : hw); ++shift) {
                const int col = G.cum[(size_t)d] + hw + shift;
                const int tt = t + shift * G.inter[d] * S;
                if (tt < 0 || tt >= N || pat[tt] == orc::PAT_NONE) continue;
                acc += conbuf[(size_t)tt * G.Lw + col];
            }
            const float v = acc + b[d] * bias;
            out[(size_t)t * D + d] = output_tanh ? orc::tanh_act(v) : v;
        }
    }
}

// err (D x N) is turned into tanh' * err in place when output_tanh is set; ex is P x N;
// dW = [P x Lw | D]
void orc_cnn_backward(int P, int D, int S, int T, int causal, int output_tanh, float bias, const int *half_width,
                      const int *interval, const char *pat, const float *weights, const float *x, const float *out,
                      float *err, float *conbuf, float *ex, float *dW) {
    const ConvGeom G(P, D, S, T, causal, half_width, interval);
    const int N = T * S;
    if (output_tanh)
        for (size_t i = 0; i < (size_t)D * N; ++i) err[i] = orc::tanh_deriv(out[i]) * err[i];
    std::memset(conbuf, 0, sizeof(float) * (size_t)G.Lw * N);
    for (int t = 0; t < N; ++t) {
        if (pat[t] == orc::PAT_NONE) continue;
        for (int d = 0; d < D; ++d) {
            const int hw = G.hw[d];
            for (int shift = -hw; shift <= (causal > 0 ? 0 : hw); ++shift) {
                const int col = G.cum[(size_t)d] + hw + shift;
                const int tt = t + shift * G.inter[d] * S;
                if (tt < 0 || tt >= N || pat[tt] == orc::PAT_NONE) continue;
                conbuf[(size_t)tt * G.Lw + col] = err[(size_t)t * D + d];
            }
        }
    }
    if (ex) orc::mat_product(ex, P, N, G.Lw, weights, false, conbuf, false, false);
    orc::mat_product(dW, P, G.Lw, N, x, false, conbuf, true, false);
    // bias: (bias * ones) * err^T over every slot, padding included
    std::vector<float> ones((size_t)N, bias);
    orc::mat_product(dW + (size_t)P * G.Lw, 1, D, N, ones.data(), false, err, true, false);
}

// ctx is C x N: conditioning frame frame_index[slot] of the slot's sequence, optionally normalised
void orc_wavnetc_load_context(int C, int S, int N, int max_feature_length, int resolution_one, const float *source,
                              const float *frame_index, const float *mean_std, const char *pat, float *ctx) {
    for (int t = 0; t < N; ++t)
        for (int c = 0; c < C; ++c) {
            float v = 0.0f;
            if (pat[t] != orc::PAT_NONE) {
                const int feat = resolution_one ? t : (int)(frame_index[t] * S + (t % S));
                if (frame_index[t] >= max_feature_length) {
                    v = 0.0f;
                } else if (mean_std) {
                    const float sd = mean_std[c + C];
                    v = (float)((source[(size_t)feat * C + c] - mean_std[c]) / (sd < 1e-5f ? 1.0 : (double)sd));
                } else {
                    v = source[(size_t)feat * C + c];
                }
            }
            ctx[(size_t)t * C + c] = v;
        }
}

// D = layer size; conv is 2D x N; core (2D x N) and ctx_tanh (2D x N) are outputs; out is D x N.
// C == 0: no conditioning (weights / ctx unused).
void orc_wavnetc_forward(int D, int C, int N, const char *pat, const float *weights, const float *ctx,
                         const float *conv, float *core, float *ctx_tanh, float *out) {
    const int D2 = 2 * D;
    if (C == 0) std::memset(core, 0, sizeof(float) * (size_t)D2 * N);
    else orc::mat_product(core, D2, N, C, weights, true, ctx, false, false);
    for (size_t i = 0; i < (size_t)D2 * N; ++i) {
        if (pat[i / D2] == orc::PAT_NONE) {
            core[i] = 0.0f;
            ctx_tanh[i] = 0.0f;
        } else {
            ctx_tanh[i] = orc::tanh_act(core[i]);
            core[i] = conv[i] + ctx_tanh[i];
        }
    }
    for (int t = 0; t < N; ++t)
        for (int d = 0; d < D; ++d)
            out[(size_t)t * D + d] = (pat[t] == orc::PAT_NONE)
                                         ? 0.0f
                                         : orc::tanh_act(core[(size_t)t * D2 + d]) * orc::logistic(core[(size_t)t * D2 + D + d]);
}

// gradient of z = tanh(y1) * sigmoid(y2) w.r.t. the 2D pre-activations `pre`, written to prev_err
void orc_gated_backward(int D, int N, const char *pat, const float *pre, const float *err, float *prev_err) {
    const int D2 = 2 * D;
    for (int t = 0; t < N; ++t)
        for (int j = 0; j < D2; ++j) {
            float v = 0.0f;
            if (pat[t] != orc::PAT_NONE) {
                if (j < D) {
                    const float th = orc::tanh_act(pre[(size_t)t * D2 + j]);
                    v = (1.0f - th * th) * orc::logistic(pre[(size_t)t * D2 + j + D]) * err[(size_t)t * D + j];
                } else {
                    const float sg = orc::logistic(pre[(size_t)t * D2 + j]);
                    v = orc::tanh_act(pre[(size_t)t * D2 + j - D]) * (sg * (1.0f - sg)) * err[(size_t)t * D + j - D];
                }
            }
            prev_err[(size_t)t * D2 + j] = v;
        }
}

void orc_gated_forward(int D, int N, const char *pat, const float *pre, float *out) {
    for (int t = 0; t < N; ++t)
        for (int d = 0; d < D; ++d)
            out[(size_t)t * D + d] = (pat[t] == orc::PAT_NONE)
                                         ? 0.0f
                                         : orc::tanh_act(pre[(size_t)t * 2 * D + d]) * orc::logistic(pre[(size_t)t * 2 * D + D + d]);
}

// ctx_tanh holds tanh(X_c) on entry and the gradient w.r.t. X_c on return; ctx_grad (C x N) may be NULL,
// otherwise W * g is added to it.
void orc_wavnetc_backward(int D, int C, int N, const char *pat, const float *weights, const float *ctx,
                          const float *core, float *ctx_tanh, const float *err, float *prev_err, float *dW,
                          float *ctx_grad) {
    const int D2 = 2 * D;
    orc_gated_backward(D, N, pat, core, err, prev_err);
    if (C == 0) return;
    for (size_t i = 0; i < (size_t)D2 * N; ++i) ctx_tanh[i] = orc::tanh_deriv(ctx_tanh[i]) * prev_err[i];
    orc::mat_product(dW, C, D2, N, ctx, false, ctx_tanh, true, false);
    if (ctx_grad) orc::mat_product(ctx_grad, C, N, D2, weights, false, ctx_tanh, false, true);
}

// frame-rate gradient: sum of the sample-rate gradients inside each frame
void orc_wavnetc_sum_context_grad(int C, int S, int resolution, int n_frames_slots, int N, const char *pat_frames,
                                  const char *pat, const float *ctx_grad, float *frame_grad) {
    for (int f = 0; f < n_frames_slots; ++f)
        for (int c = 0; c < C; ++c) {
            float *o = &frame_grad[(size_t)f * C + c];
            if (pat_frames[f] == orc::PAT_NONE) {
                *o = 0.0f;
                continue;
            }
            *o = 0.0f;  // the driver zero-fills the frame-rate buffer right before
            const int rel = f / S, s = f % S;
            for (int i = 0; i < resolution; ++i) {
                const int idx = (rel * resolution + i) * S + s;
                if (idx < N && pat[idx] != orc::PAT_NONE) *o += ctx_grad[(size_t)idx * C + c];
            }
        }
}

// out = sum of inputs; errors and errors_from_skip are cleared for the backward pass
void orc_skipadd_forward(long count, int n_in, const float *const *inputs, float *out, float *errors,
                         float *errors_from_skip) {
    for (long i = 0; i < count; ++i) {
        errors[i] = 0.0f;
        errors_from_skip[i] = 0.0f;
        float acc = 0.0f;
        for (int k = 0; k < n_in; ++k) acc += inputs[k][i];
        out[i] = acc;
    }
}

// errors += errors_from_skip; predecessors in reverse order: skip layers accumulate, others are overwritten
void orc_skipadd_backward(long count, float *errors, const float *errors_from_skip, int n_pre, float *const *targets,
                          const int *target_is_skip) {
    for (long i = 0; i < count; ++i) errors[i] = errors_from_skip[i] + errors[i];
    for (int k = n_pre - 1; k >= 0; --k)
        for (long i = 0; i < count; ++i) {
            if (target_is_skip[k]) targets[k][i] = errors[i] + targets[k][i];
            else targets[k][i] = errors[i];
        }
}

}  // extern "C"
