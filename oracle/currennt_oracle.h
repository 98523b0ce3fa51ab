// C entry points of the CPU oracle -- TEST INFRASTRUCTURE ONLY (see oracle_common.h).
// All buffers are host memory, fp32, laid out exactly as the reference lays them out:
// an activation of a layer of size D is a column-major D x (T*S) matrix, column (t*S+s).
#ifndef CURRENNT_ORACLE_H
#define CURRENNT_ORACLE_H

#ifdef __cplusplus
extern "C" {
#endif

typedef struct {
    int P;      /* size of the preceding layer                                  */
    int L;      /* layer size (sum over both directions when bidirectional)     */
    int bidir;  /* 0 unidirectional, 1 bidirectional                            */
    int S;      /* parallel sequences                                           */
    int T;      /* curMaxSeqLength of the fraction                              */
    int Tmin;   /* curMinSeqLength of the fraction                              */
    float bias; /* the layer's constant bias input                              */
} orc_lstm_desc;

/* Per-direction state; every buffer is H x (T*S), H = L or L/2. */
typedef struct {
    float *ni, *ig, *fg, *og; /* gate activations (pre-activations until the forward pass overwrites them) */
    float *c;                 /* cell states                                                               */
    float *h;                 /* block outputs                                                              */
    float *herr;              /* output errors of this direction, receives the recurrent terms in place     */
    float *dni, *dig, *dfg, *dog; /* clipped gate deltas                                                    */
    float *cerr;              /* cell-state errors (unclipped)                                              */
} orc_lstm_dir;

/* scalar helpers (for unit tests of the scalar semantics) */
// Worker threads for the large loops (default 1).  Outputs are shared out whole, so results do not change.
void orc_set_threads(int n);
int orc_get_threads(void);

float orc_logistic(float x);
float orc_tanh(float x);
float orc_safe_exp(float x);
float orc_safe_log(float x);
float orc_log_add(float x, float y);

/* generic column-major product, reference summation order */
void orc_mat_product(float *C, int m, int n, int k, const float *A, int tA, const float *B, int tB,
                     int accumulate);

/* LSTM (LstmLayer.cu).  `out` is L x (T*S). For a unidirectional layer fw->h may alias `out`. */
void orc_lstm_forward(const orc_lstm_desc *d, const float *weights, const char *patTypes, const float *x,
                      orc_lstm_dir *fw, orc_lstm_dir *bw, float *out);
/* `outerr` is L x (T*S) (read only; it is split/copied into herr).  `ex` (P x T*S) may be NULL. */
void orc_lstm_backward(const orc_lstm_desc *d, const float *weights, const char *patTypes, const float *x,
                       const float *outerr, orc_lstm_dir *fw, orc_lstm_dir *bw, float *ex,
                       float *weightUpdates);
long orc_lstm_weight_count(int P, int L, int bidir);

/* Feed-forward layer (FeedForwardLayer.cu). act: 0 identity, 1 tanh, 2 logistic, 3 relu.
   weights = [P x D col-major | D bias]. */
void orc_dense_forward(int P, int D, int N, int act, float bias, const float *weights, const float *x,
                       float *y);
/* err (D x N) is turned into deltas in place; ex (P x N) may be NULL; dW has P*D + D entries. */
void orc_dense_backward(int P, int D, int N, int act, float bias, const float *weights, const float *x,
                        const float *y, float *err, float *ex, float *dW);

/* SSE post output layer (SsePostOutputLayer.cu) */
float orc_sse_error(int D, int N, const char *patTypes, const float *y, const float *target);
void orc_sse_backward(int D, int N, const char *patTypes, const float *y, const float *target, float *err);

/* Mixture-density post-output layer (MDNUnit.cu, MDNLayer.cu).  F = T*S frames, Lp = size of the layer
   feeding the MDN, Lt = size of the target vector.  A mixture unit with M components over D target
   dimensions reads columns [startD, startD + M + 2*M*D) of the input: weights, means, log-std.
   para = [F*M weights | F*M*D means | F*M*D std]; tmp = [F*M log-likelihoods | F log-sums]. */
void orc_mdn_mixture_forward(int F, int Lp, int startD, int M, int D, float var_floor, const char *pat,
                             const float *x, float *para);
float orc_mdn_mixture_error(int F, int Lt, int startDOut, int M, int D, const char *pat, const float *target,
                            const float *para, float *tmp);
void orc_mdn_mixture_backward(int F, int Lp, int Lt, int startD, int startDOut, int M, int D, float var_floor,
                              const char *pat, const float *target, const float *para, const float *tmp,
                              float *errors);
void orc_softmax_forward(int F, int Lp, int startD, int K, float temperature, const char *pat, const float *x,
                         float *prob);
float orc_softmax_error(int F, int Lt, int startDOut, int K, long prob_capacity, const char *pat,
                        const float *target, const float *prob);
void orc_softmax_backward(int F, int Lp, int Lt, int startD, int startDOut, int K, const char *pat,
                          const float *target, const float *prob, float *errors);

/* WaveNet building blocks (CNNLayer.cu 1-D path, wavNetCore.cu, GatedActLayer.cu, SkipAddLayer.cu).
   N = T*S slots.  CNN filter d has half width half_width[d] (2*hw+1 weight columns) and tap interval
   interval[d]; weights = [P x Lw column-major | D bias], Lw = sum(2*hw+1). */
int orc_cnn_total_width(int D, const int *half_width);
void orc_cnn_forward(int P, int D, int S, int T, int causal, int output_tanh, float bias, const int *half_width,
                     const int *interval, const char *pat, const float *weights, const float *x, float *conbuf,
                     float *out);
void orc_cnn_backward(int P, int D, int S, int T, int causal, int output_tanh, float bias, const int *half_width,
                      const int *interval, const char *pat, const float *weights, const float *x, const float *out,
                      float *err, float *conbuf, float *ex, float *dW);
void orc_wavnetc_load_context(int C, int S, int N, int max_feature_length, int resolution_one, const float *source,
                              const float *frame_index, const float *mean_std, const char *pat, float *ctx);
void orc_wavnetc_forward(int D, int C, int N, const char *pat, const float *weights, const float *ctx,
                         const float *conv, float *core, float *ctx_tanh, float *out);
void orc_wavnetc_backward(int D, int C, int N, const char *pat, const float *weights, const float *ctx,
                          const float *core, float *ctx_tanh, const float *err, float *prev_err, float *dW,
                          float *ctx_grad);
void orc_wavnetc_sum_context_grad(int C, int S, int resolution, int n_frames_slots, int N, const char *pat_frames,
                                  const char *pat, const float *ctx_grad, float *frame_grad);
void orc_gated_forward(int D, int N, const char *pat, const float *pre, float *out);
void orc_gated_backward(int D, int N, const char *pat, const float *pre, const float *err, float *prev_err);
void orc_skipadd_forward(long count, int n_in, const float *const *inputs, float *out, float *errors,
                         float *errors_from_skip);
void orc_skipadd_backward(long count, float *errors, const float *errors_from_skip, int n_pre, float *const *targets,
                          const int *target_is_skip);

/* DFT log-amplitude loss (helpers/FFTMat.cu, layers/DFTErrorPostoutputLayer.cu); transforms follow cuFFT's
   R2C / C2R conventions (unnormalised, n/2+1 bins, imaginary parts of DC and Nyquist ignored by C2R). */
int orc_dft_frame_count(int signal_length, int frame_length, int frame_shift);
void orc_dft_r2c(int n, const float *in, float *out);
void orc_dft_c2r(int n, const float *in, float *out);
float orc_dft_spectral_loss(int dis_type, int fft_length, int frame_length, int frame_shift, int window_type,
                            int max_length, int length, float gamma, float log_floor, const float *source,
                            const float *target, float *grad);
float orc_dft_phase_loss(int fft_length, int frame_length, int frame_shift, int window_type, int max_length,
                         int length, float zeta, const float *source, const float *target, float *grad);
float orc_dft_logamp_loss(int fft_length, int frame_length, int frame_shift, int window_type, int max_length,
                          int length, float gamma, float log_floor, const float *source, const float *target,
                          float *grad);

/* MDN sigmoid unit (layers/MDNUnit.cu:198-225, 539-676, 3553-3856): K columns, one target per column */
void orc_sigmoid_forward(int F, int Lp, int startD, int K, const char *pat, const float *x, float *prob);
float orc_sigmoid_error(int F, int Lt, int startDOut, int K, int continuous, const char *pat, const float *target,
                        const float *prob);
void orc_sigmoid_backward(int F, int Lp, int Lt, int startD, int startDOut, int K, int continuous, const char *pat,
                          const float *target, const float *prob, float *errors);

/* weight update of the training loop (optimizers/Optimizer.cu:186-198, optimizers/SteepestDescentOptimizer.cu) */
void orc_opt_accumulate(long n, const float *layer_updates, float *cur_updates, int add);
void orc_opt_adjust_gradient(int option, long n, float *g, float *stats, const float *mask, float frac_length,
                             float beta1_accum, float beta2_accum);
void orc_opt_update_weights(long n, float *weights, float *g, float *deltas, const float *mask, float learning_rate,
                            float momentum);
float orc_opt_next_beta_accum(float accum, int which);

#ifdef __cplusplus
}
#endif
#endif
