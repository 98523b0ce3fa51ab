/* C ABI of the gfx950 (MI355X) implementation of CURRENNT's backward hot path.
 *
 * Every entry point takes plain device pointers and sizes; no C++ or PyTorch types cross this
 * boundary.  All buffers are fp32 and use the reference's layouts:
 *   - an activation / error buffer of a layer of size D is a column-major D x (T*S) matrix whose
 *     column index is t*S + s  (time-major, S parallel sequences interleaved);
 *   - patTypes is char[T*S], values 0 none (padding), 1 first, 2 normal, 3 last (Types.hpp:35-38);
 *   - weight vectors keep the reference's order  input | bias | internal.
 * `stream` is a hipStream_t passed as void*; every call only enqueues work on that stream.
 * Every function returns CNT_OK or an error code; cnt_last_error() gives the message of the
 * calling thread's last failure.  A handle must be used by one thread at a time.
 *
 * Paths in the comments are relative to CURRENNT_codes/currennt_lib/src of the reference.
 */
#ifndef CURRENNT_HIP_H
#define CURRENNT_HIP_H

#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { CNT_OK = 0, CNT_ERR_ARG = 1, CNT_ERR_HIP = 2, CNT_ERR_STATE = 3, CNT_ERR_DEVICE = 4 };

enum { CNT_ACT_IDENTITY = 0, CNT_ACT_TANH = 1, CNT_ACT_LOGISTIC = 2, CNT_ACT_RELU = 3 };

int cnt_version(void);
const char *cnt_last_error(void);

/* ---- per-kernel timing ----------------------------------------------------------------------------
 * The reference has no profiler hooks (it prints wall-clock per epoch, currennt/src/main.cpp:302-317).
 * cnt_profile_enable(1) clears earlier records and makes every launch site bracket its kernels with
 * HIP events on the launch stream; cnt_profile_get(i, ...) waits for the events and returns the i-th
 * label (order of first use), its launch count and summed duration in ms, or CNT_ERR_ARG past the end. */
int cnt_profile_enable(int on);
int cnt_profile_get(int index, char *label, int label_cap, int *launches, float *total_ms);
/* Measurement hook without a counterpart in the reference: the time of one hop of a word between two workgroups the
 * way the recursion kernels exchange data -- a store and a polling load that bypasses the per-CU cache -- on the
 * same XCD (through its L2) or on two XCDs (through the memory side), with (with_compute) or without the arithmetic
 * a recursion step does between receiving and sending.  T times this is the floor of a T-step recursion spread
 * over compute units.  Synchronous; *hop_us (host memory) receives microseconds per hop. */
int cnt_probe_hop_latency(void *stream, int same_xcd, int with_compute, int rounds, float *hop_us);
/* The same hop for a message of `kilobytes` (4, 8, 12 or 16) between two workgroups of four waves on one XCD: every
 * lane polls its 16-byte pieces until all carry the round's tag, the waves meet at a barrier, the workgroup answers.
 * 4 KB is what a workgroup of a 256-cell recursion receives per step today; 16 KB is what the forward recursion would
 * receive if it exchanged partial pre-activations of the four gates instead of outputs. */
int cnt_probe_hop_message(void *stream, int kilobytes, int rounds, float *hop_us);
/* Test hook: the scalar activation functions as the kernels evaluate them, out[i] = f(x[i]) for n device floats.
 * which = 0: logistic, 1: tanh (activation_functions/Logistic.cuh, Tanh.cuh: exp and a true quotient, clamped at
 * +-88.72); 2, 3: the same two from the hardware's exp2 and reciprocal, which only the forward LSTM recursion uses
 * (within 4e-6 / 8e-6 absolute of the former, not bit-identical). */
int cnt_probe_activation(void *stream, int which, long n, const float *x, float *out);

/* ---- helpers::Matrix product seam -------------------------------------------------------------
 * Replaces helpers::Matrix<Gpu>::assignProduct / addProduct (helpers/Matrix.cu:353-377, which call
 * cublas::multiplyMatrices, helpers/cublas.cu:52-84).  Column-major, C is m x n, inner size k.
 * transA: A is stored k x m;  transB: B is stored n x k.  (transA && transB) is rejected, as in
 * the reference.  accumulate != 0 adds to C. */
int cnt_matrix_product(void *stream, float *C, int m, int n, int k, const float *A, int transA,
                       const float *B, int transB, int accumulate);

/* ---- feed-forward layer ------------------------------------------------------------------------
 * FeedForwardLayer<TDevice,TActFn>::computeForwardPass  (layers/FeedForwardLayer.cu:1060-1101)
 * weights = [P x D column-major | D bias weights];  y = act(W^T x + bias * b). N = T*S columns. */
int cnt_dense_forward(void *stream, int P, int D, int N, int act, float bias, const float *weights,
                      const float *x, float *y);
/* FeedForwardLayer::computeBackwardPass (layers/FeedForwardLayer.cu:1633-1738, functors :105-138).
 * err (D x N) holds the output errors on entry and the deltas act'(y)*err on return (all slots,
 * padding included, as the reference does); prev_err (P x N) is overwritten with W*delta and may
 * be NULL; weight_updates (P*D + D) is overwritten with [x * delta^T | bias * sum delta]. */
int cnt_dense_backward(void *stream, int P, int D, int N, int act, float bias, const float *weights,
                       const float *x, const float *y, float *err, float *prev_err,
                       float *weight_updates);

/* The two halves of cnt_dense_backward, for callers that schedule them on different streams: the error
 * half (delta in place, prev_err) is what the next layer's backward waits for; the weight half
 * (weight_updates from x and the deltas) has no consumer before the optimizer.  The reference has no such
 * split; calling both in this order on one stream is cnt_dense_backward.
 * Device memory: the weight half of a narrow layer over a long input (P*D up to 64 K floats, N in the thousands)
 * sums split partial products through a scratch buffer of 16 MB per stream, which the library allocates the first
 * time such a product runs on a stream and keeps; the same holds for cnt_cnn_backward_weights and
 * cnt_wavnetc_backward_weights.  Apart from that, only the *_create calls allocate. */
int cnt_dense_backward_errors(void *stream, int P, int D, int N, int act, const float *weights, const float *y,
                              float *err, float *prev_err);
int cnt_dense_backward_weights(void *stream, int P, int D, int N, float bias, const float *x, const float *err,
                               float *weight_updates);
/* The scratch buffer of `stream` for those split products (16 MB of device memory), allocated now instead of
 * inside the first product that wants it, and freed again (the stream must be idle).  No counterpart in the
 * reference, whose cuBLAS handle owns its workspace.  A product that finds no buffer and cannot get one (out of
 * memory, a stream under capture) adds its splits atomically instead. */
int cnt_gemm_reserve(void *stream);
int cnt_gemm_release(void *stream);
/* How many such buffers the library holds at the moment.  That allocation is the only one any entry point other
 * than a *_create call makes, so a caller (or a test) that sees the same number before and after a pass knows that
 * the pass allocated nothing.  No counterpart in the reference. */
int cnt_gemm_scratch_buffers(void);
/* cnt_dense_backward_weights for callers that cannot allocate device memory (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc): same arguments, same result, but the split partial products go
 * through an 8 MB array that is part of the library's code object (one copy per GPU, held until the process ends),
 * so the call allocates nothing.  No counterpart in the reference.  Limit: P*D + D <= 2 097 152 floats, larger
 * layers are refused with CNT_ERR_ARG.  All calls on one GPU share that array: calls that overlap in time on one
 * GPU (different streams or threads) race; calls on one stream are ordered and safe. */
int cnt_dense_backward_weights_static(void *stream, int P, int D, int N, float bias, const float *x, const float *err,
                                      float *weight_updates);

/* ---- SSE post-output layer ---------------------------------------------------------------------
 * SsePostOutputLayer::computeBackwardPass (layers/SsePostOutputLayer.cu:224-267):
 * err = y - target, exactly 0 on padding slots. */
int cnt_sse_backward(void *stream, int D, int N, const char *patTypes, const float *y,
                     const float *target, float *err);
/* SsePostOutputLayer::calculateError (layers/SsePostOutputLayer.cu:166-210): 0.5 * sum (t-y)^2 over
 * non-padding slots, written to *result_dev (device memory, one float). */
int cnt_sse_error(void *stream, int D, int N, const char *patTypes, const float *y,
                  const float *target, float *result_dev);

/* ---- LSTM layer --------------------------------------------------------------------------------
 * LstmLayer<TDevice> (layers/LstmLayer.cu).  The handle owns what the reference keeps in its two
 * forward_backward_info_t members (layers/LstmLayer.hpp:99-133): per direction the gate
 * activations, cell states, block outputs, output errors, gate deltas and cell-state errors, each
 * H x (maxT*S).  The caller owns weights, weight updates, inputs, outputs and error buffers. */
typedef struct cnt_lstm cnt_lstm;

typedef struct {
    int P;       /* preceding layer size                                    */
    int L;       /* layer size; bidirectional layers use L/2 per direction  */
    int bidir;   /* 0 "lstm", 1 "blstm" (LayerFactory.cu:104-110)           */
    int S;       /* parallel sequences                                      */
    int maxT;    /* maxSeqLength the buffers are allocated for              */
    float bias;  /* the layer's constant bias input ("bias" in the JSON)    */
} cnt_lstm_desc;

/* LstmLayer::LstmLayer (layers/LstmLayer.cu:1078-1268): allocates the per-direction state.  Layers with 64, 128,
 * 256 or 512 cells per direction and at most 32 parallel sequences run their recursions as persistent kernels;
 * any other geometry runs them step by step (one batched recurrent product and one cell kernel per time step, the
 * reference's own schedule), with the same results.
 * With 64, 128 or 256 cells per direction both recursions run on teams of workgroups that share one XCD's L2: a job
 * is a direction and up to four sequences, its team exchanges each step's outputs (forward) or partial errors
 * (backward) through that L2, and the launch asks for a little more than half of a compute unit's LDS so that every
 * workgroup of a team gets a compute unit of its own (two on one unit take their steps at the same moments and cost
 * a fifth of the step time).  Environment, read when a handle is created: CNT_LSTM_LOCAL=0 / CNT_LSTM_FWD_LOCAL=0
 * (the kernels that exchange across XCDs instead), CNT_LSTM_SPREAD_LDS=<bytes> (the LDS request, 0: none),
 * CNT_LSTM_LOCAL_JB=16 (16 instead of 8 cells per workgroup for 256-cell layers), CNT_LSTM_WARM=1 (a full-bandwidth
 * read of the states into the memory-side cache in front of the backward recursion), CNT_LSTM_MEM_DELAY=<units of 64
 * clocks> (how long the backward recursion's memory wave sleeps after a step's barrier), CNT_LSTM_STEPWISE=1. */
int cnt_lstm_create(const cnt_lstm_desc *desc, cnt_lstm **out);
int cnt_lstm_destroy(cnt_lstm *h);
/* LstmLayer::loadSequences (layers/LstmLayer.cu:1488-1533): records the fraction's geometry and
 * zero-fills the stored output-gate deltas.  patTypes is device memory, char[curMaxT*S], and must
 * stay valid until the next call of this function.  For a fraction with much padding (curMinT at most 3/4 of
 * curMaxT, at least 2048 slots) it also lists the valid slots, on the stream, and cnt_lstm_backward_weights then sums
 * over those only -- the deltas are zero on padding slots, so no result changes (CNT_LSTM_SKIP_PADDING=0, read at
 * cnt_lstm_create: never). */
int cnt_lstm_load_sequences(cnt_lstm *h, void *stream, const char *patTypes, int curMaxT, int curMinT);
/* LstmLayer::computeForwardPass(nnState) (layers/LstmLayer.cu:1743-1949).
 * x is P x (T*S); outputs is L x (T*S). */
int cnt_lstm_forward(cnt_lstm *h, void *stream, const float *weights, const float *x, float *outputs);
/* LstmLayer::computeBackwardPass(nnState) (layers/LstmLayer.cu:2066-2382).
 * output_errors is L x (T*S).  For a unidirectional layer the recurrent error terms are added to
 * it in place, which is what the reference's buffer swap (:2086-2087, :2378-2381) leaves behind.
 * prev_errors (P x T*S) is overwritten and may be NULL.  weight_updates has the size and layout of
 * the weight vector and is overwritten.  `outputs` is the buffer cnt_lstm_forward filled. */
int cnt_lstm_backward(cnt_lstm *h, void *stream, const float *weights, const float *x,
                      const float *outputs, float *output_errors, float *prev_errors,
                      float *weight_updates);
/* The two halves of cnt_lstm_backward (layers/LstmLayer.cu:2066-2334 and :2337-2375), for callers that put
 * the weight gradients on another stream: the second half only reads x and the handle's state. */
int cnt_lstm_backward_errors(cnt_lstm *h, void *stream, const float *weights, float *output_errors,
                             float *prev_errors);
int cnt_lstm_backward_weights(cnt_lstm *h, void *stream, const float *x, float *weight_updates);
/* The product at the end of the first half on its own (layers/LstmLayer.cu:2298-2334): prev_errors =
 * sum over gates and directions of W_in * delta.  cnt_lstm_backward_errors with prev_errors == NULL runs only the
 * recursion; a caller can then start cnt_lstm_backward_weights on another stream as soon as the recursion is
 * done and compute the preceding layer's errors meanwhile. */
int cnt_lstm_backward_prev_errors(cnt_lstm *h, void *stream, const float *weights, float *prev_errors);
/* The same two pieces over a part of the fraction, for callers that overlap the end of a layer's recursion with the
 * products that follow it (the reference runs the recursion step by step, layers/LstmLayer.cu:2136-2252, and the
 * product over the whole fraction, :2298-2334; splitting either changes no result).
 * cnt_lstm_backward_errors_range runs steps [step_begin, step_end) of the curMaxT steps of the recursion; the
 * ranges of one pass must be launched in order on one stream, the first from step 0.  The handle keeps the step the
 * pass stands at: a range that starts anywhere else is refused (CNT_ERR_ARG), and a pass that is abandoned half way
 * -- a range from step 0, cnt_lstm_backward_errors, cnt_lstm_forward or cnt_lstm_load_sequences before step curMaxT
 * was reached -- is dropped cleanly (the partial errors it left in the mailbox are discarded).  Only where
 * cnt_lstm_backward_can_split returns 1 (layers whose backward recursion runs as one persistent kernel per group of
 * sequences); elsewhere it is an error.
 * cnt_lstm_backward_steps_done: the time steps [t_begin, t_end) whose deltas are final once `steps` steps have run
 * (both directions have passed them), i.e. what cnt_lstm_backward_prev_errors_range may already compute:
 * prev_errors columns of the time steps [t_begin, t_end) only.
 * (The library's own network sequencer does not split: on MI355X the second launch's cold start cost more than the
 * overlap gained for the benchmark model.) */
int cnt_lstm_backward_can_split(const cnt_lstm *h);
int cnt_lstm_backward_errors_range(cnt_lstm *h, void *stream, const float *weights, float *output_errors,
                                   int step_begin, int step_end);
int cnt_lstm_backward_steps_done(const cnt_lstm *h, int steps, int *t_begin, int *t_end);
int cnt_lstm_backward_prev_errors_range(cnt_lstm *h, void *stream, const float *weights, float *prev_errors,
                                        int t_begin, int t_end);
/* Device pointer to one internal buffer.  dir: 0 forward, 1 backward states.  which:
 * 0 niActs 1 igActs 2 fgActs 3 ogActs 4 cellStates 5 tmpOutputs 6 tmpOutputErrors
 * 7 niDeltas 8 igDeltas 9 fgDeltas 10 ogDeltas 11 cellStateErrors.  NULL if out of range. */
/* Bounds of the recursion kernels' waits (no counterpart in the reference, which has no inter-workgroup waits):
 * spin_limit = poll rounds a workgroup tries before it gives up and stops the whole recursion (default 2^22;
 * the failure surfaces at cnt_lstm_check); poll_delay_* = pause before the first poll of a step in units of 64
 * clocks.  Defaults come from the geometry (and CNT_LSTM_SPIN_LIMIT / CNT_LSTM_POLL_DELAY[_FWD]).  A tiny
 * spin_limit lets a test exercise the give-up path without any kernel hanging. */
int cnt_lstm_set_wait_bounds(cnt_lstm *h, unsigned spin_limit, int poll_delay_backward, int poll_delay_forward);
float *cnt_lstm_state(cnt_lstm *h, int dir, int which);
long cnt_lstm_weight_count(int P, int L, int bidir);
/* Waits for the stream and reports whether a recursion kernel of this handle gave up waiting for a
 * neighbouring workgroup (CNT_ERR_DEVICE; the results of that pass are invalid).  The reference has
 * no counterpart: its per-step launches cannot stall on each other.
 * Failure contract of the handle: a recursion that gives up ends normally (no kernel hangs or faults) and latches
 * the failure in host-visible memory.  It is returned, once, by this call or by the NEXT call of any kind into the
 * same handle after the failed launch has ended (cnt_lstm_load_sequences, _forward, _backward*, ...), so a caller
 * that never calls cnt_lstm_check still sees CNT_ERR_DEVICE, one call late.  The launch after that heals the
 * handle's mailboxes; nothing has to be recreated. */
int cnt_lstm_check(cnt_lstm *h, void *stream);

/* ---- mixture-density post-output layer ----------------------------------------------------------
 * MDNLayer<TDevice> with MDNUnit_sigmoid, MDNUnit_softmax (flat) and MDNUnit_mixture (untied variance) units
 * (layers/MDNLayer.cu, layers/MDNUnit.cu).  The handle owns what the units keep between calls: the
 * distribution parameters (m_paraVec) and the per-mixture log-likelihoods and log-sums (m_tmpPat).
 * `config` is the content of the reference's binary mdn config: [n, (startD, endD, startDOut, endDOut,
 * type) x n] as floats (layers/MDNLayer.cu:286-324); type 0 = sigmoid (one target per column), -1 = softmax,
 * > 0 = number of Gaussians (layers/MDNLayer.hpp:35-36).  Other unit types and tied variances are rejected.
 * cnt_mdn_calculate_error adds up the units' errors as the reference does: the mixture and softmax units
 * contribute their summed negative log-likelihood, a sigmoid unit its cross entropy divided by the number
 * of non-padding frames (layers/MDNUnit.cu:3821). */
typedef struct cnt_mdn cnt_mdn;

typedef struct {
    int Lp;            /* size of the layer feeding the MDN layer            */
    int Lt;            /* size of the MDN layer = target dimension           */
    int S;             /* parallel sequences                                 */
    int maxT;          /* maxSeqLength                                       */
    int tie_variance;  /* --tieVariance; only 0 is supported                 */
    int sigmoid_continuous; /* sigmoid units: targets are probabilities (the layer's conValSig flag, MDNLayer.cu:466) */
} cnt_mdn_desc;

/* MDNLayer::MDNLayer (layers/MDNLayer.cu:280-324, 457-545). */
int cnt_mdn_create(const cnt_mdn_desc *desc, const float *config, int config_len, cnt_mdn **out);
int cnt_mdn_destroy(cnt_mdn *h);
/* Variance floor of a mixture unit.  The reference derives it from data -- MDNUnit_mixture::initPreOutput
 * (layers/MDNUnit.cu:5146-5234: vFloorPara (1e-4) times the mean standard deviation of the target dimensions) --
 * and only when the network file holds no "weights" section (NeuralNetwork.cpp:1047-1048, :3649-3664); it is 0 for
 * a network that starts from trained weights.  That pass over the training targets is not part of this library: a
 * caller that trains from scratch computes the statistic (the reference's own mean / variance file, e.g.) and hands
 * the floor over here; left alone it is 0, as when training resumes from a weights file. */
int cnt_mdn_set_var_floor(cnt_mdn *h, int unit, float var_floor);
/* Layer::loadSequences: records the fraction's pattern types (device memory, char[curMaxT*S]). */
int cnt_mdn_load_sequences(cnt_mdn *h, void *stream, const char *patTypes, int curMaxT);
/* MDNLayer::computeForwardPass (layers/MDNLayer.cu:841-852): nn_outputs is Lp x (T*S). */
int cnt_mdn_forward(cnt_mdn *h, void *stream, const float *nn_outputs);
/* MDNLayer::calculateError (layers/MDNLayer.cu:797-827): targets is Lt x (T*S); the negative
 * log-likelihood summed over units and frames is written to *result_dev (device memory).  It also
 * stores the posteriors' ingredients that cnt_mdn_backward reads, as the reference does. */
int cnt_mdn_calculate_error(cnt_mdn *h, void *stream, const float *targets, float *result_dev);
/* MDNLayer::computeBackwardPass (layers/MDNLayer.cu:875-917): prev_errors is the preceding layer's
 * whole error buffer, Lp x (maxT*S); it is zero-filled and then receives every unit's gradient. */
int cnt_mdn_backward(cnt_mdn *h, void *stream, const float *targets, float *prev_errors);
/* MDNLayer::calculateError followed by MDNLayer::computeBackwardPass (layers/MDNLayer.cu:797-827, :875-917) as one
 * call, for trainers that always run both: *result_dev, the units' buffers and prev_errors end up as after the two
 * calls above.  A mixture unit of at most 16 components over at most 64 target dimensions (sizes and start columns
 * multiples of four, buffers 16-byte aligned) reads its parameters once for both steps; any other layer runs the two
 * calls one after the other. */
int cnt_mdn_error_backward(cnt_mdn *h, void *stream, const float *targets, float *result_dev, float *prev_errors);
/* Device pointer to a unit's buffer. which: 0 parameters (softmax: F*K probabilities; mixture:
 * [F*M weights | F*M*D means | F*M*D std]), 1 mixture log-likelihoods [F*M | F].  *count receives the
 * number of floats in use for the current fraction. */
float *cnt_mdn_unit_buffer(cnt_mdn *h, int unit, int which, long *count);

/* ---- 1-D (dilated, optionally causal) convolution layer -------------------------------------------
 * CNNLayer<TDevice>, 1-D path (layers/CNNLayer.cu).  Filter d has half width half_width[d]
 * ("window_width", 2*hw+1 weight columns, the columns after the centre are dead when causal) and tap
 * interval interval[d] ("window_tap_interval").  weights = [P x Lw column-major | D bias] with
 * Lw = sum(2*hw+1): the layout the reference stores under "internal" (:971-978).  The 2-D
 * (window_height) path and repeat_padding are not built; at most 8 live taps per filter. */
typedef struct cnt_cnn cnt_cnn;
typedef struct {
    int P;            /* preceding layer size                   */
    int D;            /* number of filters = layer size         */
    int S;            /* parallel sequences                     */
    int maxT;         /* maxSeqLength                           */
    int causal;       /* "causal"                               */
    int output_tanh;  /* "tanhoutput" (default 1 in the reference, layers/CNNLayer.cu:932) */
    float bias;       /* the layer's constant bias input        */
} cnt_cnn_desc;
int cnt_cnn_create(const cnt_cnn_desc *desc, const int *half_width, const int *interval, cnt_cnn **out);
int cnt_cnn_destroy(cnt_cnn *h);
long cnt_cnn_weight_count(const cnt_cnn *h);
/* CNNLayer::computeForwardPass (layers/CNNLayer.cu:1099-1224): outputs (D x T*S); padding slots are left
 * untouched, as in the reference. */
int cnt_cnn_forward(cnt_cnn *h, void *stream, const char *patTypes, int curT, const float *weights,
                    const float *x, float *outputs);
/* CNNLayer::computeBackwardPass (layers/CNNLayer.cu:1409-1597): output_errors becomes tanh'(y)*err in
 * place when output_tanh is set; prev_errors is the preceding layer's whole error buffer
 * (P x maxT*S, cleared beyond the current slots, may be NULL); weight_updates is overwritten. */
int cnt_cnn_backward(cnt_cnn *h, void *stream, const char *patTypes, int curT, const float *weights,
                     const float *x, const float *outputs, float *output_errors, float *prev_errors,
                     float *weight_updates);

/* The two halves of cnt_cnn_backward for callers that put the weight gradients on another stream (the reference
 * has no such split): _errors = tanh derivative in place and prev_errors; _weights reads x and the finished
 * output_errors.  Calling both in this order on one stream (delta_applied = 0) is cnt_cnn_backward.
 * delta_applied != 0: output_errors already holds tanh'(y) * error (see cnt_wavnetc_backward_errors). */
int cnt_cnn_backward_errors(cnt_cnn *h, void *stream, const char *patTypes, int curT, const float *weights,
                            const float *outputs, float *output_errors, float *prev_errors, int delta_applied);
int cnt_cnn_backward_weights(cnt_cnn *h, void *stream, const char *patTypes, int curT, const float *x,
                             const float *output_errors, float *weight_updates);

/* ---- gated activation, conditioned ("wavnetc") and plain ("gatedact") ------------------------------
 * WavNetCore<TDevice> (layers/wavNetCore.cu) and GatedActLayer<TDevice> (layers/GatedActLayer.cu).
 * D = layer size, the preceding layer has 2D units; C = contextDim; N = T*S slots.
 * The caller owns the buffers the reference keeps as members: core_buf (m_coreBuf, 2D x N),
 * ctx_tanh (m_contextTanhBuf, 2D x N), ctx (the first core's m_contextBuf, C x N). */
/* loadLinguisticFeature (layers/wavNetCore.cu:143-190, driver :455-492): ctx[slot] = source frame
 * frame_index[slot] of the slot's sequence (or slot itself when resolution_one), optionally
 * (x - mean) / std with mean_std = [C means | C std]; 0 on padding slots. */
int cnt_wavnetc_load_context(void *stream, int C, int S, int N, int max_feature_length, int resolution_one,
                             const float *source, const float *frame_index, const float *mean_std,
                             const char *patTypes, float *ctx);
/* WavNetCore::computeForwardPass (layers/wavNetCore.cu:629-711). weights is C x 2D column-major.
 * ctx_tanh may be NULL outside training.  C == 0: unconditioned. */
int cnt_wavnetc_forward(void *stream, int D, int C, int N, const char *patTypes, const float *weights,
                        const float *ctx, const float *conv_outputs, float *core_buf, float *ctx_tanh,
                        float *outputs);
/* WavNetCore::computeBackwardPass (layers/wavNetCore.cu:801-916): prev_errors (2D x N) is overwritten;
 * ctx_tanh is overwritten with the gradient w.r.t. W^T ctx; weight_updates (C x 2D) is overwritten;
 * if ctx_grad (C x N, the first core's m_contextGraBuf) is given, W * gradient is added to it. */
int cnt_wavnetc_backward(void *stream, int D, int C, int N, const char *patTypes, const float *weights,
                         const float *ctx, const float *core_buf, float *ctx_tanh, const float *output_errors,
                         float *prev_errors, float *weight_updates, float *ctx_grad);
/* The two halves of cnt_wavnetc_backward (same split as above): _errors = prev_errors, the gradient left in
 * ctx_tanh and the optional context gradient; _weights = weight_updates from ctx and that gradient.
 * prev_tanh_outputs (may be NULL): the outputs of the preceding layer when that is a cnn layer with tanh output;
 * prev_errors then receives that layer's delta tanh'(y) * error right away, which saves the pass over the buffer
 * that cnt_cnn_backward_errors would make (call it with delta_applied = 1). */
int cnt_wavnetc_backward_errors(void *stream, int D, int C, int N, const char *patTypes, const float *weights,
                                const float *core_buf, float *ctx_tanh, const float *output_errors, float *prev_errors,
                                float *ctx_grad, const float *prev_tanh_outputs);
int cnt_wavnetc_backward_weights(void *stream, int D, int C, int N, const float *ctx, const float *ctx_tanh,
                                 float *weight_updates);
/* SumGradientsForExternalInput (layers/wavNetCore.cu:237-270, driver :895-913): frame_grad (C x
 * n_frame_slots) = sum of ctx_grad over the `resolution` samples of each frame. */
int cnt_wavnetc_sum_context_grad(void *stream, int C, int S, int resolution, int n_frame_slots, int N,
                                 const char *pat_frames, const char *patTypes, const float *ctx_grad,
                                 float *frame_grad);
/* GatedActLayer::computeForwardPass / computeBackwardPass (layers/GatedActLayer.cu:177-263). */
int cnt_gatedact_forward(void *stream, int D, int N, const char *patTypes, const float *pre, float *outputs);
int cnt_gatedact_backward(void *stream, int D, int N, const char *patTypes, const float *pre,
                          const float *output_errors, float *prev_errors);

/* ---- skip-add ---------------------------------------------------------------------------------------
 * SkipAddLayer<TDevice> (layers/SkipAddLayer.cu).  `inputs` / `targets` are HOST arrays of device
 * pointers (at most 8).  Forward (:186-240): outputs = sum of inputs, errors and errors_from_skip
 * (SkipLayer::outputErrorsFromSkipLayer) are cleared.  Backward (:305-346): errors += errors_from_skip;
 * predecessors in reverse order: a skip layer's errors_from_skip buffer (target_is_skip = 1) is added
 * to, any other layer's error buffer is overwritten. */
int cnt_skipadd_forward(void *stream, long count, int n_in, const float *const *inputs, float *outputs,
                        float *errors, float *errors_from_skip);
int cnt_skipadd_backward(void *stream, long count, float *errors, const float *errors_from_skip, int n_pre,
                         float *const *targets, const int *target_is_skip);

/* ---- DFT (multi-resolution STFT spectral) loss ------------------------------------------------------
 * DFTPostoutputLayer<TDevice> with helpers::FFTMat (layers/DFTErrorPostoutputLayer.cu, helpers/FFTMat.cu)
 * for the amplitude / spectrum distances specDisType 0..6 (helpers/FFTMat.hpp:29-35; distance functors
 * helpers/FFTMat.cu:473-628, gradients :760-900) and up to three resolutions ("fftLength/frameLength/frameShift" with suffix "", "2",
 * "3", layers/DFTErrorPostoutputLayer.cu:752-845).  The layer has size 1; a waveform occupies max_length
 * consecutive floats.  The reference handles one waveform per fraction; here n_waves waveforms with their
 * own lengths can be processed by one call (waveform w at offset w*max_length).  FFT lengths must be
 * powers of two in 32..4096. */
typedef struct cnt_dft cnt_dft;
typedef struct {
    int n_res;
    int fft_length[3], frame_length[3], frame_shift[3];
    int window_type[3];  /* 0 Hann (the reference's default), 1 square */
    float gamma;         /* "gamma": weight of the spectral amplitude loss            */
    float log_floor;     /* "logSpecAmpFloor", 1e-5 by default (helpers/FFTMat.hpp:53) */
    int spec_dis_type;   /* "specDisType": 0 log-amplitude MSE, 1 KLD, 2 amplitude MSE, 3 log
                            spectral MSE, 4 spectral MSE, 5 amplitude ratio, 6 Itakura-Saito  */
    int max_length;      /* maxSeqLength in samples                                   */
    int max_waves;       /* waveforms per call, 1..32                                 */
    float zeta;          /* "zeta": weight of the phase distance; 0 = none (the reference's default,
                            layers/DFTErrorPostoutputLayer.cu:324, :613)              */
    int phase_dis_type;  /* "phaseDisType"; 0 = cosine distance (helpers/FFTMat.cu:630-656, :862-878),
                            the only one built                                        */
} cnt_dft_desc;
int cnt_dft_create(const cnt_dft_desc *desc, cnt_dft **out);
int cnt_dft_destroy(cnt_dft *h);
/* DFTPostoutputLayer::computeForwardPass in training mode (layers/DFTErrorPostoutputLayer.cu:1782-1839,
 * :1186-1244): computes the loss of every waveform and resolution into errors_dev[w*n_res + r] (device
 * memory) AND the gradient w.r.t. the source samples, which is kept inside the handle, as the reference
 * keeps it in m_fftDiffData.  lengths is a host array.  Samples at or beyond a waveform's length count as 0.
 * With zeta > 0 (layers/DFTErrorPostoutputLayer.cu:1246-1295, :1672) errors_dev holds 2*n_waves*n_res floats:
 * the phase distances follow at errors_dev[n_waves*n_res + w*n_res + r], and the kept gradient is
 * gamma * amplitude part + zeta * phase part. */
int cnt_dft_forward(cnt_dft *h, void *stream, int n_waves, const int *lengths, const float *source,
                    const float *target, float *errors_dev);
/* DFTPostoutputLayer::computeBackwardPass (layers/DFTErrorPostoutputLayer.cu:1849-1885, :1699-1714):
 * prev_errors (n_waves x max_length) = sum over resolutions of the stored gradients, 0 beyond each length. */
int cnt_dft_backward(cnt_dft *h, void *stream, float *prev_errors);

/* ---- network sequencer ------------------------------------------------------------------------------
 * NeuralNetwork<TDevice> for the layer types of this library (NeuralNetwork.cpp): "input", "feedforward_identity /
 * _tanh / _logistic / _relu", "lstm", "blstm", "skipini", "skipadd" (with "preSkipLayer"), "cnn" (1-D), "wavnetc",
 * "gatedact", "feedback" (one step back, fed by one softmax unit), "skipcat" (with "preSkipLayerDim"),
 * "externalloader" and the post-output layers "sse", "mdn" and "dft" (keys fftLength / frameLength / frameShift /
 * windowType with suffix "", "2", "3", beta, gamma, zeta, specDisType, phaseDisType, logSpecAmpFloor; one waveform per
 * fraction, i.e. parallel_sequences = 1); layers may run at a lower time "resolution" (layers/Layer.cu:254-305), and a
 * layer flagged "wavenetConditionInputLayer" feeds the wavnetc layers (NeuralNetwork.cpp:544-561).  json_text is the
 * text of a network file: "layers" in order, optionally "weights" with the "input" / "bias" / "internal" arrays of
 * every trainable layer (layers/TrainableLayer.cu:135-220).  Without "weights" the weights are zero until the caller
 * fills them (cnt_network_weights, cnt_network_randomize).  All weights of the network, and all weight updates, are
 * one device array each, layers in file order, each layer's vector in the layout of its own entry points above. */
typedef struct cnt_network cnt_network;
typedef struct {
    const float *mdn_config; /* content of the --mdn_config file (see cnt_mdn_create); NULL without an mdn layer */
    int mdn_config_len;
    int tie_variance;        /* --tieVariance; only 0 is supported                                               */
    int no_overlap;          /* != 0: weight gradients on the caller's stream instead of streams of the network's */
} cnt_network_options;
typedef struct {
    char name[64];
    char type[32];
    int size;
    long weight_offset;              /* of this layer inside the network's weight array            */
    long n_input, n_bias, n_internal; /* lengths of the three sections of its weight vector         */
    float *outputs;                  /* device, size x (maxSeqLength*S); a post-output layer keeps the targets here */
    float *output_errors;            /* device, same shape; NULL for the input and post-output layers */
    int resolution;                  /* "resolution": the layer has one slot per so many time steps; its buffers hold
                                        size x (ceil(maxSeqLength / resolution) * S) floats                      */
} cnt_layer_info;
/* NeuralNetwork::NeuralNetwork (NeuralNetwork.cpp:374-609, :805-812).  options may be NULL. */
int cnt_network_create(const char *json_text, int parallel_sequences, int max_seq_length,
                       const cnt_network_options *options, cnt_network **out);
int cnt_network_destroy(cnt_network *net);
int cnt_network_info(cnt_network *net, int *n_layers, int *input_size, int *output_size, long *n_weights);
int cnt_network_layer_info(cnt_network *net, int index, cnt_layer_info *info);
float *cnt_network_weights(cnt_network *net);        /* device, n_weights floats */
float *cnt_network_weight_updates(cnt_network *net); /* device, n_weights floats */
/* Uniform weights in (-range, range) from a seeded Mersenne twister (the reference draws from its own generator,
 * layers/TrainableLayer.cu:221-300; the streams differ). */
int cnt_network_randomize(cnt_network *net, unsigned seed, float range);
/* Conditioning features of the wavnetc layers, contextDim x (maxSeqLength*S) in device memory, one column per
 * slot (what the reference's first wavnetc layer builds in m_contextBuf from the layer flagged
 * "wavenetConditionInputLayer", layers/wavNetCore.cu:455-492; cnt_wavnetc_load_context does that step).  The
 * pointer is kept, not the data. */
int cnt_network_set_context(cnt_network *net, const float *ctx);
/* External data of an "externalloader" layer (layers/ExternalLoader.cu:58-110, :205-250; the reference reads the
 * fraction's files there): data is [frame][sequence][dimension] in device memory with max_frames frames per
 * sequence; slot (t', s) of the layer takes the frame whose index the network's input layer (size 1) holds at time
 * step t' * resolution.  mean_std = [size means | size standard deviations] ("externalDataMV") or NULL.  The
 * pointers are kept, not the data. */
int cnt_network_set_external_input(cnt_network *net, int layer_index, const float *data, int max_frames,
                                   const float *mean_std);
/* NeuralNetwork::loadSequences (NeuralNetwork.cpp:1367-1417): records the fraction's geometry and pattern types
 * (device memory, char[T*S], kept by pointer), copies inputs (input size x T*S) and targets (post-output size x T*S)
 * when given, and passes the call on to the layers that keep per-fraction state.  When Tmin < T (some sequence is
 * shorter than the fraction) it also lists the fraction's valid slots from the pattern types, on the stream: the
 * weight gradients of the dense and recurrent layers then sum over those slots only, which changes no result (every
 * layer's deltas are zero on padding slots).  The pattern types are therefore read at this call as well as during the
 * passes: change them only through another cnt_network_load_sequences. */
int cnt_network_load_sequences(cnt_network *net, void *stream, int T, int Tmin, const char *patTypes,
                               const float *inputs, const float *targets);
/* NeuralNetwork::computeForwardPass in training mode (NeuralNetwork.cpp:1419-1471, :1734-1760). */
int cnt_network_forward(cnt_network *net, void *stream);
/* NeuralNetwork::calculateError (NeuralNetwork.cpp:2897-2990): the post-output layer's error into *loss_dev. */
int cnt_network_calculate_error(cnt_network *net, void *stream, float *loss_dev);
/* NeuralNetwork::computeBackwardPass (NeuralNetwork.cpp:2744-2800, :2864-2895): layers in reverse order.  The
 * layers' weight gradients run on streams of the network's own (same priority as any other stream), ordered after
 * the error computations they depend on; small layers of one shape share a launch.  On return the caller's stream
 * has been made to wait for those streams, so weight updates are complete in stream order. */
int cnt_network_backward(cnt_network *net, void *stream);
/* cnt_lstm_check for every LSTM layer (all of them are looked at; the first failure is returned).  Failure contract
 * of the network: a pass in which a recursion gave up cannot reach the weights -- the failed launch sets a device
 * flag that the optimizer kernel of cnt_network_update reads, so even an update that was enqueued before the host
 * could see the failure leaves weights and optimizer state (momentum, statistics, Adam's bias-correction products,
 * which live in device memory for that reason) untouched -- and CNT_ERR_DEVICE is returned by this call or by the next
 * cnt_network_load_sequences / _forward / _backward / _update after the failed launch has ended (the library records
 * an event behind every recursion launch and reports nothing before that event has passed).  The report clears the
 * flag in the order of the stream it is made on, so the calls of a pass belong on one stream, of any kind. */
int cnt_network_check(cnt_network *net, void *stream);
/* cnt_lstm_set_wait_bounds for the LSTM layer at `layer_index` of the network (CNT_ERR_ARG for any other layer).  No
 * counterpart in the reference; like that call it exists so that a test can force one layer's recursion to give up
 * without any kernel hanging. */
int cnt_network_set_wait_bounds(cnt_network *net, int layer_index, unsigned spin_limit, int poll_delay_backward,
                                int poll_delay_forward);
/* One optimizer step over all weights in a single launch (see cnt_opt_step; the network keeps the optimizer's
 * current updates, deltas, statistics and Adam's accumulated betas).  If a layer of the network file carries its
 * own "learningRate" (layers/TrainableLayer.cu:110-111), the step is one launch per trainable layer instead. */
int cnt_network_update(cnt_network *net, void *stream, int option, float learning_rate, float momentum,
                       float frac_length);
/* NeuralNetwork::exportLayers + exportWeights (NeuralNetwork.cpp:2993-3040): the layer objects as they stood in the
 * network file plus the current weights.  *needed receives the size including the terminating 0; nothing is
 * written if cap is smaller (call once with buf = NULL to learn the size). */
int cnt_network_export_json(cnt_network *net, char *buf, size_t cap, size_t *needed);

/* ---- weight update of the training loop (optimizer step on device) ------------------------------------
 * optimizer option numbers are the reference's (MacroDefine.hpp:33-37): 0 plain SGD, 1 AdaGrad,
 * 2 gradient averaged over the fraction, 3 stochastic AdaGrad (statistics only), 4 SGD with decaying
 * learning rate (the decay is host logic; treated as 0 here), 5 Adam.  `stats` holds one float per weight
 * for AdaGrad (the reference initialises it to 1e-6, optimizers/Optimizer.cu:427-433) and interleaved
 * (m, v) pairs for Adam (zero-initialised, :443-447).  `mask` is the optional weight mask (NULL = none).
 *
 * cnt_opt_accumulate: per-fraction copy (add = 0) or accumulation (add != 0) of a layer's weightUpdates()
 * into the optimizer's current weight updates (optimizers/Optimizer.cu:186-198). */
int cnt_opt_accumulate(void *stream, long n, const float *layer_updates, float *cur_updates, int add);
/* The gradient adjustment SteepestDescentOptimizer::_updateWeights applies before the update
 * (optimizers/SteepestDescentOptimizer.cu:312-405; functors :119-203).  frac_length is the fraction's
 * fracTimeLength(); beta?_accum are m_adamBeta?Accum AFTER this call's multiplication by beta
 * (cnt_opt_next_beta_accum reproduces that float-times-double product, :345-349). */
int cnt_opt_adjust_gradient(void *stream, int option, long n, float *cur_updates, float *stats, const float *mask,
                            float frac_length, float beta1_accum, float beta2_accum);
/* UpdateWeightFn / UpdateWeightFn_withMask (optimizers/SteepestDescentOptimizer.cu:41-98, :408-436):
 * NaN / Inf gradients are zeroed in place, delta = momentum*delta - lr*g, w = (w + delta) [* mask].
 * A negative learning rate skips the update, as the reference does (:283-285). */
int cnt_opt_update_weights(void *stream, long n, float *weights, float *cur_updates, float *weight_deltas,
                           const float *mask, float learning_rate, float momentum);
/* The three calls above (copy, adjust, update) for one layer in a single pass over its weights; same
 * results, a third of the memory traffic.  For the hybrid online/batch mode, where the reference updates
 * after every fraction (optimizers/Optimizer.cu:229-231). */
int cnt_opt_step(void *stream, int option, long n, float *weights, const float *layer_updates, float *cur_updates,
                 float *stats, float *weight_deltas, const float *mask, float frac_length, float beta1_accum,
                 float beta2_accum, float learning_rate, float momentum);
float cnt_opt_next_beta_accum(float accum, int which);

/* ---- the .nc data path (NetCDF reader and fraction builder; host memory only) ------------------------
 * data_sets::DataSet's constructor for ONE .nc file (data_sets/DataSet.cpp:1376-1907): reads the
 * dimensions and seqLengths / seqTags, keeps the first max(1, int(numSeqs * fraction)) sequences, cuts a
 * sequence longer than 1.5 * truncate_seq into segments of truncate_seq (0 = off), and in training mode
 * sorts the segments by ascending length (stable here; the reference's std::sort leaves ties unspecified).
 * Classic (CDF-1) and 64-bit-offset (CDF-2) files are read without libnetcdf. */
typedef struct cnt_dataset cnt_dataset;
typedef struct {
    int parallel_sequences; /* S: sequences per fraction                         */
    int training_mode;      /* != 0: sort by length (Configuration::trainingMode) */
    int truncate_seq;       /* --truncate_seq, 0 = off                             */
    float fraction;         /* --train_fraction etc., in (0, 1]                    */
} cnt_dataset_desc;
int cnt_dataset_open(const char *nc_path, const cnt_dataset_desc *desc, cnt_dataset **out);
int cnt_dataset_close(cnt_dataset *d);
/* DataSet::_shuffleSequences and _shuffleFractions (data_sets/DataSet.cpp:491-514), which the reference runs at the
 * start of every epoch when --shuffle_sequences / --shuffle_fractions are set (:1026-1031): the order of the
 * sequences is permuted, then the order of the groups of parallel_sequences consecutive sequences.  One generator
 * per data set, seeded by the first call (--random_seed); the permutations are seeded and repeatable but not the
 * reference's own, whose draws come from boost's generators. */
int cnt_dataset_shuffle(cnt_dataset *d, int shuffle_sequences, int shuffle_fractions, unsigned seed);
/* DataSet::totalSequences / inputPatternSize / outputPatternSize / isClassificationData / totalTimesteps /
 * minSeqLength / maxSeqLength (data_sets/DataSet.hpp); any pointer may be NULL. */
int cnt_dataset_info(cnt_dataset *d, int *num_sequences, int *input_size, int *output_size, int *is_classification,
                     long *total_timesteps, int *min_len, int *max_len);
/* one entry of the (sorted) segment list: length, index of the segment inside its utterance, tag */
int cnt_dataset_sequence(cnt_dataset *d, int index, int *length, int *original_seq_idx, char *tag, int tag_cap);
/* DataSet::_makeFractionTask(firstSeqIdx) (data_sets/DataSet.cpp:642-1022) in two steps.  _shape gives
 * numSequences, maxSeqLength, minSeqLength and fracTimeLength of the fraction that starts at first_seq;
 * _fill writes, into host buffers the caller sized from it, patTypes[maxLen*S] (0 none, 1 first, 2 normal,
 * 3 last), inputs[maxLen*S*inputSize] and targets[maxLen*S*outputSize] (regression) or
 * target_classes[maxLen*S] (classification, -1 on padding): slot t*S+i holds time step t of the i-th
 * sequence, padding slots are zero. */
int cnt_dataset_fraction_shape(cnt_dataset *d, int first_seq, int *num_seqs, int *max_len, int *min_len,
                               int *total_length);
int cnt_dataset_fraction_fill(cnt_dataset *d, int first_seq, char *patTypes, float *inputs, float *targets,
                              int *target_classes);

#ifdef __cplusplus
}
#endif
#endif
