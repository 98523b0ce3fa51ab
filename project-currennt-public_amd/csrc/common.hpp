// Shared declarations of the gfx950 backward-pass library: error plumbing, scalar device
// functions with the reference's exact clamping rules, and the internal kernel launch API.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "../../include/currennt_hip.h"

namespace cnt {

// ----- error plumbing: nothing throws across the C ABI ------------------------------------------
void set_error(const char *fmt, ...);
const char *last_error();

#define CNT_HIP(expr)                                                                        \
    do {                                                                                     \
        hipError_t _e = (expr);                                                              \
        if (_e != hipSuccess) {                                                              \
            ::cnt::set_error("%s failed: %s (%s:%d)", #expr, hipGetErrorString(_e), __FILE__, \
                             __LINE__);                                                      \
            return CNT_ERR_HIP;                                                              \
        }                                                                                    \
    } while (0)

#define CNT_REQUIRE(cond, ...)           \
    do {                                 \
        if (!(cond)) {                   \
            ::cnt::set_error(__VA_ARGS__); \
            return CNT_ERR_ARG;          \
        }                                \
    } while (0)

#define CNT_TRY(expr)            \
    do {                         \
        int _s = (expr);         \
        if (_s != CNT_OK) return _s; \
    } while (0)

// ----- scalar semantics ---------------------------------------------------------------------------
// Reference: activation_functions/{Logistic,Maxmin1,Tanh}.cuh, helpers/{limitedError,safeExp,
// NumericLimits}.cuh.  tanh is 2*logistic(2x)-1 and the logistic saturates outside +-88.722839.
namespace lim {
constexpr float kMin = 1.1754944e-038f;
constexpr float kMax = 3.4028235e+038f;
constexpr float kExpLimit = 88.722839f;
constexpr float kLogZero = -1e30f;
constexpr float kLSmall = -0.5e10f;
constexpr float kMinLarg = 1.1754944e-038f;
constexpr float kMinLogExp = -69.0776f;
}  // namespace lim

__device__ __forceinline__ float logistic(float x) {
    if (x < lim::kExpLimit) {
        if (x > -lim::kExpLimit) return 1.0f / (1.0f + expf(-x));
        return 0.0f;
    }
    return 1.0f;
}
// The same functions from the hardware's exp2 and reciprocal (the library routines above spend about twenty instructions
// on denormal results and on an exactly rounded quotient), for the forward recursion, where the five of them per cell
// and time step sit on the critical path of every step.  Not bit-identical to the functions above: exp2 and rcp are
// good to 1 ulp each, but the argument -1.4427 * x is rounded to fp32 before the exponential, which alone is a
// relative error of |x| * 6e-8 in exp(-x).  The result stays within 4e-6 absolute of the exact logistic function
// (8e-6 for tanh) over the whole unclamped range, which tests/test_gpu_core.py checks against the CPU functions.
__device__ __forceinline__ float logistic_quick(float x) {
    if (x < lim::kExpLimit) {
        if (x > -lim::kExpLimit) return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504088896341f * x));
        return 0.0f;
    }
    return 1.0f;
}
__device__ __forceinline__ float tanh_quick(float x) { return 2.0f * logistic_quick(2.0f * x) - 1.0f; }
__device__ __forceinline__ float logistic_deriv(float y) { return y * (1.0f - y); }
__device__ __forceinline__ float tanh_act(float x) { return 2.0f * logistic(2.0f * x) - 1.0f; }
__device__ __forceinline__ float tanh_deriv(float y) { return 1.0f - y * y; }
__device__ __forceinline__ float clip1(float e) { return e < -1.0f ? -1.0f : (e > 1.0f ? 1.0f : e); }
__device__ __forceinline__ float safe_exp(float x) {
    if (x <= lim::kLogZero) return 0.0f;
    if (x >= lim::kExpLimit) return lim::kMax;
    return expf(x);
}
__device__ __forceinline__ float safe_log(float x) { return x < lim::kMinLarg ? lim::kLogZero : logf(x); }
__device__ __forceinline__ float log_add(float x, float y) {
    const float hi = x > y ? x : y;
    const float lo = x > y ? y : x;
    if ((lo - hi) < lim::kMinLogExp) return hi < lim::kLSmall ? lim::kLogZero : hi;
    return (float)((double)hi + log(1.0 + (double)expf(lo - hi)));
}

enum Act { ACT_IDENTITY = 0, ACT_TANH = 1, ACT_LOGISTIC = 2, ACT_RELU = 3 };
__device__ __forceinline__ float act_fn(int act, float a) {
    switch (act) {
        case ACT_TANH: return tanh_act(a);
        case ACT_LOGISTIC: return logistic(a);
        case ACT_RELU: return a > 0.0f ? a : 0.0f;
        default: return a;
    }
}
__device__ __forceinline__ float act_deriv(int act, float y) {
    switch (act) {
        case ACT_TANH: return tanh_deriv(y);
        case ACT_LOGISTIC: return logistic_deriv(y);
        case ACT_RELU: return y > 0.0f ? 1.0f : 0.0f;
        default: return 1.0f;
    }
}

// ----- optional per-kernel timing (capi.hip) -------------------------------------------------------
// When enabled through cnt_profile_enable, every ProfileScope brackets the launches made inside it
// with a pair of HIP events on the launch stream; cnt_profile_get sums them per label.
struct ProfileScope {
    ProfileScope(hipStream_t stream, const char *label);
    ~ProfileScope();
    hipStream_t stream_;
    int slot_;
};

// ----- GEMM (gemm.hip) ------------------------------------------------------------------------------
// C (m x n, column-major, ldc) = sum over segments of opA(A_i) * opB(B_i), optionally added to C.
// An operand is described by where element (row, kk) lives: row-contiguous (ptr[kk*ld + row]) or
// k-contiguous (ptr[row*ld + kk]).
constexpr int kGemmMaxSeg = 8;
constexpr int kGemmMaxProb = 8;

enum GemmEpilogue {
    EPI_STORE = 0,          // C = acc
    EPI_ADD = 1,            // C += acc
    EPI_ATOMIC = 2,         // atomicAdd(C, acc)   (split-K; C zeroed by the caller)
    EPI_BIAS_ACT = 3,       // C = act(acc + bias_scale * bias_vec[row])
    EPI_BIAS_ACT_SKIP = 4,  // as above, but columns whose pattern type is "none" are left untouched
    EPI_CONTEXT = 5,        // th = tanh(acc); aux_out = th; C = aux_in + th; both 0 on "none" columns
    EPI_PARTIAL = 6,        // split-K without atomics: every split stores its m x n partial product into the
                            // launcher's scratch, and a second kernel sums the splits into C (set by gemm_plan)
    EPI_STORE_DELTA = 8,    // C = acc * act'(aux_in): the product that writes a dense layer's output errors turns them
                            // into that layer's deltas on the way out (aux_in = the layer's outputs, layout of C)
    EPI_FAN = 7             // a skip layer's backward step in the epilogue of the product that writes the layer's
                            // errors: e = aux_in + acc (aux_in may be NULL), C = e, and e goes on to fan_n buffers of
                            // C's layout -- added to those flagged in fan_is_skip, stored over the others
};

struct GemmProblem {
    const float *A[kGemmMaxSeg];
    const float *B[kGemmMaxSeg];
    int b_shift[kGemmMaxSeg];  // masked mode: time-slot shift of the B operand per operand pair
    float *C;
    const float *bias_vec;
    const float *aux_in;  // EPI_CONTEXT, EPI_STORE_DELTA: same layout as C
    float *aux_out;       // EPI_CONTEXT, may be NULL
    float *rowsum_out;    // GemmArgs::rowsum: receives rowsum_scale * sum_k B(j, k), j < n
    float rowsum_scale;
    int k_trim;           // GemmArgs::k_order: 0 all listed k lines, 1 without those of the first time step, 2 without the last one's
    int k_shift;          // GemmArgs::k_order: added to every listed line (an operand pair that starts at a later slot)
};

// The slots of a fraction in the order "valid ones first, ascending; then the padding slots, ascending" (device
// memory: n_slots indices and three counts), made from the pattern types by slot_order_build.  The errors
// and deltas of every layer are zero on padding slots, so a sum over the slots may skip them.
struct SlotOrder {
    const int *order;
    const int *count;  // [0] valid slots, [1] those of the first time step, [2] those of the last time step
};
int slot_order_build(hipStream_t stream, const char *pat, int n_slots, int slots_per_step, int *order, int *count);

// Masked mode (dilated convolutions without a materialised column buffer): one index of the B operand is a
// time slot u -- its row index (b_time_on_k = 0) or its k index (b_time_on_k = 1).  The element is read from
// slot u + b_shift and counts only if pat[u] != 0, 0 <= u + b_shift < n_slots and pat[u + b_shift] != 0;
// otherwise it is 0.  This is exactly the set of entries the reference scatters into its column buffer
// (layers/CNNLayer.cu:182-237).
struct GemmArgs {
    int m, n, k;
    int lda, ldb, ldc;
    int a_kcontig, b_kcontig;  // 1: element (row,kk) at ptr[row*ld+kk]; 0: ptr[kk*ld+row]
    int nseg, nprob, splitk;
    int epilogue, act;
    float bias_scale;
    int masked, b_time_on_k, n_slots;
    const char *pat;  // masked mode and the *_SKIP / CONTEXT epilogues
    GemmProblem prob[kGemmMaxProb];
    const char *label;  // name under which the launch is timed when profiling is on (may be NULL)
    // Split-K products with a small output (EPI_ATOMIC, splitk = 0): `overwrite_ok` allows gemm_plan to choose
    // EPI_PARTIAL, which overwrites C instead of adding to a cleared C.  With `rowsum` (one operand pair, unmasked)
    // the same pass also sums every problem's B operand over k into that problem's rowsum_out -- the bias gradient
    // of a dense layer, for which the atomic path needs a separate column-sum launch.  gemm_plan clears `rowsum`
    // where it does not choose EPI_PARTIAL.
    int overwrite_ok;
    int rowsum;
    int fan_n;                   // EPI_FAN: device tables of fan_n targets and their flags
    float *const *fan_targets;
    const int *fan_is_skip;
    float *partial;        // scratch of splitk * partial_stride floats: the stream's buffer (set by gemm_plan) or the caller's
    size_t partial_stride;  // floats per split: nprob * m * n (+ nprob * n with rowsum)
    int xcd_map;            // set by gemm_launch: workgroups pick their tile by XCD (gemm_kernel.hpp)
    // A product over the slots of a fraction (weight gradients) that leaves the padding slots out (both in device memory,
    // or both NULL): only the k lines k_order[lo .. lo + n) of the operands are read, the others being all zero in at least
    // one operand.  k_count[0] = number of listed lines; with GemmProblem::k_trim = 1 the problem leaves out the first
    // k_count[1] of them (the lines of the first time step), with 2 the last k_count[2] (those of the last time step).  The
    // launcher uses the list where both operands are row-contiguous and 16-byte aligned and the tile is 64 x 64, and
    // multiplies all k lines otherwise -- so the operands' base pointers must be valid for both readings.
    const int *k_order;
    const int *k_count;
};

// Resolves splitk = 0 (chosen by the launcher) and, where the arguments allow it and it pays, switches an
// EPI_ATOMIC product to EPI_PARTIAL.  A caller that needs to know whether C must be cleared first calls this
// before gemm_launch and looks at args.epilogue; gemm_launch calls it for everyone else.
void gemm_plan(GemmArgs &args, hipStream_t stream);
// whether a product with these operands can take the EPI_FAN epilogue (operand kinds, alignment)
bool gemm_fan_supported(const GemmArgs &args);
int gemm_launch(hipStream_t stream, const GemmArgs &args);
// Frees the split-K scratch buffer that the launcher keeps for `stream` (for owners of a stream about to destroy
// it; the stream must be idle).  Buffers of streams never released stay until the process ends.
void gemm_release_stream(hipStream_t stream);
// Allocates the split-K scratch buffer of `stream` now instead of inside the first product that wants it.
int gemm_reserve_stream(hipStream_t stream);
// number of split-K scratch buffers the library holds at the moment (one per stream that has needed or reserved one)
int gemm_scratch_buffers();
// cnt_dense_backward_weights with the partial products in a scratch array that is part of the code object
int gemm_dense_weights_static(hipStream_t stream, int P, int D, int N, float bias, const float *x, const float *err,
                              float *weight_updates);

// Convenience: single problem, BLAS-like transposes on column-major matrices.
int gemm_simple(hipStream_t stream, float *C, int m, int n, int k, const float *A, bool transA,
                const float *B, bool transB, bool accumulate);

// cnt_opt_step with a device flag in front of it: when *veto is non-zero at the time the kernel runs (a recursion of
// the pass that produced the gradients gave up), the step changes nothing.
int opt_step_guarded(hipStream_t stream, int option, long n, float *weights, const float *layer_updates, float *cur_updates,
                     float *stats, float *weight_deltas, const float *mask, float frac_length, float beta1_accum,
                     float beta2_accum, float learning_rate, float momentum, const int *veto, const float *accum_dev);
// Adam's bias-correction products (two floats in device memory, both 1 before the first step) advanced by one step,
// unless *veto is non-zero; opt_step_guarded reads them in place of its two float arguments when accum_dev is given.
int opt_adam_advance(hipStream_t stream, float *accum_dev, const int *veto);
// LSTM handles of a network share one such flag: a recursion that gives up also sets *veto (until the owner clears it).
void lstm_set_veto(cnt_lstm *h, int *veto);
// non-zero if a recursion of this handle has given up since the last report (no synchronisation: it only sees
// launches that have already ended); the report clears the mark
// cnt_lstm_backward_weights in two parts that write disjoint ranges (1: input weights, 2: the rest)
int lstm_backward_weights_parts(cnt_lstm *h, hipStream_t stream, const float *x, float *weight_updates, int parts);
int lstm_take_failure(cnt_lstm *h);
// makes `other` wait for the recursion launched last on this handle's device (the event the library records behind
// every recursion launch anyway): what a stream needs that consumes the recursion's results, without another event
// record on the launching stream
int lstm_wait_recursion(cnt_lstm *h, hipStream_t other);
int lstm_is_persistent(const cnt_lstm *h);  // its recursions are single launches (not the step-by-step schedule)
int report_failure(cnt_network *net, hipStream_t stream);

// ----- error halves that also do the backward step of the skip layer in front of them ----------------
// A skip layer adds what its linkers left in its side buffer to the errors its following layer wrote, and hands the
// sum on (layers/SkipAddLayer.cu:305-346).  When that following layer is a dense or convolution layer, the sum and
// the hand-over happen in the epilogue of the product that computes those errors, instead of in a launch of their
// own.  `targets` / `is_skip` are device tables of `n` entries; `from_skip` is the side buffer or NULL.
struct FanOut {
    int n;
    float *const *targets;
    const int *is_skip;
    const float *from_skip;
};
// *fused tells whether the step was done (operands that the fan epilogue does not exist for, or a convolution
// with several filter groups, leave it to the caller).
int dense_backward_errors_fan(hipStream_t stream, int P, int D, int N, int act, const float *weights, const float *y,
                              float *err, float *prev_err, const FanOut *fan, bool *fused, int prev_act = ACT_IDENTITY,
                              const float *prev_y = nullptr);
// (prev_act, prev_y): the preceding layer is a dense layer with that activation and those outputs, and nothing but
// this product writes its output errors: the product stores act'(prev_y) * error, the preceding layer's deltas, and
// that layer's own backward step then runs with ACT_IDENTITY.  The same for a recurrent layer's error product:
int lstm_prev_errors_delta(cnt_lstm *h, hipStream_t stream, const float *weights, float *prev_errors, int prev_act,
                           const float *prev_y);
// The slots of the fraction a recurrent layer has loaded, valid ones first (nullptr: none known); the layer's weight
// gradients then skip the padding slots.  cnt_lstm_load_sequences forgets it.
void lstm_set_slot_order(cnt_lstm *h, const SlotOrder *order);
// Error path of one WaveNet residual block in one launch (skip 1x1 layer, the skip layer in front of it, the 1x1
// layer behind the gated unit, the gated unit): see wavenet_block_errors_kernel.
bool wavenet_block_errors_supported(int R, int K);
// `fold` (optional): the convolution layer above the block, whose error product (two live taps) is added to the
// block's summed errors inside the same launch instead of being written to the closing skip layer first
bool cnn_foldable(const cnt_cnn *h, int R);
int wavenet_block_errors(hipStream_t stream, int R, int K, int N, const char *patTypes, const float *skip_weights,
                         const float *out_weights, const float *skip_errors, float *total, const FanOut *fan,
                         const float *core_buf, float *ctx_tanh, const float *conv_tanh_outputs, float *conv_errors,
                         const cnt_cnn *fold, const float *fold_weights, const float *fold_deltas, float *colsum_partial);
// workgroups of that launch = rows of `colsum_partial` ([rows][2R]: per-workgroup sums of conv_errors over the samples)
int wavenet_block_rows(int N, bool fold);
int wavnetc_context_grad(hipStream_t stream, int D, int C, int N, const float *weights, const float *ctx_tanh,
                         float *ctx_grad);
int cnn_backward_errors_fan(cnt_cnn *h, hipStream_t stream, const char *patTypes, int curT, const float *weights,
                            const float *outputs, float *output_errors, float *prev_errors, int delta_applied,
                            const FanOut *fan, bool *fused);

// ----- weight-gradient halves of several layers of one shape in one launch --------------------------
// For the network sequencer: `count` (<= kGemmMaxProb) dense layers with the same P, D, N, or wavnetc layers with the
// same D, C, N and one context buffer, as the problems of one product.  Same results as `count` calls of
// cnt_dense_backward_weights / cnt_wavnetc_backward_weights.
int dense_backward_weights_batch(hipStream_t stream, int P, int D, int N, int count, const float *bias,
                                 const float *const *x, const float *const *err, float *const *weight_updates, const SlotOrder *order = nullptr);
int wavnetc_backward_weights_batch(hipStream_t stream, int D, int C, int N, int count, const float *ctx,
                                   const float *const *ctx_tanh, float *const *weight_updates);
// Convolution layers with one filter group each and the same sizes, window and causality (dilations may differ):
// cnn_batch_taps gives the live taps of such a layer (0: not batchable, several filter groups), and `count` layers
// with count * taps <= kGemmMaxProb go into one product.
int cnn_batch_taps(const cnt_cnn *h);
bool cnn_batch_compatible(const cnt_cnn *a, const cnt_cnn *b);
int cnn_backward_weights_batch(cnt_cnn *const *h, int count, hipStream_t stream, const char *patTypes, int curT,
                               const float *const *x, const float *const *output_errors, float *const *weight_updates,
                               const float *const *colsum_partial = nullptr, const int *colsum_rows = nullptr);

// ----- small streaming kernels (elementwise.hip) ----------------------------------------------------
int fill_zero(hipStream_t stream, float *p, size_t count);
// two buffers in one launch
int fill_zero_pair(hipStream_t stream, float *p, size_t count, float *q, size_t count_q);
// What a network does on the device when a fraction is loaded, as ONE launch: up to kLoadClears buffers zeroed (the
// recurrent layers' stored output-gate deltas) and, when `order` is given, the fraction's slot order built (as
// slot_order_build does).
constexpr int kLoadClears = 8;
struct LoadClears {
    float *ptr[kLoadClears];
    unsigned long long count[kLoadClears];  // floats, multiples of four, 16-byte aligned buffers
    int n;
};
int load_clear_and_order(hipStream_t stream, const LoadClears &clears, const char *pat, int n_slots, int slots_per_step,
                         int *order, int *count);
// cnt_lstm_load_sequences without the clearing launch: the caller clears what `clears` lists afterwards (false: the list
// is full or a buffer does not qualify, and the handle has launched its own clear)
int lstm_load_sequences_collect(cnt_lstm *h, hipStream_t stream, const char *patTypes, int curMaxT, int curMinT,
                                LoadClears &clears);
int fill_words(hipStream_t stream, unsigned *p, size_t count, unsigned word);
// out[d] += scale * sum over the N columns of a D x N column-major matrix (out pre-zeroed by the caller)
int column_sum(hipStream_t stream, const float *v, int D, int N, float scale, float *out);

}  // namespace cnt
