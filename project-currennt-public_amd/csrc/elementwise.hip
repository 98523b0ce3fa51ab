// Streaming kernels of the dense and SSE layers plus small utilities.
//
// Reference behaviour: layers/FeedForwardLayer.cu (:105-138 functors, :1633-1738 backward driver,
// :1060-1101 forward) and layers/SsePostOutputLayer.cu (:94-136, :166-267).
#include "common.hpp"

#include <algorithm>

namespace cnt {
namespace {

// the first n4 groups of four floats as 16-byte stores (n4 = 0 for a buffer that is not 16-byte aligned), the rest
// one by one
__global__ void fill_zero_kernel(float *__restrict__ p, size_t count, size_t n4) {
    const size_t first = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = first; i < n4; i += stride) reinterpret_cast<float4 *>(p)[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    for (size_t i = 4 * n4 + first; i < count; i += stride) p[i] = 0.0f;
}

__global__ void fill_zero_pair_kernel(float *__restrict__ p, size_t count, float *__restrict__ q, size_t count_q) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < count + count_q; i += stride) {
        if (i < count) p[i] = 0.0f;
        else q[i - count] = 0.0f;
    }
}

__global__ void fill_words_kernel(unsigned *__restrict__ p, size_t count, unsigned word) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) p[i] = word;
}

// delta = act'(y) * err in place, on every slot (the reference does not mask padding here)
// (as above: n4 groups of four floats through 16-byte accesses, the rest one by one)
__global__ void dense_delta_kernel(float *__restrict__ err, const float *__restrict__ y, size_t count, int act, size_t n4) {
    const size_t first = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = first; i < n4; i += stride) {
        const float4 yv = reinterpret_cast<const float4 *>(y)[i];
        float4 e = reinterpret_cast<float4 *>(err)[i];
        e.x = act_deriv(act, yv.x) * e.x;
        e.y = act_deriv(act, yv.y) * e.y;
        e.z = act_deriv(act, yv.z) * e.z;
        e.w = act_deriv(act, yv.w) * e.w;
        reinterpret_cast<float4 *>(err)[i] = e;
    }
    for (size_t i = 4 * n4 + first; i < count; i += stride) err[i] = act_deriv(act, y[i]) * err[i];
}

// out[d] += scale * sum_i v[d + i*D]; out is zeroed by the caller.  A block is 64 rows x 4 column lanes (one
// wave per lane, 256-byte row segments); every lane strides over the columns with eight loads in flight, the
// four partial sums meet in LDS and leave as one atomic per row and block.  The number of blocks is kept near
// 512: atomics to one address serialise, and with thousands of blocks they, not the reads, set the run time.
__global__ __launch_bounds__(256) void column_sum_kernel(const float *__restrict__ v, int D, int N, float scale,
                                                         float *__restrict__ out) {
    __shared__ float part[4][64];
    const int tx = threadIdx.x, ty = threadIdx.y;
    const int d = blockIdx.x * 64 + tx;
    const int stride = 4 * gridDim.y;
    float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
    if (d < D) {
        int i = blockIdx.y * 4 + ty;
        for (; i + 7 * stride < N; i += 8 * stride) {
            float x[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) x[u] = v[(size_t)(i + u * stride) * D + d];
            a0 += scale * x[0]; a1 += scale * x[1]; a2 += scale * x[2]; a3 += scale * x[3];
            a0 += scale * x[4]; a1 += scale * x[5]; a2 += scale * x[6]; a3 += scale * x[7];
        }
        for (; i < N; i += stride) a0 += scale * v[(size_t)i * D + d];
    }
    part[ty][tx] = (a0 + a1) + (a2 + a3);
    __syncthreads();
    if (ty == 0 && d < D) atomicAdd(out + d, (part[0][tx] + part[1][tx]) + (part[2][tx] + part[3][tx]));
}

__global__ void sse_backward_kernel(int D, size_t count, const char *__restrict__ pat, const float *__restrict__ y,
                                    const float *__restrict__ tgt, float *__restrict__ err) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) err[i] = (pat[i / D] == 0) ? 0.0f : (y[i] - tgt[i]);
}

__global__ void sse_error_kernel(int D, size_t count, const char *__restrict__ pat, const float *__restrict__ y,
                                 const float *__restrict__ tgt, float *__restrict__ result) {
    __shared__ float part[4];
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    float acc = 0.0f;
    for (; i < count; i += stride) {
        if (pat[i / D] == 0) continue;
        const float diff = tgt[i] - y[i];
        acc += diff * diff;
    }
    for (int o = 32; o > 0; o >>= 1) acc += __shfl_down(acc, o);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = acc;
    __syncthreads();
    if (threadIdx.x == 0) atomicAdd(result, 0.5f * (part[0] + part[1] + part[2] + part[3]));
}

inline int stream_blocks(size_t count) {
    size_t b = (count + 255) / 256;
    if (b > 4096) b = 4096;
    if (b < 1) b = 1;
    return (int)b;
}

// One workgroup: every thread counts the valid slots of its contiguous share, the counts are scanned (inside a wave by
// shuffles, the waves' totals through LDS), and the thread then writes its valid slots from its offset among the valid
// ones and its padding slots from its offset among the padding ones, behind all valid ones.  The pattern types are read
// eight at a time, so that a thread waits for memory once per eight slots and not once per slot.
constexpr int kOrderThreads = 1024;
__device__ __forceinline__ void slot_order_block(const char *__restrict__ pat, int n, int per_step, int *__restrict__ order,
                                                 int *__restrict__ count) {
    __shared__ int wave_total[kOrderThreads / 64];
    __shared__ int edge_count[2];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int share = (n + kOrderThreads - 1) / kOrderThreads;
    const int lo = min(tid * share, n), hi = min(lo + share, n);
    if (tid < 2) edge_count[tid] = 0;
    __syncthreads();
    int valid = 0, in_first = 0, in_last = 0;
    for (int c = lo; c < hi; c += 8) {
        char v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = pat[min(c + j, n - 1)];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int i = c + j;
            const int is = i < hi && v[j] != 0;
            valid += is;
            in_first += is && i < per_step;
            in_last += is && i >= n - per_step;
        }
    }
    if (in_first) atomicAdd(&edge_count[0], in_first);
    if (in_last) atomicAdd(&edge_count[1], in_last);
    int incl = valid;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int v = __shfl_up(incl, d);
        if (lane >= d) incl += v;
    }
    if (lane == 63) wave_total[wave] = incl;
    __syncthreads();
    int before = 0, total = 0;
#pragma unroll
    for (int w = 0; w < kOrderThreads / 64; ++w) {
        if (w < wave) before += wave_total[w];
        total += wave_total[w];
    }
    int at_valid = before + incl - valid;      // valid slots before this thread's share
    int at_pad = total + (lo - at_valid);      // padding slots before it, behind all valid ones
    for (int c = lo; c < hi; c += 8) {
        char v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = pat[min(c + j, n - 1)];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int i = c + j;
            if (i >= hi) continue;
            if (v[j] != 0) order[at_valid++] = i;
            else order[at_pad++] = i;
        }
    }
    if (tid == 0) {
        count[0] = total;
        count[1] = edge_count[0];
        count[2] = edge_count[1];
    }
}

__global__ __launch_bounds__(kOrderThreads) void slot_order_kernel(const char *__restrict__ pat, int n, int per_step,
                                                                   int *__restrict__ order, int *__restrict__ count) {
    slot_order_block(pat, n, per_step, order, count);
}

// workgroup 0 builds the slot order (when there is one to build), the others zero the listed buffers with 16-byte stores
__global__ __launch_bounds__(kOrderThreads) void load_clear_and_order_kernel(const LoadClears c, const char *__restrict__ pat,
                                                                             int n, int per_step, int *__restrict__ order,
                                                                             int *__restrict__ count) {
    if (blockIdx.x == 0) {
        if (order) slot_order_block(pat, n, per_step, order, count);
        return;
    }
    const size_t first = (size_t)(blockIdx.x - 1) * kOrderThreads + threadIdx.x;
    const size_t stride = (size_t)(gridDim.x - 1) * kOrderThreads;
    for (int b = 0; b < c.n; ++b) {
        float4 *p = reinterpret_cast<float4 *>(c.ptr[b]);
        const size_t n4 = c.count[b] / 4;
        for (size_t i = first; i < n4; i += stride) p[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    }
}

}  // namespace

int load_clear_and_order(hipStream_t stream, const LoadClears &clears, const char *pat, int n_slots, int slots_per_step,
                         int *order, int *count) {
    CNT_REQUIRE(clears.n >= 0 && clears.n <= kLoadClears, "load_clear_and_order: %d buffers", clears.n);
    CNT_REQUIRE(!order || (pat && count && n_slots > 0 && slots_per_step > 0), "load_clear_and_order: bad slot order argument");
    if (clears.n == 0 && !order) return CNT_OK;
    size_t floats = 0;
    for (int b = 0; b < clears.n; ++b) floats += clears.count[b];
    const unsigned fill_blocks = clears.n ? (unsigned)std::min<size_t>((floats / 4 + kOrderThreads - 1) / kOrderThreads, 1024) : 0;
    hipLaunchKernelGGL(load_clear_and_order_kernel, dim3(1 + fill_blocks), dim3(kOrderThreads), 0, stream, clears, pat, n_slots,
                       slots_per_step, order, count);
    CNT_HIP(hipGetLastError());
    return CNT_OK;
}

int slot_order_build(hipStream_t stream, const char *pat, int n_slots, int slots_per_step, int *order, int *count) {
    CNT_REQUIRE(pat && order && count && n_slots > 0 && slots_per_step > 0, "slot_order_build: bad argument");
    hipLaunchKernelGGL(slot_order_kernel, dim3(1), dim3(kOrderThreads), 0, stream, pat, n_slots, slots_per_step, order, count);
    CNT_HIP(hipGetLastError());
    return CNT_OK;
}

int fill_zero(hipStream_t stream, float *p, size_t count) {
    if (count == 0) return CNT_OK;
    const size_t n4 = (reinterpret_cast<uintptr_t>(p) & 15) == 0 ? count / 4 : 0;
    hipLaunchKernelGGL(fill_zero_kernel, dim3(stream_blocks(n4 ? n4 + 3 : count)), dim3(256), 0, stream, p, count, n4);
    CNT_HIP(hipGetLastError());
    return CNT_OK;
}

int fill_zero_pair(hipStream_t stream, float *p, size_t count, float *q, size_t count_q) {
    if (count + count_q == 0) return CNT_OK;
    hipLaunchKernelGGL(fill_zero_pair_kernel, dim3(stream_blocks(count + count_q)), dim3(256), 0, stream, p, count, q,
                       count_q);
    CNT_HIP(hipGetLastError());
    return CNT_OK;
}

int fill_words(hipStream_t stream, unsigned *p, size_t count, unsigned word) {
    if (count == 0) return CNT_OK;
    hipLaunchKernelGGL(fill_words_kernel, dim3(stream_blocks(count)), dim3(256), 0, stream, p, count, word);
    CNT_HIP(hipGetLastError());
    return CNT_OK;
}

int column_sum(hipStream_t stream, const float *v, int D, int N, float scale, float *out) {
    const int gx = (D + 63) / 64;
    int gy = (N + 31) / 32;  // at least eight columns per lane
    gy = std::min(gy, std::max(1, 512 / gx));
    gy = std::max(gy, 1);
    hipLaunchKernelGGL(column_sum_kernel, dim3(gx, gy), dim3(64, 4), 0, stream, v, D, N, scale, out);
    CNT_HIP(hipGetLastError());
    return CNT_OK;
}

}  // namespace cnt

extern "C" {

int cnt_dense_forward(void *stream_, int P, int D, int N, int act, float bias, const float *weights, const float *x,
                      float *y) {
    using namespace cnt;
    CNT_REQUIRE(weights && x && y, "dense_forward: null argument");
    CNT_REQUIRE(P > 0 && D > 0 && N > 0, "dense_forward: non-positive size");
    CNT_REQUIRE(act >= 0 && act <= 3, "dense_forward: unknown activation %d", act);
    GemmArgs ga = {};
    ga.m = D; ga.n = N; ga.k = P;
    ga.a_kcontig = 1; ga.lda = P;
    ga.b_kcontig = 1; ga.ldb = P;
    ga.ldc = D;
    ga.nseg = 1; ga.nprob = 1; ga.splitk = 1;
    ga.epilogue = EPI_BIAS_ACT; ga.act = act; ga.bias_scale = bias;
    ga.prob[0].A[0] = weights; ga.prob[0].B[0] = x; ga.prob[0].C = y;
    ga.prob[0].bias_vec = weights + (size_t)P * D;
    ga.label = "gemm:dense_forward";
    return gemm_launch(static_cast<hipStream_t>(stream_), ga);
}

int cnt_dense_backward_errors(void *stream, int P, int D, int N, int act, const float *weights, const float *y,
                              float *err, float *prev_err) {
    return cnt::dense_backward_errors_fan(static_cast<hipStream_t>(stream), P, D, N, act, weights, y, err, prev_err, nullptr,
                                          nullptr);
}

extern "C++" int cnt::dense_backward_errors_fan(hipStream_t stream, int P, int D, int N, int act, const float *weights,
                                                const float *y, float *err, float *prev_err, const FanOut *fan,
                                                bool *fused, int prev_act, const float *prev_y) {
    if (fused) *fused = false;
    CNT_REQUIRE(weights && y && err, "dense_backward_errors: null argument");
    CNT_REQUIRE(P > 0 && D > 0 && N > 0, "dense_backward_errors: non-positive size");
    CNT_REQUIRE(act >= 0 && act <= 3, "dense_backward_errors: unknown activation %d", act);
    const size_t count = (size_t)D * N;
    if (act != ACT_IDENTITY) {
        ProfileScope prof(stream, "dense_delta");
        const size_t n4 = ((reinterpret_cast<uintptr_t>(err) | reinterpret_cast<uintptr_t>(y)) & 15) == 0 ? count / 4 : 0;
        hipLaunchKernelGGL(dense_delta_kernel, dim3(stream_blocks(n4 ? n4 + 3 : count)), dim3(256), 0, stream, err, y, count,
                           act, n4);
        CNT_HIP(hipGetLastError());
    }
    if (prev_err) {
        GemmArgs ga = {};
        ga.m = P; ga.n = N; ga.k = D;
        ga.a_kcontig = 0; ga.lda = P;
        ga.b_kcontig = 1; ga.ldb = D;
        ga.ldc = P;
        ga.nseg = 1; ga.nprob = 1; ga.splitk = 1; ga.epilogue = EPI_STORE;
        ga.prob[0].A[0] = weights; ga.prob[0].B[0] = err; ga.prob[0].C = prev_err;
        if (prev_act != ACT_IDENTITY && prev_y && !fan) {
            ga.epilogue = EPI_STORE_DELTA;
            ga.act = prev_act;
            ga.prob[0].aux_in = prev_y;
        }
        if (fan && fused && gemm_fan_supported(ga)) {
            ga.epilogue = EPI_FAN;
            ga.fan_n = fan->n; ga.fan_targets = fan->targets; ga.fan_is_skip = fan->is_skip;
            ga.prob[0].aux_in = fan->from_skip;
            *fused = true;
        }
        ga.label = "gemm:dense_prev_errors";
        CNT_TRY(gemm_launch(stream, ga));
    }
    return CNT_OK;
}

int cnt_dense_backward_weights(void *stream, int P, int D, int N, float bias, const float *x, const float *err,
                               float *weight_updates) {
    return cnt::dense_backward_weights_batch(static_cast<hipStream_t>(stream), P, D, N, 1, &bias, &x, &err,
                                             &weight_updates);
}

extern "C++" int cnt::dense_backward_weights_batch(hipStream_t stream, int P, int D, int N, int count, const float *bias,
                                                   const float *const *x, const float *const *err,
                                                   float *const *weight_updates, const SlotOrder *order) {
    CNT_REQUIRE(count >= 1 && count <= kGemmMaxProb, "dense_backward_weights: %d layers in one launch, supported 1..%d",
                count, kGemmMaxProb);
    CNT_REQUIRE(bias && x && err && weight_updates, "dense_backward_weights: null argument");
    CNT_REQUIRE(P > 0 && D > 0 && N > 0, "dense_backward_weights: non-positive size");
    GemmArgs ga = {};
    ga.m = P; ga.n = D; ga.k = N;
    ga.a_kcontig = 0; ga.lda = P;
    ga.b_kcontig = 0; ga.ldb = D;
    ga.ldc = P;
    ga.nseg = 1; ga.nprob = count; ga.epilogue = EPI_ATOMIC;
    ga.splitk = 0;  // chosen by the launcher
    for (int z = 0; z < count; ++z) {
        CNT_REQUIRE(x[z] && err[z] && weight_updates[z], "dense_backward_weights: null argument");
        ga.prob[z].A[0] = x[z]; ga.prob[z].B[0] = err[z]; ga.prob[z].C = weight_updates[z];
        ga.prob[z].rowsum_out = weight_updates[z] + (size_t)P * D;
        ga.prob[z].rowsum_scale = bias[z];
    }
    if (order && order->order) {
        // the deltas are zero on padding slots: the sum over the slots leaves them out
        ga.k_order = order->order;
        ga.k_count = order->count;
    }
    ga.label = "gemm:dense_dW";
    // narrow layers: the launcher sums partial products instead of adding atomically, which overwrites the
    // weight part and brings the bias part (row sums of the errors) along
    ga.overwrite_ok = 1;
    ga.rowsum = 1;
    gemm_plan(ga, stream);
    if (ga.epilogue == EPI_PARTIAL) return gemm_launch(stream, ga);
    for (int z = 0; z < count; ++z) CNT_TRY(fill_zero(stream, weight_updates[z], (size_t)P * D + D));
    CNT_TRY(gemm_launch(stream, ga));
    for (int z = 0; z < count; ++z)
        CNT_TRY(column_sum(stream, err[z], D, N, bias[z], weight_updates[z] + (size_t)P * D));
    return CNT_OK;
}

int cnt_dense_backward_weights_static(void *stream, int P, int D, int N, float bias, const float *x, const float *err,
                                      float *weight_updates) {
    using namespace cnt;
    CNT_REQUIRE(x && err && weight_updates, "dense_backward_weights_static: null argument");
    CNT_REQUIRE(P > 0 && D > 0 && N > 0, "dense_backward_weights_static: non-positive size");
    return gemm_dense_weights_static(static_cast<hipStream_t>(stream), P, D, N, bias, x, err, weight_updates);
}

int cnt_gemm_reserve(void *stream) { return cnt::gemm_reserve_stream(static_cast<hipStream_t>(stream)); }

int cnt_gemm_scratch_buffers(void) { return cnt::gemm_scratch_buffers(); }

int cnt_gemm_release(void *stream) {
    cnt::gemm_release_stream(static_cast<hipStream_t>(stream));
    return CNT_OK;
}

int cnt_dense_backward(void *stream, int P, int D, int N, int act, float bias, const float *weights, const float *x,
                       const float *y, float *err, float *prev_err, float *weight_updates) {
    using namespace cnt;
    CNT_REQUIRE(x && weight_updates, "dense_backward: null argument");
    CNT_TRY(cnt_dense_backward_errors(stream, P, D, N, act, weights, y, err, prev_err));
    return cnt_dense_backward_weights(stream, P, D, N, bias, x, err, weight_updates);
}

int cnt_sse_backward(void *stream_, int D, int N, const char *patTypes, const float *y, const float *target,
                     float *err) {
    using namespace cnt;
    CNT_REQUIRE(patTypes && y && target && err, "sse_backward: null argument");
    CNT_REQUIRE(D > 0 && N > 0, "sse_backward: non-positive size");
    const size_t count = (size_t)D * N;
    hipLaunchKernelGGL(sse_backward_kernel, dim3(stream_blocks(count)), dim3(256), 0,
                       static_cast<hipStream_t>(stream_), D, count, patTypes, y, target, err);
    CNT_HIP(hipGetLastError());
    return CNT_OK;
}

int cnt_sse_error(void *stream_, int D, int N, const char *patTypes, const float *y, const float *target,
                  float *result_dev) {
    using namespace cnt;
    CNT_REQUIRE(patTypes && y && target && result_dev, "sse_error: null argument");
    CNT_REQUIRE(D > 0 && N > 0, "sse_error: non-positive size");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    CNT_TRY(fill_zero(stream, result_dev, 1));
    const size_t count = (size_t)D * N;
    int blocks = stream_blocks(count);
    if (blocks > 512) blocks = 512;
    hipLaunchKernelGGL(sse_error_kernel, dim3(blocks), dim3(256), 0, stream, D, count, patTypes, y, target,
                       result_dev);
    CNT_HIP(hipGetLastError());
    return CNT_OK;
}

}  // extern "C"
