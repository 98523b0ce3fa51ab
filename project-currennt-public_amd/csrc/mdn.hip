// Mixture-density post-output layer for gfx950: flat softmax units and untied-variance Gaussian
// mixture units.
//
// Reference behaviour: layers/MDNLayer.cu (config parsing :280-324, unit creation :457-545,
// calculateError :797-827, forward :841-852, backward :875-917) and layers/MDNUnit.cu (functors
// :227-296, :333-405, :437-470, :503-530, :683-750, :921-1000, :1003-1063, :2096-2325; drivers
// :4170-4339, :4685-4754, :5249-5420, :6036-6193, :6195-6416).
//
// The reference walks the F x Lp activation matrix with 4-6 one-element-per-thread launches per
// call.  Here every call is one streaming kernel per unit: one 64-lane wave owns one frame, lanes run
// along the frame's contiguous columns, and the per-frame reductions (offset, normaliser,
// per-mixture distance, log-sum) are wave shuffles.  HBM traffic per call is one read of the
// unit's columns plus one write of its result.
//
// Kept on purpose: the mixture-weight gradient of a padding frame is "zeroed" at index t*M+m
// instead of t*Lp+startD+m (MDNUnit.cu:2199-2200); on the reference's sequential host backend that
// zero lands after the value it collides with, so the colliding mixture-weight gradient of an
// earlier valid frame reads 0.  The kernels reproduce exactly that outcome without a race.
#include "common.hpp"

#include <algorithm>

#include <cmath>
#include <cstring>
#include <new>
#include <vector>

namespace cnt {
namespace {

constexpr float kSkipMarker = lim::kMax;
constexpr int kFramesPerBlock = 4;

__device__ __forceinline__ float wave_sum(float v) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}
__device__ __forceinline__ float wave_min(float v) {
    for (int o = 32; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ float wave_max(float v) {
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}

// offset = (min + max) / 2 with the reference's start values, exp((x - offset)/T), normalise.
// `in` points at the K inputs of the frame, `out` at its K outputs.
__device__ __forceinline__ void softmax_frame(const float *__restrict__ in, float *__restrict__ out, int K,
                                              float temperature, int lane) {
    float mx = lim::kMin, mn = lim::kMax;
    for (int k = lane; k < K; k += 64) {
        const float v = in[k];
        mn = fminf(mn, v);
        mx = fmaxf(mx, v);
    }
    mn = wave_min(mn);
    mx = wave_max(mx);
    const float offset = 0.5f * (mn + mx);
    float sum = 0.0f;
    for (int k = lane; k < K; k += 64) {
        const float e = safe_exp((in[k] - offset) / temperature);
        out[k] = e;
        sum += e;
    }
    sum = wave_sum(sum);
    if (sum == kSkipMarker) return;
    for (int k = lane; k < K; k += 64) out[k] = out[k] / sum;  // each lane re-reads its own writes
}

struct UnitGeom {
    int F, Lp, Lt;
    int startD, startDOut;
    int M, D;  // softmax unit: M = classes, D unused
    float var_floor, temperature;
    long capacity;  // allocated elements of the unit's parameter buffer
};

// ---- sigmoid unit (layers/MDNUnit.cu:198-225, 563-596, 634-676): M columns, one target per column -------
__global__ void sigmoid_forward_kernel(UnitGeom g, const char *__restrict__ pat, const float *__restrict__ x,
                                       float *__restrict__ prob) {
    const size_t n = (size_t)g.F * g.M;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const size_t f = i / g.M;
        const int k = (int)(i % g.M);
        prob[i] = pat[f] == 0 ? 0.0f : logistic(x[f * g.Lp + g.startD + k]);
    }
}

// sums[0] += binary cross entropy of the valid frames, sums[1] += number of valid frames
__global__ void sigmoid_error_kernel(UnitGeom g, int continuous, const char *__restrict__ pat,
                                     const float *__restrict__ target, const float *__restrict__ prob,
                                     float *__restrict__ sums) {
    const size_t n = (size_t)g.F * g.M;
    float v = 0.0f, cnt = 0.0f;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const size_t f = i / g.M;
        const int k = (int)(i % g.M);
        if (pat[f] == 0) continue;
        if (k == 0) cnt += 1.0f;
        const float p = prob[i], pr = (float)(1.0 - p);
        const float d = target[f * g.Lt + g.startDOut + k];
        if (continuous) {
            const float p1 = logf(fmaxf(lim::kMin, p)), p2 = logf(fmaxf(lim::kMin, pr));
            v += (float)(-1.0 * d * p1 - (1 - d) * p2);
        } else {
            const float b = d > 0 ? p : 1 - p;
            v += -logf(fmaxf(lim::kMin, b));
        }
    }
    v = wave_sum(v);
    cnt = wave_sum(cnt);
    if ((threadIdx.x & 63) == 0) {
        if (v != 0.0f) atomicAdd(sums, v);
        if (cnt != 0.0f) atomicAdd(sums + 1, cnt);
    }
}

// the unit's error is the summed cross entropy divided by the number of valid frames (MDNUnit.cu:3821)
__global__ void sigmoid_error_finish_kernel(const float *__restrict__ sums, float *__restrict__ result) {
    if (threadIdx.x == 0 && blockIdx.x == 0) *result += sums[0] / sums[1];
}

__global__ void sigmoid_backward_kernel(UnitGeom g, int continuous, const char *__restrict__ pat,
                                        const float *__restrict__ target, const float *__restrict__ prob,
                                        float *__restrict__ errors) {
    const size_t n = (size_t)g.F * g.M;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    for (; i < n; i += (size_t)gridDim.x * blockDim.x) {
        const size_t f = i / g.M;
        const int k = (int)(i % g.M);
        float e = 0.0f;
        if (pat[f] != 0) {
            const float p = prob[i], d = target[f * g.Lt + g.startDOut + k];
            e = continuous ? p - d : (d > 0 ? -1 + p : p);
        }
        errors[f * g.Lp + g.startD + k] = e;
    }
}

// ---- softmax unit -----------------------------------------------------------------------------------
__global__ void softmax_forward_kernel(UnitGeom g, const char *__restrict__ pat, const float *__restrict__ x,
                                       float *__restrict__ prob) {
    const int lane = threadIdx.x & 63;
    const int f = blockIdx.x * kFramesPerBlock + (threadIdx.x >> 6);
    if (f >= g.F) return;
    float *row = prob + (size_t)f * g.M;
    if (pat[f] == 0) {
        for (int k = lane; k < g.M; k += 64) row[k] = kSkipMarker;
        return;
    }
    softmax_frame(x + (size_t)f * g.Lp + g.startD, row, g.M, g.temperature, lane);
}

__global__ void softmax_error_kernel(UnitGeom g, const char *__restrict__ pat, const float *__restrict__ target,
                                     const float *__restrict__ prob, float *__restrict__ result) {
    const int f = blockIdx.x * blockDim.x + threadIdx.x;
    float v = 0.0f;
    if (f < g.F && pat[f] != 0) {
        const int ti = (int)target[(size_t)f * g.Lt + g.startDOut];
        const long idx = (long)f * g.M + ti;
        float p = 1.0f;
        if (idx < g.capacity && idx >= 0) p = fmaxf(lim::kMin, prob[idx]);
        v = -logf(p);
    }
    v = wave_sum(v);
    if ((threadIdx.x & 63) == 0 && v != 0.0f) atomicAdd(result, v);
}

__global__ void softmax_backward_kernel(UnitGeom g, const char *__restrict__ pat, const float *__restrict__ target,
                                        const float *__restrict__ prob, float *__restrict__ errors) {
    const int lane = threadIdx.x & 63;
    const int f = blockIdx.x * kFramesPerBlock + (threadIdx.x >> 6);
    if (f >= g.F) return;
    float *e = errors + (size_t)f * g.Lp + g.startD;
    if (pat[f] == 0) {
        // never written by the reference; the layer's zero fill is what remains
        for (int k = lane; k < g.M; k += 64) e[k] = 0.0f;
        return;
    }
    const float t = target[(size_t)f * g.Lt + g.startDOut];
    const float *p = prob + (size_t)f * g.M;
    for (int k = lane; k < g.M; k += 64) {
        const bool hit = (double)((t - k) * (t - k)) < 0.0001;
        e[k] = hit ? (-1 + p[k]) : p[k];
    }
}

// the same with 16-byte accesses (M, the row pitches and the unit's first column multiples of four): an item is four
// classes of one frame, and a thread has several items in flight
__global__ __launch_bounds__(256) void softmax_backward_vec4_kernel(UnitGeom g, const char *__restrict__ pat,
                                                                    const float *__restrict__ target,
                                                                    const float *__restrict__ prob, float *__restrict__ errors) {
    const int per_frame = g.M / 4;
    const size_t items = (size_t)g.F * per_frame;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < items; i += stride) {
        const size_t f = i / per_frame;
        const int k = (int)(i % per_frame) * 4;
        float4 v = {0.0f, 0.0f, 0.0f, 0.0f};
        if (pat[f] != 0) {
            const float t = target[f * g.Lt + g.startDOut];
            v = *reinterpret_cast<const float4 *>(prob + f * g.M + k);
            float *e = reinterpret_cast<float *>(&v);
#pragma unroll
            for (int q = 0; q < 4; ++q)
                if ((double)((t - (k + q)) * (t - (k + q))) < 0.0001) e[q] += -1.0f;
        }
        *reinterpret_cast<float4 *>(errors + f * g.Lp + g.startD + k) = v;
    }
}

// ---- mixture unit -----------------------------------------------------------------------------------
// para = [F*M weights | F*M*D means | F*M*D std], offsets by the CURRENT frame count F.
__global__ void mixture_forward_kernel(UnitGeom g, const char *__restrict__ pat, const float *__restrict__ x,
                                       float *__restrict__ para) {
    const int lane = threadIdx.x & 63;
    const int f = blockIdx.x * kFramesPerBlock + (threadIdx.x >> 6);
    if (f >= g.F) return;
    const int MD = g.M * g.D;
    float *w = para + (size_t)f * g.M;
    float *mean = para + (size_t)g.F * g.M + (size_t)f * MD;
    float *sd = para + (size_t)g.F * g.M * (1 + g.D) + (size_t)f * MD;
    if (pat[f] == 0) {
        for (int k = lane; k < g.M; k += 64) w[k] = kSkipMarker;
        for (int i = lane; i < MD; i += 64) sd[i] = kSkipMarker;  // means stay untouched
        return;
    }
    const float *in = x + (size_t)f * g.Lp + g.startD;
    softmax_frame(in, w, g.M, 1.0f, lane);
    for (int i = lane; i < MD; i += 64) {
        mean[i] = in[g.M + i];
        const float b = safe_exp(in[g.M + MD + i]);
        sd[i] = b < g.var_floor ? g.var_floor : b;
    }
}

// tmp = [F*M per-mixture log-likelihoods | F log-sums]; result accumulates -sum of log-sums
__global__ void mixture_error_kernel(UnitGeom g, const char *__restrict__ pat, const float *__restrict__ target,
                                     const float *__restrict__ para, float *__restrict__ tmp,
                                     float *__restrict__ result) {
    const int lane = threadIdx.x & 63;
    const int f = blockIdx.x * kFramesPerBlock + (threadIdx.x >> 6);
    if (f >= g.F) return;
    const int M = g.M, D = g.D;
    if (pat[f] == 0) {
        for (int m = lane; m < M; m += 64) tmp[(size_t)f * M + m] = 0.0f;  // distance pass writes 0, the rest skips
        return;
    }
    const float *t = target + (size_t)f * g.Lt + g.startDOut;
    const float *mean = para + (size_t)g.F * M + (size_t)f * M * D;
    const float *sd = para + (size_t)g.F * M * (1 + D) + (size_t)f * M * D;
    const float gauss_const = (float)(D * log(2 * 3.141215) / 2.0);  // the reference's own value of pi
    float lsum = lim::kLogZero;
    for (int m = 0; m < M; ++m) {
        float dist = 0.0f, logsd = 0.0f;
        for (int d = lane; d < D; d += 64) {
            const float s = sd[m * D + d], diff = t[d] - mean[m * D + d];
            dist += diff * diff / (s * s) * 0.5f;
            logsd += safe_log(s);
        }
        dist = wave_sum(dist);
        logsd = wave_sum(logsd);
        float lp = logf(para[(size_t)f * M + m]) - dist - gauss_const - logsd;
        if (lp < lim::kLSmall) lp = lim::kLSmall;
        lsum = log_add(lsum, lp);
        if (lane == 0) tmp[(size_t)f * M + m] = lp;
    }
    if (lane == 0) {
        tmp[(size_t)g.F * M + f] = lsum;
        atomicAdd(result, -lsum);
    }
}

// The same error pass for units whose data can be moved 16 bytes at a time (the condition of the VEC4 backward
// kernel below).  Four lanes share a mixture component: lane (m, p) reads the 16-byte vectors p, p+4, ... of the
// component's means and deviations, so one load instruction of the wave covers 64 contiguous bytes of sixteen
// components; the four partial sums meet through two DPP steps instead of one six-step wave reduction per component.
// The log-sum over the components is max + log(sum exp(. - max)) over the wave (the reference's running log_add in
// another order: terms below e^-69 of the largest drop out either way).  A wave takes one frame (a frame is one chain
// of loads, reductions and transcendentals; two frames in turn per wave are 1-2 % slower), and the eight
// waves of a workgroup add their frames' log-sums in LDS, so the single result word receives one atomic per 8
// frames -- 6000 atomics on one address, which serialise, were what the first kernel's time went to.
constexpr int kErrFramesPerWave = 1;
constexpr int kErrWaves = 8;
__global__ __launch_bounds__(64 * kErrWaves) void mixture_error_vec_kernel(UnitGeom g, const char *__restrict__ pat,
                                                                const float *__restrict__ target,
                                                                const float *__restrict__ para, float *__restrict__ tmp,
                                                                float *__restrict__ result) {
    __shared__ float lp_sh[kErrWaves][64];
    __shared__ float block_sum[kErrWaves];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int M = g.M, D = g.D, MD = M * D, DV = D / 4;
    const int p = lane & 3, ml = lane >> 2;  // lane (ml, p): component ml of the pass, quarter p
    const float gauss_const = (float)(D * log(2 * 3.141215) / 2.0);  // the reference's own value of pi
    float wave_total = 0.0f;
    for (int i = 0; i < kErrFramesPerWave; ++i) {
        const int f = (blockIdx.x * kErrWaves + wave) * kErrFramesPerWave + i;
        if (f >= g.F) break;
        if (pat[f] == 0) {
            for (int m = lane; m < M; m += 64) tmp[(size_t)f * M + m] = 0.0f;  // distance pass writes 0, the rest skips
            continue;
        }
        const float4 *t4 = reinterpret_cast<const float4 *>(target + (size_t)f * g.Lt + g.startDOut);
        const float4 *mean4 = reinterpret_cast<const float4 *>(para + (size_t)g.F * M + (size_t)f * MD);
        const float4 *sd4 = reinterpret_cast<const float4 *>(para + (size_t)g.F * M * (1 + D) + (size_t)f * MD);
        float mx = lim::kLogZero;
        float lp_mine[4];  // component lane + 64*pass, held by lanes below M - 64*pass after the exchange
        int npass = 0;
        for (int m0 = 0; m0 < M; m0 += 16, ++npass) {
            const int m = m0 + ml;
            float dist = 0.0f, logsd = 0.0f;
            if (m < M) {
                // sixteen vectors of a component per round, four per lane, all twelve loads of a lane requested
                // before the first is used (a loop over v alone waits for memory once per vector)
                for (int v0 = 0; v0 < DV; v0 += 16) {
                    float4 s[4], mu[4], tv[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const int v = min(v0 + p + 4 * q, DV - 1);
                        s[q] = sd4[m * DV + v]; mu[q] = mean4[m * DV + v]; tv[q] = t4[v];
                    }
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        if (v0 + p + 4 * q >= DV) continue;
                        const float d0 = tv[q].x - mu[q].x, d1 = tv[q].y - mu[q].y, d2 = tv[q].z - mu[q].z, d3 = tv[q].w - mu[q].w;
                        dist += d0 * d0 / (s[q].x * s[q].x) * 0.5f; dist += d1 * d1 / (s[q].y * s[q].y) * 0.5f;
                        dist += d2 * d2 / (s[q].z * s[q].z) * 0.5f; dist += d3 * d3 / (s[q].w * s[q].w) * 0.5f;
                        logsd += safe_log(s[q].x) + safe_log(s[q].y) + safe_log(s[q].z) + safe_log(s[q].w);
                    }
                }
            }
            // the four quarters of a component sit in one quad
            dist += __shfl_xor(dist, 1); logsd += __shfl_xor(logsd, 1);
            dist += __shfl_xor(dist, 2); logsd += __shfl_xor(logsd, 2);
            if (m < M && p == 0) {
                float lp = logf(para[(size_t)f * M + m]) - dist - gauss_const - logsd;
                if (lp < lim::kLSmall) lp = lim::kLSmall;
                tmp[(size_t)f * M + m] = lp;
                lp_sh[wave][ml] = lp;
            }
            // one component per lane for the log-sum (lanes 0..15 of this pass); same wave, so no barrier
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            const float lp = (lane < 16 && m0 + lane < M) ? lp_sh[wave][lane] : lim::kLogZero;
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            if (npass < 4) lp_mine[npass] = lp;
            mx = fmaxf(mx, lp);
        }
        mx = wave_max(mx);
        float se = 0.0f;
        for (int q = 0; q < npass && q < 4; ++q)
            if (lane < 16 && 16 * q + lane < M) se += expf(lp_mine[q] - mx);
        se = wave_sum(se);
        const float lsum = mx + logf(se);
        if (lane == 0) {
            tmp[(size_t)g.F * M + f] = lsum;
            wave_total -= lsum;
        }
    }
    if (lane == 0) block_sum[wave] = wave_total;
    __syncthreads();
    if (threadIdx.x == 0) {
        float v = 0.0f;
#pragma unroll
        for (int w = 0; w < kErrWaves; w += 2) v += block_sum[w] + block_sum[w + 1];
        if (v != 0.0f) atomicAdd(result, v);
    }
}

// VEC4: the mean / std part moves 16 bytes per lane (D, M, Lp, Lt and both start columns multiples of four and all
// buffers 16-byte aligned, so that four consecutive dimensions of one mixture component sit in one aligned vector)
template <bool VEC4>
__global__ void mixture_backward_kernel(UnitGeom g, const char *__restrict__ pat, const float *__restrict__ target,
                                        const float *__restrict__ para, const float *__restrict__ tmp,
                                        float *__restrict__ errors) {
    const int lane = threadIdx.x & 63;
    const int f = blockIdx.x * kFramesPerBlock + (threadIdx.x >> 6);
    if (f >= g.F) return;
    const int M = g.M, D = g.D, MD = M * D, Lp = g.Lp;
    const int unit_cols = M + 2 * MD;
    float *e = errors + (size_t)f * Lp + g.startD;
    if (pat[f] == 0) {
        // The reference zeroes index f*M+m for this frame's mixture weights.  Where that index is a column
        // of this unit the outcome is decided by the owner of the column (see below); elsewhere the zero
        // is written as is.  This frame's own columns end up 0: weights by the layer's zero fill, means and
        // std by the second pass.
        for (int m = lane; m < M; m += 64) {
            const long idx = (long)f * M + m;
            const int col = (int)(idx % Lp);
            if (col < g.startD || col >= g.startD + unit_cols) errors[idx] = 0.0f;
        }
        for (int i = lane; i < unit_cols; i += 64) e[i] = 0.0f;
        return;
    }
    const float lsum = tmp[(size_t)g.F * M + f];
    for (int m = lane; m < M; m += 64) {
        const float post = safe_exp(tmp[(size_t)f * M + m] - lsum);
        float v = para[(size_t)f * M + m] - post;
        // a padding frame fd with fd*M + m' == this index overwrites the value with 0 afterwards
        const long idx = (long)f * Lp + g.startD + m;
        const long fd = idx / M;
        if (fd < g.F && pat[fd] == 0) v = 0.0f;
        e[m] = v;
    }
    const float *t = target + (size_t)f * g.Lt + g.startDOut;
    const float *mean = para + (size_t)g.F * M + (size_t)f * MD;
    const float *sd = para + (size_t)g.F * M * (1 + D) + (size_t)f * MD;
    if (VEC4) {
        for (int i = 4 * lane; i < MD; i += 256) {
            const int m = i / D, d = i - m * D;
            const float post = safe_exp(tmp[(size_t)f * M + m] - lsum);
            const float4 mu4 = *reinterpret_cast<const float4 *>(mean + i);
            const float4 s4 = *reinterpret_cast<const float4 *>(sd + i);
            const float4 t4 = *reinterpret_cast<const float4 *>(t + d);
            const float mu[4] = {mu4.x, mu4.y, mu4.z, mu4.w}, sv[4] = {s4.x, s4.y, s4.z, s4.w};
            const float tv[4] = {t4.x, t4.y, t4.z, t4.w};
            float em[4], es[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                em[q] = post * (mu[q] - tv[q]) / sv[q] / sv[q];
                es[q] = (sv[q] > g.var_floor) ? post - em[q] * (mu[q] - tv[q]) : 0.0f;
            }
            *reinterpret_cast<float4 *>(e + M + i) = make_float4(em[0], em[1], em[2], em[3]);
            *reinterpret_cast<float4 *>(e + M + MD + i) = make_float4(es[0], es[1], es[2], es[3]);
        }
        return;
    }
    for (int i = lane; i < MD; i += 64) {
        const int m = i / D, d = i - m * D;
        const float post = safe_exp(tmp[(size_t)f * M + m] - lsum);
        const float mu = mean[i], s = sd[i], tv = t[d];
        const float e_mu = post * (mu - tv) / s / s;
        e[M + i] = e_mu;
        e[M + MD + i] = (s > g.var_floor) ? post - e_mu * (mu - tv) : 0.0f;
    }
}

// Error and gradient of a mixture unit in ONE pass over its parameters (MDNUnit_mixture::calculateError followed by
// ::computeBackward, layers/MDNUnit.cu:6036-6193, :6195-6416), for units of at most sixteen components and 64 target
// dimensions whose data moves 16 bytes at a time.  A wave takes a frame; lane (m, p) holds the 16-byte vectors p, p+4,
// p+8, p+12 of component m's means and deviations and of the targets in registers, so the 1936 parameters of a
// benchmark frame are read once: the component's log-likelihood comes out of two quad steps, the frame's log-sum out
// of a wave maximum and a wave sum, and the posterior turns the same registers into the errors.  What the two separate
// kernels leave behind is left behind here as well (per-component log-likelihoods and log-sums in tmp, the summed
// negative log-likelihood), with the same arithmetic as mixture_error_vec_kernel and mixture_backward_kernel<true>.
constexpr int kFusedWaves = 8;  // measured on MI355X at 6000 frames: 4 -> 33.8 us, 8 -> 25.6 us, 16 -> 29.4 us
__global__ __launch_bounds__(64 * kFusedWaves) void mixture_error_backward_kernel(UnitGeom g, const char *__restrict__ pat,
                                                                                 const float *__restrict__ target,
                                                                                 const float *__restrict__ para,
                                                                                 float *__restrict__ tmp,
                                                                                 float *__restrict__ result,
                                                                                 float *__restrict__ errors,
                                                                                 float *__restrict__ loss_acc,
                                                                                 unsigned *__restrict__ loss_ticket,
                                                                                 unsigned total_workgroups) {
    __shared__ float block_sum[kFusedWaves];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int M = g.M, D = g.D, MD = M * D, DV = D / 4, Lp = g.Lp;
    const int p = lane & 3, m = lane >> 2;
    const int unit_cols = M + 2 * MD;
    const int f = blockIdx.x * kFusedWaves + wave;
    float wave_total = 0.0f;
    if (f < g.F) {
        float *e = errors + (size_t)f * Lp + g.startD;
        if (pat[f] == 0) {
            // as in the two kernels: the distance pass leaves 0, the gradient pass the zeros described there
            for (int k = lane; k < M; k += 64) {
                tmp[(size_t)f * M + k] = 0.0f;
                const long idx = (long)f * M + k;
                const int col = (int)(idx % Lp);
                if (col < g.startD || col >= g.startD + unit_cols) errors[idx] = 0.0f;
            }
            for (int i = lane; i < unit_cols; i += 64) e[i] = 0.0f;
        } else {
            const float gauss_const = (float)(D * log(2 * 3.141215) / 2.0);  // the reference's own value of pi
            const float4 *t4 = reinterpret_cast<const float4 *>(target + (size_t)f * g.Lt + g.startDOut);
            const float4 *mean4 = reinterpret_cast<const float4 *>(para + (size_t)g.F * M + (size_t)f * MD);
            const float4 *sd4 = reinterpret_cast<const float4 *>(para + (size_t)g.F * M * (1 + D) + (size_t)f * MD);
            const bool live = m < M;
            const int mc = live ? m : 0;
            float4 s[4], mu[4], tv[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int v = min(p + 4 * q, DV - 1);
                s[q] = sd4[mc * DV + v]; mu[q] = mean4[mc * DV + v]; tv[q] = t4[v];
            }
            const float weight = para[(size_t)f * M + mc];
            float dist = 0.0f, logsd = 0.0f;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                if (p + 4 * q >= DV) continue;
                const float d0 = tv[q].x - mu[q].x, d1 = tv[q].y - mu[q].y, d2 = tv[q].z - mu[q].z, d3 = tv[q].w - mu[q].w;
                dist += d0 * d0 / (s[q].x * s[q].x) * 0.5f; dist += d1 * d1 / (s[q].y * s[q].y) * 0.5f;
                dist += d2 * d2 / (s[q].z * s[q].z) * 0.5f; dist += d3 * d3 / (s[q].w * s[q].w) * 0.5f;
                logsd += safe_log(s[q].x) + safe_log(s[q].y) + safe_log(s[q].z) + safe_log(s[q].w);
            }
            dist += __shfl_xor(dist, 1); logsd += __shfl_xor(logsd, 1);
            dist += __shfl_xor(dist, 2); logsd += __shfl_xor(logsd, 2);
            float lp = logf(weight) - dist - gauss_const - logsd;
            if (lp < lim::kLSmall) lp = lim::kLSmall;
            if (live && p == 0) tmp[(size_t)f * M + m] = lp;
            const float mx = wave_max(live ? lp : lim::kLogZero);
            const float se = wave_sum((live && p == 0) ? expf(lp - mx) : 0.0f);
            const float lsum = mx + logf(se);
            if (lane == 0) {
                tmp[(size_t)g.F * M + f] = lsum;
                wave_total = -lsum;
            }
            const float post = safe_exp(lp - lsum);
            if (live) {
                if (p == 0) {
                    float v = weight - post;
                    // a padding frame fd with fd*M + m' == this index overwrites the value with 0 afterwards
                    const long idx = (long)f * Lp + g.startD + m;
                    const long fd = idx / M;
                    if (fd < g.F && pat[fd] == 0) v = 0.0f;
                    e[m] = v;
                }
                float4 *em4 = reinterpret_cast<float4 *>(e + M + (size_t)m * D);
                float4 *es4 = reinterpret_cast<float4 *>(e + M + MD + (size_t)m * D);
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int v = p + 4 * q;
                    if (v >= DV) continue;
                    const float muv[4] = {mu[q].x, mu[q].y, mu[q].z, mu[q].w}, sv[4] = {s[q].x, s[q].y, s[q].z, s[q].w};
                    const float tt[4] = {tv[q].x, tv[q].y, tv[q].z, tv[q].w};
                    float em[4], es[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        em[k] = post * (muv[k] - tt[k]) / sv[k] / sv[k];
                        es[k] = (sv[k] > g.var_floor) ? post - em[k] * (muv[k] - tt[k]) : 0.0f;
                    }
                    em4[v] = make_float4(em[0], em[1], em[2], em[3]);
                    es4[v] = make_float4(es[0], es[1], es[2], es[3]);
                }
            }
        }
    }
    if (lane == 0) block_sum[wave] = wave_total;
    __syncthreads();
    if (threadIdx.x == 0) {
        float v = 0.0f;
#pragma unroll
        for (int w = 0; w < kFusedWaves; w += 2) v += block_sum[w] + block_sum[w + 1];
        // The workgroups of a call (of all its units' launches) add into an accumulator of the handle; the one that
        // finishes last hands the sum to the caller and leaves accumulator and ticket counter at zero for the next
        // call, so that no launch has to clear the caller's result first.
        // No fence (a device-scope fence writes the L2 back, which costs more than the kernel): the ticket is taken
        // only after the add has returned its old value, i.e. has been performed where every XCD's atomics meet.
        const float before = __hip_atomic_fetch_add(loss_acc, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        unsigned one = 1u;
        asm volatile("" : "+v"(one) : "v"(before));  // the ticket's operand depends on the returned value
        if (__hip_atomic_fetch_add(loss_ticket, one, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == total_workgroups - 1u) {
            *result = __hip_atomic_exchange(loss_acc, 0.0f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(loss_ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

}  // namespace
}  // namespace cnt

// ---------------------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------------------
struct cnt_mdn_unit {
    int type;  // >0 mixtures, -1 softmax, 0 sigmoid
    int startD, endD, startDOut, endDOut;
    int M, D;
    float var_floor;
    float *para, *tmp;
    long para_capacity, tmp_capacity;
};

struct cnt_mdn {
    cnt_mdn_desc desc;
    std::vector<cnt_mdn_unit> units;
    const char *pat;
    int T;
    bool covers_all_columns;
    float *loss_acc;         // cnt_mdn_error_backward: the call's running sum (device), zero between calls
    unsigned *loss_ticket;   // and the count of workgroups that have added to it
};

extern "C" {

int cnt_mdn_destroy(cnt_mdn *h) {
    if (!h) return CNT_OK;
    for (auto &u : h->units) {
        if (u.para) (void)hipFree(u.para);
        if (u.tmp) (void)hipFree(u.tmp);
    }
    if (h->loss_acc) (void)hipFree(h->loss_acc);
    delete h;
    return CNT_OK;
}

int cnt_mdn_create(const cnt_mdn_desc *desc, const float *config, int config_len, cnt_mdn **out) {
    using namespace cnt;
    CNT_REQUIRE(desc && config && out, "mdn_create: null argument");
    CNT_REQUIRE(desc->Lp > 0 && desc->Lt > 0 && desc->S > 0 && desc->maxT > 0, "mdn_create: non-positive size");
    CNT_REQUIRE(config_len >= 1, "mdn_create: empty configuration");
    const int n = (int)config[0];
    // same consistency rule as the reference's reader (MDNLayer.cu:303-305)
    CNT_REQUIRE(config_len == n * 5 + 1, "Number of parameter != 1st parameter * 5 + 1");
    cnt_mdn *h = new (std::nothrow) cnt_mdn();
    CNT_REQUIRE(h != nullptr, "mdn_create: out of host memory");
    h->desc = *desc;
    h->pat = nullptr;
    h->T = 0;
    const long maxF = (long)desc->maxT * desc->S;
    std::vector<char> covered((size_t)desc->Lp, 0);
    for (int i = 0; i < n; ++i) {
        cnt_mdn_unit u = {};
        u.startD = (int)config[1 + i * 5]; u.endD = (int)config[2 + i * 5];
        u.startDOut = (int)config[3 + i * 5]; u.endDOut = (int)config[4 + i * 5];
        u.type = (int)config[5 + i * 5];
        const int cols = u.endD - u.startD, dims = u.endDOut - u.startDOut;
        bool ok = u.startD >= 0 && u.endD <= desc->Lp && cols > 0 && u.startDOut >= 0 && u.endDOut <= desc->Lt && dims > 0;
        if (ok && u.type == -1) {
            u.M = cols; u.D = 1;
            u.para_capacity = maxF * u.M;
            u.tmp_capacity = 0;
            ok = (dims == 1);
        } else if (ok && u.type == 0) {
            u.M = cols; u.D = 1;
            u.para_capacity = maxF * u.M;
            u.tmp_capacity = 2;  // cross-entropy sum and frame count
            ok = (dims == cols);
        } else if (ok && u.type > 0) {
            u.M = u.type; u.D = dims;
            ok = !desc->tie_variance && cols == u.M * (1 + 2 * u.D);
            u.para_capacity = maxF * u.M * (1 + 2 * u.D);
            u.tmp_capacity = maxF * (u.M + 1);
        } else {
            ok = false;
        }
        if (!ok) {
            set_error("mdn_create: unit %d (type %d, columns %d..%d, targets %d..%d) is not supported: only sigmoid (0, one "
                      "target per column), flat softmax (-1) and untied-variance mixture units (>0 with columns = "
                      "M*(1+2*D)) are built",
                      i, u.type, u.startD, u.endD, u.startDOut, u.endDOut);
            cnt_mdn_destroy(h);
            return CNT_ERR_ARG;
        }
        hipError_t err = hipMalloc(reinterpret_cast<void **>(&u.para), (size_t)u.para_capacity * sizeof(float));
        if (err == hipSuccess) err = hipMemset(u.para, 0, (size_t)u.para_capacity * sizeof(float));
        if (err == hipSuccess && u.tmp_capacity) {
            err = hipMalloc(reinterpret_cast<void **>(&u.tmp), (size_t)u.tmp_capacity * sizeof(float));
            if (err == hipSuccess) err = hipMemset(u.tmp, 0, (size_t)u.tmp_capacity * sizeof(float));
        }
        h->units.push_back(u);
        if (err != hipSuccess) {
            set_error("mdn_create: %s", hipGetErrorString(err));
            cnt_mdn_destroy(h);
            return CNT_ERR_HIP;
        }
        for (int c = u.startD; c < u.endD; ++c) covered[(size_t)c] = 1;
    }
    h->covers_all_columns = true;
    for (char c : covered) h->covers_all_columns = h->covers_all_columns && c;
    {
        hipError_t err = hipMalloc(reinterpret_cast<void **>(&h->loss_acc), 256);
        if (err == hipSuccess) err = hipMemset(h->loss_acc, 0, 256);
        if (err != hipSuccess) {
            set_error("mdn_create: %s", hipGetErrorString(err));
            cnt_mdn_destroy(h);
            return CNT_ERR_HIP;
        }
        h->loss_ticket = reinterpret_cast<unsigned *>(h->loss_acc) + 32;
    }
    *out = h;
    return CNT_OK;
}

int cnt_mdn_set_var_floor(cnt_mdn *h, int unit, float var_floor) {
    using namespace cnt;
    CNT_REQUIRE(h && unit >= 0 && unit < (int)h->units.size(), "mdn_set_var_floor: no such unit");
    h->units[(size_t)unit].var_floor = var_floor;
    return CNT_OK;
}

int cnt_mdn_load_sequences(cnt_mdn *h, void *stream, const char *patTypes, int curMaxT) {
    using namespace cnt;
    (void)stream;
    CNT_REQUIRE(h && patTypes, "mdn_load_sequences: null argument");
    CNT_REQUIRE(curMaxT >= 1 && curMaxT <= h->desc.maxT, "mdn_load_sequences: curMaxT %d outside 1..%d", curMaxT,
                h->desc.maxT);
    h->pat = patTypes;
    h->T = curMaxT;
    return CNT_OK;
}

float *cnt_mdn_unit_buffer(cnt_mdn *h, int unit, int which, long *count) {
    if (!h || unit < 0 || unit >= (int)h->units.size()) return nullptr;
    cnt_mdn_unit &u = h->units[(size_t)unit];
    const long F = (long)h->T * h->desc.S;
    if (which == 0) {
        if (count) *count = u.type <= 0 ? F * u.M : F * u.M * (1 + 2 * u.D);
        return u.para;
    }
    if (which == 1 && u.tmp && u.type > 0) {
        if (count) *count = F * (u.M + 1);
        return u.tmp;
    }
    return nullptr;
}

static cnt::UnitGeom unit_geom(const cnt_mdn *h, const cnt_mdn_unit &u) {
    cnt::UnitGeom g;
    g.F = h->T * h->desc.S; g.Lp = h->desc.Lp; g.Lt = h->desc.Lt;
    g.startD = u.startD; g.startDOut = u.startDOut; g.M = u.M; g.D = u.D;
    g.var_floor = u.var_floor; g.temperature = 1.0f;
    g.capacity = u.para_capacity;
    return g;
}

int cnt_mdn_forward(cnt_mdn *h, void *stream_, const float *nn_outputs) {
    using namespace cnt;
    CNT_REQUIRE(h && nn_outputs, "mdn_forward: null argument");
    CNT_REQUIRE(h->T > 0, "mdn_forward: load_sequences has not been called");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    for (auto &u : h->units) {
        const UnitGeom g = unit_geom(h, u);
        const dim3 grid((g.F + kFramesPerBlock - 1) / kFramesPerBlock), block(64 * kFramesPerBlock);
        if (u.type == 0) {
            ProfileScope prof(stream, "mdn_sigmoid_forward");
            const size_t n = (size_t)g.F * g.M;
            hipLaunchKernelGGL(sigmoid_forward_kernel, dim3((unsigned)std::min<size_t>((n + 255) / 256, 4096)), dim3(256), 0,
                               stream, g, h->pat, nn_outputs, u.para);
        } else if (u.type == -1) {
            ProfileScope prof(stream, "mdn_softmax_forward");
            hipLaunchKernelGGL(softmax_forward_kernel, grid, block, 0, stream, g, h->pat, nn_outputs, u.para);
        } else {
            ProfileScope prof(stream, "mdn_mixture_forward");
            hipLaunchKernelGGL(mixture_forward_kernel, grid, block, 0, stream, g, h->pat, nn_outputs, u.para);
        }
        CNT_HIP(hipGetLastError());
    }
    return CNT_OK;
}

int cnt_mdn_calculate_error(cnt_mdn *h, void *stream_, const float *targets, float *result_dev) {
    using namespace cnt;
    CNT_REQUIRE(h && targets && result_dev, "mdn_calculate_error: null argument");
    CNT_REQUIRE(h->T > 0, "mdn_calculate_error: load_sequences has not been called");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    CNT_TRY(fill_zero(stream, result_dev, 1));
    for (auto &u : h->units) {
        const UnitGeom g = unit_geom(h, u);
        if (u.type == 0) {
            ProfileScope prof(stream, "mdn_sigmoid_error");
            const size_t n = (size_t)g.F * g.M;
            CNT_TRY(fill_zero(stream, u.tmp, 2));
            hipLaunchKernelGGL(sigmoid_error_kernel, dim3((unsigned)std::min<size_t>((n + 255) / 256, 1024)), dim3(256), 0,
                               stream, g, h->desc.sigmoid_continuous, h->pat, targets, u.para, u.tmp);
            hipLaunchKernelGGL(sigmoid_error_finish_kernel, dim3(1), dim3(64), 0, stream, u.tmp, result_dev);
        } else if (u.type == -1) {
            ProfileScope prof(stream, "mdn_softmax_error");
            hipLaunchKernelGGL(softmax_error_kernel, dim3((g.F + 255) / 256), dim3(256), 0, stream, g, h->pat, targets,
                               u.para, result_dev);
        } else {
            ProfileScope prof(stream, "mdn_mixture_error");
            auto aligned = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
            const bool vec4 = g.D % 4 == 0 && g.M % 4 == 0 && g.M <= 64 && g.Lt % 4 == 0 && g.startDOut % 4 == 0 &&
                              aligned(targets) && aligned(u.para);
            if (vec4) {
                const int per_block = kErrWaves * kErrFramesPerWave;
                hipLaunchKernelGGL(mixture_error_vec_kernel, dim3((g.F + per_block - 1) / per_block), dim3(64 * kErrWaves), 0, stream, g,
                                   h->pat, targets, u.para, u.tmp, result_dev);
            } else {
                const dim3 grid((g.F + kFramesPerBlock - 1) / kFramesPerBlock), block(64 * kFramesPerBlock);
                hipLaunchKernelGGL(mixture_error_kernel, grid, block, 0, stream, g, h->pat, targets, u.para, u.tmp,
                                   result_dev);
            }
        }
        CNT_HIP(hipGetLastError());
    }
    return CNT_OK;
}

// calculateError and computeBackwardPass of the layer in one call: the same results in result_dev, the units' buffers
// and prev_errors as cnt_mdn_calculate_error followed by cnt_mdn_backward.  A mixture unit of at most sixteen components
// and 64 target dimensions with 16-byte aligned data takes both steps in one pass over its parameters; every other
// unit runs its two kernels one after the other.
int cnt_mdn_error_backward(cnt_mdn *h, void *stream_, const float *targets, float *result_dev, float *prev_errors) {
    using namespace cnt;
    CNT_REQUIRE(h && targets && result_dev && prev_errors, "mdn_error_backward: null argument");
    CNT_REQUIRE(h->T > 0, "mdn_error_backward: load_sequences has not been called");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    auto aligned = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    bool all_fused = true;
    for (auto &u : h->units) {
        const UnitGeom g = unit_geom(h, u);
        const bool fused = u.type > 0 && g.M <= 16 && g.D <= 64 && g.D % 4 == 0 && g.M % 4 == 0 && g.Lp % 4 == 0 &&
                           g.Lt % 4 == 0 && g.startD % 4 == 0 && g.startDOut % 4 == 0 && aligned(targets) &&
                           aligned(u.para) && aligned(prev_errors);
        all_fused = all_fused && fused;
    }
    if (!all_fused) {
        CNT_TRY(cnt_mdn_calculate_error(h, stream_, targets, result_dev));
        return cnt_mdn_backward(h, stream_, targets, prev_errors);
    }
    const size_t used = (size_t)h->T * h->desc.S * h->desc.Lp;
    const size_t cap = (size_t)h->desc.maxT * h->desc.S * h->desc.Lp;
    if (!h->covers_all_columns) CNT_TRY(fill_zero(stream, prev_errors, used));
    if (cap > used) CNT_TRY(fill_zero(stream, prev_errors + used, cap - used));
    unsigned total = 0;
    for (auto &u : h->units) total += (unsigned)((unit_geom(h, u).F + kFusedWaves - 1) / kFusedWaves);
    for (auto &u : h->units) {
        const UnitGeom g = unit_geom(h, u);
        ProfileScope prof(stream, "mdn_mixture_error_backward");
        hipLaunchKernelGGL(mixture_error_backward_kernel, dim3((g.F + kFusedWaves - 1) / kFusedWaves), dim3(64 * kFusedWaves), 0,
                           stream, g, h->pat, targets, u.para, u.tmp, result_dev, prev_errors, h->loss_acc, h->loss_ticket, total);
        CNT_HIP(hipGetLastError());
    }
    return CNT_OK;
}

int cnt_mdn_backward(cnt_mdn *h, void *stream_, const float *targets, float *prev_errors) {
    using namespace cnt;
    CNT_REQUIRE(h && targets && prev_errors, "mdn_backward: null argument");
    CNT_REQUIRE(h->T > 0, "mdn_backward: load_sequences has not been called");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const size_t used = (size_t)h->T * h->desc.S * h->desc.Lp;
    const size_t cap = (size_t)h->desc.maxT * h->desc.S * h->desc.Lp;
    // MDNLayer::computeBackwardPass zero-fills the whole preceding error buffer first.  The unit kernels
    // write every column they own for every current frame, so only what they do not cover is filled.
    if (!h->covers_all_columns) CNT_TRY(fill_zero(stream, prev_errors, used));
    if (cap > used) CNT_TRY(fill_zero(stream, prev_errors + used, cap - used));
    for (auto &u : h->units) {
        const UnitGeom g = unit_geom(h, u);
        const dim3 grid((g.F + kFramesPerBlock - 1) / kFramesPerBlock), block(64 * kFramesPerBlock);
        if (u.type == 0) {
            ProfileScope prof(stream, "mdn_sigmoid_backward");
            const size_t n = (size_t)g.F * g.M;
            hipLaunchKernelGGL(sigmoid_backward_kernel, dim3((unsigned)std::min<size_t>((n + 255) / 256, 4096)), dim3(256), 0,
                               stream, g, h->desc.sigmoid_continuous, h->pat, targets, u.para, prev_errors);
        } else if (u.type == -1) {
            ProfileScope prof(stream, "mdn_softmax_backward");
            const bool vec4 = g.M % 4 == 0 && g.Lp % 4 == 0 && g.startD % 4 == 0 &&
                              (reinterpret_cast<uintptr_t>(u.para) & 15) == 0 && (reinterpret_cast<uintptr_t>(prev_errors) & 15) == 0;
            if (vec4) {
                const size_t items = (size_t)g.F * (g.M / 4);
                hipLaunchKernelGGL(softmax_backward_vec4_kernel, dim3((unsigned)std::min<size_t>((items + 255) / 256, 2048)),
                                   dim3(256), 0, stream, g, h->pat, targets, u.para, prev_errors);
            } else {
                hipLaunchKernelGGL(softmax_backward_kernel, grid, block, 0, stream, g, h->pat, targets, u.para,
                                   prev_errors);
            }
        } else {
            ProfileScope prof(stream, "mdn_mixture_backward");
            auto aligned = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
            const bool vec4 = g.D % 4 == 0 && g.M % 4 == 0 && g.Lp % 4 == 0 && g.Lt % 4 == 0 && g.startD % 4 == 0 &&
                              g.startDOut % 4 == 0 && aligned(targets) && aligned(u.para) && aligned(prev_errors);
            if (vec4)
                hipLaunchKernelGGL(mixture_backward_kernel<true>, grid, block, 0, stream, g, h->pat, targets, u.para,
                                   u.tmp, prev_errors);
            else
                hipLaunchKernelGGL(mixture_backward_kernel<false>, grid, block, 0, stream, g, h->pat, targets, u.para,
                                   u.tmp, prev_errors);
        }
        CNT_HIP(hipGetLastError());
    }
    return CNT_OK;
}

}  // extern "C"
