// WaveNet building blocks for gfx950: 1-D dilated (causal) convolution layer, conditioned gated
// activation ("wavnetc"), its unconditioned twin ("gatedact"), and the skip-add fan-in / fan-out.
//
// Reference behaviour: layers/CNNLayer.cu (functors :78-246, forward :1099-1224, backward :1409-1597),
// layers/wavNetCore.cu (functors :69-270, forward :629-711, backward :801-916),
// layers/GatedActLayer.cu (:64-121, :177-263), layers/SkipAddLayer.cu (:186-240, :305-346).
//
// The reference materialises a (sum of window widths) x (T*S) column buffer per layer, zero-fills it
// and scatters the deltas into it before two matrix products.  Here the column buffer never exists:
// every window tap is one operand pair of the MFMA GEMM whose B-side loader applies the tap's time
// shift and the padding mask while staging the tile, so the deltas are read straight from the error
// buffer.  The dead "future" tap of a causal window is never computed; its gradient columns are the
// zeros of the weight-update clear.  The elementwise parts are fused streaming kernels.
#include "common.hpp"

#include <cstring>
#include <new>
#include <vector>

namespace cnt {
namespace {

inline int stream_blocks(size_t count) {
    size_t b = (count + 255) / 256;
    if (b > 8192) b = 8192;
    if (b < 1) b = 1;
    return (int)b;
}

__global__ void tanh_delta_kernel(float *__restrict__ err, const float *__restrict__ y, size_t count) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) err[i] = tanh_deriv(y[i]) * err[i];
}

// conditioning frame of every slot (wavNetCore.cu:143-190)
__global__ void load_context_kernel(int C, int S, size_t count, int max_feature_length, int resolution_one,
                                    const float *__restrict__ source, const float *__restrict__ frame_index,
                                    const float *__restrict__ mean_std, const char *__restrict__ pat,
                                    float *__restrict__ ctx) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) {
        const int t = (int)(i / C), c = (int)(i % C);
        float v = 0.0f;
        if (pat[t] != 0) {
            const float fi = frame_index[t];
            const int feat = resolution_one ? t : (int)(fi * S + (t % S));
            if (fi >= max_feature_length) {
                v = 0.0f;
            } else if (mean_std) {
                const float sd = mean_std[c + C];
                v = (float)((source[(size_t)feat * C + c] - mean_std[c]) / (sd < 1e-5f ? 1.0 : (double)sd));
            } else {
                v = source[(size_t)feat * C + c];
            }
        }
        ctx[i] = v;
    }
}

// z = tanh(y1) * sigmoid(y2), 0 on padding slots; pre is 2D x N
__global__ void gated_forward_kernel(int D, size_t count, const char *__restrict__ pat, const float *__restrict__ pre,
                                     float *__restrict__ out) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) {
        const size_t t = i / D, d = i % D;
        out[i] = (pat[t] == 0) ? 0.0f : tanh_act(pre[t * 2 * D + d]) * logistic(pre[t * 2 * D + D + d]);
    }
}

// unconditioned core: core = conv (0 on padding), ctx_tanh = 0
__global__ void core_copy_kernel(int D2, size_t count, const char *__restrict__ pat, const float *__restrict__ conv,
                                 float *__restrict__ core, float *__restrict__ ctx_tanh) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) {
        core[i] = (pat[i / D2] == 0) ? 0.0f : conv[i] + 0.0f;
        if (ctx_tanh) ctx_tanh[i] = 0.0f;
    }
}

// One thread per (slot, d): both halves of the gate gradient from the same three loads, and -- when the
// core is conditioned -- the gradient through tanh(X_c) written over ctx_tanh in the same pass.
// prev_out (optional): outputs of a preceding layer with tanh output; its delta tanh'(y) * error is then written
// instead of the error.
template <int V> struct Pack;
template <> struct Pack<1> { typedef float type; };
template <> struct Pack<4> { typedef float4 type; };

// VEC consecutive channels per thread (VEC = 4: 16-byte accesses, for D % 4 == 0 and 16-byte aligned buffers)
template <int VEC>
__global__ void gated_backward_kernel(int D, size_t count, const char *__restrict__ pat, const float *__restrict__ pre,
                                      const float *__restrict__ err, float *__restrict__ prev_err,
                                      float *__restrict__ ctx_tanh, const float *__restrict__ prev_out) {
    typedef typename Pack<VEC>::type V;
    const size_t groups = count / VEC;
    const size_t per_slot = (size_t)D / VEC;
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < groups; i += stride) {
        const size_t t = i / per_slot, d = (i % per_slot) * VEC;
        const size_t i1 = t * 2 * D + d, i2 = i1 + D;
        float g1[VEC], g2[VEC];
#pragma unroll
        for (int q = 0; q < VEC; ++q) g1[q] = g2[q] = 0.0f;
        if (pat[t] != 0) {
            const V p1 = *reinterpret_cast<const V *>(pre + i1), p2 = *reinterpret_cast<const V *>(pre + i2);
            const V ev = *reinterpret_cast<const V *>(err + t * D + d);
            const float *a1 = reinterpret_cast<const float *>(&p1), *a2 = reinterpret_cast<const float *>(&p2);
            const float *e = reinterpret_cast<const float *>(&ev);
#pragma unroll
            for (int q = 0; q < VEC; ++q) {
                const float th = tanh_act(a1[q]);
                const float sg = logistic(a2[q]);
                g1[q] = (1.0f - th * th) * sg * e[q];
                g2[q] = th * (sg * (1.0f - sg)) * e[q];
            }
        }
        V o1, o2;
        float *w1 = reinterpret_cast<float *>(&o1), *w2 = reinterpret_cast<float *>(&o2);
        if (prev_out) {
            const V y1 = *reinterpret_cast<const V *>(prev_out + i1), y2 = *reinterpret_cast<const V *>(prev_out + i2);
            const float *b1 = reinterpret_cast<const float *>(&y1), *b2 = reinterpret_cast<const float *>(&y2);
#pragma unroll
            for (int q = 0; q < VEC; ++q) {
                w1[q] = tanh_deriv(b1[q]) * g1[q];
                w2[q] = tanh_deriv(b2[q]) * g2[q];
            }
        } else {
#pragma unroll
            for (int q = 0; q < VEC; ++q) {
                w1[q] = g1[q];
                w2[q] = g2[q];
            }
        }
        *reinterpret_cast<V *>(prev_err + i1) = o1;
        *reinterpret_cast<V *>(prev_err + i2) = o2;
        if (ctx_tanh) {
            const V c1 = *reinterpret_cast<const V *>(ctx_tanh + i1), c2 = *reinterpret_cast<const V *>(ctx_tanh + i2);
            const float *b1 = reinterpret_cast<const float *>(&c1), *b2 = reinterpret_cast<const float *>(&c2);
#pragma unroll
            for (int q = 0; q < VEC; ++q) {
                w1[q] = tanh_deriv(b1[q]) * g1[q];
                w2[q] = tanh_deriv(b2[q]) * g2[q];
            }
            *reinterpret_cast<V *>(ctx_tanh + i1) = o1;
            *reinterpret_cast<V *>(ctx_tanh + i2) = o2;
        }
    }
}

int launch_gated_backward(hipStream_t stream, int D, size_t count, const char *pat, const float *pre, const float *err,
                          float *prev_err, float *ctx_tanh, const float *prev_out) {
    auto aligned = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    const bool vec4 = D % 4 == 0 && aligned(pre) && aligned(err) && aligned(prev_err) && aligned(ctx_tanh) &&
                      aligned(prev_out);
    if (vec4)
        hipLaunchKernelGGL(gated_backward_kernel<4>, dim3(stream_blocks(count / 4)), dim3(256), 0, stream, D, count, pat,
                           pre, err, prev_err, ctx_tanh, prev_out);
    else
        hipLaunchKernelGGL(gated_backward_kernel<1>, dim3(stream_blocks(count)), dim3(256), 0, stream, D, count, pat, pre,
                           err, prev_err, ctx_tanh, prev_out);
    CNT_HIP(hipGetLastError());
    return CNT_OK;
}

// ---------------------------------------------------------------------------------------------------
// Error path of one residual block in one launch: the 1x1 layer that feeds the skip sum (R -> K), the skip layer in
// front of it (adds what later layers handed to it and hands the sum on), the 1x1 layer behind the gated unit
// (R -> R) and the gated unit itself.  Run layer by layer this is a product that writes R x N errors, a second
// product that reads them and writes R x N, and an elementwise pass that reads those; here the R x N intermediates
// stay in registers.
//
// A wave owns 16 samples.  Both products are computed transposed, D[channel][sample] = sum_k W[k][channel] *
// E[sample][k], with v_mfma_f32_16x16x4f32: a lane then holds, for ITS sample (lane % 16), four consecutive channels
// per accumulator (channel = 16*tile + 4*(lane/16) + v), i.e. 16-byte pieces of the sample-major buffers, and the sum
// over k may run in any order: instruction (j, i) takes k = 16j + 4*(lane/16) + i from both operands.  With that order
// the B operand of the first product is K/16 16-byte loads per lane straight from the error buffer (64 contiguous
// bytes per sample and load), and the accumulators of the first product ARE the B operand of the second (register i
// of tile j).  The weights sit in LDS in the order the A operand wants them, one 16-byte read per four instructions.
struct BlockErrArgs {
    int N;
    const char *pat;
    const float *w_skip;     // [K][R]: weights of the R -> K layer (element (k, r) at k*R + r)
    const float *w_out;      // [R][R]: weights of the R -> R layer
    const float *e_skip;     // K x N: errors at the outputs of the R -> K layer
    const float *from_skip;  // R x N or null: what later layers handed to the skip layer
    float *total;            // R x N: the skip layer's summed errors (= the R -> R layer's output errors)
    int fan_n;
    float *const *fan_targets;
    const int *fan_is_skip;
    const float *pre;        // 2R x N: pre-activations of the gated unit
    const float *conv_tanh;  // 2R x N or null: outputs of a convolution layer with tanh output
    float *ctx_tanh;         // 2R x N or null: tanh of the conditioning part, overwritten with its gradient
    float *deltas;           // 2R x N: errors (or deltas) of the convolution layer
    // folded convolution (two live taps, R inputs, 2R filters) whose errors go to the block's closing skip layer:
    const float *conv_w[2];      // weight of (filter 0, tap q); filter d at + d*conv_ld, input channel p at + p
    int conv_ld;
    int conv_shift[2];           // tap q reads the delta of slot n + conv_shift[q]
    const float *conv_deltas;    // 2R x N deltas of that convolution layer
    float *colsum;               // optional, [workgroups][2R]: this workgroup's sums of `deltas` over its samples
};

typedef float f32x4v __attribute__((ext_vector_type(4)));

template <int R, int K, bool CONV>
__global__ __launch_bounds__(CONV ? 512 : 256, (CONV || K > 128) ? 1 : 2) void wavenet_block_errors_kernel(const BlockErrArgs a) {
    static_assert(R % 16 == 0 && K % 16 == 0 && R <= 128, "block geometry");
    constexpr int NT = CONV ? 512 : 256;  // the folded convolution's weights take 2 x 2R x R words of LDS more
    constexpr int RT = R / 16;  // channel tiles
    constexpr int KJ = K / 16, RJ = R / 16, CJ = 2 * R / 16;
    // A operands: [tile][j][lane = 16*quarter + channel in tile][i] = W[16j + 4*quarter + i][16*tile + channel]
    __shared__ __attribute__((aligned(16))) float w1[RT * KJ * 64 * 4];
    __shared__ __attribute__((aligned(16))) float w2[RT * RJ * 64 * 4];
    // one tap of the folded convolution at a time: with both taps the workgroup would hold 112 KB of the compute unit's
    // 160 KB and nothing that wants 64 KB (a weight-gradient product on another stream) could run next to it
    __shared__ __attribute__((aligned(16))) float wc[CONV ? RT * CJ * 64 * 4 : 4];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int quarter = lane >> 4, col = lane & 15;
    const int n_raw = (blockIdx.x * (NT / 64) + wave) * 16 + col;
    const bool ok = n_raw < a.N;
    const size_t n = ok ? n_raw : a.N - 1;  // lanes past the end compute on the last sample and store nothing

    // every global read that does not depend on a product is requested up front
    constexpr int T1 = K * R / 4, T2 = R * R / 4, TC = 2 * R * R / 4;  // 16-byte pieces
    constexpr int F1 = (T1 + NT - 1) / NT, F2 = (T2 + NT - 1) / NT, FC = CONV ? (TC + NT - 1) / NT : 0;
    float4 s1[F1], s2[F2];
#pragma unroll
    for (int q = 0; q < F1; ++q)
        if (q * NT + tid < T1) s1[q] = reinterpret_cast<const float4 *>(a.w_skip)[q * NT + tid];
#pragma unroll
    for (int q = 0; q < F2; ++q)
        if (q * NT + tid < T2) s2[q] = reinterpret_cast<const float4 *>(a.w_out)[q * NT + tid];
    float4 b1[KJ];
    {
        const float4 *src = reinterpret_cast<const float4 *>(a.e_skip + n * K + 4 * quarter);
#pragma unroll
        for (int j = 0; j < KJ; ++j) b1[j] = src[4 * j];
    }
    float4 side[RT];
    if (a.from_skip) {
#pragma unroll
        for (int t = 0; t < RT; ++t) side[t] = *reinterpret_cast<const float4 *>(a.from_skip + n * R + 16 * t + 4 * quarter);
    }
    const bool live = a.pat[n] != 0;
    auto stage = [](float *w, int J, int idx4, const float4 &v) {
        // element (k, ch .. ch+3): same k, four neighbouring channels of one tile
        const int k = idx4 * 4 / R, ch = idx4 * 4 % R;
        float *dst = w + ((((ch / 16) * J + k / 16) * 4 + ((k >> 2) & 3)) * 16 + ch % 16) * 4 + (k & 3);
        dst[0] = v.x; dst[4] = v.y; dst[8] = v.z; dst[12] = v.w;
    };
#pragma unroll
    for (int q = 0; q < F1; ++q)
        if (q * NT + tid < T1) stage(w1, KJ, q * NT + tid, s1[q]);
#pragma unroll
    for (int q = 0; q < F2; ++q)
        if (q * NT + tid < T2) stage(w2, RJ, q * NT + tid, s2[q]);
    // folded convolution: tap q contributes sum_d Wc[d][tap q][p] * delta[slot n + shift q][d], counted only where both
    // slots are inside the fraction and not padding (the rule of the convolution layer's own error product)
    float4 bc[CONV ? 2 : 1][CONV ? CJ : 1];
    float4 sc1[FC > 0 ? FC : 1];  // the second tap's weights wait in registers until the first tap's products are done
    if (CONV) {
        float4 sc0[FC > 0 ? FC : 1];
#pragma unroll
        for (int q = 0; q < FC; ++q) {
            const int idx4 = q * NT + tid;
            if (idx4 < TC) {
                const size_t at = (size_t)(idx4 * 4 / R) * a.conv_ld + idx4 * 4 % R;
                sc0[q] = *reinterpret_cast<const float4 *>(a.conv_w[0] + at);
                sc1[q] = *reinterpret_cast<const float4 *>(a.conv_w[1] + at);
            }
        }
#pragma unroll
        for (int q = 0; q < FC; ++q)
            if (q * NT + tid < TC) stage(wc, CJ, q * NT + tid, sc0[q]);
#pragma unroll
        for (int tap = 0; tap < 2; ++tap) {
            const long long src = (long long)n + a.conv_shift[tap];
            const bool inside = src >= 0 && src < a.N;
            const size_t sc = inside ? (size_t)src : n;
            const bool keep = live && inside && a.pat[sc] != 0;
            const float4 *p = reinterpret_cast<const float4 *>(a.conv_deltas + sc * 2 * R + 4 * quarter);
#pragma unroll
            for (int j = 0; j < CJ; ++j) {
                const float4 v = p[4 * j];
                bc[tap][j] = keep ? v : float4{0.0f, 0.0f, 0.0f, 0.0f};
            }
        }
    }
    // the gate's pre-activations and the first target's old values are requested before the products start
    float4 p1[RT], p2[RT], old0[RT];
    const bool add_first = ok && a.fan_n > 0 && a.fan_is_skip[0] != 0;
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        const size_t at = n * 2 * R + 16 * t + 4 * quarter;
        p1[t] = *reinterpret_cast<const float4 *>(a.pre + at);
        p2[t] = *reinterpret_cast<const float4 *>(a.pre + at + R);
        if (add_first) old0[t] = *reinterpret_cast<const float4 *>(a.fan_targets[0] + n * R + 16 * t + 4 * quarter);
    }
    __syncthreads();

    f32x4v e[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        f32x4v acc0 = {0, 0, 0, 0}, acc1 = {0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < KJ; ++j) {
            const float4 w = *reinterpret_cast<const float4 *>(&w1[((t * KJ + j) * 64 + lane) * 4]);
            acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(w.x, b1[j].x, acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(w.y, b1[j].y, acc1, 0, 0, 0);
            acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(w.z, b1[j].z, acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(w.w, b1[j].w, acc1, 0, 0, 0);
        }
        if (CONV) {
#pragma unroll
            for (int j = 0; j < CJ; ++j) {
                const float4 w = *reinterpret_cast<const float4 *>(&wc[((t * CJ + j) * 64 + lane) * 4]);
                acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(w.x, bc[0][j].x, acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(w.y, bc[0][j].y, acc1, 0, 0, 0);
                acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(w.z, bc[0][j].z, acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(w.w, bc[0][j].w, acc1, 0, 0, 0);
            }
        }
        e[t] = acc0 + acc1;
    }
    if (CONV) {
        __syncthreads();  // every wave is done with the first tap's weights
#pragma unroll
        for (int q = 0; q < FC; ++q)
            if (q * NT + tid < TC) stage(wc, CJ, q * NT + tid, sc1[q]);
        __syncthreads();
#pragma unroll
        for (int t = 0; t < RT; ++t) {
            f32x4v acc0 = e[t], acc1 = {0, 0, 0, 0};
#pragma unroll
            for (int j = 0; j < CJ; ++j) {
                const float4 w = *reinterpret_cast<const float4 *>(&wc[((t * CJ + j) * 64 + lane) * 4]);
                acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(w.x, bc[1][j].x, acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(w.y, bc[1][j].y, acc1, 0, 0, 0);
                acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(w.z, bc[1][j].z, acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(w.w, bc[1][j].w, acc1, 0, 0, 0);
            }
            e[t] = acc0 + acc1;
        }
    }
    // the skip layer's step: add the side buffer, keep the sum, hand it on
    if (a.from_skip) {
#pragma unroll
        for (int t = 0; t < RT; ++t) {
            e[t][0] += side[t].x; e[t][1] += side[t].y; e[t][2] += side[t].z; e[t][3] += side[t].w;
        }
    }
    if (ok) {
#pragma unroll
        for (int t = 0; t < RT; ++t)
            *reinterpret_cast<float4 *>(a.total + n * R + 16 * t + 4 * quarter) = float4{e[t][0], e[t][1], e[t][2], e[t][3]};
        for (int q = 0; q < a.fan_n; ++q) {
            float *tgt = a.fan_targets[q];
            if (a.fan_is_skip[q]) {
                float4 old[RT];
#pragma unroll
                for (int t = 0; t < RT; ++t)
                    old[t] = q == 0 ? old0[t] : *reinterpret_cast<const float4 *>(tgt + n * R + 16 * t + 4 * quarter);
#pragma unroll
                for (int t = 0; t < RT; ++t)
                    *reinterpret_cast<float4 *>(tgt + n * R + 16 * t + 4 * quarter) =
                        float4{e[t][0] + old[t].x, e[t][1] + old[t].y, e[t][2] + old[t].z, e[t][3] + old[t].w};
            } else {
#pragma unroll
                for (int t = 0; t < RT; ++t)
                    *reinterpret_cast<float4 *>(tgt + n * R + 16 * t + 4 * quarter) = float4{e[t][0], e[t][1], e[t][2], e[t][3]};
            }
        }
    }

    // second product: errors at the gated unit's outputs
    f32x4v u[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        f32x4v acc0 = {0, 0, 0, 0}, acc1 = {0, 0, 0, 0};
#pragma unroll
        for (int j = 0; j < RJ; ++j) {
            const float4 w = *reinterpret_cast<const float4 *>(&w2[((t * RJ + j) * 64 + lane) * 4]);
            acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(w.x, e[j][0], acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(w.y, e[j][1], acc1, 0, 0, 0);
            acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(w.z, e[j][2], acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(w.w, e[j][3], acc1, 0, 0, 0);
        }
        u[t] = acc0 + acc1;
    }

    // the gated unit (see gated_backward_kernel), four channels at a time
    float4 cs1[RT], cs2[RT];  // what this lane writes to `deltas`, for the bias gradient of the convolution layer
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        const size_t at = n * 2 * R + 16 * t + 4 * quarter;
        const float *a1 = reinterpret_cast<const float *>(&p1[t]), *a2 = reinterpret_cast<const float *>(&p2[t]);
        float g1[4], g2[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const float th = tanh_act(a1[q]);
            const float sg = logistic(a2[q]);
            const float ev = u[t][q];
            g1[q] = live ? (1.0f - th * th) * sg * ev : 0.0f;
            g2[q] = live ? th * (sg * (1.0f - sg)) * ev : 0.0f;
        }
        float4 o1 = {g1[0], g1[1], g1[2], g1[3]}, o2 = {g2[0], g2[1], g2[2], g2[3]};
        if (a.conv_tanh) {
            const float4 y1 = *reinterpret_cast<const float4 *>(a.conv_tanh + at);
            const float4 y2 = *reinterpret_cast<const float4 *>(a.conv_tanh + at + R);
            o1 = float4{tanh_deriv(y1.x) * g1[0], tanh_deriv(y1.y) * g1[1], tanh_deriv(y1.z) * g1[2], tanh_deriv(y1.w) * g1[3]};
            o2 = float4{tanh_deriv(y2.x) * g2[0], tanh_deriv(y2.y) * g2[1], tanh_deriv(y2.z) * g2[2], tanh_deriv(y2.w) * g2[3]};
        }
        if (ok) {
            *reinterpret_cast<float4 *>(a.deltas + at) = o1;
            *reinterpret_cast<float4 *>(a.deltas + at + R) = o2;
        }
        cs1[t] = ok ? o1 : float4{0.0f, 0.0f, 0.0f, 0.0f};
        cs2[t] = ok ? o2 : float4{0.0f, 0.0f, 0.0f, 0.0f};
        if (a.ctx_tanh) {
            const float4 c1 = *reinterpret_cast<const float4 *>(a.ctx_tanh + at);
            const float4 c2 = *reinterpret_cast<const float4 *>(a.ctx_tanh + at + R);
            const float4 q1 = {tanh_deriv(c1.x) * g1[0], tanh_deriv(c1.y) * g1[1], tanh_deriv(c1.z) * g1[2], tanh_deriv(c1.w) * g1[3]};
            const float4 q2 = {tanh_deriv(c2.x) * g2[0], tanh_deriv(c2.y) * g2[1], tanh_deriv(c2.z) * g2[2], tanh_deriv(c2.w) * g2[3]};
            if (ok) {
                *reinterpret_cast<float4 *>(a.ctx_tanh + at) = q1;
                *reinterpret_cast<float4 *>(a.ctx_tanh + at + R) = q2;
            }
        }
    }
    if (a.colsum) {
        // sums over the wave's sixteen samples (lanes that share lane / 16), then over the workgroup's waves
        __shared__ float csum[NT / 64][2 * R];
        auto over_samples = [](float v) {
            v += __shfl_xor(v, 1); v += __shfl_xor(v, 2); v += __shfl_xor(v, 4); v += __shfl_xor(v, 8);
            return v;
        };
#pragma unroll
        for (int t = 0; t < RT; ++t) {
            const float4 u1 = {over_samples(cs1[t].x), over_samples(cs1[t].y), over_samples(cs1[t].z), over_samples(cs1[t].w)};
            const float4 u2 = {over_samples(cs2[t].x), over_samples(cs2[t].y), over_samples(cs2[t].z), over_samples(cs2[t].w)};
            if (col == 0) {
                *reinterpret_cast<float4 *>(&csum[wave][16 * t + 4 * quarter]) = u1;
                *reinterpret_cast<float4 *>(&csum[wave][R + 16 * t + 4 * quarter]) = u2;
            }
        }
        __syncthreads();
        if (tid < 2 * R) {
            float v = 0.0f;
#pragma unroll
            for (int w = 0; w < NT / 64; ++w) v += csum[w][tid];
            a.colsum[(size_t)blockIdx.x * 2 * R + tid] = v;
        }
    }
}

// out[d] = scale * sum over rows of partial[row][d] (the second half of a column sum whose first half rode in
// wavenet_block_errors_kernel); overwrites
constexpr int kColsumGroups = 4;
__global__ __launch_bounds__(64 * kColsumGroups) void colsum_finish_kernel(const float *__restrict__ partial, int rows, int D,
                                                                           float scale, float *__restrict__ out) {
    // 64 columns per block, four groups of lanes over the rows, eight loads in flight per lane.  Four waves and few registers:
    // a block finds room on a compute unit that a block-error workgroup (which leaves a tenth of the registers) occupies;
    // with sixteen waves it waited for that launch to end.
    constexpr int G = kColsumGroups;
    __shared__ float part[G][64];
    const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
    const int d = blockIdx.x * 64 + tx;
    float acc = 0.0f;
    if (d < D) {
        int r = ty;
        for (; r + 7 * G < rows; r += 8 * G) {
            float x[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) x[u] = partial[(size_t)(r + G * u) * D + d];
            acc += ((x[0] + x[1]) + (x[2] + x[3])) + ((x[4] + x[5]) + (x[6] + x[7]));
        }
        for (; r < rows; r += G) acc += partial[(size_t)r * D + d];
    }
    part[ty][tx] = acc;
    __syncthreads();
    if (ty == 0 && d < D) {
        float v = 0.0f;
#pragma unroll
        for (int q = 0; q < G; ++q) v += part[q][tx];
        out[d] = scale * v;
    }
}

struct FillList {
    float *ptr[kGemmMaxProb];
    unsigned long long count[kGemmMaxProb];
    int n;
};
// zeroes up to kGemmMaxProb small buffers in one launch (blockIdx.y = buffer)
__global__ void fill_zero_list_kernel(const FillList f) {
    float *p = f.ptr[blockIdx.y];
    const size_t count = f.count[blockIdx.y];
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < count; i += (size_t)gridDim.x * blockDim.x) p[i] = 0.0f;
}

typedef void (*block_err_kernel_t)(const BlockErrArgs);
block_err_kernel_t pick_block_errors_kernel(int R, int K, bool conv) {
#define CNT_BLOCK_KERNEL(r, k) \
    if (R == r && K == k) return conv ? wavenet_block_errors_kernel<r, k, true> : wavenet_block_errors_kernel<r, k, false>;
    CNT_BLOCK_KERNEL(64, 128)
    CNT_BLOCK_KERNEL(64, 256)
    CNT_BLOCK_KERNEL(64, 64)
    CNT_BLOCK_KERNEL(32, 128)
    CNT_BLOCK_KERNEL(32, 64)
    CNT_BLOCK_KERNEL(32, 32)
#undef CNT_BLOCK_KERNEL
    return nullptr;
}

__global__ void sum_context_grad_kernel(int C, int S, int resolution, size_t count, int N,
                                        const char *__restrict__ pat_frames, const char *__restrict__ pat,
                                        const float *__restrict__ ctx_grad, float *__restrict__ frame_grad) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) {
        const int f = (int)(i / C), c = (int)(i % C);
        float acc = 0.0f;
        if (pat_frames[f] != 0) {
            const int rel = f / S, s = f % S;
            for (int k = 0; k < resolution; ++k) {
                const int idx = (rel * resolution + k) * S + s;
                if (idx < N && pat[idx] != 0) acc += ctx_grad[(size_t)idx * C + c];
            }
        }
        frame_grad[i] = acc;
    }
}

constexpr int kSkipMaxFan = 8;
struct SkipPtrs {
    const float *in[kSkipMaxFan];
    float *target[kSkipMaxFan];
    int is_skip[kSkipMaxFan];
    int n;
};

__global__ void skipadd_forward_kernel(size_t count, SkipPtrs p, float *__restrict__ out, float *__restrict__ errors,
                                       float *__restrict__ errors_from_skip) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) {
        float acc = 0.0f;
        for (int k = 0; k < p.n; ++k) acc += p.in[k][i];
        out[i] = acc;
        if (errors) errors[i] = 0.0f;
        if (errors_from_skip) errors_from_skip[i] = 0.0f;
    }
}

__global__ void skipadd_backward_kernel(size_t count, SkipPtrs p, float *__restrict__ errors,
                                        const float *__restrict__ errors_from_skip) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) {
        const float e = errors_from_skip[i] + errors[i];
        errors[i] = e;
        for (int k = p.n - 1; k >= 0; --k) {
            if (p.is_skip[k]) p.target[k][i] = e + p.target[k][i];
            else p.target[k][i] = e;
        }
    }
}

}  // namespace
}  // namespace cnt

// ---------------------------------------------------------------------------------------------------
// CNN layer handle: filters grouped into runs of equal half width and tap interval
// ---------------------------------------------------------------------------------------------------
struct cnt_cnn_group {
    int d0, d1;   // filter range
    int hw, dil;  // half width, tap interval
    int col0;     // first weight column of the run
};

struct cnt_cnn {
    cnt_cnn_desc desc;
    int Lw;
    std::vector<cnt_cnn_group> groups;
};

extern "C" {

int cnt_cnn_create(const cnt_cnn_desc *desc, const int *half_width, const int *interval, cnt_cnn **out) {
    using namespace cnt;
    CNT_REQUIRE(desc && half_width && interval && out, "cnn_create: null argument");
    CNT_REQUIRE(desc->P > 0 && desc->D > 0 && desc->S > 0 && desc->maxT > 0, "cnn_create: non-positive size");
    cnt_cnn *h = new (std::nothrow) cnt_cnn();
    CNT_REQUIRE(h != nullptr, "cnn_create: out of host memory");
    h->desc = *desc;
    int col = 0;
    for (int d = 0; d < desc->D; ++d) {
        const int hw = half_width[d], dil = interval[d];
        const int taps = desc->causal > 0 ? hw + 1 : 2 * hw + 1;
        if (hw < 0 || dil < 1 || taps > kGemmMaxSeg) {
            set_error("cnn_create: filter %d has half width %d, tap interval %d; supported: interval >= 1 and at most %d "
                      "live taps per filter", d, hw, dil, kGemmMaxSeg);
            delete h;
            return CNT_ERR_ARG;
        }
        if (h->groups.empty() || h->groups.back().hw != hw || h->groups.back().dil != dil) {
            cnt_cnn_group g = {d, d + 1, hw, dil, col};
            h->groups.push_back(g);
        } else {
            h->groups.back().d1 = d + 1;
        }
        col += 2 * hw + 1;
    }
    h->Lw = col;
    *out = h;
    return CNT_OK;
}

int cnt_cnn_destroy(cnt_cnn *h) {
    delete h;
    return CNT_OK;
}

long cnt_cnn_weight_count(const cnt_cnn *h) { return h ? (long)h->desc.P * h->Lw + h->desc.D : 0; }

int cnt_cnn_forward(cnt_cnn *h, void *stream_, const char *patTypes, int curT, const float *weights, const float *x,
                    float *outputs) {
    using namespace cnt;
    CNT_REQUIRE(h && patTypes && weights && x && outputs, "cnn_forward: null argument");
    CNT_REQUIRE(curT >= 1 && curT <= h->desc.maxT, "cnn_forward: curT %d outside 1..%d", curT, h->desc.maxT);
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const cnt_cnn_desc &d = h->desc;
    const int P = d.P, D = d.D, S = d.S, N = curT * S;
    for (const cnt_cnn_group &g : h->groups) {
        GemmArgs ga = {};
        ga.m = g.d1 - g.d0; ga.n = N; ga.k = P;
        ga.a_kcontig = 1; ga.lda = (2 * g.hw + 1) * P;  // filter d, tap column c: weights[(col0 + (d-d0)*(2hw+1) + c) * P + p]
        ga.b_kcontig = 1; ga.ldb = P;
        ga.ldc = D;
        ga.nprob = 1; ga.splitk = 1;
        ga.epilogue = EPI_BIAS_ACT_SKIP; ga.act = d.output_tanh ? ACT_TANH : ACT_IDENTITY; ga.bias_scale = d.bias;
        ga.masked = 1; ga.b_time_on_k = 0; ga.n_slots = N; ga.pat = patTypes;
        int seg = 0;
        for (int shift = -g.hw; shift <= (d.causal > 0 ? 0 : g.hw); ++shift, ++seg) {
            ga.prob[0].A[seg] = weights + (size_t)(g.col0 + g.hw + shift) * P;
            ga.prob[0].B[seg] = x;
            ga.prob[0].b_shift[seg] = shift * g.dil * S;
        }
        ga.nseg = seg;
        ga.prob[0].C = outputs + g.d0;
        ga.prob[0].bias_vec = weights + (size_t)P * h->Lw + g.d0;
        ga.label = "gemm:cnn_forward";
        CNT_TRY(gemm_launch(stream, ga));
    }
    return CNT_OK;
}

int cnt_cnn_backward_errors(cnt_cnn *h, void *stream, const char *patTypes, int curT, const float *weights,
                            const float *outputs, float *output_errors, float *prev_errors, int delta_applied) {
    return cnt::cnn_backward_errors_fan(h, static_cast<hipStream_t>(stream), patTypes, curT, weights, outputs, output_errors,
                                        prev_errors, delta_applied, nullptr, nullptr);
}

extern "C++" int cnt::cnn_backward_errors_fan(cnt_cnn *h, hipStream_t stream, const char *patTypes, int curT,
                                              const float *weights, const float *outputs, float *output_errors,
                                              float *prev_errors, int delta_applied, const FanOut *fan, bool *fused) {
    if (fused) *fused = false;
    CNT_REQUIRE(h && patTypes && weights && outputs && output_errors, "cnn_backward_errors: null argument");
    CNT_REQUIRE(curT >= 1 && curT <= h->desc.maxT, "cnn_backward_errors: curT %d outside 1..%d", curT, h->desc.maxT);
    const cnt_cnn_desc &d = h->desc;
    const int P = d.P, D = d.D, S = d.S, N = curT * S;
    const size_t count = (size_t)D * N;

    if (d.output_tanh && !delta_applied) {
        ProfileScope prof(stream, "cnn_tanh_delta");
        hipLaunchKernelGGL(tanh_delta_kernel, dim3(stream_blocks(count)), dim3(256), 0, stream, output_errors, outputs,
                           count);
        CNT_HIP(hipGetLastError());
    }

    if (prev_errors) {
        // the reference clears the whole preceding error buffer, then overwrites the current slots
        const size_t used = (size_t)P * N, cap = (size_t)P * d.maxT * S;
        if (cap > used) CNT_TRY(fill_zero(stream, prev_errors + used, cap - used));
        bool first = true;
        for (const cnt_cnn_group &g : h->groups) {
            GemmArgs ga = {};
            ga.m = P; ga.n = N; ga.k = g.d1 - g.d0;
            ga.a_kcontig = 0; ga.lda = (2 * g.hw + 1) * P;
            ga.b_kcontig = 1; ga.ldb = D;
            ga.ldc = P;
            ga.nprob = 1; ga.splitk = 1;
            ga.epilogue = first ? EPI_STORE : EPI_ADD;
            ga.masked = 1; ga.b_time_on_k = 0; ga.n_slots = N; ga.pat = patTypes;
            int seg = 0;
            for (int shift = -g.hw; shift <= (d.causal > 0 ? 0 : g.hw); ++shift, ++seg) {
                ga.prob[0].A[seg] = weights + (size_t)(g.col0 + g.hw + shift) * P;
                ga.prob[0].B[seg] = output_errors + g.d0;
                // column (slot u, tap shift) of the reference's buffer holds the delta of slot u - shift*dil*S
                ga.prob[0].b_shift[seg] = -shift * g.dil * S;
            }
            ga.nseg = seg;
            ga.prob[0].C = prev_errors;
            if (fan && fused && h->groups.size() == 1 && gemm_fan_supported(ga)) {
                ga.epilogue = EPI_FAN;
                ga.fan_n = fan->n; ga.fan_targets = fan->targets; ga.fan_is_skip = fan->is_skip;
                ga.prob[0].aux_in = fan->from_skip;
                *fused = true;
            }
            ga.label = "gemm:cnn_prev_errors";
            CNT_TRY(gemm_launch(stream, ga));
            first = false;
        }
    }
    return CNT_OK;
}

extern "C++" int cnt::cnn_batch_taps(const cnt_cnn *h) {
    if (!h || h->groups.size() != 1) return 0;
    const cnt_cnn_group &g = h->groups[0];
    return h->desc.causal > 0 ? g.hw + 1 : 2 * g.hw + 1;
}

extern "C++" bool cnt::cnn_batch_compatible(const cnt_cnn *a, const cnt_cnn *b) {
    if (cnn_batch_taps(a) == 0 || cnn_batch_taps(a) != cnn_batch_taps(b)) return false;
    const cnt_cnn_group &ga = a->groups[0], &gb = b->groups[0];
    return a->desc.P == b->desc.P && a->desc.D == b->desc.D && a->desc.S == b->desc.S && a->Lw == b->Lw &&
           (a->desc.causal > 0) == (b->desc.causal > 0) && ga.hw == gb.hw && ga.d0 == gb.d0 && ga.d1 == gb.d1 &&
           ga.col0 == gb.col0;
}

extern "C++" int cnt::cnn_backward_weights_batch(cnt_cnn *const *h, int count, hipStream_t stream, const char *patTypes,
                                                 int curT, const float *const *x, const float *const *output_errors,
                                                 float *const *weight_updates, const float *const *colsum_partial,
                                                 const int *colsum_rows) {
    CNT_REQUIRE(h && patTypes && x && output_errors && weight_updates && count >= 1, "cnn_backward_weights: null argument");
    const int taps = cnn_batch_taps(h[0]);
    CNT_REQUIRE(taps > 0 && count * taps <= kGemmMaxProb, "cnn_backward_weights: %d layers of %d taps in one launch", count,
                taps);
    for (int z = 0; z < count; ++z) {
        CNT_REQUIRE(cnn_batch_compatible(h[0], h[z]), "cnn_backward_weights: layers of different shapes in one launch");
        CNT_REQUIRE(x[z] && output_errors[z] && weight_updates[z], "cnn_backward_weights: null argument");
        CNT_REQUIRE(curT >= 1 && curT <= h[z]->desc.maxT, "cnn_backward_weights: curT %d outside 1..%d", curT,
                    h[z]->desc.maxT);
    }
    const cnt_cnn_desc &d = h[0]->desc;
    const cnt_cnn_group &g0 = h[0]->groups[0];
    const int P = d.P, D = d.D, S = d.S, N = curT * S;
    {
        FillList fl = {};
        size_t most = 0;
        for (int z = 0; z < count; ++z) {
            fl.ptr[z] = weight_updates[z];
            fl.count[z] = (size_t)P * h[z]->Lw + D;
            most = std::max(most, (size_t)fl.count[z]);
        }
        fl.n = count;
        hipLaunchKernelGGL(fill_zero_list_kernel, dim3((unsigned)std::min<size_t>((most + 255) / 256, 256), count), dim3(256), 0,
                           stream, fl);
        CNT_HIP(hipGetLastError());
    }
    GemmArgs ga = {};
    ga.m = P; ga.n = g0.d1 - g0.d0; ga.k = N;
    ga.a_kcontig = 0; ga.lda = P;
    ga.b_kcontig = 0; ga.ldb = D;
    ga.ldc = (2 * g0.hw + 1) * P;
    ga.nseg = 1;
    ga.epilogue = EPI_ATOMIC;
    ga.masked = 1; ga.b_time_on_k = 1; ga.n_slots = N; ga.pat = patTypes;
    int pr = 0;
    for (int z = 0; z < count; ++z) {
        const cnt_cnn_group &g = h[z]->groups[0];
        for (int shift = -g.hw; shift <= (d.causal > 0 ? 0 : g.hw); ++shift, ++pr) {
            ga.prob[pr].A[0] = x[z];
            ga.prob[pr].B[0] = output_errors[z] + g.d0;
            ga.prob[pr].b_shift[0] = -shift * g.dil * S;
            ga.prob[pr].C = weight_updates[z] + (size_t)(g.col0 + g.hw + shift) * P;
        }
    }
    ga.nprob = pr;
    ga.splitk = 0;  // chosen by the launcher
    ga.overwrite_ok = 1;
    ga.label = "gemm:cnn_dW";
    CNT_TRY(gemm_launch(stream, ga));
    for (int z = 0; z < count; ++z) {
        float *bias_grad = weight_updates[z] + (size_t)P * h[z]->Lw;
        if (colsum_partial && colsum_partial[z] && colsum_rows[z] > 0) {
            // the launch that wrote these deltas summed them per workgroup
            hipLaunchKernelGGL(colsum_finish_kernel, dim3((D + 63) / 64), dim3(64 * kColsumGroups), 0, stream, colsum_partial[z],
                               colsum_rows[z], D, h[z]->desc.bias, bias_grad);
            CNT_HIP(hipGetLastError());
        } else {
            CNT_TRY(column_sum(stream, output_errors[z], D, N, h[z]->desc.bias, bias_grad));
        }
    }
    return CNT_OK;
}

int cnt_cnn_backward_weights(cnt_cnn *h, void *stream_, const char *patTypes, int curT, const float *x,
                             const float *output_errors, float *weight_updates) {
    using namespace cnt;
    CNT_REQUIRE(h && patTypes && x && output_errors && weight_updates, "cnn_backward_weights: null argument");
    CNT_REQUIRE(curT >= 1 && curT <= h->desc.maxT, "cnn_backward_weights: curT %d outside 1..%d", curT, h->desc.maxT);
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const cnt_cnn_desc &d = h->desc;
    const int P = d.P, D = d.D, S = d.S, N = curT * S;

    CNT_TRY(fill_zero(stream, weight_updates, (size_t)P * h->Lw + D));
    for (const cnt_cnn_group &g : h->groups) {
        GemmArgs ga = {};
        ga.m = P; ga.n = g.d1 - g.d0; ga.k = N;
        ga.a_kcontig = 0; ga.lda = P;
        ga.b_kcontig = 0; ga.ldb = D;
        ga.ldc = (2 * g.hw + 1) * P;
        ga.nseg = 1;
        ga.epilogue = EPI_ATOMIC;
        ga.masked = 1; ga.b_time_on_k = 1; ga.n_slots = N; ga.pat = patTypes;
        int pr = 0;
        for (int shift = -g.hw; shift <= (d.causal > 0 ? 0 : g.hw); ++shift, ++pr) {
            ga.prob[pr].A[0] = x;
            ga.prob[pr].B[0] = output_errors + g.d0;
            ga.prob[pr].b_shift[0] = -shift * g.dil * S;
            ga.prob[pr].C = weight_updates + (size_t)(g.col0 + g.hw + shift) * P;
        }
        ga.nprob = pr;
        ga.splitk = 0;  // chosen by the launcher
        ga.overwrite_ok = 1;  // every tap's P x (d1 - d0) block is written whole; the rest stays as cleared above
        ga.label = "gemm:cnn_dW";
        CNT_TRY(gemm_launch(stream, ga));
    }
    // bias gradient over every slot, padding included, as the reference's ones-vector product does
    return column_sum(stream, output_errors, D, N, d.bias, weight_updates + (size_t)P * h->Lw);
}

int cnt_cnn_backward(cnt_cnn *h, void *stream, const char *patTypes, int curT, const float *weights, const float *x,
                     const float *outputs, float *output_errors, float *prev_errors, float *weight_updates) {
    using namespace cnt;
    CNT_REQUIRE(x && weight_updates, "cnn_backward: null argument");
    CNT_TRY(cnt_cnn_backward_errors(h, stream, patTypes, curT, weights, outputs, output_errors, prev_errors, 0));
    return cnt_cnn_backward_weights(h, stream, patTypes, curT, x, output_errors, weight_updates);
}

// ---------------------------------------------------------------------------------------------------
// Conditioned / unconditioned gated activation
// ---------------------------------------------------------------------------------------------------
int cnt_wavnetc_load_context(void *stream_, int C, int S, int N, int max_feature_length, int resolution_one,
                             const float *source, const float *frame_index, const float *mean_std,
                             const char *patTypes, float *ctx) {
    using namespace cnt;
    CNT_REQUIRE(source && frame_index && patTypes && ctx, "wavnetc_load_context: null argument");
    CNT_REQUIRE(C > 0 && S > 0 && N > 0, "wavnetc_load_context: non-positive size");
    const size_t count = (size_t)C * N;
    hipLaunchKernelGGL(load_context_kernel, dim3(stream_blocks(count)), dim3(256), 0, static_cast<hipStream_t>(stream_),
                       C, S, count, max_feature_length, resolution_one, source, frame_index, mean_std, patTypes, ctx);
    CNT_HIP(hipGetLastError());
    return CNT_OK;
}

int cnt_gatedact_forward(void *stream_, int D, int N, const char *patTypes, const float *pre, float *outputs) {
    using namespace cnt;
    CNT_REQUIRE(patTypes && pre && outputs, "gatedact_forward: null argument");
    CNT_REQUIRE(D > 0 && N > 0, "gatedact_forward: non-positive size");
    const size_t count = (size_t)D * N;
    ProfileScope prof(static_cast<hipStream_t>(stream_), "gated_forward");
    hipLaunchKernelGGL(gated_forward_kernel, dim3(stream_blocks(count)), dim3(256), 0,
                       static_cast<hipStream_t>(stream_), D, count, patTypes, pre, outputs);
    CNT_HIP(hipGetLastError());
    return CNT_OK;
}

int cnt_gatedact_backward(void *stream_, int D, int N, const char *patTypes, const float *pre, const float *output_errors,
                          float *prev_errors) {
    using namespace cnt;
    CNT_REQUIRE(patTypes && pre && output_errors && prev_errors, "gatedact_backward: null argument");
    CNT_REQUIRE(D > 0 && N > 0, "gatedact_backward: non-positive size");
    const size_t count = (size_t)D * N;
    ProfileScope prof(static_cast<hipStream_t>(stream_), "gated_backward");
    return launch_gated_backward(static_cast<hipStream_t>(stream_), D, count, patTypes, pre, output_errors, prev_errors,
                                 nullptr, nullptr);
}

int cnt_wavnetc_forward(void *stream_, int D, int C, int N, const char *patTypes, const float *weights, const float *ctx,
                        const float *conv_outputs, float *core_buf, float *ctx_tanh, float *outputs) {
    using namespace cnt;
    CNT_REQUIRE(patTypes && conv_outputs && core_buf && outputs, "wavnetc_forward: null argument");
    CNT_REQUIRE(D > 0 && N > 0 && C >= 0, "wavnetc_forward: bad size");
    CNT_REQUIRE(C == 0 || (weights && ctx), "wavnetc_forward: conditioning needs weights and context");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const size_t count2 = (size_t)2 * D * N;
    if (C == 0) {
        hipLaunchKernelGGL(core_copy_kernel, dim3(stream_blocks(count2)), dim3(256), 0, stream, 2 * D, count2, patTypes,
                           conv_outputs, core_buf, ctx_tanh);
        CNT_HIP(hipGetLastError());
    } else {
        // X_c = W^T ctx with the tanh, the sum with the convolution output and the padding mask in the epilogue
        GemmArgs ga = {};
        ga.m = 2 * D; ga.n = N; ga.k = C;
        ga.a_kcontig = 1; ga.lda = C;
        ga.b_kcontig = 1; ga.ldb = C;
        ga.ldc = 2 * D;
        ga.nseg = 1; ga.nprob = 1; ga.splitk = 1;
        ga.epilogue = EPI_CONTEXT; ga.pat = patTypes;
        ga.prob[0].A[0] = weights; ga.prob[0].B[0] = ctx; ga.prob[0].C = core_buf;
        ga.prob[0].aux_in = conv_outputs; ga.prob[0].aux_out = ctx_tanh;
        ga.label = "gemm:wavnetc_context";
        CNT_TRY(gemm_launch(stream, ga));
    }
    return cnt_gatedact_forward(stream_, D, N, patTypes, core_buf, outputs);
}

extern "C++" bool cnt::wavenet_block_errors_supported(int R, int K) { return pick_block_errors_kernel(R, K, false) != nullptr; }

extern "C++" int cnt::wavenet_block_rows(int N, bool fold) { return fold ? (N + 127) / 128 : (N + 63) / 64; }

extern "C++" bool cnt::cnn_foldable(const cnt_cnn *h, int R) {
    // one run of filters, causal, two live taps, R inputs and 2R filters
    return h && h->groups.size() == 1 && h->desc.causal > 0 && h->groups[0].hw == 1 && h->groups[0].d0 == 0 &&
           h->groups[0].d1 == h->desc.D && h->desc.P == R && h->desc.D == 2 * R;
}

extern "C++" int cnt::wavenet_block_errors(hipStream_t stream, int R, int K, int N, const char *patTypes,
                                           const float *skip_weights, const float *out_weights, const float *skip_errors,
                                           float *total, const FanOut *fan, const float *core_buf, float *ctx_tanh,
                                           const float *conv_tanh_outputs, float *conv_errors, const cnt_cnn *fold,
                                           const float *fold_weights, const float *fold_deltas, float *colsum_partial) {
    block_err_kernel_t k = pick_block_errors_kernel(R, K, fold != nullptr);
    CNT_REQUIRE(k != nullptr, "wavenet_block_errors: no kernel for %d residual and %d skip channels", R, K);
    CNT_REQUIRE(N > 0 && patTypes && skip_weights && out_weights && skip_errors && total && core_buf && conv_errors,
                "wavenet_block_errors: null argument");
    BlockErrArgs a = {};
    a.N = N; a.pat = patTypes; a.w_skip = skip_weights; a.w_out = out_weights; a.e_skip = skip_errors;
    a.total = total;
    if (fan) { a.from_skip = fan->from_skip; a.fan_n = fan->n; a.fan_targets = fan->targets; a.fan_is_skip = fan->is_skip; }
    a.pre = core_buf; a.conv_tanh = conv_tanh_outputs; a.ctx_tanh = ctx_tanh; a.deltas = conv_errors;
    a.colsum = colsum_partial;
    auto aligned = [](const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
    if (fold) {
        CNT_REQUIRE(cnn_foldable(fold, R) && fold_weights && fold_deltas && aligned(fold_weights) && aligned(fold_deltas),
                    "wavenet_block_errors: this convolution layer cannot be folded into the block");
        const cnt_cnn_group &g = fold->groups[0];
        const int P = fold->desc.P;
        a.conv_ld = (2 * g.hw + 1) * P;
        for (int tap = 0; tap < 2; ++tap) {
            const int shift = -tap;  // taps at shift 0 and -1 (cnn_backward_errors_fan)
            a.conv_w[tap] = fold_weights + (size_t)(g.col0 + g.hw + shift) * P;
            a.conv_shift[tap] = -shift * g.dil * fold->desc.S;
        }
        a.conv_deltas = fold_deltas;
    }
    CNT_REQUIRE(aligned(skip_weights) && aligned(out_weights) && aligned(skip_errors) && aligned(total) &&
                aligned(a.from_skip) && aligned(core_buf) && aligned(ctx_tanh) && aligned(conv_tanh_outputs) &&
                aligned(conv_errors), "wavenet_block_errors: buffers must be 16-byte aligned");
    ProfileScope prof(stream, fold ? "wavenet_block_errors+cnn" : "wavenet_block_errors");
    hipLaunchKernelGGL(k, dim3(wavenet_block_rows(N, fold != nullptr)), dim3(fold ? 512 : 256), 0, stream, a);
    CNT_HIP(hipGetLastError());
    return CNT_OK;
}

extern "C++" int cnt::wavnetc_context_grad(hipStream_t stream, int D, int C, int N, const float *weights,
                                           const float *ctx_tanh, float *ctx_grad) {
    GemmArgs ga = {};
    ga.m = C; ga.n = N; ga.k = 2 * D;
    ga.a_kcontig = 0; ga.lda = C;
    ga.b_kcontig = 1; ga.ldb = 2 * D;
    ga.ldc = C;
    ga.nseg = 1; ga.nprob = 1; ga.splitk = 1; ga.epilogue = EPI_ADD;
    ga.prob[0].A[0] = weights; ga.prob[0].B[0] = ctx_tanh; ga.prob[0].C = ctx_grad;
    ga.label = "gemm:wavnetc_ctx_grad";
    return gemm_launch(stream, ga);
}

int cnt_wavnetc_backward_errors(void *stream_, int D, int C, int N, const char *patTypes, const float *weights,
                                const float *core_buf, float *ctx_tanh, const float *output_errors, float *prev_errors,
                                float *ctx_grad, const float *prev_tanh_outputs) {
    using namespace cnt;
    CNT_REQUIRE(patTypes && core_buf && output_errors && prev_errors, "wavnetc_backward: null argument");
    CNT_REQUIRE(D > 0 && N > 0 && C >= 0, "wavnetc_backward: bad size");
    CNT_REQUIRE(C == 0 || ctx_tanh, "wavnetc_backward: conditioning needs the tanh buffer");
    CNT_REQUIRE(!ctx_grad || weights, "wavnetc_backward: the context gradient needs the weights");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const size_t count = (size_t)D * N;
    {
        ProfileScope prof(stream, "gated_backward");
        CNT_TRY(launch_gated_backward(stream, D, count, patTypes, core_buf, output_errors, prev_errors,
                                      C > 0 ? ctx_tanh : nullptr, prev_tanh_outputs));
    }
    if (C > 0 && ctx_grad) CNT_TRY(wavnetc_context_grad(stream, D, C, N, weights, ctx_tanh, ctx_grad));
    return CNT_OK;
}

int cnt_wavnetc_backward_weights(void *stream, int D, int C, int N, const float *ctx, const float *ctx_tanh,
                                 float *weight_updates) {
    return cnt::wavnetc_backward_weights_batch(static_cast<hipStream_t>(stream), D, C, N, 1, ctx, &ctx_tanh, &weight_updates);
}

extern "C++" int cnt::wavnetc_backward_weights_batch(hipStream_t stream, int D, int C, int N, int count, const float *ctx,
                                                     const float *const *ctx_tanh, float *const *weight_updates) {
    CNT_REQUIRE(count >= 1 && count <= kGemmMaxProb, "wavnetc_backward_weights: %d layers in one launch, supported 1..%d",
                count, kGemmMaxProb);
    CNT_REQUIRE(D > 0 && N > 0 && C >= 0, "wavnetc_backward_weights: bad size");
    if (C == 0) return CNT_OK;
    CNT_REQUIRE(ctx && ctx_tanh && weight_updates, "wavnetc_backward_weights: null argument");
    GemmArgs ga = {};
    ga.m = C; ga.n = 2 * D; ga.k = N;
    ga.a_kcontig = 0; ga.lda = C;
    ga.b_kcontig = 0; ga.ldb = 2 * D;
    ga.ldc = C;
    ga.nseg = 1; ga.nprob = count; ga.epilogue = EPI_ATOMIC;
    ga.splitk = 0;  // chosen by the launcher
    for (int z = 0; z < count; ++z) {
        CNT_REQUIRE(ctx_tanh[z] && weight_updates[z], "wavnetc_backward_weights: null argument");
        ga.prob[z].A[0] = ctx; ga.prob[z].B[0] = ctx_tanh[z]; ga.prob[z].C = weight_updates[z];
    }
    ga.label = "gemm:wavnetc_dW";
    ga.overwrite_ok = 1;  // the product covers all C x 2D weights
    gemm_plan(ga, stream);
    if (ga.epilogue != EPI_PARTIAL)
        for (int z = 0; z < count; ++z) CNT_TRY(fill_zero(stream, weight_updates[z], (size_t)C * 2 * D));
    return gemm_launch(stream, ga);
}

int cnt_wavnetc_backward(void *stream, int D, int C, int N, const char *patTypes, const float *weights, const float *ctx,
                         const float *core_buf, float *ctx_tanh, const float *output_errors, float *prev_errors,
                         float *weight_updates, float *ctx_grad) {
    using namespace cnt;
    CNT_REQUIRE(C == 0 || (weights && ctx && ctx_tanh && weight_updates),
                "wavnetc_backward: conditioning needs weights, context, tanh buffer and weight updates");
    CNT_TRY(cnt_wavnetc_backward_errors(stream, D, C, N, patTypes, weights, core_buf, ctx_tanh, output_errors, prev_errors,
                                        ctx_grad, nullptr));
    return cnt_wavnetc_backward_weights(stream, D, C, N, ctx, ctx_tanh, weight_updates);
}

int cnt_wavnetc_sum_context_grad(void *stream_, int C, int S, int resolution, int n_frame_slots, int N,
                                 const char *pat_frames, const char *patTypes, const float *ctx_grad,
                                 float *frame_grad) {
    using namespace cnt;
    CNT_REQUIRE(pat_frames && patTypes && ctx_grad && frame_grad, "wavnetc_sum_context_grad: null argument");
    CNT_REQUIRE(C > 0 && S > 0 && resolution > 0 && n_frame_slots > 0 && N > 0, "wavnetc_sum_context_grad: bad size");
    const size_t count = (size_t)C * n_frame_slots;
    hipLaunchKernelGGL(sum_context_grad_kernel, dim3(stream_blocks(count)), dim3(256), 0,
                       static_cast<hipStream_t>(stream_), C, S, resolution, count, N, pat_frames, patTypes, ctx_grad,
                       frame_grad);
    CNT_HIP(hipGetLastError());
    return CNT_OK;
}

// ---------------------------------------------------------------------------------------------------
// Skip-add
// ---------------------------------------------------------------------------------------------------
int cnt_skipadd_forward(void *stream_, long count, int n_in, const float *const *inputs, float *outputs,
                        float *errors, float *errors_from_skip) {
    using namespace cnt;
    CNT_REQUIRE(inputs && outputs, "skipadd_forward: null argument");
    CNT_REQUIRE(count > 0 && n_in >= 1 && n_in <= kSkipMaxFan, "skipadd_forward: %d inputs, supported 1..%d", n_in,
                kSkipMaxFan);
    SkipPtrs p = {};
    p.n = n_in;
    for (int k = 0; k < n_in; ++k) {
        CNT_REQUIRE(inputs[k], "skipadd_forward: null input %d", k);
        p.in[k] = inputs[k];
    }
    ProfileScope prof(static_cast<hipStream_t>(stream_), "skipadd_forward");
    hipLaunchKernelGGL(skipadd_forward_kernel, dim3(stream_blocks((size_t)count)), dim3(256), 0,
                       static_cast<hipStream_t>(stream_), (size_t)count, p, outputs, errors, errors_from_skip);
    CNT_HIP(hipGetLastError());
    return CNT_OK;
}

int cnt_skipadd_backward(void *stream_, long count, float *errors, const float *errors_from_skip, int n_pre,
                         float *const *targets, const int *target_is_skip) {
    using namespace cnt;
    CNT_REQUIRE(errors && errors_from_skip && targets && target_is_skip, "skipadd_backward: null argument");
    CNT_REQUIRE(count > 0 && n_pre >= 1 && n_pre <= kSkipMaxFan, "skipadd_backward: %d predecessors, supported 1..%d",
                n_pre, kSkipMaxFan);
    SkipPtrs p = {};
    p.n = n_pre;
    for (int k = 0; k < n_pre; ++k) {
        CNT_REQUIRE(targets[k], "skipadd_backward: null target %d", k);
        p.target[k] = targets[k];
        p.is_skip[k] = target_is_skip[k];
    }
    ProfileScope prof(static_cast<hipStream_t>(stream_), "skipadd_backward");
    hipLaunchKernelGGL(skipadd_backward_kernel, dim3(stream_blocks((size_t)count)), dim3(256), 0,
                       static_cast<hipStream_t>(stream_), (size_t)count, p, errors, errors_from_skip);
    CNT_HIP(hipGetLastError());
    return CNT_OK;
}

}  // extern "C"
