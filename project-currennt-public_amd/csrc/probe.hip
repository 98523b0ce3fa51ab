// Measurement hook: the latency floor of one step of a recursion that is spread over compute units.
//
// However a recurrent layer is cut up, a time step ends with every compute unit that holds a slice of the recurrent
// weights having told every other one its share -- one hop through memory that both sides can see -- and the next
// step cannot start before that.  This kernel measures that hop the way the recursion kernels make it (a store, and
// a polling load that bypasses the per-CU cache), between two workgroups on the same XCD (through its L2) or on
// different XCDs (through the memory side), optionally with the arithmetic of a step between receiving and sending:
// a round trip through LDS, the cell update's chain of about twenty dependent operations, and the thirty-two
// v_mfma_f32_4x4x1 of a 256-cell slice's product.  T times the result is the time below which no schedule of a
// T-step recursion can get on this machine; the benchmark prints it next to what the recursion kernel takes.
#include "common.hpp"

namespace cnt {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(64) void hop_probe_kernel(unsigned *ctl, unsigned *mail, int rounds, int same_xcd, int with_compute,
                                                       long long *ticks) {
    __shared__ int role_sh;
    __shared__ float lds[64];
    if (threadIdx.x == 0) {
        const unsigned xcd = __builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20) & 15u;  // XCC_ID
        int r = -1;
        if (xcd == 0u) {
            const unsigned t = atomicAdd(&ctl[0], 1u);
            if (t == 0u || (same_xcd && t == 1u)) r = (int)t;
        } else if (!same_xcd) {  // any XCD other than the first role's
            if (atomicAdd(&ctl[1], 1u) == 0u) r = 1;
        }
        role_sh = r;
    }
    __syncthreads();
    const int r = role_sh;
    if (r < 0) return;
    // word 0 is written by role 0 and read by role 1, word 64 the other way; stores to another XCD go to the device-
    // coherent level, stores inside an XCD stay in its L2
    unsigned *mine = mail + (r ? 64 : 0), *theirs = mail + (r ? 0 : 64);
    float carry = 1.0f;
    f32x4 acc = {0, 0, 0, 0};
    const long long t0 = wall_clock64();
    bool ok = true;
    for (int i = 1; i <= rounds && ok; ++i) {
        for (int half = 0; half < 2; ++half) {
            const bool sender = (half == 0) == (r == 0);
            if (sender) {
                if (with_compute) {
                    // what a step does between the arrival of the partial errors and the departure of its own
                    lds[threadIdx.x] = carry;
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
                    __builtin_amdgcn_s_barrier();
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
                    float v = lds[(threadIdx.x + 1) & 63];
#pragma unroll
                    for (int q = 0; q < 20; ++q) v = v * 0.999f + 0.001f;
#pragma unroll
                    for (int q = 0; q < 32; ++q) acc = __builtin_amdgcn_mfma_f32_4x4x1f32(v, carry, acc, 0, 0, 0);
                    carry = acc[0] * 1e-30f + 1.0f;
                }
                if (threadIdx.x == 0) {
                    const unsigned word = (unsigned)i + (carry == 12345.0f ? 1u : 0u);
                    if (same_xcd) asm volatile("global_store_dword %0, %1, off" ::"v"(mine), "v"(word) : "memory");
                    else asm volatile("global_store_dword %0, %1, off sc1" ::"v"(mine), "v"(word) : "memory");
                }
            } else {
                unsigned v = 0, spins = 0;
                do {
                    asm volatile("global_load_dword %0, %1, off sc1\n s_waitcnt vmcnt(0)" : "=v"(v) : "v"(theirs) : "memory");
                } while (v != (unsigned)i && ++spins < (1u << 20));
                if (v != (unsigned)i) ok = false;  // every wait is bounded: the kernel always ends
            }
        }
    }
    if (threadIdx.x == 0) {
        ticks[r] = wall_clock64() - t0;
        if (!ok) ticks[2] = 1;
    }
}

// The same hop for a message of `pieces` x 4 KB between two workgroups of four waves on one XCD, the way a recursion
// step receives: every lane polls its 16-byte pieces (all in flight together) until each carries the round's tag, the
// waves meet at a barrier, then the workgroup answers with a message of the same size.  4 KB is what a workgroup of a
// 256-cell recursion receives per step when outputs (forward, gather form) or partial errors (backward) travel;
// 16 KB is what it would receive if the forward recursion sent partial pre-activations of four gates instead.
__global__ __launch_bounds__(256) void hop_message_kernel(unsigned *ctl, unsigned *mail, int rounds, int pieces, long long *ticks) {
    __shared__ int role_sh;
    typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
    if (threadIdx.x == 0) {
        const unsigned xcd = __builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20) & 15u;  // XCC_ID
        int r = -1;
        if (xcd == 0u) {
            const unsigned t = atomicAdd(&ctl[0], 1u);
            if (t < 2u) r = (int)t;
        }
        role_sh = r;
    }
    __syncthreads();
    const int r = role_sh;
    if (r < 0) return;
    const size_t words = (size_t)pieces * 1024;  // per direction
    unsigned *mine = mail + (r ? words : 0), *theirs = mail + (r ? 0 : words);
    const long long t0 = wall_clock64();
    bool ok = true;
    for (int i = 1; i <= rounds && ok; ++i) {
        for (int half = 0; half < 2; ++half) {
            const bool sender = (half == 0) == (r == 0);
            if (sender) {
                const u32x4 v = {(unsigned)i, (unsigned)i, (unsigned)i, (unsigned)i};
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    if (q < pieces)
                        asm volatile("global_store_dwordx4 %0, %1, off" ::"v"(mine + (size_t)q * 1024 + threadIdx.x * 4), "v"(v) : "memory");
            } else {
                unsigned spins = 0;
                bool all = false;
                do {
                    u32x4 w[4];
                    unsigned worst = (unsigned)i;
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        if (q < pieces)
                            asm volatile("global_load_dwordx4 %0, %1, off sc1" : "=v"(w[q]) : "v"(theirs + (size_t)q * 1024 + threadIdx.x * 4) : "memory");
                    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        if (q >= pieces) continue;
                        asm volatile("" : "+v"(w[q]));
                        if (w[q].x != (unsigned)i || w[q].y != (unsigned)i || w[q].z != (unsigned)i || w[q].w != (unsigned)i) worst = 0u;
                    }
                    all = __builtin_amdgcn_ballot_w64(worst != (unsigned)i) == 0;
                } while (!all && ++spins < (1u << 20));
                if (!all) ok = false;  // every wait is bounded: the kernel always ends
                __syncthreads();
            }
        }
    }
    if (threadIdx.x == 0) {
        ticks[r] = wall_clock64() - t0;
        if (!ok) ticks[2] = 1;
    }
}

// the activation functions as the recursion kernels evaluate them, element by element (a test hook)
__global__ void activations_kernel(size_t n, const float *__restrict__ x, float *__restrict__ out, int which) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const float v = x[i];
    out[i] = which == 0 ? logistic(v) : which == 1 ? tanh_act(v) : which == 2 ? logistic_quick(v) : tanh_quick(v);
}

}  // namespace
}  // namespace cnt

extern "C" int cnt_probe_activation(void *stream, int which, long n, const float *x, float *out) {
    using namespace cnt;
    CNT_REQUIRE(which >= 0 && which <= 3, "probe_activation: function %d, known 0..3", which);
    CNT_REQUIRE(n >= 0 && (n == 0 || (x && out)), "probe_activation: bad argument");
    if (n == 0) return CNT_OK;
    hipLaunchKernelGGL(activations_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       (size_t)n, x, out, which);
    CNT_HIP(hipGetLastError());
    return CNT_OK;
}

extern "C" int cnt_probe_hop_latency(void *stream_, int same_xcd, int with_compute, int rounds, float *hop_us) {
    using namespace cnt;
    CNT_REQUIRE(hop_us, "probe_hop_latency: null argument");
    CNT_REQUIRE(rounds >= 1 && rounds <= 100000, "probe_hop_latency: 1..100000 rounds");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    unsigned *buf = nullptr;
    CNT_HIP(hipMalloc(reinterpret_cast<void **>(&buf), 4096));
    int status = CNT_OK;
    long long host_ticks[3] = {0, 0, 0};
    do {
        if (hipMemsetAsync(buf, 0, 4096, stream) != hipSuccess) { status = CNT_ERR_HIP; break; }
        unsigned *ctl = buf, *mail = buf + 64;
        long long *ticks = reinterpret_cast<long long *>(buf + 512);
        // 256 small workgroups spread over every XCD; two of them take the roles, the others end at once
        hipLaunchKernelGGL(hop_probe_kernel, dim3(256), dim3(64), 0, stream, ctl, mail, rounds, same_xcd != 0, with_compute != 0,
                           ticks);
        if (hipGetLastError() != hipSuccess || hipStreamSynchronize(stream) != hipSuccess ||
            hipMemcpy(host_ticks, ticks, sizeof(host_ticks), hipMemcpyDeviceToHost) != hipSuccess)
            status = CNT_ERR_HIP;
    } while (false);
    (void)hipFree(buf);
    if (status != CNT_OK) {
        set_error("probe_hop_latency: HIP call failed: %s", hipGetErrorString(hipGetLastError()));
        return status;
    }
    if (host_ticks[2] != 0 || host_ticks[0] == 0 || host_ticks[1] == 0) {
        set_error("probe_hop_latency: the two workgroups did not meet (placement or visibility)");
        return CNT_ERR_DEVICE;
    }
    // 100 MHz clock; a round is two hops
    *hop_us = (float)((double)(host_ticks[0] > host_ticks[1] ? host_ticks[0] : host_ticks[1]) * 0.01 / rounds / 2.0);
    return CNT_OK;
}

extern "C" int cnt_probe_hop_message(void *stream_, int kilobytes, int rounds, float *hop_us) {
    using namespace cnt;
    CNT_REQUIRE(hop_us, "probe_hop_message: null argument");
    CNT_REQUIRE(rounds >= 1 && rounds <= 100000, "probe_hop_message: 1..100000 rounds");
    CNT_REQUIRE(kilobytes == 4 || kilobytes == 8 || kilobytes == 12 || kilobytes == 16, "probe_hop_message: 4, 8, 12 or 16 KB");
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const int pieces = kilobytes / 4;
    const size_t bytes = 8192 + (size_t)2 * pieces * 4096;
    unsigned *buf = nullptr;
    CNT_HIP(hipMalloc(reinterpret_cast<void **>(&buf), bytes));
    int status = CNT_OK;
    long long host_ticks[3] = {0, 0, 0};
    do {
        if (hipMemsetAsync(buf, 0, bytes, stream) != hipSuccess) { status = CNT_ERR_HIP; break; }
        unsigned *ctl = buf, *mail = buf + 2048;
        long long *ticks = reinterpret_cast<long long *>(buf + 512);
        hipLaunchKernelGGL(hop_message_kernel, dim3(256), dim3(256), 0, stream, ctl, mail, rounds, pieces, ticks);
        if (hipGetLastError() != hipSuccess || hipStreamSynchronize(stream) != hipSuccess ||
            hipMemcpy(host_ticks, ticks, sizeof(host_ticks), hipMemcpyDeviceToHost) != hipSuccess)
            status = CNT_ERR_HIP;
    } while (false);
    (void)hipFree(buf);
    if (status != CNT_OK) {
        set_error("probe_hop_message: HIP call failed: %s", hipGetErrorString(hipGetLastError()));
        return status;
    }
    if (host_ticks[2] != 0 || host_ticks[0] == 0 || host_ticks[1] == 0) {
        set_error("probe_hop_message: the two workgroups did not meet (placement or visibility)");
        return CNT_ERR_DEVICE;
    }
    *hop_us = (float)((double)(host_ticks[0] > host_ticks[1] ? host_ticks[0] : host_ticks[1]) * 0.01 / rounds / 2.0);
    return CNT_OK;
}
