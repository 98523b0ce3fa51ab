// fp32 MFMA matrix product for gfx950.
//
// This is the seam that the reference reaches through helpers::Matrix::assignProduct/addProduct
// (helpers/Matrix.cu:353-377 -> helpers/cublas.cu:52-84).  One kernel covers every operand
// orientation, K-concatenated accumulation over several operand pairs (the eight W_in * delta
// products of a BLSTM become one pass), several independent problems per launch, split-K for the
// long-K weight-gradient shapes, and a fused bias + activation epilogue for the dense forward.
//
// Tiling: T x T x 32 per workgroup with T = 128 or 64, four 64-lane waves in a 2 x 2 arrangement, each wave
// owning a T/2 x T/2 block as tiles of v_mfma_f32_32x32x2_f32.  An operand tile sits in LDS in the
// orientation it has in memory, so that staging never transposes: k-contiguous operands as [row][k] with
// a (BK+4)-float pitch (16-byte fragment reads, conflict free), row-contiguous operands as [k][row]
// (4-byte fragment reads along consecutive rows).  A transposing store of the latter into [row][k]
// costs a 16-way LDS bank conflict.
// The MFMA operands are swapped (the B tile feeds the instruction's A port) so that lane%32 walks
// along the column-major output's contiguous dimension and every store is a 128-byte segment.
#include "gemm_kernel.hpp"

#include <algorithm>
#include <cstdlib>
#include <mutex>
#include <vector>

namespace cnt {
namespace {

inline int pick_vec(const GemmArgs &a, bool for_a) {
    const int ld = for_a ? a.lda : a.ldb;
    const bool kc = for_a ? a.a_kcontig : a.b_kcontig;
    const int extent = kc ? a.k : (for_a ? a.m : a.n);
    int v = 4;
    while (v > 1) {
        bool ok = (ld % v == 0) && (extent % v == 0);
        for (int p = 0; ok && p < a.nprob; ++p)
            for (int s = 0; ok && s < a.nseg; ++s) {
                const float *ptr = for_a ? a.prob[p].A[s] : a.prob[p].B[s];
                ok = (reinterpret_cast<uintptr_t>(ptr) % (4 * v)) == 0;
            }
        if (ok) break;
        v >>= 1;
    }
    return v;
}

// Tile edge.  128 x 128 tiles give the most MFMA work per byte staged, but a launch that yields only a few of
// them per compute unit leaves the machine waiting on memory latency (one or two workgroups of four waves per
// CU) and on the last, partly filled round of workgroups.  Measured on MI355X, 64 x 64 tiles -- four times as
// many workgroups -- are faster for every product of the benchmark networks (the acoustic model's 512 x 5880
// error products by 1.4x, the WaveNet layers' K = 64..384 products over 32 000 slots by 2x); the large tile is
// kept for launches that fill the machine many times over anyway.
int pick_tile(const GemmArgs &a) {
    static const int forced = [] { const char *e = std::getenv("CNT_GEMM_TILE"); return e ? std::atoi(e) : 0; }();
    if (forced == 64 || forced == 128) return forced;
    const long t128 = (long)((a.m + 127) / 128) * ((a.n + 127) / 128) * a.splitk * a.nprob;
    return t128 < 2048 ? 64 : 128;
}

// ----- split-K through partial products ---------------------------------------------------------------------
// Weight gradients of narrow layers over long inputs (a 64 x 128 output summed over 32 000 slots) need a few
// hundred splits to fill the machine, and with the atomic epilogue every output element then receives a few
// hundred atomic adds; atomics to one address serialise, and they, not the loads, set the run time of such a
// launch.  Here every split stores its partial product with plain stores into a scratch buffer and a second,
// small kernel sums the splits into C.  That also replaces the clearing launch in front of the atomic path and,
// for dense layers, the separate column sum for the bias gradient (the splits carry the row sums of B along).
constexpr size_t kSplitScratchFloats = (size_t)4 << 20;  // 16 MB per (device, stream)
constexpr long kPartialMaxOutput = 128 << 10;            // floats of output (all problems) up to which it pays

struct SplitScratch {
    int device;
    hipStream_t stream;
    float *buf;
};
std::mutex g_split_mu;  // held while a product and its reduction are enqueued, so that they stay adjacent
std::vector<SplitScratch> g_split_scratch;

// One scratch buffer per stream: launches on a stream execute in order, so the next product on the same stream
// cannot overwrite partial sums that a reduction has yet to read.  Kept until gemm_release_stream.
float *split_scratch_find(hipStream_t stream) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return nullptr;
    for (const SplitScratch &e : g_split_scratch)
        if (e.device == dev && e.stream == stream) return e.buf;
    return nullptr;
}

// the stream's buffer, allocated now if the stream has none; NULL when the allocation is refused (out of memory,
// a stream under capture): the caller then takes the atomic path
float *split_scratch(hipStream_t stream) {
    if (float *buf = split_scratch_find(stream)) return buf;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return nullptr;
    float *buf = nullptr;
    if (hipMalloc(reinterpret_cast<void **>(&buf), kSplitScratchFloats * sizeof(float)) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    g_split_scratch.push_back({dev, stream, buf});
    return buf;
}

// ----- scratch that is part of the loaded code object, for callers that must not allocate ---------------------
// Every device the library runs on holds its own copy of this array at its own address until the process ends.
// In host code the array's name is only a handle for hipGetSymbolAddress: the address a kernel may use is looked
// up once per device and kept in g_static_ptr.
constexpr size_t kStaticScratchFloats = (size_t)2 << 20;  // 8 MB
constexpr int kMaxDevices = 64;
static __device__ __align__(256) float scratch[kStaticScratchFloats];
float *g_static_ptr[kMaxDevices];

// device address of the current device's copy of `scratch` (NULL with the error text set on failure)
float *static_scratch() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        set_error("static scratch: no current device");
        return nullptr;
    }
    std::lock_guard<std::mutex> lock(g_split_mu);
    if (!g_static_ptr[dev]) {
        void *ptr = nullptr;
        const hipError_t err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (err != hipSuccess || !ptr) {
            set_error("static scratch: hipGetSymbolAddress: %s", hipGetErrorString(err));
            return nullptr;
        }
        g_static_ptr[dev] = static_cast<float *>(ptr);
    }
    return g_static_ptr[dev];
}

// 32 consecutive outputs per block, the splits dealt to eight groups of 32 threads whose sums meet in LDS; four
// loads in flight per thread
constexpr int kReduceOutputs = 32;
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const GemmArgs args) {
    constexpr int G = 256 / kReduceOutputs;
    __shared__ float part[G][kReduceOutputs];
    const int tx = threadIdx.x % kReduceOutputs, g = threadIdx.x / kReduceOutputs;
    const size_t mn = (size_t)args.m * args.n;
    const size_t products = mn * args.nprob;
    const size_t total = products + (args.rowsum ? (size_t)args.n * args.nprob : 0);
    const size_t e = (size_t)blockIdx.x * kReduceOutputs + tx;
    float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f, a3 = 0.0f;
    if (e < total) {
        const float *__restrict__ p = args.partial + e;
        const size_t st = args.partial_stride;
        int s = g;
        for (; s + 3 * G < args.splitk; s += 4 * G) {
            const float x0 = p[(size_t)s * st], x1 = p[(size_t)(s + G) * st];
            const float x2 = p[(size_t)(s + 2 * G) * st], x3 = p[(size_t)(s + 3 * G) * st];
            a0 += x0; a1 += x1; a2 += x2; a3 += x3;
        }
        for (; s < args.splitk; s += G) a0 += p[(size_t)s * st];
    }
    part[g][tx] = (a0 + a1) + (a2 + a3);
    __syncthreads();
    if (g == 0 && e < total) {
        float v = 0.0f;
#pragma unroll
        for (int q = 0; q < G; ++q) v += part[q][tx];
        if (e < products) {
            const size_t z = e / mn, r = e % mn;
            args.prob[z].C[(r / args.m) * args.ldc + r % args.m] = v;
        } else {
            const size_t z = (e - products) / args.n, j = (e - products) % args.n;
            args.prob[z].rowsum_out[j] = args.prob[z].rowsum_scale * v;
        }
    }
}

}  // namespace

bool gemm_fan_supported(const GemmArgs &a) {
    return !a.a_kcontig && a.b_kcontig && a.nprob == 1 && pick_vec(a, true) == 4 && pick_vec(a, false) == 4;
}

void gemm_release_stream(hipStream_t stream) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) return;
    std::lock_guard<std::mutex> lock(g_split_mu);
    for (size_t i = 0; i < g_split_scratch.size(); ++i)
        if (g_split_scratch[i].device == dev && g_split_scratch[i].stream == stream) {
            (void)hipFree(g_split_scratch[i].buf);
            g_split_scratch.erase(g_split_scratch.begin() + (long)i);
            return;
        }
}

int gemm_reserve_stream(hipStream_t stream) {
    std::lock_guard<std::mutex> lock(g_split_mu);
    CNT_REQUIRE(split_scratch(stream) != nullptr, "gemm: no memory for the split-K scratch buffer");
    return CNT_OK;
}

int gemm_scratch_buffers() {
    std::lock_guard<std::mutex> lock(g_split_mu);
    return (int)g_split_scratch.size();
}

void gemm_plan(GemmArgs &args, hipStream_t stream) {
    if (args.splitk != 0) return;
    // Long-K products with a small output (weight gradients): cut K so that the launch has about
    // `target` workgroups of 64 x 64 tiles, but leave every workgroup at least eight k-iterations -- each
    // one ends with an atomic add (or a store) of its whole tile, and those, not the products, dominate short
    // ranges.
    // Outputs of one or two tiles per problem (the WaveNet layers' 64 x 64 ... 80 x 128 weights) take twice the
    // workgroups: measured on MI355X next to the error chain of the same pass, 1024 workgroups end the stack's backward
    // pass 4% sooner than 512, and 1536 or more (where the partial products no longer fit the scratch buffer and the
    // launch adds atomically) 4-8% later; the acoustic model's wide outputs are best at 768 (2.249 / 2.232 / 2.219 / 2.246 /
    // 2.243 ms at 512 / 640 / 768 / 896 / 1024 with the loader of constant offsets; they were best at 512 before it).
    static const int forced_target = [] { const char *e = std::getenv("CNT_GEMM_SPLIT_TARGET"); return e ? std::atoi(e) : 0; }();
    const long tiles = (long)((args.m + 63) / 64) * ((args.n + 63) / 64) * args.nprob;
    // (768 only where a launch has at least 64 tiles to begin with: the WaveNet stack's 256 x 256 output layers over
    // 32 000 samples, 16 tiles, are better off with 512: 2.724 against 2.736 ms)
    const int target = forced_target > 0 ? forced_target : ((long)args.m * args.n <= 16384 ? 1024 : tiles >= 64 ? 768 : 512);
    const long kt = ((long)args.k + BK - 1) / BK * args.nseg;
    long s = (target + tiles - 1) / tiles;
    s = std::min(s, std::max(1L, kt / 8));
    s = std::max(1L, s);
    // no empty split: every split of the partial-product path has to write its share
    while (s > 1 && (s - 1) * ((kt + s - 1) / s) >= kt) --s;
    args.splitk = (int)s;
    static const bool partial_on = [] { const char *e = std::getenv("CNT_GEMM_PARTIAL"); return !e || std::atoi(e) != 0; }();
    const long out = (long)args.m * args.n * args.nprob;
    const size_t stride = (size_t)out + (args.rowsum ? (size_t)args.n * args.nprob : 0);
    const bool rowsum_ok = !args.rowsum || (args.nseg == 1 && !args.masked);
    bool partial = partial_on && args.epilogue == EPI_ATOMIC && args.overwrite_ok && rowsum_ok && s >= 8 &&
                   out <= kPartialMaxOutput && stride * (size_t)s <= kSplitScratchFloats;
    if (partial && !args.partial) {
        // the stream's scratch buffer: reserved by its owner, else allocated on first use; without one (allocation
        // refused) the product adds atomically
        std::lock_guard<std::mutex> lock(g_split_mu);
        args.partial = split_scratch(stream);
        partial = args.partial != nullptr;
    }
    if (partial) {
        args.epilogue = EPI_PARTIAL;
        args.partial_stride = stride;
    } else {
        args.rowsum = 0;  // the caller sums the rows itself
    }
}

int gemm_launch(hipStream_t stream, const GemmArgs &args_in) {
    GemmArgs args = args_in;
    CNT_REQUIRE(args.m > 0 && args.n > 0 && args.k > 0, "gemm: empty problem %d x %d x %d", args.m, args.n,
                args.k);
    CNT_REQUIRE(args.nseg >= 1 && args.nseg <= kGemmMaxSeg, "gemm: %d operand pairs, supported 1..%d",
                args.nseg, kGemmMaxSeg);
    CNT_REQUIRE(args.nprob >= 1 && args.nprob <= kGemmMaxProb, "gemm: %d problems, supported 1..%d",
                args.nprob, kGemmMaxProb);
    CNT_REQUIRE(args.splitk >= 0 && (args.splitk == 1 || args.epilogue == EPI_ATOMIC || args.epilogue == EPI_PARTIAL),
                "gemm: split-K needs the atomic epilogue");
    CNT_REQUIRE(args.epilogue != EPI_STORE_DELTA || (args.splitk == 1 && args.prob[0].aux_in != nullptr),
                "gemm: the delta epilogue needs the preceding layer's outputs and no split");
    CNT_REQUIRE(args.epilogue != EPI_FAN || (gemm_fan_supported(args) && args.splitk == 1),
                "gemm: the fan epilogue exists for one unsplit problem with 16-byte row-contiguous A and k-contiguous B");
    CNT_REQUIRE(args.epilogue != EPI_PARTIAL || (args.splitk >= 1 && args.partial_stride > 0 && args.partial),
                "gemm: the partial-product epilogue is chosen by gemm_plan only");
    for (int p = 0; p < args.nprob; ++p) {
        CNT_REQUIRE(args.prob[p].C != nullptr, "gemm: null output");
        for (int s = 0; s < args.nseg; ++s)
            CNT_REQUIRE(args.prob[p].A[s] && args.prob[p].B[s], "gemm: null operand");
    }
    // the unmasked loaders address an operand through 32-bit byte offsets beside a base that moves along k
    const auto reachable = [](long rows, long ld, int kcontig) {
        return (kcontig ? rows * ld : BK * ld + rows) * (long)sizeof(float) < (1L << 32);
    };
    CNT_REQUIRE(args.masked || (reachable(args.m, args.lda, args.a_kcontig) && reachable(args.n, args.ldb, args.b_kcontig)),
                "gemm: operands of 4 GiB and more are not supported (%d x %d x %d, lda %d, ldb %d)", args.m, args.n, args.k,
                args.lda, args.ldb);
    const int va = pick_vec(args, true), vb = pick_vec(args, false);
    gemm_plan(args, stream);
    if (args.epilogue != EPI_PARTIAL) args.rowsum = 0;
    const int tile = pick_tile(args);
    static const bool use_lines = [] { const char *e = std::getenv("CNT_GEMM_K_ORDER"); return !e || std::atoi(e) != 0; }();
    if (!use_lines) args.k_order = nullptr;
    // a list of k lines is used where the kernel that reads through it exists, and ignored otherwise (the lines it leaves
    // out are zero)
    if (args.k_order && !(args.k_count && !args.masked && !args.a_kcontig && !args.b_kcontig && va == 4 && vb == 4 && tile == 64 &&
                          args.epilogue != EPI_FAN && args.k < (1 << 24) && args.lda < (1 << 22) && args.ldb < (1 << 22)))
        args.k_order = nullptr;
    const int tiles = ((args.m + tile - 1) / tile) * ((args.n + tile - 1) / tile);
    dim3 grid(tiles, args.splitk, args.nprob);
    // XCD-aware placement (gemm_kernel.hpp) for launches of several problems: measured with FETCH_SIZE on MI355X it
    // cuts what the L2s fetch 2.2-2.6x for the WaveNet stack's batched weight gradients (a convolution's two taps and
    // a stack's conditioning projections share an operand) and ends that pass 0.5% sooner.  For one problem per launch
    // it cuts the fetches 2-4x as well (the acoustic model's weight gradients: 270 -> 68 MB) and the products run 1%
    // faster, but that model's pass came out 0.7% slower in every run, so single problems keep the launch order
    // (CNT_GEMM_XCD_MAP=2 maps them too, 0 maps nothing).
    static const int xcd_map = [] { const char *e = std::getenv("CNT_GEMM_XCD_MAP"); return e ? std::atoi(e) : 1; }();
    args.xcd_map = (xcd_map == 2 || (xcd_map == 1 && args.nprob > 1)) && (long)tiles * args.splitk * args.nprob >= 16 ? 1 : 0;
    ProfileScope prof(stream, args.label ? args.label : "gemm");
    std::unique_lock<std::mutex> split_lock(g_split_mu, std::defer_lock);
    // a product and its reduction stay adjacent on the stream
    if (args.epilogue == EPI_PARTIAL) split_lock.lock();
    if (va == 4) gemm_dispatch_va4(args, grid, stream, args.a_kcontig, vb, args.b_kcontig, tile);
    else if (va == 2) gemm_dispatch_va2(args, grid, stream, args.a_kcontig, vb, args.b_kcontig, tile);
    else if (args.a_kcontig) gemm_dispatch_va1k(args, grid, stream, vb, args.b_kcontig, tile);
    else gemm_dispatch_va1r(args, grid, stream, vb, args.b_kcontig, tile);
    CNT_HIP(hipGetLastError());
    if (args.epilogue == EPI_PARTIAL) {
        const size_t total = args.partial_stride;
        hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)((total + kReduceOutputs - 1) / kReduceOutputs)), dim3(256),
                           0, stream, args);
        CNT_HIP(hipGetLastError());
    }
    return CNT_OK;
}

// A dense layer's weight gradient (dW = x * delta^T, P x D, plus the bias part: bias * row sums of delta) as a
// split-K product whose partial products go through the code object's own scratch array: no allocation at all.
int gemm_dense_weights_static(hipStream_t stream, int P, int D, int N, float bias, const float *x, const float *err,
                              float *weight_updates) {
    const size_t stride = (size_t)P * D + D;
    CNT_REQUIRE(stride <= kStaticScratchFloats,
                "dense_backward_weights_static: %d x %d weights + %d biases = %zu floats exceed the static scratch of %zu "
                "floats; use cnt_dense_backward_weights", P, D, D, stride, kStaticScratchFloats);
    float *buf = static_scratch();
    if (!buf) return CNT_ERR_HIP;
    GemmArgs ga = {};
    ga.m = P; ga.n = D; ga.k = N;
    ga.a_kcontig = 0; ga.lda = P;
    ga.b_kcontig = 0; ga.ldb = D;
    ga.ldc = P;
    ga.nseg = 1; ga.nprob = 1;
    ga.prob[0].A[0] = x; ga.prob[0].B[0] = err; ga.prob[0].C = weight_updates;
    ga.prob[0].rowsum_out = weight_updates + (size_t)P * D;
    ga.prob[0].rowsum_scale = bias;
    ga.label = "gemm:dense_dW_static";
    ga.rowsum = 1;
    // as many splits as the usual plan takes, as far as their partial products fit into the array
    GemmArgs probe = ga;
    probe.epilogue = EPI_ATOMIC; probe.splitk = 0; probe.overwrite_ok = 0;
    gemm_plan(probe, stream);
    size_t splits = (size_t)probe.splitk;
    if (splits * stride > kStaticScratchFloats) splits = kStaticScratchFloats / stride;
    const long kt = ((long)N + BK - 1) / BK;
    while (splits > 1 && ((long)splits - 1) * ((kt + (long)splits - 1) / (long)splits) >= kt) --splits;  // no empty split
    ga.splitk = (int)splits;
    ga.epilogue = EPI_PARTIAL;
    ga.partial = buf;
    ga.partial_stride = stride;
    return gemm_launch(stream, ga);
}

int gemm_simple(hipStream_t stream, float *C, int m, int n, int k, const float *A, bool transA,
                const float *B, bool transB, bool accumulate) {
    GemmArgs a = {};
    a.m = m; a.n = n; a.k = k;
    // column-major A (m x k, lda=m) is row-contiguous; transposed storage (k x m, lda=k) is k-contiguous
    a.a_kcontig = transA ? 1 : 0;
    a.lda = transA ? k : m;
    // column-major B (k x n, ldb=k) is k-contiguous; transposed storage (n x k, ldb=n) is row-contiguous
    a.b_kcontig = transB ? 0 : 1;
    a.ldb = transB ? n : k;
    a.ldc = m;
    a.nseg = 1; a.nprob = 1; a.splitk = 1;
    a.epilogue = accumulate ? EPI_ADD : EPI_STORE;
    a.prob[0].A[0] = A;
    a.prob[0].B[0] = B;
    a.prob[0].C = C;
    return gemm_launch(stream, a);
}

}  // namespace cnt
