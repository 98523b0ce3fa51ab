// Kernel template and launch ladder of the fp32 MFMA matrix product (design notes: gemm.hip).
#pragma once

#include "common.hpp"

namespace cnt {
namespace {

constexpr int BK = 32;  // k depth of a staged tile (16 measured 5-8% slower on the acoustic model's products: twice the
                        // barriers per flop); the tile edge (rows of A = columns of B per workgroup) is a template
                        // parameter: 128 or 64
constexpr int PITCH = BK + 4;
constexpr int NTHREADS = 256;

typedef float f32x16 __attribute__((ext_vector_type(16)));

// workgroup barrier that orders LDS traffic only; global loads issued before it stay in flight
__device__ __forceinline__ void lds_only_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

template <int V>
struct VecT;
template <>
struct VecT<1> { typedef float type; };
template <>
struct VecT<2> { typedef float2 type; };
template <>
struct VecT<4> { typedef float4 type; };

// Stages one ROWS-row x BK-k operand tile: global -> registers -> LDS.
//
// A load always executes, on a clamped address, and what decides whether its vector counts (inside the matrix; in
// masked mode: both pattern bytes non-zero and the shifted slot inside the fraction) is only LOOKED AT in store(),
// one k-iteration later.  Nothing between a load and the LDS store a whole iteration later touches the loaded
// registers -- neither the data nor the two pattern bytes -- so the only wait the loop needs is "all but the newest
// tile have arrived"; zeroing the vector right after the load would make every iteration wait for its own loads.
template <int VEC, bool KCONTIG, int ROWS>
struct TileStage {
    static constexpr int NLOAD = (ROWS * BK) / (NTHREADS * VEC);
    static_assert(NLOAD >= 1, "tile too small for this vector width");
    typename VecT<VEC>::type r[NLOAD];
    bool inside_[NLOAD];      // known at load time (indices only)
    char pat_own_[NLOAD], pat_src_[NLOAD];  // masked mode: loaded next to the data, looked at in store()

    // shift / pat / n_slots: masked mode (pat == nullptr switches it off); time_on_k selects which index is
    // the time slot
    __device__ __forceinline__ void load(const float *__restrict__ base, int ld, int row0, int k0,
                                         int rows_total, int k_total, int tid, const char *__restrict__ pat = nullptr,
                                         int shift = 0, int n_slots = 0, bool time_on_k = false) {
        if (KCONTIG) {
            constexpr int TPR = BK / VEC;        // threads per row
            constexpr int RPP = NTHREADS / TPR;  // rows per pass
            const int kq = (tid % TPR) * VEC;
            const int rr = tid / TPR;
#pragma unroll
            for (int p = 0; p < NLOAD; ++p) {
                const int row = row0 + rr + p * RPP;
                typename VecT<VEC>::type v = {};
                pat_own_[p] = 1; pat_src_[p] = 1;
                if (!pat) {
                    inside_[p] = row < rows_total && (k0 + kq) < k_total;
                    const int rc = min(row, rows_total - 1), kc = (k0 + kq) < k_total ? k0 + kq : 0;
                    v = *reinterpret_cast<const typename VecT<VEC>::type *>(base + (size_t)rc * ld + kc);
                } else if (!time_on_k) {
                    // the row is the time slot, so the whole vector is kept or dropped
                    const int rc = min(row, rows_total - 1), kc = (k0 + kq) < k_total ? k0 + kq : 0;
                    const int src = rc + shift;
                    const int sc = min(max(src, 0), n_slots - 1);
                    inside_[p] = row < rows_total && (k0 + kq) < k_total && src == sc;
                    v = *reinterpret_cast<const typename VecT<VEC>::type *>(base + (size_t)sc * ld + kc);
                    pat_own_[p] = pat[rc]; pat_src_[p] = pat[sc];
                } else {
                    inside_[p] = true;
                    if (row < rows_total && (k0 + kq) < k_total) {
                        // vector along k = consecutive time slots: element-wise masking
                        float *e = reinterpret_cast<float *>(&v);
#pragma unroll
                        for (int j = 0; j < VEC; ++j) {
                            const int u = k0 + kq + j, src = u + shift;
                            if (pat[u] != 0 && src >= 0 && src < n_slots && pat[src] != 0)
                                e[j] = base[(size_t)row * ld + src];
                        }
                    }
                }
                r[p] = v;
            }
        } else {
            constexpr int TPK = ROWS / VEC;      // threads per k line
            constexpr int KPP = NTHREADS / TPK;  // k lines per pass
            const int rq = (tid % TPK) * VEC;
            const int kk = tid / TPK;
#pragma unroll
            for (int p = 0; p < NLOAD; ++p) {
                const int k = k0 + kk + p * KPP;
                typename VecT<VEC>::type v = {};
                pat_own_[p] = 1; pat_src_[p] = 1;
                if (!pat) {
                    inside_[p] = k < k_total && (row0 + rq) < rows_total;
                    const int kc = min(k, k_total - 1), rc = (row0 + rq) < rows_total ? row0 + rq : 0;
                    v = *reinterpret_cast<const typename VecT<VEC>::type *>(base + (size_t)kc * ld + rc);
                } else if (time_on_k) {
                    // the k line is the time slot
                    const int kc = min(k, k_total - 1), rc = (row0 + rq) < rows_total ? row0 + rq : 0;
                    const int src = kc + shift;
                    const int sc = min(max(src, 0), n_slots - 1);
                    inside_[p] = k < k_total && (row0 + rq) < rows_total && src == sc;
                    v = *reinterpret_cast<const typename VecT<VEC>::type *>(base + (size_t)sc * ld + rc);
                    pat_own_[p] = pat[kc]; pat_src_[p] = pat[sc];
                } else {
                    inside_[p] = true;
                    if (k < k_total && (row0 + rq) < rows_total) {
                        float *e = reinterpret_cast<float *>(&v);
#pragma unroll
                        for (int j = 0; j < VEC; ++j) {
                            const int u = row0 + rq + j, src = u + shift;
                            if (pat[u] != 0 && src >= 0 && src < n_slots && pat[src] != 0)
                                e[j] = base[(size_t)k * ld + src];
                        }
                    }
                }
                r[p] = v;
            }
        }
    }

    __device__ __forceinline__ typename VecT<VEC>::type kept(int p) const {
        const bool keep = inside_[p] && pat_own_[p] != 0 && pat_src_[p] != 0;
        return keep ? r[p] : typename VecT<VEC>::type{};
    }

    // k values [k_first, k_first + BK/2) of tile row `row`, in MFMA issue order
    static __device__ __forceinline__ void fragment(const float *__restrict__ lds, int row, int k_first,
                                                    float (&f)[BK / 2]) {
        if (KCONTIG) {
            const float *p = lds + row * PITCH + k_first;
#pragma unroll
            for (int q = 0; q < BK / 8; ++q) {
                const float4 v = *reinterpret_cast<const float4 *>(p + 4 * q);
                f[4 * q] = v.x; f[4 * q + 1] = v.y; f[4 * q + 2] = v.z; f[4 * q + 3] = v.w;
            }
        } else {
#pragma unroll
            for (int q = 0; q < BK / 2; ++q) f[q] = lds[(k_first + q) * ROWS + row];
        }
    }

    __device__ __forceinline__ void store(float *__restrict__ lds, int tid) const {
        if (KCONTIG) {
            constexpr int TPR = BK / VEC;
            constexpr int RPP = NTHREADS / TPR;
            const int kq = (tid % TPR) * VEC;
            const int rr = tid / TPR;
#pragma unroll
            for (int p = 0; p < NLOAD; ++p)
                *reinterpret_cast<typename VecT<VEC>::type *>(lds + (rr + p * RPP) * PITCH + kq) = kept(p);
        } else {
            constexpr int TPK = ROWS / VEC;
            constexpr int KPP = NTHREADS / TPK;
            const int rq = (tid % TPK) * VEC;
            const int kk = tid / TPK;
#pragma unroll
            for (int p = 0; p < NLOAD; ++p)
                *reinterpret_cast<typename VecT<VEC>::type *>(lds + (kk + p * KPP) * ROWS + rq) = kept(p);
        }
    }
};

// The unmasked loader.  What a thread loads differs from tile to tile only by the tile's k
// offset, so everything per thread is computed once: `voff`, the byte offset of its vector inside the operand at k = 0
// (row clamped into the matrix), as a 32-bit offset beside a 64-bit base that is uniform over the workgroup -- the
// address form that costs no vector arithmetic per load -- and which of its vectors lie inside the matrix.  A tile
// needs masking only at the matrix edge or in the last, partly filled k tile of an operand pair; both are uniform over
// the workgroup (`special`), every other tile is stored as it arrived.
template <int VEC, bool KCONTIG, int ROWS>
struct FastStage {
    static constexpr int NLOAD = (ROWS * BK) / (NTHREADS * VEC);
    typedef typename VecT<VEC>::type vec_t;
    vec_t r[NLOAD];
    unsigned voff[NLOAD];    // byte offsets at k = 0
    unsigned koff[NLOAD];    // what has to be taken off voff to reach k position 0 of the tile (used in a k tail only)
    int kpos[NLOAD];         // first k of the vector inside the tile
    bool row_ok[NLOAD];
    bool edge;               // uniform: some row of this tile lies outside the matrix
    int k_valid;             // uniform: k values of the tile in registers that lie inside the operand pair

    __device__ __forceinline__ void init(int ld, int row0, int rows_total, int tid) {
        edge = row0 + ROWS > rows_total;
        if (KCONTIG) {
            constexpr int TPR = BK / VEC, RPP = NTHREADS / TPR;
            const int kq = (tid % TPR) * VEC, rr = tid / TPR;
#pragma unroll
            for (int p = 0; p < NLOAD; ++p) {
                const int row = row0 + rr + p * RPP;
                row_ok[p] = row < rows_total;
                voff[p] = (unsigned)(((size_t)min(row, rows_total - 1) * ld + kq) * sizeof(float));
                koff[p] = (unsigned)(kq * sizeof(float));
                kpos[p] = kq;
            }
        } else {
            constexpr int TPK = ROWS / VEC, KPP = NTHREADS / TPK;
            const int rq = (tid % TPK) * VEC, kk = tid / TPK;
#pragma unroll
            for (int p = 0; p < NLOAD; ++p) {
                const int k = kk + p * KPP;
                row_ok[p] = (row0 + rq) < rows_total;
                const int rc = row_ok[p] ? row0 + rq : 0;
                voff[p] = (unsigned)(((size_t)k * ld + rc) * sizeof(float));
                koff[p] = (unsigned)((size_t)k * ld * sizeof(float));
                kpos[p] = k;
            }
        }
    }
    // base = the operand at the tile's first k (uniform), kv = valid k values of the tile
    __device__ __forceinline__ void load(const float *__restrict__ base, int kv) {
        k_valid = kv;
        const char *b = reinterpret_cast<const char *>(base);
        if (kv >= BK) {
#pragma unroll
            for (int p = 0; p < NLOAD; ++p) r[p] = *reinterpret_cast<const vec_t *>(b + voff[p]);
        } else {
            // partly filled tile: a vector beyond the operand's k extent is read from k position 0 instead (in bounds)
            // and dropped at the store
#pragma unroll
            for (int p = 0; p < NLOAD; ++p)
                r[p] = *reinterpret_cast<const vec_t *>(b + (kpos[p] < kv ? voff[p] : voff[p] - koff[p]));
        }
    }
    __device__ __forceinline__ void store(float *__restrict__ lds, int tid) const {
        const bool special = edge || k_valid < BK;
        if (KCONTIG) {
            constexpr int TPR = BK / VEC, RPP = NTHREADS / TPR;
            const int kq = (tid % TPR) * VEC, rr = tid / TPR;
#pragma unroll
            for (int p = 0; p < NLOAD; ++p) {
                vec_t v = r[p];
                if (special && !(row_ok[p] && kpos[p] < k_valid)) v = vec_t{};
                *reinterpret_cast<vec_t *>(lds + (rr + p * RPP) * PITCH + kq) = v;
            }
        } else {
            constexpr int TPK = ROWS / VEC, KPP = NTHREADS / TPK;
            const int rq = (tid % TPK) * VEC, kk = tid / TPK;
#pragma unroll
            for (int p = 0; p < NLOAD; ++p) {
                vec_t v = r[p];
                if (special && !(row_ok[p] && kpos[p] < k_valid)) v = vec_t{};
                *reinterpret_cast<vec_t *>(lds + (kk + p * KPP) * ROWS + rq) = v;
            }
        }
    }
};

// The unmasked loader for row-contiguous operands whose k lines are picked through a list (16-byte vectors only): tile k
// line j is line idx[j] of the operand.  The indices of a tile are loaded one iteration ahead by the kernel (both operands
// share them) and handed to load(); everything else is FastStage.
template <int ROWS>
struct GatherStage {
    static constexpr int NLOAD = (ROWS * BK) / (NTHREADS * 4);
    static constexpr int TPK = ROWS / 4, KPP = NTHREADS / TPK;
    float4 r[NLOAD];
    unsigned roff;   // byte offset of the thread's four rows inside a k line (clamped into the matrix)
    int kk;          // the thread's first k line inside a tile; its others follow at a distance of KPP
    bool row_ok;
    bool edge;       // uniform: some row of this tile lies outside the matrix
    int k_valid;     // uniform: k lines of the tile in registers that are listed

    __device__ __forceinline__ void init(int row0, int rows_total, int tid) {
        edge = row0 + ROWS > rows_total;
        const int rq = (tid % TPK) * 4;
        kk = tid / TPK;
        row_ok = (row0 + rq) < rows_total;
        roff = (unsigned)((row_ok ? row0 + rq : 0) * sizeof(float));
    }
    // line_bytes and the indices are below 2^24 and the operand below 4 GiB (checked by the launcher): a 24-bit multiply-add
    // gives the 32-bit offset beside the uniform base
    __device__ __forceinline__ void load(const float *__restrict__ operand, unsigned line_bytes, const int (&idx)[NLOAD], int kv) {
        k_valid = kv;
        const char *b = reinterpret_cast<const char *>(operand);
#pragma unroll
        for (int p = 0; p < NLOAD; ++p)
            r[p] = *reinterpret_cast<const float4 *>(b + (__umul24((unsigned)idx[p], line_bytes) + roff));
    }
    __device__ __forceinline__ void store(float *__restrict__ lds, int tid) const {
        const bool special = edge || k_valid < BK;
        const int rq = (tid % TPK) * 4;
#pragma unroll
        for (int p = 0; p < NLOAD; ++p) {
            float4 v = r[p];
            if (special && !(row_ok && kk + p * KPP < k_valid)) v = float4{0.0f, 0.0f, 0.0f, 0.0f};
            *reinterpret_cast<float4 *>(lds + (kk + p * KPP) * ROWS + rq) = v;
        }
    }
};

// MASKED selects the time-shifted, padding-masked B loader at compile time: its per-element predication is a lot
// of code, and four copies of it (two prologue fetches, two in the unrolled loop) inside the plain kernels would
// push their hot loop out of the instruction cache.
// FAN: the EPI_FAN epilogue, a kernel of its own (instantiated for 16-byte row-contiguous A and k-contiguous B only,
// the shapes of the error products that use it) so that its registers and code stay out of every other product.
// GATHER: the k lines of both (row-contiguous, 16-byte aligned) operands are those a list names (GemmArgs::k_order).
template <int VA, bool AK, int VB, bool BK_, bool MASKED, int TILE, bool FAN = false, bool GATHER = false>
__global__ __launch_bounds__(NTHREADS) void gemm_f32_kernel(const GemmArgs args) {
    constexpr int BM = TILE, BN = TILE;
    constexpr int WT = TILE / 2;   // edge of a wave's block (waves are arranged 2 x 2)
    constexpr int NB = WT / 32;    // 32 x 32 MFMA tiles per wave and dimension
    __shared__ __attribute__((aligned(16))) float lds_a[2][BM * PITCH];
    __shared__ __attribute__((aligned(16))) float lds_b[2][BN * PITCH];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave & 1, wn = wave >> 1;

    // Which tile, k range and problem this workgroup takes.  Workgroups go to the eight XCDs in turn, in launch
    // order, and each XCD has its own L2: the workgroups one XCD receives take CONSECUTIVE positions of the order
    // (tile, problem, k range), with the tiles of one output walked in bands of eight rows of tiles.  What runs on one XCD
    // at a time is then a compact block of tiles of one k range (its operand panels are fetched into that L2 once
    // instead of once per XCD) and, for several problems per launch, the same k range of neighbouring problems
    // (which share an operand where a layer's taps or a stack's layers read the same input).
    const int tiles_m = (args.m + BM - 1) / BM;
    int tile = blockIdx.x, split_id = blockIdx.y, prob_id = blockIdx.z;
    if (args.xcd_map) {
        const unsigned total = gridDim.x * gridDim.y * gridDim.z;
        const unsigned at = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
        const unsigned per = total / 8, rem = total % 8, xcd = at % 8, slot = at / 8;
        const unsigned pos = xcd < rem ? xcd * (per + 1) + slot : rem * (per + 1) + (xcd - rem) * per + slot;
        const unsigned in_output = pos % gridDim.x, rest = pos / gridDim.x;
        prob_id = (int)(rest % gridDim.z);
        split_id = (int)(rest / gridDim.z);
        const int tiles_n = (int)gridDim.x / tiles_m;
        const int band = (int)in_output / (8 * tiles_n), off = (int)in_output % (8 * tiles_n);
        const int rows = min(tiles_m - 8 * band, 8);
        tile = (8 * band + off % rows) + (off / rows) * tiles_m;
    }
    const int m0 = (tile % tiles_m) * BM;
    const int n0 = (tile / tiles_m) * BN;
    const GemmProblem &pb = args.prob[prob_id];

    // iteration space: segments x k-tiles, cut into splitk contiguous ranges
    // the listed k lines this problem takes: all of them, or all but the first / last time step's
    int k_extent = args.k, k_lo = 0;
    if (GATHER) {
        k_extent = args.k_count[0];
        if (pb.k_trim == 1) { k_lo = args.k_count[1]; k_extent -= k_lo; }
        else if (pb.k_trim == 2) k_extent -= args.k_count[2];
        k_extent = max(k_extent, 0);
    }
    const int kt_per_seg = (k_extent + BK - 1) / BK;
    const int total_it = kt_per_seg * args.nseg;
    const int per_split = (total_it + args.splitk - 1) / args.splitk;
    const int it_begin = split_id * per_split;
    const int it_end = min(total_it, it_begin + per_split);
    // (a split left without k lines by a short list still has its partial product to write)
    if (it_begin >= it_end && !(GATHER && args.epilogue == EPI_PARTIAL)) return;

    f32x16 acc[NB][NB];
#pragma unroll
    for (int i = 0; i < NB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    // Two register sets per operand: tile it+1 waits in one of them while tile it+2 is being fetched into the
    // other, so that a global load has two k-iterations of MFMA work (about 4000 clocks) to arrive in; with one
    // workgroup per compute unit, which is what the benchmark's shapes give, nothing else hides that latency.
    // The loop is unrolled by two so that the sets swap roles without register copies, and its barrier orders
    // LDS only (__syncthreads() would also drain the loads in flight).
    const char *mask_pat = MASKED ? args.pat : nullptr;
    constexpr bool kStoreEarly = true;

    // sum of the B operand over this split's k range, per row (dense bias gradient); kept by the waves with wm == 0
    const bool rowsum = args.rowsum != 0;
    float rs[NB];
#pragma unroll
    for (int j = 0; j < NB; ++j) rs[j] = 0.0f;

    const int frag_row = lane & 31;
    constexpr int FK = BK / 2;  // k values per half-wave and tile
    const int frag_k = (lane >> 5) * FK;

    // `fetch_next(a, b)` loads the next tile of the walk into a pair of register sets; after the last tile it loads
    // that one again, so that the count of loads in flight is the same on every path.
    auto run = [&](auto &a0, auto &b0, auto &a1, auto &b1, auto &fetch_next) __attribute__((always_inline)) {
        fetch_next(a0, b0);
        fetch_next(a1, b1);
        a0.store(lds_a[0], tid);
        b0.store(lds_b[0], tid);
        lds_only_barrier();
        // one k-iteration on LDS buffer `cur`; `held` carries tile it+1, `recv` receives tile it+2
        auto iterate = [&](int it, int cur, auto &held_a, auto &held_b, auto &recv_a, auto &recv_b) __attribute__((always_inline)) {
            fetch_next(recv_a, recv_b);
            __builtin_amdgcn_sched_barrier(0);  // keep the loads ahead of the MFMA block: the scheduler would sink them
            if (kStoreEarly && it + 1 < it_end) {
                // the tile that arrived during the last iteration goes to the other LDS buffer (free since the barrier)
                // while this iteration's fragments are on their way, not behind the last MFMA
                held_a.store(lds_a[cur ^ 1], tid);
                held_b.store(lds_b[cur ^ 1], tid);
                __builtin_amdgcn_sched_barrier(0);
            }

            float fa[NB][FK], fb[NB][FK];
#pragma unroll
            for (int i = 0; i < NB; ++i) {
                TileStage<VA, AK, TILE>::fragment(lds_a[cur], wm * WT + i * 32 + frag_row, frag_k, fa[i]);
                TileStage<VB, BK_, TILE>::fragment(lds_b[cur], wn * WT + i * 32 + frag_row, frag_k, fb[i]);
            }
#pragma unroll
            for (int kk = 0; kk < FK; ++kk) {
#pragma unroll
                for (int i = 0; i < NB; ++i) {
#pragma unroll
                    for (int j = 0; j < NB; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[j][kk], fa[i][kk], acc[i][j], 0, 0, 0);
                }
            }
            if (rowsum) {
#pragma unroll
                for (int j = 0; j < NB; ++j)
#pragma unroll
                    for (int kk = 0; kk < FK; ++kk) rs[j] += fb[j][kk];
            }

            if (!kStoreEarly && it + 1 < it_end) {
                held_a.store(lds_a[cur ^ 1], tid);
                held_b.store(lds_b[cur ^ 1], tid);
            }
            lds_only_barrier();
        };
        for (int it = it_begin; it < it_end; it += 2) {
            iterate(it, 0, a1, b1, a0, b0);
            if (it + 1 < it_end) iterate(it + 1, 1, a0, b0, a1, b1);
        }
    };
    if constexpr (GATHER) {
        static_assert(VA == 4 && VB == 4 && !AK && !BK_ && !MASKED, "the gathering loader is for two row-contiguous operands");
        GatherStage<TILE> ga0, ga1, gb0, gb1;
        ga0.init(m0, args.m, tid); ga1.init(m0, args.m, tid);
        gb0.init(n0, args.n, tid); gb1.init(n0, args.n, tid);
        constexpr int NL = GatherStage<TILE>::NLOAD, KPP = GatherStage<TILE>::KPP;
        const int *__restrict__ order = args.k_order + k_lo;
        const int k_shift = pb.k_shift;
        const unsigned a_line = (unsigned)(args.lda * sizeof(float)), b_line = (unsigned)(args.ldb * sizeof(float));
        int seg = it_begin / kt_per_seg, kin = it_begin % kt_per_seg, left = it_end - it_begin - 1;
        const float *pa = pb.A[seg], *pbb = pb.B[seg];
        // the k lines of the cursor's tile, loaded while the tile before it is being requested
        int idx[NL];
        auto lines_of = [&](int tile) __attribute__((always_inline)) {
#pragma unroll
            for (int p = 0; p < NL; ++p) idx[p] = order[max(min(tile * BK + ga0.kk + p * KPP, k_extent - 1), 0)] + k_shift;
        };
        lines_of(kin);
        auto fetch_next = [&](GatherStage<TILE> &qa, GatherStage<TILE> &qb) __attribute__((always_inline)) {
            const int kv = min(BK, k_extent - kin * BK);
            qa.load(pa, a_line, idx, kv);
            qb.load(pbb, b_line, idx, kv);
            if (left > 0) {
                --left;
                if (++kin == kt_per_seg) {
                    kin = 0; ++seg;
                    pa = pb.A[seg]; pbb = pb.B[seg];
                }
            }
            lines_of(kin);
        };
        if (it_begin < it_end) run(ga0, gb0, ga1, gb1, fetch_next);
    } else if constexpr (MASKED) {
        TileStage<VA, AK, TILE> sa0, sa1;
        TileStage<VB, BK_, TILE> sb0, sb1;
        int next_it = it_begin;
        auto fetch_next = [&](TileStage<VA, AK, TILE> &ra, TileStage<VB, BK_, TILE> &rb) __attribute__((always_inline)) {
            const int it = min(next_it, it_end - 1);
            ++next_it;
            const int seg = it / kt_per_seg;
            const int k0 = (it % kt_per_seg) * BK;
            ra.load(pb.A[seg], args.lda, m0, k0, args.m, args.k, tid);
            rb.load(pb.B[seg], args.ldb, n0, k0, args.n, args.k, tid, mask_pat, pb.b_shift[seg], args.n_slots,
                    args.b_time_on_k != 0);
        };
        run(sa0, sb0, sa1, sb1, fetch_next);
    } else {
        // the tile cursor: operand pair `seg`, k tile `kin` inside it; the operands' base pointers are looked up only
        // when the pair changes
        FastStage<VA, AK, TILE> qa0, qa1;
        FastStage<VB, BK_, TILE> qb0, qb1;
        qa0.init(args.lda, m0, args.m, tid); qa1.init(args.lda, m0, args.m, tid);
        qb0.init(args.ldb, n0, args.n, tid); qb1.init(args.ldb, n0, args.n, tid);
        int seg = it_begin / kt_per_seg, kin = it_begin % kt_per_seg, left = it_end - it_begin - 1;
        const float *pa = pb.A[seg], *pbb = pb.B[seg];
        const size_t ka = AK ? 1 : (size_t)args.lda, kb = BK_ ? 1 : (size_t)args.ldb;  // floats per k step
        auto fetch_next = [&](FastStage<VA, AK, TILE> &qa, FastStage<VB, BK_, TILE> &qb) __attribute__((always_inline)) {
            const int kv = min(BK, args.k - kin * BK);
            qa.load(pa + (size_t)kin * BK * ka, kv);
            qb.load(pbb + (size_t)kin * BK * kb, kv);
            if (left > 0) {
                --left;
                if (++kin == kt_per_seg) {
                    kin = 0; ++seg;
                    pa = pb.A[seg]; pbb = pb.B[seg];
                }
            }
        };
        run(qa0, qb0, qa1, qb1, fetch_next);
    }

    // epilogue: lane%32 runs along m (contiguous), the 16 accumulators along n
    float *__restrict__ C = pb.C;
    const int half = lane >> 5;
    if (args.epilogue == EPI_PARTIAL) {
        // this split's partial product, m x n column-major without padding, after those of the problems before it
        float *__restrict__ P = args.partial + (size_t)split_id * args.partial_stride +
                                (size_t)prob_id * args.m * args.n;
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            const int m = m0 + wm * WT + i * 32 + frag_row;
            if (m >= args.m) continue;
#pragma unroll
            for (int j = 0; j < NB; ++j) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int n = n0 + wn * WT + j * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                    if (n < args.n) P[(size_t)n * args.m + m] = acc[i][j][r];
                }
            }
        }
        if (rowsum && wm == 0 && m0 == 0) {
            float *__restrict__ R = args.partial + (size_t)split_id * args.partial_stride +
                                    (size_t)args.nprob * args.m * args.n + (size_t)prob_id * args.n;
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                const float s = rs[j] + __shfl_xor(rs[j], 32);
                const int n = n0 + wn * WT + j * 32 + frag_row;
                if (half == 0 && n < args.n) R[n] = s;
            }
        }
        return;
    }
    if (FAN) {
        // All loads of a 32 x 32 tile's sixteen values per lane are issued before anything is stored: the compiler
        // cannot know that the buffers do not overlap and would otherwise wait for memory once per value.
#pragma unroll
        for (int i = 0; i < NB; ++i) {
            const int m = m0 + wm * WT + i * 32 + frag_row;
#pragma unroll
            for (int j = 0; j < NB; ++j) {
                size_t idx[16];
                bool ok[16];
                float e[16], old[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int n = n0 + wn * WT + j * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                    ok[r] = m < args.m && n < args.n;
                    idx[r] = ok[r] ? (size_t)n * args.ldc + m : 0;
                    old[r] = (ok[r] && pb.aux_in) ? pb.aux_in[idx[r]] : 0.0f;
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    e[r] = pb.aux_in ? old[r] + acc[i][j][r] : acc[i][j][r];
                    if (ok[r]) C[idx[r]] = e[r];
                }
                for (int q = 0; q < args.fan_n; ++q) {
                    float *__restrict__ t = args.fan_targets[q];
                    if (args.fan_is_skip[q]) {
#pragma unroll
                        for (int r = 0; r < 16; ++r) old[r] = ok[r] ? t[idx[r]] : 0.0f;
#pragma unroll
                        for (int r = 0; r < 16; ++r)
                            if (ok[r]) t[idx[r]] = e[r] + old[r];
                    } else {
#pragma unroll
                        for (int r = 0; r < 16; ++r)
                            if (ok[r]) t[idx[r]] = e[r];
                    }
                }
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
        const int m = m0 + wm * WT + i * 32 + frag_row;
        if (m >= args.m) continue;
        float bterm = 0.0f;
        if (args.epilogue == EPI_BIAS_ACT || args.epilogue == EPI_BIAS_ACT_SKIP)
            bterm = args.bias_scale * pb.bias_vec[m];
#pragma unroll
        for (int j = 0; j < NB; ++j) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int n = n0 + wn * WT + j * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                if (n >= args.n) continue;
                const size_t idx = (size_t)n * args.ldc + m;
                float *dst = C + idx;
                const float v = acc[i][j][r];
                switch (args.epilogue) {
                    case EPI_STORE: *dst = v; break;
                    case EPI_STORE_DELTA: *dst = v * act_deriv(args.act, pb.aux_in[idx]); break;
                    case EPI_ADD: *dst = *dst + v; break;
                    case EPI_ATOMIC: atomicAdd(dst, v); break;

                    case EPI_BIAS_ACT: *dst = act_fn(args.act, v + bterm); break;
                    case EPI_BIAS_ACT_SKIP:
                        if (args.pat[n] != 0) *dst = act_fn(args.act, v + bterm);
                        break;
                    default: {  // EPI_CONTEXT
                        const bool valid = args.pat[n] != 0;
                        const float th = valid ? tanh_act(v) : 0.0f;
                        if (pb.aux_out) pb.aux_out[idx] = th;
                        *dst = valid ? pb.aux_in[idx] + th : 0.0f;
                    } break;
                }
            }
        }
    }
}

template <int VA, bool AK, int VB, bool BK_, int TILE>
void launch_m(const GemmArgs &a, dim3 grid, hipStream_t s) {
    if (a.epilogue == EPI_FAN) {
        // gemm_launch has checked that the operands are of the one kind this exists for
        if constexpr (VA == 4 && !AK && VB == 4 && BK_) {
            if (a.masked)
                hipLaunchKernelGGL((gemm_f32_kernel<VA, AK, VB, BK_, true, TILE, true>), grid, dim3(NTHREADS), 0, s, a);
            else
                hipLaunchKernelGGL((gemm_f32_kernel<VA, AK, VB, BK_, false, TILE, true>), grid, dim3(NTHREADS), 0, s, a);
        }
        return;
    }
    if (a.k_order) {
        // gemm_launch has checked that the operands are of the one kind this exists for
        if constexpr (VA == 4 && !AK && VB == 4 && !BK_ && TILE == 64)
            hipLaunchKernelGGL((gemm_f32_kernel<VA, AK, VB, BK_, false, TILE, false, true>), grid, dim3(NTHREADS), 0, s, a);
        return;
    }
    if (a.masked) hipLaunchKernelGGL((gemm_f32_kernel<VA, AK, VB, BK_, true, TILE>), grid, dim3(NTHREADS), 0, s, a);
    else hipLaunchKernelGGL((gemm_f32_kernel<VA, AK, VB, BK_, false, TILE>), grid, dim3(NTHREADS), 0, s, a);
}
template <int VA, bool AK, int VB, bool BK_>
void launch_t(const GemmArgs &a, dim3 grid, hipStream_t s, int tile) {
    if (tile == 64) launch_m<VA, AK, VB, BK_, 64>(a, grid, s);
    else launch_m<VA, AK, VB, BK_, 128>(a, grid, s);
}
template <int VA, bool AK, int VB>
void launch_b(const GemmArgs &a, dim3 grid, hipStream_t s, bool bk, int tile) {
    if (bk) launch_t<VA, AK, VB, true>(a, grid, s, tile);
    else launch_t<VA, AK, VB, false>(a, grid, s, tile);
}
template <int VA, bool AK>
void launch_vb(const GemmArgs &a, dim3 grid, hipStream_t s, int vb, bool bk, int tile) {
    if (vb == 4) launch_b<VA, AK, 4>(a, grid, s, bk, tile);
    else if (vb == 2) launch_b<VA, AK, 2>(a, grid, s, bk, tile);
    else launch_b<VA, AK, 1>(a, grid, s, bk, tile);
}
template <int VA>
void launch_ak(const GemmArgs &a, dim3 grid, hipStream_t s, bool ak, int vb, bool bk, int tile) {
    if (ak) launch_vb<VA, true>(a, grid, s, vb, bk, tile);
    else launch_vb<VA, false>(a, grid, s, vb, bk, tile);
}

}  // namespace

// One translation unit per A-operand vector width instantiates its share of the kernels (they compile in
// parallel); gemm.hip dispatches on the width.
void gemm_dispatch_va4(const GemmArgs &a, dim3 grid, hipStream_t s, bool ak, int vb, bool bk, int tile);
void gemm_dispatch_va2(const GemmArgs &a, dim3 grid, hipStream_t s, bool ak, int vb, bool bk, int tile);
void gemm_dispatch_va1k(const GemmArgs &a, dim3 grid, hipStream_t s, int vb, bool bk, int tile);
void gemm_dispatch_va1r(const GemmArgs &a, dim3 grid, hipStream_t s, int vb, bool bk, int tile);

}  // namespace cnt
