// LSTM layer for gfx950: forward recursion, BPTT error recursion, and the batched contractions.
//
// Reference behaviour: layers/LstmLayer.cu  (forward :57-208, :1743-1949; backward :210-648,
// :2066-2382; sequence loading :1488-1533; weight layout :1136-1169, :1218-1268).
//
// The reference launches four small matrix products and one elementwise functor per time step and
// direction.  Here each direction is ONE persistent kernel ("chain"): G = H/JB workgroups each own
// JB cells for the whole sequence, keep their slice of the recurrent weight matrix in registers as
// MFMA operands for all T steps, carry the per-cell recurrent state (cell error, forget-gate
// activation, gate deltas) in registers, and exchange the only truly shared quantity of a step
// through a small device-memory mailbox:
//   forward : block outputs h[t] (H x S), gathered by every workgroup;
//   backward: each workgroup multiplies its own 4*JB gate deltas with its weight slice and
//             scatters partial output errors to the owners of the receiving cells (H x S words per
//             workgroup instead of the 4H x S a gather of the deltas would need).
// Mailbox words are plain 4-byte floats; a reserved NaN pattern means "not written yet", so a word validates
// itself and neither tags nor fences sit on the critical path.  Words are moved 16 bytes at a time, polled with
// loads that bypass the non-coherent caches, and handed back as empty after use; four slots rotate.  Every
// poll loop is bounded: when the bound is hit the workgroup raises a device flag and every workgroup drains
// out.  Inside a workgroup, waves specialise (polling waves that never store, product / cell waves that never
// wait for a store, one memory wave for all ordinary loads and stores), see the kernels' comments.
//
// The dense work that does not sit on the recursion is batched over all time steps on the MFMA
// GEMM: input projections (8 problems, one launch), the error to the preceding layer
// (one K-concatenated product), input and recurrent weight gradients (split-K), and one streaming
// reduction for bias and peephole gradients.
#include "common.hpp"

#include <cstdlib>
#include <cstring>
#include <new>
#include <type_traits>
#include <vector>
#include <utility>
#include <algorithm>
#include <mutex>

namespace cnt {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned long long u64;

constexpr int kThreads = 256;
constexpr int kWaves = 4;

struct DirPtrs {
    float *ni, *ig, *fg, *og, *c, *h;
    float *herr, *dni, *dig, *dfg, *dog, *cerr;
    const float *w_int;    // gate 0 block of this direction; gate g at + g*L*H
    const float *b[4];     // bias weights per gate
    const float *peep[3];  // ig, fg, og peepholes
    float *fmail;          // forward: kMailSlots slots of H*S plain words
    float *bmail;          // backward: kMailSlots slots of plain words
};

struct ChainParams {
    int H, L, S, T, Tmin, ndir;
    float bias;
    const char *pat;
    DirPtrs d[2];
    float *out;           // forward: L x (T*S) layer outputs (NULL when it aliases d[0].h)
    const float *outerr;  // backward: L x (T*S) output errors
    float *herr_out;      // backward, unidirectional: where the summed error is written back
    unsigned spin_limit;
    int *abort_flag;
    int xcd_pack;
    long long *phase_ticks;  // optional diagnostic: per workgroup accumulated phase durations (100 MHz ticks)
    int poll_delay, poll_gap;  // s_sleep units before the first poll of a step / between polls
    int mem_delay;             // XCD-local backward recursion: s_sleep units before the memory wave's work of a step
    int poll_delay_fwd;
    int *latch;  // host-visible mark "a recursion of this handle gave up" (pinned host memory), never cleared by kernels
    int *veto;   // optional device flag shared by a network's handles, set together with the latch
    // XCD-local backward recursion: jobs = (direction, group of sequences), see lstm_local.hpp
    int njobs;
    struct { int dir, seq0, nseq; } job[8];
    unsigned *ctl;   // placement counters, zero at launch
    float *lmail;    // one mailbox per job
    float *flmail;   // the same for the XCD-local forward recursion
    // XCD-local backward recursion over a range of its steps: [step_begin, step_end) of 0 .. T.  A launch that starts
    // at a later step takes what the step before it left: the carried cell-state terms from the state arrays, the
    // partial errors from the mailbox (which nothing may touch in between).
    int step_begin, step_end;
};

// A workgroup that gives up: every workgroup of the launch sees the device flag and drains; the host sees the latch
// at its next call into the handle, the optimizer step of a network sees the veto flag.
__device__ __forceinline__ void raise_abort(const ChainParams &p) {
    __hip_atomic_store(p.abort_flag, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(p.latch, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    if (p.veto) __hip_atomic_store(p.veto, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also drains every outstanding
// global load and store of the wave, which would put the HBM latency of the look-ahead loads and the
// acknowledgement of the result stores on the recursion's critical path.  No thread of a workgroup
// reads global data written by another thread of the same launch except through the mailbox.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

__device__ __forceinline__ bool map_block(const ChainParams &p, int G, int &dir, int &me) {
    const int b = blockIdx.x;
    if (p.xcd_pack) {
        // workgroups are dealt round-robin to the 8 XCDs; keep one chain inside one XCD's L2
        const int xcd = b & 7;
        if (xcd >= p.ndir) return false;
        dir = xcd;
        me = b >> 3;
    } else {
        dir = b % p.ndir;
        me = b / p.ndir;
    }
    return me < G;
}

// ---------------------------------------------------------------------------------------------------
// Backward (error) recursion.
//
// The partial output errors travel through a mailbox of plain 4-byte words, laid out
// [slot][receiving workgroup][sending workgroup][sequence][cell of the receiver]:
//   * a word that holds kEmpty (an all-ones NaN pattern no product can yield) has not been written yet;
//     a sender stores the JB values of one (receiver, sequence) pair as 16-byte vectors, a receiver polls
//     its contiguous G*S*JB words with 16-byte loads and validates every word on its own;
//   * after reading, the receiving workgroup puts kEmpty back.  Four slots rotate (step % 4); the ordering
//     argument for the reset of a slot against its next use is given with the kernel's wave roles below.
// A launch that runs to its end leaves every word empty, so the host fills the mailbox with kEmpty once and
// again only after a launch that gave up.
// ---------------------------------------------------------------------------------------------------
constexpr unsigned kEmpty = 0xFFFFFFFFu;
constexpr int kMailSlots = 4;
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

// s_waitcnt vmcnt(0) (expcnt and lgkmcnt left at their maxima) as a builtin, so that the compiler's own wait
// insertion sees that nothing is outstanding afterwards and adds no waits of its own for older loads.
__device__ __forceinline__ void wait_all_vmem() { __builtin_amdgcn_s_waitcnt(0x0F70); }

// N 16-byte loads that bypass the non-coherent caches (device scope), all in flight together, then one wait.
// Inline assembly because the polled words change under the compiler's feet: the loads may neither be
// hoisted out of the polling loop nor merged.
template <int N>
__device__ __forceinline__ void poll_load(const float *base, unsigned byte_off, unsigned q_stride_bytes,
                                          u32x4 (&w)[N]) {
#pragma unroll
    for (int q = 0; q < N; ++q) {
        const float *bq = reinterpret_cast<const float *>(reinterpret_cast<const char *>(base) +
                                                          (size_t)q * q_stride_bytes);
        asm volatile("global_load_dwordx4 %0, %1, %2 sc1" : "=v"(w[q]) : "v"(byte_off), "s"(bq) : "memory");
    }
    wait_all_vmem();
#pragma unroll
    for (int q = 0; q < N; ++q) asm volatile("" : "+v"(w[q]));  // consumers stay behind the wait
}

// 16-byte store written through to the device-coherent level (cache policy bit 4 = sc1).  A compiler builtin,
// unlike the loads above, so that the compiler's own wait counting knows the store is in flight.
__device__ __forceinline__ void store128_device(__amdgpu_buffer_rsrc_t rsrc, unsigned byte_off, u32x4 v) {
    __builtin_amdgcn_raw_buffer_store_b128(v, rsrc, (int)byte_off, 0, 16);
}
// ---------------------------------------------------------------------------------------------------
// Forward recursion.  HT = H/64, JB = cells per workgroup, NT = ceil(S/16).
//
// Every workgroup needs the block outputs h[t-1] of ALL cells.  They travel through a mailbox of plain
// 4-byte words laid out [slot][cell / 4][sequence][cell % 4]; a word that holds kEmpty has not been written.
// Four slots rotate.  The producer of a word empties it again two steps after writing it -- by then every
// workgroup has consumed it, because a workgroup can only publish h[t] after it has seen h[t-1] of all others
// -- and drains its stores before it publishes again, so a reader that has seen h[t-1] can never find the
// value of four steps earlier in the slot of h[t].  The host fills the mailbox with kEmpty before each launch.
//
// Waves and their roles (one LDS-only barrier per step):
//   gather waves (4)   wait, poll h[t-1] straight into MFMA B operands (each wave a quarter of the source
//                      cells), multiply with their register-resident weight slice, leave the partial
//                      pre-activations in LDS.  They issue no stores.
//   cell waves (CW)    after the barrier: add the four partials to the input projection, run the gate / cell
//                      update of JB x S elements, publish h[t], empty the slot of h[t-2], leave the step's
//                      results in LDS.
//   memory wave (1)    loads the input projections two steps ahead and hands them over through LDS one step
//                      ahead; writes the results of the finished step to the state arrays and the layer output.
// ---------------------------------------------------------------------------------------------------
constexpr int fwd_cell_waves(int JB, int NT) { return (JB * 16 * NT + 63) / 64; }
constexpr int fwd_threads(int JB, int NT) { return kThreads + 64 * fwd_cell_waves(JB, NT) + 64; }

template <int HT, int JB, int NT>
__global__ __launch_bounds__(fwd_threads(JB, NT)) void lstm_forward_chain(const ChainParams p) {
    constexpr int H = 64 * HT;
    constexpr int G = H / JB;
    constexpr int NS = 16 * NT;
    constexpr int MT = (4 * JB) / 16;  // output tiles: rows are (gate, cell)
    constexpr int KS = H / 16;         // k-steps of 4 per gather wave (each covers H/4 source cells)
    constexpr int KV = KS / 4;         // 16-byte vectors (4 source cells) per lane and column tile
    constexpr int EL = JB * NS;        // (cell, sequence) elements, padded
    constexpr int CW = fwd_cell_waves(JB, NT);
    constexpr int EPAD = 64 * CW;
    static_assert((4 * JB) % 16 == 0 && KS % 4 == 0, "JB must be a multiple of 4, H of 64");
    enum { R_NI = 0, R_IG, R_FG, R_OG, R_C, R_H, NRES };

    int dir, me;
    if (!map_block(p, G, dir, me)) return;
    const DirPtrs &D = p.d[dir];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int S = p.S, T = p.T;
    const int j0 = me * JB;
    const int n = S * H;

    __shared__ float red[2][kWaves][4 * JB][NS + 1];  // partial pre-activations, by step parity
    __shared__ float pre[2][4][EPAD];                 // input projections of the step, by step parity
    __shared__ int pre_dummy[2][EPAD];
    __shared__ float res[2][NRES][EPAD];              // results of the step, by step parity
    __shared__ int res_flags[2][EPAD];                // bit 0: gate activations to store, bit 1: cell state to store
    __shared__ int wait_failed;
    if (threadIdx.x == 0) wait_failed = 0;

    auto slot_of = [&](int step) { return dir ? (T - 1 - step) : step; };
    const unsigned slot_words = (unsigned)H * S;
    const __amdgpu_buffer_rsrc_t mail =
        __builtin_amdgcn_make_buffer_rsrc(D.fmail, 0, (int)(kMailSlots * slot_words * sizeof(float)), 0x00020000);

    if (wave == kWaves + CW) {
        // ------------------------------------------------------------------ memory wave
        constexpr int EIT = CW;
        struct StepIn { float a[4]; char pat; };
        int cs[EIT], cj[EIT];
        bool valid[EIT];
#pragma unroll
        for (int it = 0; it < EIT; ++it) {
            const int id = it * 64 + lane;
            cs[it] = id / JB; cj[it] = id % JB;
            valid[it] = id < EL && cs[it] < S;
        }
        auto load_step = [&](int step, StepIn (&v)[EIT]) {
            const int t = slot_of(step);
#pragma unroll
            for (int it = 0; it < EIT; ++it) {
                v[it] = StepIn{{0, 0, 0, 0}, 1};
                if (!valid[it] || step >= T) continue;
                const size_t gi = (size_t)t * n + (size_t)cs[it] * H + j0 + cj[it];
                v[it].a[0] = D.ni[gi]; v[it].a[1] = D.ig[gi]; v[it].a[2] = D.fg[gi]; v[it].a[3] = D.og[gi];
                v[it].pat = p.pat[t * S + cs[it]];
            }
        };
        auto put_pre = [&](int step, const StepIn (&v)[EIT]) {
            const int t = slot_of(step);
#pragma unroll
            for (int it = 0; it < EIT; ++it) {
                const int id = it * 64 + lane;
#pragma unroll
                for (int g = 0; g < 4; ++g) pre[step & 1][g][id] = v[it].a[g];
                pre_dummy[step & 1][id] = ((t >= p.Tmin) && (v[it].pat == 0)) ? 1 : 0;
            }
        };
        auto store_results = [&](int step) {
            const int t = slot_of(step), b = step & 1;
#pragma unroll
            for (int it = 0; it < EIT; ++it) {
                if (!valid[it]) continue;
                const int id = it * 64 + lane;
                const size_t gi = (size_t)t * n + (size_t)cs[it] * H + j0 + cj[it];
                const int flags = res_flags[b][id];
                if (flags & 1) {
                    D.ni[gi] = res[b][R_NI][id]; D.ig[gi] = res[b][R_IG][id];
                    D.fg[gi] = res[b][R_FG][id]; D.og[gi] = res[b][R_OG][id];
                }
                if (flags & 2) D.c[gi] = res[b][R_C][id];
                const float hval = res[b][R_H][id];
                D.h[gi] = hval;
                if (p.out) p.out[((size_t)t * S + cs[it]) * p.L + dir * H + j0 + cj[it]] = hval;
            }
        };
        auto run_step = [&](const int step, StepIn (&far)[EIT], const StepIn (&near)[EIT]) __attribute__((always_inline)) -> bool {
            lds_barrier();  // results of step-1 and partial sums of this step are in LDS
            if (wait_failed) return false;
            wait_all_vmem();  // whatever is still in flight was issued a step ago
            load_step(step + 2, far);
            if (step + 1 < T) put_pre(step + 1, near);
            if (step > 0) store_results(step - 1);
            return true;
        };
        StepIn in_a[EIT], in_b[EIT];
        load_step(0, in_a);
        load_step(1, in_b);
        put_pre(0, in_a);
        lds_barrier();  // start of the recursion
        for (int step = 0; step < T; step += 2) {
            if (!run_step(step, in_a, in_b)) return;
            if (step + 1 < T && !run_step(step + 1, in_b, in_a)) return;
        }
        lds_barrier();  // results of the last step
        if (wait_failed) return;
        store_results(T - 1);
        return;
    }

    if (wave >= kWaves) {
        // ------------------------------------------------------------------ cell waves
        const int id = tid - kThreads;
        const int cs = id / JB, cj = id % JB;
        const bool cell_valid = id < EL && cs < S;
        float b_ni = 0, b_ig = 0, b_fg = 0, b_og = 0, p_ig = 0, p_fg = 0, p_og = 0;
        if (cell_valid) {
            b_ni = p.bias * D.b[0][j0 + cj]; b_ig = p.bias * D.b[1][j0 + cj];
            b_fg = p.bias * D.b[2][j0 + cj]; b_og = p.bias * D.b[3][j0 + cj];
            p_ig = D.peep[0][j0 + cj]; p_fg = D.peep[1][j0 + cj]; p_og = D.peep[2][j0 + cj];
        }
        // word of this element inside a mailbox slot: [cell / 4][sequence][cell % 4]
        const unsigned my_word = ((unsigned)((j0 + cj) >> 2) * S + cs) * 4u + ((j0 + cj) & 3);
        float c_prev = 0.0f;
        wait_all_vmem();
        lds_barrier();  // start of the recursion
        for (int step = 0; step < T; ++step) {
            const bool first = (step == 0);
            const int b = step & 1;
            lds_barrier();
            if (wait_failed) return;
            // stores of the previous step (publication, reset) are complete before this step publishes
            wait_all_vmem();
            if (!cell_valid) continue;
            float a_ni = pre[b][0][id], a_ig = pre[b][1][id], a_fg = pre[b][2][id], a_og = pre[b][3][id];
            if (!first) {
#pragma unroll
                for (int w = 0; w < kWaves; ++w) {
                    a_ni += red[b][w][0 * JB + cj][cs];
                    a_ig += red[b][w][1 * JB + cj][cs];
                    a_fg += red[b][w][2 * JB + cj][cs];
                    a_og += red[b][w][3 * JB + cj][cs];
                }
            }
            float hval = 0.0f;
            int flags;
            if (pre_dummy[b][id]) {
                // the reference leaves the summed pre-activations in place on padding slots, clears the
                // cell only in the time-reversed direction and emits a zero output
                res[b][R_NI][id] = a_ni; res[b][R_IG][id] = a_ig; res[b][R_FG][id] = a_fg; res[b][R_OG][id] = a_og;
                res[b][R_C][id] = 0.0f;
                flags = (first ? 0 : 1) | (dir ? 2 : 0);
                if (dir) c_prev = 0.0f;
            } else {
                float x_ni = a_ni + b_ni, x_ig = a_ig + b_ig, x_fg = a_fg + b_fg, x_og = a_og + b_og;
                if (!first) { x_ig += c_prev * p_ig; x_fg += c_prev * p_fg; }
                const float ni = tanh_quick(x_ni), ig = logistic_quick(x_ig), fg = logistic_quick(x_fg);
                float c = ni * ig;
                if (!first) c += c_prev * fg;
                x_og += c * p_og;
                const float og = logistic_quick(x_og);
                hval = tanh_quick(c) * og;
                res[b][R_NI][id] = ni; res[b][R_IG][id] = ig; res[b][R_FG][id] = fg; res[b][R_OG][id] = og;
                res[b][R_C][id] = c;
                flags = 3;
                c_prev = c;
            }
            if (step + 1 < T) {
                unsigned bits = __float_as_uint(hval);
                if (bits == kEmpty) bits = 0x7FC00000u;
                __builtin_amdgcn_raw_buffer_store_b32(bits, mail, (int)(((unsigned)(step % kMailSlots) * slot_words + my_word) * 4u), 0, 16);
            }
            if (step >= 2 && step + 2 < T)
                __builtin_amdgcn_raw_buffer_store_b32(kEmpty, mail, (int)(((unsigned)((step + 2) % kMailSlots) * slot_words + my_word) * 4u), 0, 16);
            res[b][R_H][id] = hval;
            res_flags[b][id] = flags;
        }
        lds_barrier();  // results of the last step are in LDS
        return;
    }

    // ---------------------------------------------------------------------- gather waves
    // Recurrent weights as MFMA A operands: row (gate, cell); the k order is free as long as both operands
    // agree, and it is chosen so that the four k values of a lane and k-step group are the four cells of one
    // 16-byte mailbox vector: k-step (j, c) of lane group kq is source cell  wave*H/4 + 4*(kq + 4*j) + c.
    float wA[MT][KS];
    {
        const int i = lane & 15, kq = lane >> 4;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const int o = mt * 16 + i, g = o / JB, jj = o % JB;
            const float *wg = D.w_int + (size_t)g * p.L * H + (size_t)(j0 + jj) * H;
#pragma unroll
            for (int j = 0; j < KV; ++j)
#pragma unroll
                for (int c = 0; c < 4; ++c) wA[mt][4 * j + c] = wg[wave * (H / 4) + 4 * (kq + 4 * j) + c];
        }
    }
    long long ph0 = 0, ph3 = 0, poll_rounds = 0;
    const bool timing = p.phase_ticks != nullptr;
    const long long tk_begin = timing ? wall_clock64() : 0;
    const int kq = lane >> 4;
    wait_all_vmem();
    lds_barrier();  // start of the recursion
    lds_barrier();  // step 0 has nothing to gather

    for (int step = 1; step < T; ++step) {
        const long long tk0 = timing ? wall_clock64() : 0;
        const float *slot = D.fmail + (size_t)((step - 1) % kMailSlots) * slot_words;
        bool ok = true;
        f32x4 acc[MT][NT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = f32x4{0, 0, 0, 0};
        // h[t-1] cannot be there before the cell waves of the other workgroups are done; see the backward kernel
        for (int d = 0; d < p.poll_delay_fwd; ++d) __builtin_amdgcn_s_sleep(1);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const int s = nt * 16 + (lane & 15);
            u32x4 w[KV];
#pragma unroll
            for (int j = 0; j < KV; ++j) w[j] = u32x4{0, 0, 0, 0};
            if (s < S) {
                // vector j of this lane: cells 4*quad .. 4*quad+3 with quad = wave*H/16 + kq + 4*j
                const unsigned off = (((unsigned)(wave * (H / 16) + kq)) * S + s) * 16u;
                unsigned spins = 0;
                for (;;) {
                    poll_load<KV>(slot, off, 4u * (unsigned)S * 16u, w);
                    unsigned worst = 0;
#pragma unroll
                    for (int j = 0; j < KV; ++j) worst = max(max(worst, w[j].x), max(max(w[j].y, w[j].z), w[j].w));
                    if (timing) ++poll_rounds;
                    if (worst != kEmpty) break;
                    if (++spins > p.spin_limit) { ok = false; break; }
                    if ((spins & 255u) == 0u &&
                        __hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
                        ok = false;
                        break;
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < KV; ++j) {
                const f32x4 hv = __builtin_bit_cast(f32x4, w[j]);
#pragma unroll
                for (int c = 0; c < 4; ++c)
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(wA[mt][4 * j + c], hv[c], acc[mt][nt], 0, 0, 0);
            }
        }
        wait_all_vmem();
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    red[step & 1][wave][mt * 16 + 4 * (lane >> 4) + r][nt * 16 + (lane & 15)] = acc[mt][nt][r];
        if (!ok) wait_failed = 1;
        lds_barrier();
        if (wait_failed) {
            if (tid == 0) raise_abort(p);
            return;
        }
        if (timing) ph0 += wall_clock64() - tk0;
    }
    lds_barrier();  // results of the last step
    if (timing) ph3 = wall_clock64() - tk_begin;
    if (timing && tid == 0) {
        long long *o = p.phase_ticks + (size_t)blockIdx.x * 6;
        o[0] = ph0; o[1] = 0; o[3] = ph3; o[4] = poll_rounds;
    }
}

// Workgroup layout, nine waves in three roles that meet at two workgroup barriers per step:
//   receive waves (4)  poll the mailbox, reduce the partial errors through LDS (barrier A), run the cell update
//                      and leave the gate deltas in LDS (barrier B).  They issue no stores at all, so the only
//                      memory operations their wait counter ever covers are their own polls.
//   product waves (4)  hold the recurrent weight slice as MFMA operands; after barrier B they multiply it with
//                      the deltas and publish the partial errors.  They never wait for a store.
//   memory wave (1)    owns every other global access: two steps ahead it loads what the cell update needs,
//                      one step ahead it folds everything that does not depend on the recursion into five
//                      coefficients per cell (LDS), one step behind it writes the cell update's results to the
//                      state arrays.
// Mailbox slots rotate over four steps.  The product waves also hand the words their workgroup consumed in a
// step back as empty, and drain all of their stores once per step (right after barrier A, when only stores of
// the previous step can still be in flight), so the reset of the words consumed in step k is complete before
// this workgroup publishes in step k+1; a sender rewrites those words only in step k+3, after it has seen
// that publication.
constexpr int kBwdThreads = 2 * kThreads + 64;

template <int HT, int JB, int NT>
__global__ __launch_bounds__(kBwdThreads) void lstm_backward_chain(const ChainParams p) {
    constexpr int H = 64 * HT;
    constexpr int G = H / JB;
    constexpr int NS = 16 * NT;
    constexpr int MT = H / 64;  // 16-row tiles of receiving cells per product wave (each covers H/4)
    constexpr int KS = JB;      // k = (gate, own cell): 4*JB values, 4 per MFMA
    constexpr int EL = JB * NS; // (cell, sequence) pairs of this workgroup, padded
    constexpr int JV = JB / 4;  // 16-byte vectors per (sender, sequence) pair
    constexpr int PG = kThreads / NS;   // sender groups polled side by side
    constexpr int NPOLL = G / PG;       // senders per polling lane
    constexpr int PITCH = EL + 4;
    constexpr int EIT = (EL + 63) / 64; // elements per lane of the memory wave
    static_assert(G % PG == 0 && NPOLL >= 1 && JB % 4 == 0 && EL <= kThreads, "mailbox polling layout");
    enum { C_OG = 0, C_CE, C_NI, C_FG, C_IG, C_E, C_DOG, C_FGACT, C_DUMMY, NCOEF };

    int dir, me;
    if (!map_block(p, G, dir, me)) return;
    const DirPtrs &D = p.d[dir];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int S = p.S, T = p.T;
    const int j0 = me * JB;
    const int n = S * H;

    __shared__ __attribute__((aligned(16))) float psum[PG][PITCH];
    __shared__ float dl[4 * JB][NS + 1];
    __shared__ float coef[NCOEF][EL];
    __shared__ float res[2][EL];  // summed output error, cell error
    __shared__ int wait_failed;
    if (threadIdx.x == 0) wait_failed = 0;

    auto slot_of = [&](int step) { return dir ? step : (T - 1 - step); };
    // mailbox geometry, in floats
    const unsigned pair_words = (unsigned)S * JB;           // one (receiver, sender) pair
    const unsigned recv_words = (unsigned)G * pair_words;   // everything one receiver gets in a step
    const size_t slot_words = (size_t)G * recv_words;
    const size_t mail_bytes = kMailSlots * slot_words * sizeof(float);
    const __amdgpu_buffer_rsrc_t mail = __builtin_amdgcn_make_buffer_rsrc(D.bmail, 0, (int)mail_bytes, 0x00020000);

    if (wave == 2 * kWaves) {
        // ------------------------------------------------------------------ memory wave
        struct StepIn { float e, ni, ig, fg, og, dog_old, c, c_earlier; char pat; };
        int cs[EIT], cj[EIT];
        bool valid[EIT];
#pragma unroll
        for (int it = 0; it < EIT; ++it) {
            const int id = it * 64 + lane;
            cs[it] = id / JB; cj[it] = id % JB;
            valid[it] = id < EL && cs[it] < S;
        }
        auto load_step = [&](int step, StepIn (&v)[EIT]) {
            const int t = slot_of(step);
#pragma unroll
            for (int it = 0; it < EIT; ++it) {
                v[it] = StepIn{0, 0, 0, 0, 0, 0, 0, 0, 1};
                if (!valid[it] || step >= T) continue;
                const size_t gi = (size_t)t * n + (size_t)cs[it] * H + j0 + cj[it];
                v[it].e = p.outerr[((size_t)t * S + cs[it]) * p.L + dir * H + j0 + cj[it]];
                v[it].ni = D.ni[gi]; v[it].ig = D.ig[gi]; v[it].fg = D.fg[gi]; v[it].og = D.og[gi];
                v[it].dog_old = D.dog[gi];
                v[it].c = D.c[gi];
                if (step + 1 < T)
                    v[it].c_earlier = D.c[(size_t)slot_of(step + 1) * n + (size_t)cs[it] * H + j0 + cj[it]];
                v[it].pat = p.pat[t * S + cs[it]];
            }
        };
        auto put_coef = [&](int step, const StepIn (&v)[EIT]) {
            const int t = slot_of(step);
#pragma unroll
            for (int it = 0; it < EIT; ++it) {
                const int id = it * 64 + lane;
                if (id >= EL) continue;
                const StepIn &x = v[it];
                const float tc = tanh_act(x.c);
                coef[C_OG][id] = logistic_deriv(x.og) * tc;         // d_og = this * e + dog_old
                coef[C_CE][id] = x.og * tanh_deriv(tc);             // ce   = this * e + ...
                coef[C_NI][id] = x.ig * tanh_deriv(x.ni);           // d_ni = this * ce
                coef[C_FG][id] = logistic_deriv(x.fg) * x.c_earlier;  // d_fg = this * ce
                coef[C_IG][id] = logistic_deriv(x.ig) * x.ni;       // d_ig = this * ce
                coef[C_E][id] = x.e;
                coef[C_DOG][id] = x.dog_old;
                coef[C_FGACT][id] = x.fg;
                coef[C_DUMMY][id] = ((t >= p.Tmin) && (x.pat == 0)) ? 1.0f : 0.0f;
            }
        };
        const bool mtiming = p.phase_ticks != nullptr;
        long long mbusy = 0;
        // one step of the memory wave; `far` receives the inputs of step+2, `near` holds those of step+1
        auto run_step = [&](const int step, StepIn (&far)[EIT], const StepIn (&near)[EIT]) __attribute__((always_inline)) -> bool {
            const int t = slot_of(step);
            if (step > 0) {
                lds_barrier();  // A: partial sums are in LDS
                if (wait_failed) return false;
            }
            // everything still in flight is at least a step old: state stores and mailbox resets of the
            // previous step, inputs requested a step ago
            wait_all_vmem();
            load_step(step + 2, far);
            lds_barrier();  // B: results of this step are in LDS
            const long long tm0 = mtiming ? wall_clock64() : 0;
            // coefficients first: the receive waves need them at the next barrier A, the stores can trail
            if (step + 1 < T) put_coef(step + 1, near);
#pragma unroll
            for (int it = 0; it < EIT; ++it) {
                if (!valid[it]) continue;
                const int id = it * 64 + lane;
                const size_t gi = (size_t)t * n + (size_t)cs[it] * H + j0 + cj[it];
                D.dni[gi] = dl[0 * JB + cj[it]][cs[it]]; D.dig[gi] = dl[1 * JB + cj[it]][cs[it]];
                D.dfg[gi] = dl[2 * JB + cj[it]][cs[it]]; D.dog[gi] = dl[3 * JB + cj[it]][cs[it]];
                D.cerr[gi] = res[1][id];
                if (p.herr_out) p.herr_out[gi] = res[0][id];
                else D.herr[gi] = res[0][id];
            }
            if (mtiming) mbusy += wall_clock64() - tm0;
            return true;
        };
        StepIn in_a[EIT], in_b[EIT];
        load_step(0, in_a);
        load_step(1, in_b);
        put_coef(0, in_a);
        lds_barrier();  // start of the recursion
        for (int step = 0; step < T; step += 2) {
            if (!run_step(step, in_a, in_b)) return;
            if (step + 1 < T && !run_step(step + 1, in_b, in_a)) return;
        }
        if (mtiming && lane == 0) p.phase_ticks[(size_t)blockIdx.x * 6 + 5] = mbusy;
        return;
    }

    if (wave >= kWaves) {
        // ------------------------------------------------------------------ product waves
        const int pw = wave - kWaves;
        // recurrent weights as MFMA A operands: row = receiving ("from") cell, k = (gate, own cell)
        float wA[MT][KS];
        {
            const int i = lane & 15, kq = lane >> 4;
#pragma unroll
            for (int ks = 0; ks < KS; ++ks) {
                const int k = 4 * ks + kq, g = k / JB, jj = k % JB;
                const float *wg = D.w_int + (size_t)g * p.L * H + (size_t)(j0 + jj) * H;
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) wA[mt][ks] = wg[pw * (H / 4) + mt * 16 + i];
            }
        }
        // reset role: the same words this workgroup's receive waves poll (sequence ps, senders pg, pg + PG, ...)
        const int ptid = tid - kThreads;
        const int ps = ptid % NS, pg = ptid / NS;
        const unsigned poll_off = ((unsigned)(pg * S + ps) * JB) * 4u;
        const unsigned poll_stride = (unsigned)PG * pair_words * 4u;
        wait_all_vmem();
        lds_barrier();  // start of the recursion
        const bool timing = p.phase_ticks != nullptr;
        long long busy = 0;
        for (int step = 0; step < T; ++step) {
            if (step > 0) {
                lds_barrier();  // A
                if (wait_failed) return;
                // everything this wave stored in the previous step (partial errors, resets) is complete
                // before it publishes again; the wait hides behind the cell update of the receive waves
                wait_all_vmem();
            }
            lds_barrier();  // B: the deltas of this step are in LDS
            const long long tp0 = timing ? wall_clock64() : 0;
            if (step < T - 1) {
                // partial output errors of every receiving cell from this workgroup's deltas
                const unsigned slot_off = (unsigned)((size_t)(step % kMailSlots) * slot_words * 4u);
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    const int s = nt * 16 + (lane & 15);
                    float bv[KS];
#pragma unroll
                    for (int ks = 0; ks < KS; ++ks) bv[ks] = dl[4 * ks + (lane >> 4)][s];
                    // two tiles at a time: two independent accumulation chains keep the matrix pipe busy, and
                    // the first partial errors leave while the later tiles are still computed
#pragma unroll
                    for (int m0 = 0; m0 < MT; m0 += 2) {
                        f32x4 acc[2] = {{0, 0, 0, 0}, {0, 0, 0, 0}};
#pragma unroll
                        for (int ks = 0; ks < KS; ++ks)
#pragma unroll
                            for (int u = 0; u < 2; ++u)
                                if (m0 + u < MT)
                                    acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(wA[m0 + u][ks], bv[ks], acc[u], 0, 0, 0);
                        if (s < S) {
#pragma unroll
                            for (int u = 0; u < 2; ++u) {
                                if (m0 + u >= MT) continue;
                                // the four accumulator rows of a lane are four neighbouring receiving cells
                                const int from = pw * (H / 4) + (m0 + u) * 16 + 4 * (lane >> 4);
                                const int dst = from / JB, jd = from % JB;
                                u32x4 v = __builtin_bit_cast(u32x4, acc[u]);
                                // a NaN that happens to look like the empty marker is sent as the default NaN
                                v.x = v.x == kEmpty ? 0x7FC00000u : v.x; v.y = v.y == kEmpty ? 0x7FC00000u : v.y;
                                v.z = v.z == kEmpty ? 0x7FC00000u : v.z; v.w = v.w == kEmpty ? 0x7FC00000u : v.w;
                                store128_device(mail, slot_off + ((unsigned)dst * recv_words + (unsigned)(me * S + s) * JB + jd) * 4u, v);
                            }
                        }
                    }
                }
            }
            if (step > 0 && ps < S) {
                // the words the receive waves consumed in this step (before barrier A) are empty again
                const u32x4 empty = {kEmpty, kEmpty, kEmpty, kEmpty};
                const unsigned mine_off =
                    (unsigned)(((size_t)((step - 1) % kMailSlots) * slot_words + (size_t)me * recv_words) * 4u);
#pragma unroll
                for (int jv = 0; jv < JV; ++jv)
#pragma unroll
                    for (int q = 0; q < NPOLL; ++q)
                        store128_device(mail, mine_off + poll_off + 16u * jv + (unsigned)q * poll_stride, empty);
            }
            // `dl` is rewritten only after the next barrier A, which this wave reaches after its LDS reads
            if (timing) busy += wall_clock64() - tp0;
        }
        if (timing && tid == kThreads) p.phase_ticks[(size_t)blockIdx.x * 6 + 2] = busy;
        return;
    }

    // ---------------------------------------------------------------------- receive waves
    // polling role: sequence ps, senders pg, pg + PG, ...
    const int ps = tid % NS, pg = tid / NS;
    const bool polls = ps < S;
    const unsigned poll_off = ((unsigned)(pg * S + ps) * JB) * 4u;  // bytes inside the receiver's block
    const unsigned poll_stride = (unsigned)PG * pair_words * 4u;
    // cell-update role: element tid = (sequence cs, cell cj), cell fastest
    const bool cell_thread = tid < EL;
    const int cs = tid / JB, cj = tid % JB;
    const bool cell_valid = cell_thread && cs < S;
    float p_ig = 0, p_fg = 0, p_og = 0;
    if (cell_valid) { p_ig = D.peep[0][j0 + cj]; p_fg = D.peep[1][j0 + cj]; p_og = D.peep[2][j0 + cj]; }
    // this cell's values at the slot processed in the previous iteration
    float fg_later = 0, cerr_later = 0, dig_later = 0, dfg_later = 0;
    long long ph0 = 0, ph1 = 0, ph3 = 0, poll_rounds = 0;
    const bool timing = p.phase_ticks != nullptr;
    const long long tk_begin = timing ? wall_clock64() : 0;

    wait_all_vmem();  // peepholes are in registers before the recursion starts
    lds_barrier();    // start of the recursion: coefficients of step 0 are in LDS

    for (int step = 0; step < T; ++step) {
        const long long tk0 = timing ? wall_clock64() : 0;
        const bool first = (step == 0), last = (step == T - 1);

        if (!first) {
            const float *mine = D.bmail + (size_t)((step - 1) % kMailSlots) * slot_words + (size_t)me * recv_words;
            bool ok = true;
            if (polls) {
                u32x4 w[JV][NPOLL];
                unsigned spins = 0;
                // the partial errors cannot be there before the senders' products are done: a poll that comes back
                // incomplete costs a whole memory round trip, a poll that starts a little late only the delay
                for (int d = 0; d < p.poll_delay; ++d) __builtin_amdgcn_s_sleep(1);
                for (;;) {
                    unsigned worst = 0;
#pragma unroll
                    for (int jv = 0; jv < JV; ++jv) {
                        poll_load<NPOLL>(mine, poll_off + 16u * jv, poll_stride, w[jv]);
#pragma unroll
                        for (int q = 0; q < NPOLL; ++q)
                            worst = max(max(worst, w[jv][q].x), max(max(w[jv][q].y, w[jv][q].z), w[jv][q].w));
                    }
                    if (timing) ++poll_rounds;
                    if (worst != kEmpty) break;
                    if (++spins > p.spin_limit) { ok = false; break; }
                    if ((spins & 255u) == 0u &&
                        __hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
                        ok = false;
                        break;
                    }
                    for (int d = 0; d < p.poll_gap; ++d) __builtin_amdgcn_s_sleep(1);
                }
#pragma unroll
                for (int jv = 0; jv < JV; ++jv) {
                    f32x4 sum = {0, 0, 0, 0};
#pragma unroll
                    for (int q = 0; q < NPOLL; ++q) sum += __builtin_bit_cast(f32x4, w[jv][q]);
                    *reinterpret_cast<f32x4 *>(&psum[pg][ps * JB + 4 * jv]) = sum;
                }
            }
            // polling lanes have drained their loads; stated for all lanes so that the compiler knows nothing
            // is outstanding here
            wait_all_vmem();
            if (!ok) wait_failed = 1;
            lds_barrier();  // A
            if (wait_failed) {
                if (tid == 0) raise_abort(p);
                return;
            }
        }

        const long long tk1 = timing ? wall_clock64() : 0;
        if (cell_valid) {
            float e = coef[C_E][tid];
            if (!first) {
                // pairwise sum of the sender groups' partial errors: log2(PG) dependent additions instead of PG
                float part[PG];
#pragma unroll
                for (int q = 0; q < PG; ++q) part[q] = psum[q][tid];
#pragma unroll
                for (int q = 0; q < PG / 2; ++q) part[q] += part[q + PG / 2];
#pragma unroll
                for (int q = 0; q < PG / 4; ++q) part[q] += part[q + PG / 4];
#pragma unroll
                for (int q = 0; q < PG / 8; ++q) part[q] += part[q + PG / 8];
#pragma unroll
                for (int q = 0; q < PG / 16; ++q) part[q] += part[q + PG / 16];
                static_assert(PG == 8 || PG == 16, "pairwise sum written for 8 or 16 sender groups");
                e += part[0];
            }
            const float fg = coef[C_FGACT][tid];
            float s_ni = 0, s_ig = 0, s_fg = 0, s_og = 0, ce = 0;
            if (coef[C_DUMMY][tid] == 0.0f) {
                const float d_og = (coef[C_OG][tid] * e) + coef[C_DOG][tid];
                ce = coef[C_CE][tid] * e + p_og * d_og;
                if (!first) ce += (fg_later * cerr_later + p_ig * dig_later + p_fg * dfg_later);
                const float d_ni = coef[C_NI][tid] * ce;
                const float d_fg = last ? 0.0f : coef[C_FG][tid] * ce;
                const float d_ig = coef[C_IG][tid] * ce;
                s_ni = clip1(d_ni); s_ig = clip1(d_ig); s_fg = clip1(d_fg); s_og = clip1(d_og);
            }
            dl[0 * JB + cj][cs] = s_ni; dl[1 * JB + cj][cs] = s_ig;
            dl[2 * JB + cj][cs] = s_fg; dl[3 * JB + cj][cs] = s_og;
            res[0][tid] = e; res[1][tid] = ce;
            fg_later = fg; cerr_later = ce; dig_later = s_ig; dfg_later = s_fg;
        }
        lds_barrier();  // B
        // `dl`, `res`, `coef` and `psum` change only between the barriers of later steps
        if (timing) {
            const long long tk2 = wall_clock64();
            ph0 += tk1 - tk0; ph1 += tk2 - tk1;
        }
    }
    if (timing) ph3 = wall_clock64() - tk_begin;
    if (timing && tid == 0) {
        long long *o = p.phase_ticks + (size_t)blockIdx.x * 6;
        o[0] = ph0; o[1] = ph1; o[3] = ph3; o[4] = poll_rounds;
    }
}

#include "lstm_local.hpp"
#include "lstm_local_fwd.hpp"

// Runs in front of every recursion launch (one workgroup).  If the launch before gave up, the device flag is still
// set and mailbox words may be left over: refill the mailboxes and clear the flag, so that a handle heals without
// its owner's help.  Always: zero the placement counters of the XCD-local recursion.
struct GuardParams {
    int *abort_flag;
    unsigned *ctl;
    int nctl;
    unsigned *mail[4];
    size_t words[4];
};
// the work of one workgroup (any size)
__device__ __forceinline__ void guard_body(const GuardParams &g) {
    const bool heal = __hip_atomic_load(g.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0;
    if (heal) {
        for (int m = 0; m < 4; ++m)
            for (size_t i = threadIdx.x; i < g.words[m]; i += blockDim.x) g.mail[m][i] = kEmpty;
    }
    for (int i = threadIdx.x; i < g.nctl; i += blockDim.x) g.ctl[i] = 0u;
    __syncthreads();
    if (heal && threadIdx.x == 0) __hip_atomic_store(g.abort_flag, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__global__ __launch_bounds__(1024) void chain_guard(const GuardParams g) { guard_body(g); }

// ---------------------------------------------------------------------------------------------------
// Bias and peephole gradients: per (direction, gate, cell) sums over all patterns
// (LstmLayer.cu:524-541, 574-610, 625-646).  One thread per cell, a chunk of patterns per block.
// ---------------------------------------------------------------------------------------------------
struct SmallGradParams {
    int H, L, S, N;  // N = T*S patterns
    float bias;
    const float *dni, *dig, *dfg, *dog, *c;
    float *g_bias;  // + g*L + u
    float *g_peep;  // + k*L + u
    int dir;
    int chunk;
};

__global__ void lstm_small_grads(const SmallGradParams p) {
    const int u = blockIdx.x * blockDim.x + threadIdx.x;
    if (u >= p.H) return;
    const int i0 = blockIdx.y * p.chunk;
    const int i1 = min(p.N, i0 + p.chunk);
    const int H = p.H, S = p.S;
    float b0 = 0, b1 = 0, b2 = 0, b3 = 0, q_ig = 0, q_fg = 0, q_og = 0;
    for (int i = i0; i < i1; ++i) {
        const size_t o = (size_t)i * H + u;
        const float d_ni = p.dni[o], d_ig = p.dig[o], d_fg = p.dfg[o], d_og = p.dog[o];
        b0 += p.bias * d_ni; b1 += p.bias * d_ig; b2 += p.bias * d_fg; b3 += p.bias * d_og;
        q_og += p.c[o] * d_og;
        // input/forget peepholes look at the cell state one step earlier in processing order
        const int ie = p.dir ? i + S : i - S;
        if (ie >= 0 && ie < p.N) {
            const float ce = p.c[(size_t)ie * H + u];
            q_ig += ce * d_ig;
            q_fg += ce * d_fg;
        }
    }
    const int L = p.L;
    atomicAdd(p.g_bias + 0 * L + u, b0); atomicAdd(p.g_bias + 1 * L + u, b1);
    atomicAdd(p.g_bias + 2 * L + u, b2); atomicAdd(p.g_bias + 3 * L + u, b3);
    atomicAdd(p.g_peep + 0 * L + u, q_ig); atomicAdd(p.g_peep + 1 * L + u, q_fg);
    atomicAdd(p.g_peep + 2 * L + u, q_og);
}

// The same sums for layers whose cell count per direction is a multiple of four: a thread owns four neighbouring
// cells (16-byte loads), a wave walks whole rows of the state arrays, a workgroup's waves share a chunk of patterns
// and add up in LDS first, so that a gradient element takes one global atomic per chunk -- atomics to one address
// serialise, and with a short chunk they, not the loads, set the kernel's time.  blockIdx.z is the direction.
struct SmallGradDirs {
    int H, L, S, N, chunk;
    float bias;
    const float *dni[2], *dig[2], *dfg[2], *dog[2], *c[2];
    float *g_bias;  // + g*L + dir*H + u
    float *g_peep;  // + k*L + dir*H + u
};

__global__ __launch_bounds__(256) void lstm_small_grads_quads(const SmallGradDirs p) {
    __shared__ float acc[7][256];
    const int dir = blockIdx.z;
    const int quads = p.H / 4;
    const int qpb = min(quads, 64);     // quads per workgroup
    const int rows = 256 / qpb;         // pattern rows walked side by side
    const int tid = threadIdx.x;
    for (int k = 0; k < 7; ++k) acc[k][tid] = 0.0f;
    __syncthreads();
    const int ql = tid % qpb, r = tid / qpb;
    const int q = blockIdx.x * qpb + ql;
    if (r < rows && q < quads) {
        const int i0 = blockIdx.y * p.chunk, i1 = min(p.N, i0 + p.chunk);
        const int H = p.H, S = p.S;
        const f32x4 *dni = reinterpret_cast<const f32x4 *>(p.dni[dir]), *dig = reinterpret_cast<const f32x4 *>(p.dig[dir]);
        const f32x4 *dfg = reinterpret_cast<const f32x4 *>(p.dfg[dir]), *dog = reinterpret_cast<const f32x4 *>(p.dog[dir]);
        const f32x4 *c = reinterpret_cast<const f32x4 *>(p.c[dir]);
        f32x4 b0 = {0, 0, 0, 0}, b1 = b0, b2 = b0, b3 = b0, q_ig = b0, q_fg = b0, q_og = b0;
#pragma unroll 4
        for (int i = i0 + r; i < i1; i += rows) {
            const size_t o = ((size_t)i * H) / 4 + q;
            const f32x4 d_ni = dni[o], d_ig = dig[o], d_fg = dfg[o], d_og = dog[o];
            b0 += d_ni; b1 += d_ig; b2 += d_fg; b3 += d_og;
            q_og += c[o] * d_og;
            // input/forget peepholes look at the cell state one step earlier in processing order
            const int ie = dir ? i + S : i - S;
            if (ie >= 0 && ie < p.N) {
                const f32x4 ce = c[((size_t)ie * H) / 4 + q];
                q_ig += ce * d_ig;
                q_fg += ce * d_fg;
            }
        }
        const f32x4 v[7] = {b0 * p.bias, b1 * p.bias, b2 * p.bias, b3 * p.bias, q_ig, q_fg, q_og};
#pragma unroll
        for (int k = 0; k < 7; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) atomicAdd(&acc[k][4 * ql + e], v[k][e]);
    }
    __syncthreads();
    const int u = blockIdx.x * qpb * 4 + tid;
    if (tid < 4 * qpb && u < p.H) {
        float *gb = p.g_bias + dir * p.H + u, *gp = p.g_peep + dir * p.H + u;
        for (int k = 0; k < 4; ++k) atomicAdd(gb + k * p.L, acc[k][tid]);
        for (int k = 0; k < 3; ++k) atomicAdd(gp + k * p.L, acc[4 + k][tid]);
    }
}

// ---------------------------------------------------------------------------------------------------
// Step-by-step recursion for geometries the persistent kernels do not cover (cells per direction other than 64,
// 128, 256, 512, or more than 32 parallel sequences): per time step one batched recurrent product through the
// matrix-product kernel and one cell kernel, i.e. the reference's own schedule (LstmLayer.cu:1743-1949,
// :2066-2255).  One thread per (direction, sequence, cell).
// ---------------------------------------------------------------------------------------------------
__global__ void lstm_forward_step(const ChainParams p, int step) {
    const int H = p.H, S = p.S, n = S * H;
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= p.ndir * n) return;
    const int dir = idx / n, r = idx % n, s = r / H, j = r % H;
    const DirPtrs &D = p.d[dir];
    const int t = dir ? (p.T - 1 - step) : step;
    const int prev = dir ? t + 1 : t - 1;
    const bool first = step == 0;
    const size_t i = (size_t)t * n + (size_t)s * H + j;
    float *out = p.out ? p.out + ((size_t)t * S + s) * p.L + dir * H + j : nullptr;
    // padding is only looked for at or after the shortest sequence's end (LstmLayer.cu:1800-1803)
    if (t >= p.Tmin && p.pat[t * S + s] == 0) {
        if (dir) D.c[i] = 0.0f;  // only the time-reversed direction clears the cell state
        D.h[i] = 0.0f;
        if (out) *out = 0.0f;
        return;
    }
    const size_t ip = (size_t)prev * n + (size_t)s * H + j;
    float a_ni = D.ni[i] + p.bias * D.b[0][j];
    float a_ig = D.ig[i] + p.bias * D.b[1][j];
    float a_fg = D.fg[i] + p.bias * D.b[2][j];
    float a_og = D.og[i] + p.bias * D.b[3][j];
    float cp = 0.0f;
    if (!first) {
        cp = D.c[ip];
        a_ig += cp * D.peep[0][j];
        a_fg += cp * D.peep[1][j];
    }
    const float ni = tanh_act(a_ni), ig = logistic(a_ig), fg = logistic(a_fg);
    D.ni[i] = ni; D.ig[i] = ig; D.fg[i] = fg;
    float c = ni * ig;
    if (!first) c += cp * fg;
    D.c[i] = c;
    a_og += c * D.peep[2][j];
    const float og = logistic(a_og);
    D.og[i] = og;
    const float hv = tanh_act(c) * og;
    D.h[i] = hv;
    if (out) *out = hv;
}

// herr of both directions from the interleaved output errors (LstmLayer.cu:210-235)
__global__ void lstm_split_errors(const ChainParams p, size_t count) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < count; i += stride) {
        const size_t slot = i / p.L;
        const int v = (int)(i % p.L);
        const float e = p.outerr[i];
        if (v < p.H) p.d[0].herr[slot * p.H + v] = e;
        else p.d[1].herr[slot * p.H + v - p.H] = e;
    }
}

__global__ void lstm_backward_step(const ChainParams p, int step) {
    const int H = p.H, S = p.S, n = S * H;
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= p.ndir * n) return;
    const int dir = idx / n, r = idx % n, s = r / H, j = r % H;
    const DirPtrs &D = p.d[dir];
    const int t = dir ? step : (p.T - 1 - step);
    const int later = dir ? t - 1 : t + 1;    // the slot handled one step before this one
    const int earlier = dir ? t + 1 : t - 1;  // the slot the forward pass came from
    const bool first = step == 0, last = step == p.T - 1;
    const size_t i = (size_t)t * n + (size_t)s * H + j;
    if (t >= p.Tmin && p.pat[t * S + s] == 0) {
        D.dni[i] = 0.0f; D.dig[i] = 0.0f; D.dfg[i] = 0.0f; D.dog[i] = 0.0f;
        D.cerr[i] = 0.0f;
        return;
    }
    const float e = D.herr[i];
    const float ni = D.ni[i], ig = D.ig[i], og = D.og[i], c = D.c[i];
    const float tc = tanh_act(c);
    // the stored output-gate delta is read back before it is overwritten (LstmLayer.cu:300-310)
    const float d_og = (logistic_deriv(og) * tc * e) + D.dog[i];
    float ce = og * tanh_deriv(tc) * e + D.peep[2][j] * d_og;
    if (!first) {
        const size_t il = (size_t)later * n + (size_t)s * H + j;
        ce += (D.fg[il] * D.cerr[il] + D.peep[0][j] * D.dig[il] + D.peep[1][j] * D.dfg[il]);
    }
    const float d_ni = ig * tanh_deriv(ni) * ce;
    float d_fg = 0.0f;
    if (!last) d_fg = logistic_deriv(D.fg[i]) * D.c[(size_t)earlier * n + (size_t)s * H + j] * ce;
    const float d_ig = logistic_deriv(ig) * ni * ce;
    D.dni[i] = clip1(d_ni);
    D.dig[i] = clip1(d_ig);
    D.dfg[i] = clip1(d_fg);
    D.dog[i] = clip1(d_og);
    D.cerr[i] = ce;
}

}  // namespace
}  // namespace cnt

// ---------------------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------------------
struct cnt_lstm {
    cnt_lstm_desc desc;
    int ndir, H;
    int T, Tmin;  // current fraction
    const char *pat;
    float *state[2][12];
    float *fmail[2];       // forward recursion
    size_t fmail_words;
    float *bmail[2];       // backward recursion
    size_t bmail_words;
    int *abort_flag;
    int device;
    int JB, NT;
    unsigned spin_limit;
    int xcd_pack;   // forward recursion: one direction per XCD
    long long *phase_ticks;  // diagnostic buffer, allocated when CNT_LSTM_TIMING is set
    int poll_delay, poll_gap, poll_delay_fwd;
    int last_was_forward;  // which recursion the diagnostic buffer describes
    int bmail_dirty;       // the backward mailbox may hold words that are not empty
    int flmail_dirty;      // the same for the XCD-local forward recursion's mailbox
    cnt::SlotOrder slot_order;  // the loaded fraction's slots, valid ones first (set by the owner of the pattern types, or null)
    int *own_order;             // maxT * S indices + 4 counts: the list the handle makes itself for a fraction with much padding
    bool make_order;            // false inside a network, whose sequencer makes one list for all layers
    int stepwise;          // no persistent recursion kernel for this geometry: one product + one cell kernel per step
    int *latch_host, *latch_dev;  // pinned host word a kernel that gives up sets; read by the host without a sync
    int *veto;             // a network's shared flag (device), or NULL
    // XCD-local backward recursion
    int local;             // 1: lstm_backward_local runs the error recursion
    int njobs;
    struct { int dir, seq0, nseq; } job[8];
    unsigned *ctl;
    float *lmail;
    size_t lmail_words;
    float *flmail;         // XCD-local forward recursion: one mailbox per job
    size_t flmail_words;
    int fwd_local;
    int last_blocks;       // workgroups of the last recursion launch
    int warm;  // read the recursion's inputs once before the XCD-local backward recursion (off; CNT_LSTM_WARM=1: on)
    int spread_lds;  // dynamic LDS the XCD-local recursion asks for so that a compute unit takes one of its workgroups
    int poll_delay_local;  // pause before the first poll of a step in the XCD-local recursion, units of 64 clocks
    int mem_delay_local;   // pause of that recursion's memory wave after the step barrier, same units
    int poll_delay_fwd_local;  // the same for the XCD-local forward recursion
    // set by every recursion launch: the failure latch is taken only once the launch that may have set it has ended
    // (the device's recursion-order event, see launch_in_order), so that no workgroup of that launch can set it (or the
    // veto) again after the report
    int launch_pending;
    // backward recursion run as ranges of steps: the step the next range has to start at (0: a fresh pass)
    int next_step;
};

namespace cnt {
namespace {

typedef void (*chain_kernel_t)(const ChainParams);

template <int HT, int JB>
chain_kernel_t pick_nt(bool fwd, int NT) {
    if (NT == 1) return fwd ? (chain_kernel_t)lstm_forward_chain<HT, JB, 1> : (chain_kernel_t)lstm_backward_chain<HT, JB, 1>;
    if (NT == 2) return fwd ? (chain_kernel_t)lstm_forward_chain<HT, JB, 2> : (chain_kernel_t)lstm_backward_chain<HT, JB, 2>;
    return nullptr;
}

chain_kernel_t pick_kernel(bool fwd, int H, int JB, int NT) {
    if (H == 64 && JB == 4) return pick_nt<1, 4>(fwd, NT);
    if (H == 128 && JB == 4) return pick_nt<2, 4>(fwd, NT);
    if (H == 128 && JB == 8) return pick_nt<2, 8>(fwd, NT);
    if (H == 256 && JB == 4) return pick_nt<4, 4>(fwd, NT);
    if (H == 256 && JB == 8) return pick_nt<4, 8>(fwd, NT);
    if (H == 512 && JB == 8) return pick_nt<8, 8>(fwd, NT);
    return nullptr;
}

// cells per workgroup: measured on MI355X, H=256 runs ~3% faster with 4 (64 workgroups per direction) than with 8
int default_jb(int H) { return H >= 512 ? 8 : 4; }

size_t weight_count(int P, int L, int bidir) {
    const size_t H = L / (bidir ? 2 : 1);
    return (size_t)4 * P * L + (size_t)4 * L + (size_t)4 * L * H + (size_t)3 * L;
}

void fill_chain_params(const cnt_lstm *h, const float *weights, ChainParams &p) {
    const cnt_lstm_desc &d = h->desc;
    const int P = d.P, L = d.L, H = h->H;
    std::memset(&p, 0, sizeof(p));
    p.H = H; p.L = L; p.S = d.S; p.T = h->T; p.Tmin = h->Tmin; p.ndir = h->ndir; p.bias = d.bias;
    p.step_begin = 0; p.step_end = h->T;
    p.pat = h->pat;
    const size_t off_bias = (size_t)4 * P * L, off_int = off_bias + (size_t)4 * L;
    const size_t off_peep = off_int + (size_t)4 * L * H;
    for (int dir = 0; dir < h->ndir; ++dir) {
        DirPtrs &D = p.d[dir];
        float *const *s = h->state[dir];
        D.ni = s[0]; D.ig = s[1]; D.fg = s[2]; D.og = s[3]; D.c = s[4]; D.h = s[5];
        D.herr = s[6]; D.dni = s[7]; D.dig = s[8]; D.dfg = s[9]; D.dog = s[10]; D.cerr = s[11];
        D.w_int = weights + off_int + (size_t)dir * H * H;
        for (int g = 0; g < 4; ++g) D.b[g] = weights + off_bias + (size_t)g * L + dir * H;
        for (int k = 0; k < 3; ++k) D.peep[k] = weights + off_peep + (size_t)k * L + dir * H;
        D.fmail = h->fmail[dir];
        D.bmail = h->bmail[dir];
    }
    p.spin_limit = h->spin_limit;
    p.abort_flag = h->abort_flag;
    p.latch = h->latch_dev;
    p.veto = h->veto;
    p.njobs = h->njobs;
    for (int j = 0; j < h->njobs; ++j) { p.job[j].dir = h->job[j].dir; p.job[j].seq0 = h->job[j].seq0; p.job[j].nseq = h->job[j].nseq; }
    p.ctl = h->ctl;
    p.lmail = h->lmail;
    p.flmail = h->flmail;
    p.phase_ticks = h->phase_ticks;
    p.poll_delay = h->poll_delay; p.poll_gap = h->poll_gap; p.poll_delay_fwd = h->poll_delay_fwd;
}

// Reads the arrays a backward recursion is going to read, at full memory bandwidth, so that they sit in the
// memory-side cache when the recursion asks for them row by row.  A compute unit returns its vector loads in order
// over all of its waves: a row that has to come from HBM holds back the mailbox polls issued behind it, which costs
// the XCD-local recursion about 0.25 us per step (measured with the states evicted against just read); the pass
// itself takes some 20 us for 84 MB.
struct WarmParams {
    const void *ptr[16];
    unsigned long long bytes[16];
    int count;
};

__global__ __launch_bounds__(256) void warm_cache(const WarmParams w, const GuardParams g) {
    if (blockIdx.x == 0) guard_body(g);  // the guard in front of the recursion rides along (a launch less)
    const size_t first = ((size_t)blockIdx.x * blockDim.x + threadIdx.x) * 16, pitch = (size_t)gridDim.x * blockDim.x * 16;
    for (int a = 0; a < w.count; ++a) {
        const char *base = static_cast<const char *>(w.ptr[a]);
        for (size_t i = first; i + 16 <= w.bytes[a]; i += pitch) {
            const uint4 v = *reinterpret_cast<const uint4 *>(base + i);
            asm volatile("" ::"v"(v.x), "v"(v.y), "v"(v.z), "v"(v.w));
        }
    }
}

int warm_backward_inputs(const cnt_lstm *h, hipStream_t stream, const ChainParams &p, const GuardParams &g) {
    WarmParams w = {};
    const size_t state_bytes = (size_t)h->T * p.S * p.H * sizeof(float);
    auto add = [&](const void *ptr, size_t bytes) {
        if (ptr && (reinterpret_cast<uintptr_t>(ptr) & 15u) == 0) { w.ptr[w.count] = ptr; w.bytes[w.count] = bytes; ++w.count; }
    };
    for (int dir = 0; dir < h->ndir; ++dir) {
        const DirPtrs &D = p.d[dir];
        add(D.ni, state_bytes); add(D.ig, state_bytes); add(D.fg, state_bytes); add(D.og, state_bytes);
        add(D.c, state_bytes); add(D.dog, state_bytes);
    }
    add(p.outerr, (size_t)h->T * p.S * p.L * sizeof(float));
    ProfileScope prof(stream, "lstm_warm_states");
    hipLaunchKernelGGL(warm_cache, dim3(2048), dim3(256), 0, stream, w, g);
    CNT_HIP(hipGetLastError());
    return CNT_OK;
}

chain_kernel_t pick_local_kernel(int H, int &JB) {
    if (H == 256) {
        static const int wide = [] { const char *e = std::getenv("CNT_LSTM_LOCAL_JB"); return e ? std::atoi(e) : 8; }();
        if (wide == 16) { JB = 16; return (chain_kernel_t)lstm_backward_local<256, 16>; }
        JB = 8;
        return (chain_kernel_t)lstm_backward_local<256, 8>;
    }
    if (H == 128) { JB = 4; return (chain_kernel_t)lstm_backward_local<128, 4>; }
    if (H == 64) { JB = 4; return (chain_kernel_t)lstm_backward_local<64, 4>; }
    return nullptr;
}

// the forward recursion's kernel with the backward recursion's cells per workgroup (one mailbox geometry for both)
chain_kernel_t pick_local_forward_kernel(int H, int &JB) {
    if (H == 256) { JB = 8; return (chain_kernel_t)lstm_forward_local<256, 8>; }
    if (H == 128) { JB = 4; return (chain_kernel_t)lstm_forward_local<128, 4>; }
    if (H == 64) { JB = 4; return (chain_kernel_t)lstm_forward_local<64, 4>; }
    return nullptr;
}

// allows a kernel the dynamic LDS of the launches below (once per device and kernel)
int set_spread_lds(const cnt_lstm *h, const void *kernel) {
    if (h->spread_lds <= 0) return CNT_OK;
    static std::mutex mu;
    static std::vector<std::pair<int, const void *>> done;
    std::lock_guard<std::mutex> lock(mu);
    const std::pair<int, const void *> key(h->device, kernel);
    if (std::find(done.begin(), done.end(), key) == done.end()) {
        CNT_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, h->spread_lds));
        done.push_back(key);
    }
    return CNT_OK;
}

// Persistent recursion launches of one process run one at a time on a device.  Every workgroup of a team has to be
// resident before the team can take a step, and an XCD-local launch takes a compute unit per workgroup: two such
// launches that start together on different streams can each hold half of an XCD's compute units with half a team and
// wait for the other half until their bounded waits give up.  A launch therefore waits, in stream order, for the
// recursion launched before it (from whatever handle or stream); launches on one stream are ordered anyway and skip
// the wait.  The mutex keeps wait, launch and record of one launch together when several host threads launch.
struct RecursionOrder {
    std::mutex mu;
    hipEvent_t done = nullptr;
    hipStream_t last = nullptr;
    bool any = false;
};
RecursionOrder &recursion_order(int device) {
    static RecursionOrder order[64];
    return order[device >= 0 && device < 64 ? device : 0];
}
template <typename Launch>
int launch_in_order(cnt_lstm *h, hipStream_t stream, Launch launch) {
    RecursionOrder &o = recursion_order(h->device);
    std::lock_guard<std::mutex> lock(o.mu);
    if (!o.done) CNT_HIP(hipEventCreateWithFlags(&o.done, hipEventDisableTiming));
    if (o.any && o.last != stream) CNT_HIP(hipStreamWaitEvent(stream, o.done, 0));
    launch();
    CNT_HIP(hipGetLastError());
    // Also what lstm_take_failure asks: once this record (or a later one, which waited for it) has completed, every
    // recursion launched so far has ended.
    CNT_HIP(hipEventRecord(o.done, stream));
    o.last = stream; o.any = true;
    h->launch_pending = 1;
    return CNT_OK;
}

int launch_chain(cnt_lstm *h, hipStream_t stream, bool fwd, ChainParams &p) {
    const bool local = !fwd && h->local;
    int local_jb = 0;
    chain_kernel_t k = local ? pick_local_kernel(h->H, local_jb) : pick_kernel(fwd, h->H, h->JB, h->NT);
    CNT_REQUIRE(k != nullptr, "lstm: no recursion kernel for H=%d JB=%d S=%d", h->H, h->JB, h->desc.S);
    // heals the handle after a launch that gave up, zeroes the placement counters; in front of the XCD-local backward
    // recursion it is part of the cache-warming launch
    GuardParams g = {};
    g.abort_flag = h->abort_flag;
    g.ctl = h->ctl; g.nctl = h->ctl ? kCtlWords : 0;
    g.mail[0] = reinterpret_cast<unsigned *>(h->bmail[0]); g.words[0] = h->bmail[0] ? h->bmail_words : 0;
    g.mail[1] = reinterpret_cast<unsigned *>(h->bmail[1]); g.words[1] = h->bmail[1] ? h->bmail_words : 0;
    g.mail[2] = reinterpret_cast<unsigned *>(h->lmail); g.words[2] = h->lmail ? h->lmail_words : 0;
    g.mail[3] = reinterpret_cast<unsigned *>(h->flmail); g.words[3] = h->flmail ? h->flmail_words : 0;
    // a launch that continues a recursion in the middle: the counters are zeroed, nothing is refilled or warmed
    const bool resumes = local && p.step_begin > 0;
    CNT_REQUIRE(local || (p.step_begin == 0 && p.step_end == h->T), "lstm: only the XCD-local backward recursion runs a "
                "range of steps");
    CNT_REQUIRE(p.step_begin >= 0 && p.step_begin < p.step_end && p.step_end <= h->T, "lstm: steps %d..%d of %d",
                p.step_begin, p.step_end, h->T);
    if (local) {
        // A range that ends before T leaves its last partial errors in the mailbox for the range that continues it.  A
        // launch that starts over instead (the pass was abandoned) must not find them: the mailbox is refilled.
        CNT_REQUIRE(p.step_begin == 0 || p.step_begin == h->next_step, "lstm: the backward recursion stands at step %d, "
                    "a range cannot start at step %d", h->next_step, p.step_begin);
        if (p.step_begin == 0 && h->next_step != 0) h->bmail_dirty = 1;
        h->next_step = p.step_end < h->T ? p.step_end : 0;
    }
    const bool guard_rides = local && !fwd && h->warm && !resumes && !(h->bmail_dirty && h->lmail);
    if (!guard_rides) {
        hipLaunchKernelGGL(chain_guard, dim3(1), dim3(1024), 0, stream, g);
        CNT_HIP(hipGetLastError());
    }
    // Every word of a mailbox starts out empty.  The forward recursion across XCDs leaves its last outputs behind; the
    // backward recursions hand every word back, so their mailboxes need the fill once (and the guard above refills
    // them after a recursion that gave up).
    for (int dir = 0; dir < h->ndir; ++dir) {
        if (fwd && h->fwd_local) continue;  // that kernel's mailbox is looked after below
        if (fwd) CNT_TRY(fill_words(stream, reinterpret_cast<unsigned *>(h->fmail[dir]), h->fmail_words, kEmpty));
        else if (h->bmail_dirty && h->bmail[dir]) CNT_TRY(fill_words(stream, reinterpret_cast<unsigned *>(h->bmail[dir]), h->bmail_words, kEmpty));
    }
    if (!fwd && h->bmail_dirty && h->lmail) CNT_TRY(fill_words(stream, reinterpret_cast<unsigned *>(h->lmail), h->lmail_words, kEmpty));
    if (!fwd) h->bmail_dirty = 0;
    h->last_was_forward = fwd ? 1 : 0;
    if (local && h->warm && !resumes) {
        GuardParams none = {};
        none.abort_flag = h->abort_flag;  // with nothing to zero or refill the body only reads the flag
        CNT_TRY(warm_backward_inputs(h, stream, p, guard_rides ? g : none));
    }
    ProfileScope prof(stream, fwd ? "lstm_forward_chain" : "lstm_backward_chain");
    if (fwd && h->fwd_local) {
        // like the backward recursions, this one hands every word back as empty: the fill is needed once (the guard
        // refills after a launch that gave up)
        if (h->flmail_dirty) CNT_TRY(fill_words(stream, reinterpret_cast<unsigned *>(h->flmail), h->flmail_words, kEmpty));
        h->flmail_dirty = 0;
        int fjb = 0;
        chain_kernel_t fk = pick_local_forward_kernel(h->H, fjb);
        const int G = h->H / fjb;
        const int blocks = (h->njobs * G + 8 * (G - 1) + 7) / 8 * 8;
        h->last_blocks = blocks;
        CNT_TRY(set_spread_lds(h, reinterpret_cast<const void *>(fk)));
        p.poll_delay_fwd = h->poll_delay_fwd_local;
        return launch_in_order(h, stream, [&] {
            hipLaunchKernelGGL(fk, dim3(blocks), dim3(local_threads(h->H)), (size_t)h->spread_lds, stream, p);
        });
    }
    if (local) {
        // enough workgroups that njobs complete teams form on any spread over the XCDs
        const int G = h->H / local_jb;
        const int blocks = (h->njobs * G + 8 * (G - 1) + 7) / 8 * 8;
        h->last_blocks = blocks;
        p.poll_delay = h->poll_delay_local;
        p.mem_delay = h->mem_delay_local;
        // One workgroup per compute unit.  A team's workgroups take a step in lock-step, and two of them on one compute
        // unit share its four matrix pipes and its path to the L2 at exactly the same moments: the dispatcher, left to
        // itself, puts the 32 workgroups of a 256-cell team on 16-17 compute units, and a step then takes 1.55 us instead
        // of 1.30 us (measured on MI355X, benchmark layer: 932 -> 781 us per launch).  What keeps a second workgroup of
        // this kernel off a compute unit is its LDS request: the launch asks for a little more than half of a compute
        // unit's LDS (unused dynamic shared memory), which still leaves room for two workgroups of a matrix product
        // beside it.  CNT_LSTM_SPREAD_LDS sets the request in bytes (0: none).
        CNT_TRY(set_spread_lds(h, reinterpret_cast<const void *>(k)));
        return launch_in_order(h, stream, [&] {
            hipLaunchKernelGGL(k, dim3(blocks), dim3(local_threads(h->H)), (size_t)h->spread_lds, stream, p);
        });
    }
    const int G = h->H / h->JB;
    p.xcd_pack = fwd ? h->xcd_pack : 0;
    const int blocks = p.xcd_pack ? 8 * G : h->ndir * G;
    h->last_blocks = blocks;
    return launch_in_order(h, stream, [&] {
        hipLaunchKernelGGL(k, dim3(blocks), dim3(fwd ? kThreads + 64 * ((h->JB * 16 * h->NT + 63) / 64) + 64 : kBwdThreads), 0, stream, p);
    });
}

// The recursions of both directions step by step (see lstm_forward_step): per step the recurrent products of all
// gates and directions are one launch of the matrix-product kernel, accumulating into the slices of that step.
int stepwise_forward(cnt_lstm *h, hipStream_t stream, ChainParams &p) {
    const int H = h->H, S = h->desc.S, L = h->desc.L, n = S * H;
    const int threads = h->ndir * n;
    ProfileScope prof(stream, "lstm_forward_steps");
    for (int step = 0; step < h->T; ++step) {
        if (step > 0) {
            GemmArgs ga = {};
            ga.m = H; ga.n = S; ga.k = H;
            ga.a_kcontig = 1; ga.lda = H;  // W_int block [from + to*H]: element (to, from) at [to*H + from]
            ga.b_kcontig = 1; ga.ldb = H;
            ga.ldc = H;
            ga.nseg = 1; ga.splitk = 1; ga.epilogue = EPI_ADD;
            ga.nprob = 4 * h->ndir;
            for (int dir = 0; dir < h->ndir; ++dir) {
                const int t = dir ? (h->T - 1 - step) : step, prev = dir ? t + 1 : t - 1;
                for (int g = 0; g < 4; ++g) {
                    GemmProblem &pb = ga.prob[dir * 4 + g];
                    pb.A[0] = p.d[dir].w_int + (size_t)g * L * H;
                    pb.B[0] = p.d[dir].h + (size_t)prev * n;
                    pb.C = h->state[dir][g] + (size_t)t * n;
                }
            }
            CNT_TRY(gemm_launch(stream, ga));
        }
        hipLaunchKernelGGL(lstm_forward_step, dim3((threads + 255) / 256), dim3(256), 0, stream, p, step);
        CNT_HIP(hipGetLastError());
    }
    return CNT_OK;
}

int stepwise_backward(cnt_lstm *h, hipStream_t stream, ChainParams &p) {
    const int H = h->H, S = h->desc.S, L = h->desc.L, n = S * H;
    const int threads = h->ndir * n;
    const size_t count = (size_t)L * h->T * S;
    ProfileScope prof(stream, "lstm_backward_steps");
    if (h->ndir == 2) {
        size_t blocks = (count + 255) / 256;
        if (blocks > 4096) blocks = 4096;
        hipLaunchKernelGGL(lstm_split_errors, dim3((unsigned)blocks), dim3(256), 0, stream, p, count);
        CNT_HIP(hipGetLastError());
    } else {
        CNT_HIP(hipMemcpyAsync(p.d[0].herr, p.outerr, count * sizeof(float), hipMemcpyDeviceToDevice, stream));
    }
    for (int step = 0; step < h->T; ++step) {
        if (step > 0) {
            // herr[t] += sum over gates of W_int[g] * delta_g[later]
            GemmArgs ga = {};
            ga.m = H; ga.n = S; ga.k = H;
            ga.a_kcontig = 0; ga.lda = H;
            ga.b_kcontig = 1; ga.ldb = H;
            ga.ldc = H;
            ga.nseg = 4; ga.splitk = 1; ga.epilogue = EPI_ADD;
            ga.nprob = h->ndir;
            for (int dir = 0; dir < h->ndir; ++dir) {
                const int t = dir ? step : (h->T - 1 - step), later = dir ? t - 1 : t + 1;
                GemmProblem &pb = ga.prob[dir];
                for (int g = 0; g < 4; ++g) {
                    pb.A[g] = p.d[dir].w_int + (size_t)g * L * H;
                    pb.B[g] = h->state[dir][7 + g] + (size_t)later * n;
                }
                pb.C = p.d[dir].herr + (size_t)t * n;
            }
            CNT_TRY(gemm_launch(stream, ga));
        }
        hipLaunchKernelGGL(lstm_backward_step, dim3((threads + 255) / 256), dim3(256), 0, stream, p, step);
        CNT_HIP(hipGetLastError());
    }
    // a unidirectional layer leaves the summed errors in the caller's buffer (LstmLayer.cu:2086-2087, :2378-2381)
    if (p.herr_out)
        CNT_HIP(hipMemcpyAsync(p.herr_out, p.d[0].herr, count * sizeof(float), hipMemcpyDeviceToDevice, stream));
    return CNT_OK;
}

}  // namespace
}  // namespace cnt

extern "C" {

long cnt_lstm_weight_count(int P, int L, int bidir) { return (long)cnt::weight_count(P, L, bidir); }

int cnt_lstm_create(const cnt_lstm_desc *desc, cnt_lstm **out) {
    using namespace cnt;
    CNT_REQUIRE(desc && out, "lstm_create: null argument");
    CNT_REQUIRE(desc->P > 0 && desc->L > 0 && desc->S > 0 && desc->maxT > 0, "lstm_create: non-positive size");
    // the reference refuses odd bidirectional sizes (LstmLayer.cu:1091-1092)
    CNT_REQUIRE(!desc->bidir || desc->L % 2 == 0, "Cannot create a bidirectional layer with an odd layer size");
    const int ndir = desc->bidir ? 2 : 1;
    const int H = desc->L / ndir;
    const int NT = (desc->S + 15) / 16;
    int JB = default_jb(H);
    if (const char *e = std::getenv("CNT_LSTM_JB")) JB = std::atoi(e);
    // H in {64, 128, 256, 512} with S <= 32 run as persistent recursion kernels; everything else step by step
    const bool stepwise = pick_kernel(true, H, JB, NT) == nullptr || std::getenv("CNT_LSTM_STEPWISE") != nullptr;
    if (stepwise) JB = 1;

    cnt_lstm *h = new (std::nothrow) cnt_lstm();
    CNT_REQUIRE(h != nullptr, "lstm_create: out of host memory");
    std::memset(h, 0, sizeof(*h));
    h->desc = *desc; h->ndir = ndir; h->H = H; h->JB = JB; h->NT = NT;
    h->stepwise = stepwise ? 1 : 0;
    h->bmail_dirty = 1;
    h->flmail_dirty = 1;
    h->spin_limit = 1u << 22;
    if (const char *e = std::getenv("CNT_LSTM_SPIN_LIMIT")) h->spin_limit = (unsigned)std::strtoul(e, nullptr, 10);
    h->xcd_pack = 0;
    if (const char *e = std::getenv("CNT_LSTM_XCD_PACK")) h->xcd_pack = std::atoi(e) != 0;
    // Backward recursion: pause before the first poll of a step, in units of 64 clocks -- the time the senders need
    // for their products (32 clocks per MFMA, (H/64)*JB*NT of them per wave), the time a store takes to become
    // visible, and a share that grows with the words all workgroups publish per step (ndir * G * H * S).  Fitted to
    // the measured optima on MI355X: 14 at 64 cells (S=8, two directions), 16-18 at 128 cells, 22-24 at 256 cells
    // with 4 or 10 sequences, 28 at 256 cells with 16 sequences and for the two-layer acoustic model, whose
    // recursions share the machine with other streams' products; 512 cells are flat between 18 and 40.
    {
        const double mfma = (H / 64) * JB * NT / 2.0;
        const double words = (double)ndir * (H / JB) * H * desc->S;
        int pause = (int)(14.0 + 1.25 * mfma + words / 90000.0 + 0.5);
        h->poll_delay = pause > 40 ? 40 : pause;
    }
    // XCD-local recursion: product (about 0.3 us) and one hop through the L2 (about 0.45 us) pass between a step's
    // barrier and the arrival of the next partial errors
    // (fitted on the benchmark models with one workgroup of a team per compute unit: the acoustic model's pass takes
    // 2.41 / 2.38 / 2.35 / 2.39 / 2.47 / 2.50 ms at 8 / 9 / 10 / 11 / 12 / 13 units, the single 256-cell layer 0.355 /
    // 0.353 / 0.361 ms at 9 / 10 / 11: a pause that ends after the words have arrived costs a whole poll round less,
    // one that ends too late costs its own length)
    h->poll_delay_local = 10;
    // The memory wave's loads and stores of a step are issued once the first poll is expected back: pause of the poll
    // plus one poll round (four 16-byte loads per lane at 256 cells, two or one below).  Measured on MI355X: acoustic
    // model 2.39 / 2.53 / 2.52 / 2.36 / 2.31 / 2.32 / 2.34 / 2.36 ms at 0 / 12 / 14 / 16 / 17 / 18 / 19 / 24 units (a wave that
    // wakes while the poll is in flight is the worst case); a 128- or 64-cell BLSTM layer alone 716 / 661 / 695 / 722 us
    // and 688 / 641 / 678 / 713 us at 0 / 15 / 17 / 19 units.  With the mailbox hand-back stores in this wave as well the
    // landscape moves by one unit (2.51 / 2.35 / 2.28 / 2.30 / 2.31 / 2.34 ms at 16 / 17 / 18 / 19 / 20 / 21).  The value kept
    // is one unit behind the best one: the step in front of the best value is a cliff, the step behind it costs 0.2 %.
    // (128- and 64-cell layers alone, hand-back stores included: 679 / 647 / 657 / 676 us and 683 / 648 / 662 / 672 us at
    // 14 / 15 / 16 / 17 units.)
    h->mem_delay_local = h->poll_delay_local + (H >= 256 ? 9 : 6);
    if (const char *e = std::getenv("CNT_LSTM_MEM_DELAY")) h->mem_delay_local = std::atoi(e);
    // The full-bandwidth read of the recursion's inputs in front of it (warm_cache) was worth 0.15 ms per model pass
    // while the memory wave's loads were issued in front of the polls; with that wave's pause it costs more than it
    // gains (2.290 -> 2.282 ms without it, 0.355 -> 0.352 ms for the single layer).  CNT_LSTM_WARM=1 turns it on.
    h->make_order = true;
    if (const char *e = std::getenv("CNT_LSTM_SKIP_PADDING")) h->make_order = std::atoi(e) != 0;
    h->warm = 0;
    if (const char *e = std::getenv("CNT_LSTM_WARM")) h->warm = std::atoi(e) != 0;
    {
        // a little more than half of a compute unit's LDS (160 KB on gfx950: 82 KB); the kernel's own few KB come on top
        int per_cu = 0, dev = 0;
        if (hipGetDevice(&dev) != hipSuccess ||
            hipDeviceGetAttribute(&per_cu, hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, dev) != hipSuccess) {
            (void)hipGetLastError();
            per_cu = 0;
        }
        h->spread_lds = per_cu >= (64 << 10) ? per_cu / 2 + 2048 : 0;
        if (const char *e = std::getenv("CNT_LSTM_SPREAD_LDS")) h->spread_lds = std::atoi(e);
    }
    if (const char *e = std::getenv("CNT_LSTM_POLL_DELAY")) h->poll_delay = h->poll_delay_local = std::atoi(e);
    // forward recursion: the senders' cell update (a few hundred clocks) plus store visibility
    // measured optima on MI355X: 26 at H=256 (S=10 and S=4), 25-26 at H=128 (S=8), 24 at H=64 (S=6); two units early
    // cost a second poll round (+0.2 us per step), every unit late costs its 0.027 us
    h->poll_delay_fwd = H <= 64 ? 24 : 26;
    // the same pause for the forward recursion on XCD-local teams: measured optima 24 at 256 cells (876 us per benchmark
    // layer; 14: 887, 18: 916, 30: 963), 14-18 at 128 cells, 18 at 64 cells
    h->poll_delay_fwd_local = H >= 256 ? 24 : H >= 128 ? 16 : 18;
    if (const char *e = std::getenv("CNT_LSTM_POLL_DELAY_FWD")) h->poll_delay_fwd = h->poll_delay_fwd_local = std::atoi(e);
    if (const char *e = std::getenv("CNT_LSTM_POLL_GAP")) h->poll_gap = std::atoi(e);
    hipError_t err = hipGetDevice(&h->device);
    const size_t nstate = (size_t)H * desc->maxT * desc->S;
    const int G = H / JB;
    // mailboxes, kMailSlots slots each: forward H*S words, backward G*G*JB*S words
    h->fmail_words = stepwise ? 1 : (size_t)kMailSlots * H * desc->S;
    h->bmail_words = stepwise ? 1 : (size_t)kMailSlots * G * H * desc->S;
    for (int dir = 0; dir < ndir && err == hipSuccess; ++dir) {
        for (int w = 0; w < 12 && err == hipSuccess; ++w) {
            err = hipMalloc(reinterpret_cast<void **>(&h->state[dir][w]), nstate * sizeof(float));
            if (err == hipSuccess) err = hipMemset(h->state[dir][w], 0, nstate * sizeof(float));
        }
        if (err == hipSuccess) err = hipMalloc(reinterpret_cast<void **>(&h->fmail[dir]), h->fmail_words * sizeof(float));
        if (err == hipSuccess) err = hipMalloc(reinterpret_cast<void **>(&h->bmail[dir]), h->bmail_words * sizeof(float));
    }
    // XCD-local error recursion: 64, 128 or 256 cells per direction and sequence groups of at most four
    {
        int local_jb = 0;
        const int max_jobs = kLocalMaxJobs / ndir;  // per direction
        const int groups = desc->S < max_jobs ? desc->S : max_jobs;
        const bool fits = !stepwise && pick_local_kernel(H, local_jb) != nullptr && (desc->S + groups - 1) / groups <= kLocalSeqs;
        const char *e = std::getenv("CNT_LSTM_LOCAL");
        h->local = fits && (!e || std::atoi(e) != 0);
        if (h->local) {
            // sequences dealt to the groups as evenly as possible, in order
            for (int dir = 0; dir < ndir; ++dir) {
                int seq = 0;
                for (int q = 0; q < groups; ++q) {
                    const int cnt = desc->S / groups + (q < desc->S % groups ? 1 : 0);
                    h->job[h->njobs].dir = dir; h->job[h->njobs].seq0 = seq; h->job[h->njobs].nseq = cnt;
                    ++h->njobs;
                    seq += cnt;
                }
            }
            h->lmail_words = (size_t)h->njobs * (size_t)kMailSlots * (H / local_jb) * (H / local_jb) * kLocalSeqs * local_jb;
            if (err == hipSuccess) err = hipMalloc(reinterpret_cast<void **>(&h->lmail), h->lmail_words * sizeof(float));
            // the forward recursion on the same teams (lstm_local_fwd.hpp); CNT_LSTM_FWD_LOCAL=0: the kernel across XCDs
            h->fwd_local = 1;
            if (const char *fe = std::getenv("CNT_LSTM_FWD_LOCAL")) h->fwd_local = std::atoi(fe) != 0;
            if (h->fwd_local) {
                int fjb = 0;
                h->fwd_local = pick_local_forward_kernel(H, fjb) != nullptr;
                if (h->fwd_local) {
                    h->flmail_words = (size_t)h->njobs * local_job_words(H, fjb);
                    if (err == hipSuccess) err = hipMalloc(reinterpret_cast<void **>(&h->flmail), h->flmail_words * sizeof(float));
                }
            }
            if (err == hipSuccess) err = hipMalloc(reinterpret_cast<void **>(&h->ctl), kCtlWords * sizeof(unsigned));
            if (err == hipSuccess) err = hipMemset(h->ctl, 0, kCtlWords * sizeof(unsigned));
        }
    }
    if (err == hipSuccess && std::getenv("CNT_LSTM_TIMING"))
        err = hipMalloc(reinterpret_cast<void **>(&h->phase_ticks), 8 * 512 * 6 * sizeof(long long));
    if (err == hipSuccess && h->phase_ticks) err = hipMemset(h->phase_ticks, 0, 8 * 512 * 6 * sizeof(long long));
    if (err == hipSuccess) err = hipMalloc(reinterpret_cast<void **>(&h->own_order), ((size_t)h->desc.maxT * h->desc.S + 4) * sizeof(int));
    if (err == hipSuccess) err = hipMalloc(reinterpret_cast<void **>(&h->abort_flag), sizeof(int));
    if (err == hipSuccess) err = hipMemset(h->abort_flag, 0, sizeof(int));
    // the word a kernel that gives up sets for the host: pinned, mapped, coherent host memory
    if (err == hipSuccess) err = hipHostMalloc(reinterpret_cast<void **>(&h->latch_host), sizeof(int), hipHostMallocMapped);
    if (err == hipSuccess) {
        *h->latch_host = 0;
        err = hipHostGetDevicePointer(reinterpret_cast<void **>(&h->latch_dev), h->latch_host, 0);
    }
    if (err != hipSuccess) {
        set_error("lstm_create: %s", hipGetErrorString(err));
        cnt_lstm_destroy(h);
        return CNT_ERR_HIP;
    }
    *out = h;
    return CNT_OK;
}

int cnt_lstm_destroy(cnt_lstm *h) {
    if (!h) return CNT_OK;
    for (int dir = 0; dir < 2; ++dir) {
        for (int w = 0; w < 12; ++w)
            if (h->state[dir][w]) (void)hipFree(h->state[dir][w]);
        if (h->fmail[dir]) (void)hipFree(h->fmail[dir]);
        if (h->bmail[dir]) (void)hipFree(h->bmail[dir]);
    }
    if (h->abort_flag) (void)hipFree(h->abort_flag);
    if (h->phase_ticks) (void)hipFree(h->phase_ticks);
    if (h->lmail) (void)hipFree(h->lmail);
    if (h->flmail) (void)hipFree(h->flmail);
    if (h->ctl) (void)hipFree(h->ctl);
    if (h->own_order) (void)hipFree(h->own_order);
    if (h->latch_host) (void)hipHostFree(h->latch_host);
    delete h;
    return CNT_OK;
}

namespace {
// everything cnt_lstm_load_sequences does; the stored output-gate deltas are cleared here, or listed in `collect` for the caller
int load_sequences_impl(cnt_lstm *h, hipStream_t stream, const char *patTypes, int curMaxT, int curMinT, cnt::LoadClears *collect) {
    using namespace cnt;
    CNT_REQUIRE(h && patTypes, "lstm_load_sequences: null argument");
    CNT_REQUIRE(curMaxT >= 1 && curMaxT <= h->desc.maxT, "lstm_load_sequences: curMaxT %d outside 1..%d", curMaxT,
                h->desc.maxT);
    CNT_REQUIRE(curMinT >= 0 && curMinT <= curMaxT, "lstm_load_sequences: curMinT %d outside 0..%d", curMinT, curMaxT);
    h->T = curMaxT; h->Tmin = curMinT; h->pat = patTypes;
    h->slot_order = SlotOrder{nullptr, nullptr};
    // A fraction with much padding (the shortest sequence at most 3/4 of the longest, and enough slots for the list's one
    // launch to pay): the weight gradients sum over its valid slots only (GemmArgs::k_order).  The owner of a network's
    // pattern types hands its own list over instead (lstm_set_slot_order).
    if (h->make_order && h->own_order && (long)curMaxT * h->desc.S >= 2048 && (curMaxT - curMinT) * 4 >= curMaxT) {
        const int n = curMaxT * h->desc.S;
        int *count = h->own_order + (size_t)h->desc.maxT * h->desc.S;
        CNT_TRY(slot_order_build(stream, patTypes, n, h->desc.S, h->own_order, count));
        h->slot_order = SlotOrder{h->own_order, count};
    }
    if (h->next_step != 0) { h->bmail_dirty = 1; h->next_step = 0; }  // an abandoned partial backward pass
    const size_t nstate = (size_t)h->H * h->desc.maxT * h->desc.S;
    if (collect && nstate % 4 == 0 && collect->n + h->ndir <= kLoadClears) {
        for (int dir = 0; dir < h->ndir; ++dir) {
            collect->ptr[collect->n] = h->state[dir][10];
            collect->count[collect->n] = nstate;
            ++collect->n;
        }
        return CNT_OK;
    }
    // stored output-gate deltas of both directions, one launch
    if (h->ndir == 2) CNT_TRY(fill_zero_pair(stream, h->state[0][10], nstate, h->state[1][10], nstate));
    else CNT_TRY(fill_zero(stream, h->state[0][10], nstate));
    return CNT_OK;
}
}  // namespace

int cnt_lstm_load_sequences(cnt_lstm *h, void *stream, const char *patTypes, int curMaxT, int curMinT) {
    return load_sequences_impl(h, static_cast<hipStream_t>(stream), patTypes, curMaxT, curMinT, nullptr);
}

extern "C++" int cnt::lstm_load_sequences_collect(cnt_lstm *h, hipStream_t stream, const char *patTypes, int curMaxT,
                                                  int curMinT, LoadClears &clears) {
    return load_sequences_impl(h, stream, patTypes, curMaxT, curMinT, &clears);
}

int cnt_lstm_set_wait_bounds(cnt_lstm *h, unsigned spin_limit, int poll_delay_backward, int poll_delay_forward) {
    using namespace cnt;
    CNT_REQUIRE(h, "lstm_set_wait_bounds: null handle");
    CNT_REQUIRE(poll_delay_backward >= 0 && poll_delay_backward <= 4096 && poll_delay_forward >= 0 &&
                poll_delay_forward <= 4096, "lstm_set_wait_bounds: poll delays must be within 0..4096");
    h->spin_limit = spin_limit;
    h->poll_delay = poll_delay_backward;
    h->poll_delay_local = poll_delay_backward < 10 ? poll_delay_backward : 10;
    if (poll_delay_backward < 10) h->mem_delay_local = poll_delay_backward;
    h->poll_delay_fwd = poll_delay_forward;
    h->poll_delay_fwd_local = poll_delay_forward < 24 ? poll_delay_forward : h->poll_delay_fwd_local;
    return CNT_OK;
}

float *cnt_lstm_state(cnt_lstm *h, int dir, int which) {
    if (!h || dir < 0 || dir >= h->ndir || which < 0 || which >= 12) return nullptr;
    return h->state[dir][which];
}

static const char *kGaveUp = "lstm: a recursion kernel gave up waiting for a neighbouring workgroup; results are invalid";

extern "C++" void cnt::lstm_set_veto(cnt_lstm *h, int *veto) {
    if (h) h->veto = veto;
}

extern "C++" int cnt::lstm_is_persistent(const cnt_lstm *h) { return h && !h->stepwise ? 1 : 0; }

extern "C++" void cnt::lstm_set_slot_order(cnt_lstm *h, const SlotOrder *order) {
    if (!h) return;
    h->make_order = false;  // from now on the caller's lists (or none) are the ones that count: no list of the handle's own
    h->slot_order = order ? *order : SlotOrder{nullptr, nullptr};
}

extern "C++" int cnt::lstm_wait_recursion(cnt_lstm *h, hipStream_t other) {
    CNT_REQUIRE(h, "lstm_wait_recursion: null handle");
    RecursionOrder &o = recursion_order(h->device);
    std::lock_guard<std::mutex> lock(o.mu);
    if (o.done && o.any) CNT_HIP(hipStreamWaitEvent(other, o.done, 0));
    return CNT_OK;
}

extern "C++" int cnt::lstm_take_failure(cnt_lstm *h) {
    if (!h || !h->latch_host) return 0;
    volatile int *latch = h->latch_host;
    if (*latch == 0) return 0;
    if (h->launch_pending) {
        // the launch that set the mark may still be running: its other workgroups would set it again after the report
        RecursionOrder &o = recursion_order(h->device);
        std::lock_guard<std::mutex> lock(o.mu);
        if (o.done && hipEventQuery(o.done) != hipSuccess) {
            (void)hipGetLastError();
            return 0;  // reported by a later call, once the launch has ended
        }
        h->launch_pending = 0;
    }
    *latch = 0;
    return 1;
}

// Every entry point that launches or consumes a recursion starts with this: a recursion that gave up in an EARLIER
// call (and has ended by now) turns the current call into CNT_ERR_DEVICE, also for callers that never call
// cnt_lstm_check.  The handle itself is healed by the guard kernel in front of its next launch.  A handle that belongs to
// a network (it carries the network's veto flag) leaves the report to the network's entry points.
#define CNT_LSTM_REPORT_FAILURE(h)              \
    do {                                        \
        if (!(h)->veto && cnt::lstm_take_failure(h)) { \
            cnt::set_error("%s", kGaveUp);      \
            return CNT_ERR_DEVICE;              \
        }                                       \
    } while (0)

int cnt_lstm_check(cnt_lstm *h, void *stream) {
    using namespace cnt;
    CNT_REQUIRE(h, "lstm_check: null handle");
    CNT_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
    if (h->phase_ticks) {
        // diagnostic: mean phase durations of the last recursion over the workgroups that took part
        const int blocks = h->last_blocks;
        const bool local = h->local && !h->last_was_forward;
        const int stride = local ? 8 : 6;
        std::vector<long long> t((size_t)blocks * stride);
        CNT_HIP(hipMemcpy(t.data(), h->phase_ticks, t.size() * sizeof(long long), hipMemcpyDeviceToHost));
        double m[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        int active = 0;
        for (int b = 0; b < blocks; ++b) {
            if (t[(size_t)b * stride + 3] == 0) continue;
            ++active;
            for (int q = 0; q < stride; ++q) m[q] += (double)t[(size_t)b * stride + q];
        }
        if (local && std::getenv("CNT_LSTM_TRACE")) {
            std::vector<long long> tr((size_t)blocks * kTraceStride);
            CNT_HIP(hipMemcpy(tr.data(), h->phase_ticks + kTraceBase, tr.size() * sizeof(long long), hipMemcpyDeviceToHost));
            for (int b = 0; b < blocks; ++b) {
                if (t[(size_t)b * stride + 3] == 0) continue;
                const long long *r = &tr[(size_t)b * kTraceStride];
                std::fprintf(stderr, "trace block %d job %lld member %lld xcd %lld hwid %lld:", b, r[0], r[1], r[2], r[3]);
                for (int q = 0; q < 5 * kTraceSteps; ++q) std::fprintf(stderr, " %lld", r[4 + q]);
                std::fprintf(stderr, "\n");
            }
        }
        CNT_HIP(hipMemset(h->phase_ticks, 0, 8 * 512 * 6 * sizeof(long long)));
        const double us = active ? 0.01 / active / h->T : 0.0;
        if (h->last_was_forward)
            std::fprintf(stderr, "lstm forward per step [us]: gather waves pause+poll %.3f product %.3f barrier %.3f loop %.3f "
                         "poll rounds %.2f (T=%d, %d workgroups)\n", m[1] * us, (m[0] - m[1] - m[2]) * us, m[2] * us, m[3] * us,
                         active ? m[4] / active / h->T : 0.0, h->T, active);
        else if (local)
            std::fprintf(stderr, "lstm backward per step [us], XCD-local: cell wave wait+poll %.3f (lane 0's polls %.3f in %.2f rounds) "
                         "update+barrier %.3f loop %.3f | product waves busy %.3f | memory wave busy %.3f (T=%d, %d workgroups)\n",
                         m[0] * us, m[6] * us, active ? m[4] / active / h->T : 0.0, m[1] * us, m[3] * us, m[2] * us, m[5] * us,
                         h->T, active);
        else
            std::fprintf(stderr, "lstm backward per step [us]: receive waves wait %.3f cell %.3f loop %.3f poll rounds %.2f | "
                         "product waves busy %.3f | memory wave busy after B %.3f (T=%d, %d workgroups)\n",
                         m[0] * us, m[1] * us, m[3] * us, active ? m[4] / active / h->T : 0.0, m[2] * us, m[5] * us, h->T, active);
    }
    if (lstm_take_failure(h)) {
        set_error("%s", kGaveUp);
        return CNT_ERR_DEVICE;
    }
    return CNT_OK;
}

int cnt_lstm_forward(cnt_lstm *h, void *stream_, const float *weights, const float *x, float *outputs) {
    using namespace cnt;
    CNT_REQUIRE(h && weights && x && outputs, "lstm_forward: null argument");
    CNT_REQUIRE(h->T > 0, "lstm_forward: load_sequences has not been called");
    CNT_LSTM_REPORT_FAILURE(h);
    if (h->next_step != 0) { h->bmail_dirty = 1; h->next_step = 0; }  // new states: a partial backward pass is void
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const cnt_lstm_desc &d = h->desc;
    const int P = d.P, L = d.L, H = h->H, N = h->T * d.S;

    // input projections of all gates and directions in one launch: a_g = W_in[g]^T x
    GemmArgs ga = {};
    ga.m = H; ga.n = N; ga.k = P;
    ga.a_kcontig = 1; ga.lda = P;  // W_in block is P x H column-major: element (unit, p) at [unit*P + p]
    ga.b_kcontig = 1; ga.ldb = P;
    ga.ldc = H;
    ga.nseg = 1; ga.splitk = 1; ga.epilogue = EPI_STORE;
    ga.nprob = 4 * h->ndir;
    for (int dir = 0; dir < h->ndir; ++dir)
        for (int g = 0; g < 4; ++g) {
            GemmProblem &pb = ga.prob[dir * 4 + g];
            pb.A[0] = weights + (size_t)g * P * L + (size_t)dir * P * H;
            pb.B[0] = x;
            pb.C = h->state[dir][g];
        }
    ga.label = "gemm:lstm_input_projection";
    CNT_TRY(gemm_launch(stream, ga));

    ChainParams p;
    fill_chain_params(h, weights, p);
    // the reference lets a unidirectional layer write its outputs directly (buffer swap, :1747-1749)
    p.out = outputs;
    if (h->stepwise) return stepwise_forward(h, stream, p);
    return launch_chain(h, stream, true, p);
}

int cnt_lstm_backward_errors(cnt_lstm *h, void *stream_, const float *weights, float *output_errors,
                             float *prev_errors) {
    using namespace cnt;
    CNT_REQUIRE(h && weights && output_errors, "lstm_backward_errors: null argument");
    CNT_REQUIRE(h->T > 0, "lstm_backward_errors: load_sequences has not been called");
    CNT_LSTM_REPORT_FAILURE(h);
    hipStream_t stream = static_cast<hipStream_t>(stream_);

    // 1. error recursion (splits the interleaved output errors on the fly)
    ChainParams p;
    fill_chain_params(h, weights, p);
    p.outerr = output_errors;
    p.herr_out = (h->ndir == 1) ? output_errors : nullptr;
    if (h->stepwise) CNT_TRY(stepwise_backward(h, stream, p));
    else CNT_TRY(launch_chain(h, stream, false, p));

    // 2. error to the preceding layer
    if (prev_errors) return cnt_lstm_backward_prev_errors(h, stream_, weights, prev_errors);
    return CNT_OK;
}

int cnt_lstm_backward_prev_errors(cnt_lstm *h, void *stream_, const float *weights, float *prev_errors) {
    CNT_REQUIRE(h, "lstm_backward_prev_errors: null argument");
    return cnt_lstm_backward_prev_errors_range(h, stream_, weights, prev_errors, 0, h->T);
}

int cnt_lstm_backward_steps_done(const cnt_lstm *h, int steps, int *t_begin, int *t_end) {
    using namespace cnt;
    CNT_REQUIRE(h && t_begin && t_end, "lstm_backward_steps_done: null argument");
    CNT_REQUIRE(h->T > 0 && steps >= 0 && steps <= h->T, "lstm_backward_steps_done: %d steps of %d", steps, h->T);
    // the first direction's recursion runs from the last time step down, the second one's from the first up
    *t_begin = h->T - steps;
    *t_end = h->ndir == 2 ? steps : h->T;
    if (*t_end < *t_begin) *t_end = *t_begin;
    return CNT_OK;
}

int cnt_lstm_backward_errors_range(cnt_lstm *h, void *stream_, const float *weights, float *output_errors, int step_begin,
                                   int step_end) {
    using namespace cnt;
    CNT_REQUIRE(h && weights && output_errors, "lstm_backward_errors_range: null argument");
    CNT_REQUIRE(h->T > 0, "lstm_backward_errors_range: load_sequences has not been called");
    CNT_REQUIRE(!h->stepwise && h->local, "lstm_backward_errors_range: this layer's recursion cannot run a range of its "
                "steps (cnt_lstm_backward_can_split)");
    CNT_LSTM_REPORT_FAILURE(h);
    ChainParams p;
    fill_chain_params(h, weights, p);
    p.outerr = output_errors;
    p.herr_out = (h->ndir == 1) ? output_errors : nullptr;
    p.step_begin = step_begin; p.step_end = step_end;
    return launch_chain(h, static_cast<hipStream_t>(stream_), false, p);
}

int cnt_lstm_backward_can_split(const cnt_lstm *h) { return h && !h->stepwise && h->local ? 1 : 0; }

int cnt_lstm_backward_prev_errors_range(cnt_lstm *h, void *stream_, const float *weights, float *prev_errors, int t_begin,
                                        int t_end) {
    using namespace cnt;
    CNT_REQUIRE(h && weights && prev_errors, "lstm_backward_prev_errors: null argument");
    CNT_REQUIRE(h->T > 0, "lstm_backward_prev_errors: load_sequences has not been called");
    CNT_REQUIRE(t_begin >= 0 && t_begin <= t_end && t_end <= h->T, "lstm_backward_prev_errors: time steps %d..%d of %d",
                t_begin, t_end, h->T);
    CNT_LSTM_REPORT_FAILURE(h);
    if (t_begin == t_end) return CNT_OK;
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const cnt_lstm_desc &d = h->desc;
    const int P = d.P, L = d.L, H = h->H, S = d.S, N = (t_end - t_begin) * S;
    const size_t first = (size_t)t_begin * S;  // slots are time-major
    // e_x = sum_{dir,g} W_in[g,dir] * delta[g,dir]  (overwrite)
    {
        GemmArgs ga = {};
        ga.m = P; ga.n = N; ga.k = H;
        ga.a_kcontig = 0; ga.lda = P;
        ga.b_kcontig = 1; ga.ldb = H;
        ga.ldc = P;
        ga.nseg = 4 * h->ndir; ga.nprob = 1; ga.splitk = 1; ga.epilogue = EPI_STORE;
        for (int dir = 0; dir < h->ndir; ++dir)
            for (int g = 0; g < 4; ++g) {
                ga.prob[0].A[dir * 4 + g] = weights + (size_t)g * P * L + (size_t)dir * P * H;
                ga.prob[0].B[dir * 4 + g] = h->state[dir][7 + g] + first * H;
            }
        ga.prob[0].C = prev_errors + first * P;
        ga.label = "gemm:lstm_prev_errors";
        CNT_TRY(gemm_launch(stream, ga));
    }
    return CNT_OK;
}

// cnt_lstm_backward_prev_errors whose product also applies the derivative of the preceding (dense) layer's activation
extern "C++" int cnt::lstm_prev_errors_delta(cnt_lstm *h, hipStream_t stream, const float *weights, float *prev_errors,
                                             int prev_act, const float *prev_y) {
    CNT_REQUIRE(h && weights && prev_errors && prev_y, "lstm_prev_errors_delta: null argument");
    CNT_REQUIRE(h->T > 0, "lstm_prev_errors_delta: load_sequences has not been called");
    CNT_LSTM_REPORT_FAILURE(h);
    const cnt_lstm_desc &d = h->desc;
    const int P = d.P, L = d.L, H = h->H, N = h->T * d.S;
    GemmArgs ga = {};
    ga.m = P; ga.n = N; ga.k = H;
    ga.a_kcontig = 0; ga.lda = P;
    ga.b_kcontig = 1; ga.ldb = H;
    ga.ldc = P;
    ga.nseg = 4 * h->ndir; ga.nprob = 1; ga.splitk = 1; ga.epilogue = EPI_STORE_DELTA;
    ga.act = prev_act;
    for (int dir = 0; dir < h->ndir; ++dir)
        for (int g = 0; g < 4; ++g) {
            ga.prob[0].A[dir * 4 + g] = weights + (size_t)g * P * L + (size_t)dir * P * H;
            ga.prob[0].B[dir * 4 + g] = h->state[dir][7 + g];
        }
    ga.prob[0].C = prev_errors;
    ga.prob[0].aux_in = prev_y;
    ga.label = "gemm:lstm_prev_errors";
    return gemm_launch(stream, ga);
}

int cnt_lstm_backward_weights(cnt_lstm *h, void *stream, const float *x, float *weight_updates) {
    return cnt::lstm_backward_weights_parts(h, static_cast<hipStream_t>(stream), x, weight_updates, 3);
}

// parts: 1 = input weights, 2 = bias, recurrent and peephole weights; the two parts write disjoint ranges of the
// weight updates and may run on different streams
extern "C++" int cnt::lstm_backward_weights_parts(cnt_lstm *h, hipStream_t stream, const float *x, float *weight_updates,
                                                  int parts) {
    CNT_REQUIRE(h && x && weight_updates, "lstm_backward_weights: null argument");
    CNT_REQUIRE(h->T > 0, "lstm_backward_weights: load_sequences has not been called");
    CNT_LSTM_REPORT_FAILURE(h);
    const cnt_lstm_desc &d = h->desc;
    const int P = d.P, L = d.L, H = h->H, S = d.S, N = h->T * S;

    // 3. weight updates (overwritten every call, as the reference's transform-assign does)
    const size_t nW = weight_count(P, L, d.bidir);
    const size_t off_bias = (size_t)4 * P * L, off_int = off_bias + (size_t)4 * L;
    const size_t off_peep = off_int + (size_t)4 * L * H;
    if ((parts & 3) == 3) {
        CNT_TRY(fill_zero(stream, weight_updates, nW));
    } else {
        if (parts & 1) CNT_TRY(fill_zero(stream, weight_updates, off_bias));
        if (parts & 2) CNT_TRY(fill_zero(stream, weight_updates + off_bias, nW - off_bias));
    }
    if (parts & 1) {
        // input weights: dW_in[g,dir] (P x H) = x (P x N) * delta^T
        GemmArgs ga = {};
        ga.m = P; ga.n = H; ga.k = N;
        ga.a_kcontig = 0; ga.lda = P;
        ga.b_kcontig = 0; ga.ldb = H;
        ga.ldc = P;
        ga.nseg = 1; ga.nprob = 4 * h->ndir; ga.epilogue = EPI_ATOMIC;
        ga.splitk = 0;  // chosen by the launcher
        for (int dir = 0; dir < h->ndir; ++dir)
            for (int g = 0; g < 4; ++g) {
                GemmProblem &pb = ga.prob[dir * 4 + g];
                pb.A[0] = x;
                pb.B[0] = h->state[dir][7 + g];
                pb.C = weight_updates + (size_t)g * P * L + (size_t)dir * P * H;
            }
        if (h->slot_order.order) {
            // the deltas are zero on padding slots: the sum over the slots leaves them out
            ga.k_order = h->slot_order.order;
            ga.k_count = h->slot_order.count;
        }
        ga.label = "gemm:lstm_dW_input";
        CNT_TRY(gemm_launch(stream, ga));
    }
    if (!(parts & 2)) return CNT_OK;
    if (h->T > 1) {
        // recurrent weights: dW_int[g,dir][src + to*H] = sum h[src] at the earlier step * delta[to]
        GemmArgs ga = {};
        ga.m = H; ga.n = H; ga.k = N - S;
        ga.a_kcontig = 0; ga.lda = H;
        ga.b_kcontig = 0; ga.ldb = H;
        ga.ldc = H;
        ga.nseg = 1; ga.nprob = 4 * h->ndir; ga.epilogue = EPI_ATOMIC;
        ga.splitk = 0;  // chosen by the launcher
        for (int dir = 0; dir < h->ndir; ++dir)
            for (int g = 0; g < 4; ++g) {
                GemmProblem &pb = ga.prob[dir * 4 + g];
                const float *hbuf = h->state[dir][5];
                const float *dl = h->state[dir][7 + g];
                // forward states pair delta[t] with h[t-1]; backward states pair delta[t] with h[t+1]
                pb.A[0] = dir ? hbuf + (size_t)S * H : hbuf;
                pb.B[0] = dir ? dl : dl + (size_t)S * H;
                pb.C = weight_updates + off_int + (size_t)g * L * H + (size_t)dir * H * H;
                // with the list of valid slots: a forward state's pairs are the valid slots from the second time step on,
                // counted from there; a backward state's are the valid slots before the last time step
                pb.k_trim = dir ? 2 : 1;
                pb.k_shift = dir ? 0 : -S;
            }
        if (h->slot_order.order) {
            ga.k_order = h->slot_order.order;
            ga.k_count = h->slot_order.count;
        }
        ga.label = "gemm:lstm_dW_internal";
        CNT_TRY(gemm_launch(stream, ga));
    }
    if (H % 4 == 0) {
        SmallGradDirs sp;
        sp.H = H; sp.L = L; sp.S = S; sp.N = N; sp.bias = d.bias;
        sp.chunk = N >= 4096 ? 64 : 16;  // a short fraction still fills some tens of workgroups
        for (int dir = 0; dir < 2; ++dir) {
            const int sd = dir < h->ndir ? dir : 0;
            sp.dni[dir] = h->state[sd][7]; sp.dig[dir] = h->state[sd][8]; sp.dfg[dir] = h->state[sd][9];
            sp.dog[dir] = h->state[sd][10]; sp.c[dir] = h->state[sd][4];
        }
        sp.g_bias = weight_updates + off_bias;
        sp.g_peep = weight_updates + off_peep;
        const int quads = H / 4, qpb = quads < 64 ? quads : 64;
        dim3 grid((quads + qpb - 1) / qpb, (N + sp.chunk - 1) / sp.chunk, h->ndir);
        ProfileScope prof(stream, "lstm_small_grads");
        hipLaunchKernelGGL(lstm_small_grads_quads, grid, dim3(256), 0, stream, sp);
        CNT_HIP(hipGetLastError());
        return CNT_OK;
    }
    for (int dir = 0; dir < h->ndir; ++dir) {
        SmallGradParams sp;
        sp.H = H; sp.L = L; sp.S = S; sp.N = N; sp.bias = d.bias;
        sp.dni = h->state[dir][7]; sp.dig = h->state[dir][8]; sp.dfg = h->state[dir][9]; sp.dog = h->state[dir][10];
        sp.c = h->state[dir][4];
        sp.g_bias = weight_updates + off_bias + dir * H;
        sp.g_peep = weight_updates + off_peep + dir * H;
        sp.dir = dir;
        sp.chunk = 32;
        dim3 grid((H + 255) / 256, (N + sp.chunk - 1) / sp.chunk);
        ProfileScope prof(stream, "lstm_small_grads");
        hipLaunchKernelGGL(lstm_small_grads, grid, dim3(256), 0, stream, sp);
        CNT_HIP(hipGetLastError());
    }
    return CNT_OK;
}


int cnt_lstm_backward(cnt_lstm *h, void *stream, const float *weights, const float *x, const float *outputs,
                      float *output_errors, float *prev_errors, float *weight_updates) {
    using namespace cnt;
    CNT_REQUIRE(outputs, "lstm_backward: null argument");
    CNT_TRY(cnt_lstm_backward_errors(h, stream, weights, output_errors, prev_errors));
    return cnt_lstm_backward_weights(h, stream, x, weight_updates);
}

}  // extern "C"
