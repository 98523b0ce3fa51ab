// XCD-local BPTT error recursion (included by lstm.hip inside its anonymous namespace).
//
// The parallel sequences of a fraction are independent chains, and so are the two directions of a bidirectional
// layer.  The recursion is therefore cut into up to eight JOBS = (direction, group of at most four sequences), and
// every job is run by a TEAM of G = H/JB workgroups that sit on ONE XCD: the all-to-all exchange of a step then
// stays inside that XCD's L2 (plain stores, loads that only bypass the per-CU cache), which takes about half as
// long as a hop through the memory side, and a step moves G*G*4*JB words per job instead of G*G*S*JB per direction.
//
// Placement.  Nothing guarantees which XCD a workgroup lands on, so roles are handed out at run time: more
// workgroups are launched than needed, each reads the id of its XCD and takes a ticket there; G consecutive
// tickets of one XCD form a team, and a complete team claims the next unclaimed job.  Teams beyond an XCD's first
// give the other XCDs' first teams a head start, so that with an even spread every XCD runs one job on its own
// compute units, while any other spread still finds a team for every job: with W launched workgroups at least
// (W - 8*(G-1)) / G teams complete, whatever the spread, and the launch uses W = njobs*G + 8*(G-1).  Workgroups
// without a job end at once.
//
// Per workgroup (cells j0 .. j0+JB-1 of the job's direction, all T steps): the recurrent weights that read this
// workgroup's gate deltas, W[h][k] for every cell h of the direction and k = (gate, own cell), live in registers
// as operands of v_mfma_f32_4x4x1 (sixteen independent 4 x 4 outer products per instruction: four receiving cells
// times the four sequences of the job).  Waves and roles, ONE LDS-only barrier per step (every LDS buffer exists twice,
// by step parity):
//   cell wave (1)      polls all words addressed to the workgroup (H/64 16-byte loads per lane, in address order: lane
//                      = sender * JB + chunk), sums them in registers and across lanes, and runs the cell update of the
//                      4*JB elements straight from those registers; the step's coefficients were fetched from LDS
//                      while the poll was in flight.  It issues no stores.
//   product waves      after the barrier: multiply the fresh deltas with the weight slice, publish, hand the
//   (H/64)             consumed words back as empty.  They never wait for a load.
//   memory wave (1)    every other global access: loads the inputs of the cell update three steps ahead, folds what
//                      does not depend on the recursion into coefficients two steps ahead, writes the results of the
//                      finished step to the state arrays.
//
// Mailbox of a job: plain 4-byte words [slot][receiver][sender][sequence][cell of the receiver], kEmpty = not
// written yet, four slots, the receiver hands its words back as empty after use.  The ordering argument is the one
// given for lstm_backward_chain; a store is acknowledged once the XCD's L2 holds it, which is where the team's
// polls read.

constexpr int kLocalSeqs = 4;     // sequences of a job (padded)
constexpr int kLocalMaxJobs = 8;
constexpr int kLocalTeams = 16;   // teams counted per XCD
// control words (zero before every launch): tickets per XCD, jobs claimed, per (XCD, team) arrivals and job
constexpr int kCtlTickets = 0, kCtlClaimed = 8, kCtlArrived = 16, kCtlTeamJob = kCtlArrived + 8 * kLocalTeams;
constexpr int kCtlWords = kCtlTeamJob + 8 * kLocalTeams;
constexpr unsigned kNoJob = 0xFFFFFFFFu;

constexpr int local_threads(int H) { return (H / 64 + 2) * 64; }
constexpr size_t local_job_words(int H, int JB) {
    return (size_t)kMailSlots * (H / JB) * (H / JB) * kLocalSeqs * JB;
}

// The placement counters carry nothing but their own values (everything else a workgroup reads was written by earlier
// launches), so every access to them is a relaxed device-scope atomic: acquire or release at that scope would write
// back and invalidate the XCD's L2 at every access, also under the launches that run beside this one.
__device__ __forceinline__ unsigned ctl_load(const unsigned *p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Role of this workgroup: job * 64 + member, or -1.  Called by one thread.
__device__ int local_claim_role(const ChainParams &p, int G) {
    const unsigned xcd = __builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20) & 15u;  // XCC_ID, bits 3:0
    if (xcd >= 8u) return -1;
    const unsigned ticket = __hip_atomic_fetch_add(p.ctl + kCtlTickets + xcd, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned team = ticket / (unsigned)G, member = ticket % (unsigned)G;
    if (team >= (unsigned)kLocalTeams) return -1;
    unsigned *arrived = p.ctl + kCtlArrived + xcd * kLocalTeams + team;
    unsigned *team_job = p.ctl + kCtlTeamJob + xcd * kLocalTeams + team;
    unsigned *claimed = p.ctl + kCtlClaimed;
    const unsigned before = __hip_atomic_fetch_add(arrived, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    unsigned job = 0;  // 0: undecided, j + 1: job j, kNoJob: none
    if (before == (unsigned)G - 1u) {
        // this arrival completes the team
        if (team > 0) {
            // head start for the first teams of the other XCDs: about 20 us, or until every job is taken
            const long long t0 = wall_clock64();
            while (ctl_load(claimed) < (unsigned)p.njobs && wall_clock64() - t0 < 2000) __builtin_amdgcn_s_sleep(8);
        }
        const unsigned c = __hip_atomic_fetch_add(claimed, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        job = c < (unsigned)p.njobs ? c + 1u : kNoJob;
        __hip_atomic_store(team_job, job, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
        unsigned spins = 0;
        for (;;) {
            job = ctl_load(team_job);
            if (job != 0u) break;
            // every job is taken and this team is still incomplete: whoever completes it will find none left
            if (ctl_load(claimed) >= (unsigned)p.njobs && ctl_load(arrived) < (unsigned)G) { job = kNoJob; break; }
            if (++spins > p.spin_limit || __hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
                raise_abort(p);
                job = kNoJob;
                break;
            }
            __builtin_amdgcn_s_sleep(4);
        }
    }
    if (job == kNoJob) return -1;
    return (int)((job - 1u) * 64u + member);
}

// Sum over the lanes that share lane % JB (the senders polled side by side, JB = 4 or 8); every lane ends up with
// the total.  Inside a row of sixteen lanes by DPP rotations (a sum over all rotations of a row does not depend on
// the direction of the rotation), across the four rows by the two lane-swap instructions of gfx950: with both
// operands the same register, permlane16_swap returns {own row pair's even row, own row pair's odd row} and
// permlane32_swap {own half's ... } such that the two results add up to v[lane] + v[lane ^ 16] and
// v[lane] + v[lane ^ 32].
template <int JB>
__device__ __forceinline__ float sender_sum(float v) {
    static_assert(JB == 4 || JB == 8 || JB == 16, "cells per workgroup");
    auto dpp = [](float x, auto ctrl) {
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), decltype(ctrl)::value, 0xF, 0xF, false));
    };
    if (JB <= 8) v += dpp(v, std::integral_constant<int, 0x128>{});   // row_ror:8
    if (JB == 4) v += dpp(v, std::integral_constant<int, 0x124>{});   // row_ror:4
    {
        const unsigned u = __builtin_bit_cast(unsigned, v);
        const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
        v = __builtin_bit_cast(float, (unsigned)r[0]) + __builtin_bit_cast(float, (unsigned)r[1]);
    }
    {
        const unsigned u = __builtin_bit_cast(unsigned, v);
        const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
        v = __builtin_bit_cast(float, (unsigned)r[0]) + __builtin_bit_cast(float, (unsigned)r[1]);
    }
    return v;
}

// Diagnostic trace (CNT_LSTM_TIMING): for four steps in the middle of the recursion every workgroup records when its
// waves pass five points of a step, on the 100 MHz clock all compute units share.  32 entries per workgroup behind the
// phase counters: [0] job, [1] member, [2] XCD, [4 + 5*i + k] stamp k of traced step i.
constexpr int kTraceFirstStep = 100, kTraceSteps = 4, kTraceBase = 8 * 512, kTraceStride = 32;
__device__ __forceinline__ void trace_stamp(const ChainParams &p, int step, int k) {
    if (p.phase_ticks && step >= kTraceFirstStep && step < kTraceFirstStep + kTraceSteps)
        p.phase_ticks[kTraceBase + (size_t)blockIdx.x * kTraceStride + 4 + 5 * (step - kTraceFirstStep) + k] = wall_clock64();
}

template <int H, int JB>
__global__ __launch_bounds__(local_threads(H)) void lstm_backward_local(const ChainParams p) {
    constexpr int G = H / JB;
    constexpr int NSQ = kLocalSeqs;
    constexpr int PW = H / 64;        // product waves
    constexpr int SPW = 64 / JB;      // senders side by side in the polling wave
    constexpr int NL = G / SPW;       // 16-byte loads per polling lane
    constexpr int EL = NSQ * JB;      // (sequence, cell) elements of this workgroup: e = sequence * JB + cell
    constexpr int KW = 4 * JB;        // k extent of the product: (gate, own cell)
    constexpr int DP = KW + 4;        // pitch of a sequence's deltas in LDS (16-byte reads of four sequences: no bank shared)
    constexpr int PAIR = NSQ * JB;    // words of one (receiver, sender) pair
    constexpr int RECV = G * PAIR;    // words one receiver gets per step
    static_assert((JB == 4 || JB == 8 || JB == 16) && EL <= 64 && G % SPW == 0 && NL == PW, "local recursion geometry");
    enum { C_OG = 0, C_CE, C_NI, C_FG, C_IG, C_E, C_DOG, C_FGACT, C_DUMMY, NCOEF };

    __shared__ __attribute__((aligned(16))) float dl[2][NSQ][DP];
    __shared__ float coef[2][NCOEF][EL];
    __shared__ float res[2][2][EL];  // summed output error, cell error
    __shared__ int wait_failed;
    __shared__ int role_sh;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    if (tid == 0) {
        wait_failed = 0;
        role_sh = local_claim_role(p, G);
    }
    __syncthreads();
    const int role = role_sh;
    if (role < 0) return;
    const int job = role >> 6, me = role & 63;
    const int dir = p.job[job].dir, seq0 = p.job[job].seq0, nseq = p.job[job].nseq;
    const DirPtrs &D = p.d[dir];
    const int S = p.S, T = p.T;
    const int j0 = me * JB;
    const int n = S * H;
    float *const mailbox = p.lmail + (size_t)job * local_job_words(H, JB);
    constexpr unsigned slot_words = (unsigned)G * RECV;
    const __amdgpu_buffer_rsrc_t mail =
        __builtin_amdgcn_make_buffer_rsrc(mailbox, 0, (int)(local_job_words(H, JB) * sizeof(float)), 0x00020000);
    auto slot_of = [&](int step) { return dir ? step : (T - 1 - step); };

    if (wave == PW + 1) {
        // ------------------------------------------------------------------ memory wave
        struct StepIn { float e, ni, ig, fg, og, dog_old, c, c_earlier; char pat; };
        const int ej = lane / JB, ec = lane % JB;  // element `lane`: sequence seq0 + ej, cell j0 + ec
        const bool valid = lane < EL && ej < nseq;
        const int s = seq0 + ej;
        auto load_step = [&](int step, StepIn &v) {
            v = StepIn{0, 0, 0, 0, 0, 0, 0, 0, 1};
            if (!valid || step >= T) return;
            const int t = slot_of(step);
            const size_t gi = (size_t)t * n + (size_t)s * H + j0 + ec;
            v.e = p.outerr[((size_t)t * S + s) * p.L + dir * H + j0 + ec];
            v.ni = D.ni[gi]; v.ig = D.ig[gi]; v.fg = D.fg[gi]; v.og = D.og[gi];
            v.dog_old = D.dog[gi];
            v.c = D.c[gi];
            if (step + 1 < T) v.c_earlier = D.c[(size_t)slot_of(step + 1) * n + (size_t)s * H + j0 + ec];
            v.pat = p.pat[t * S + s];
        };
        auto put_coef = [&](int step, const StepIn &x) {
            if (lane >= EL || step >= T) return;
            const int t = slot_of(step), b = step & 1;
            const float tc = tanh_act(x.c);
            coef[b][C_OG][lane] = logistic_deriv(x.og) * tc;           // d_og = this * e + dog_old
            coef[b][C_CE][lane] = x.og * tanh_deriv(tc);               // ce   = this * e + ...
            coef[b][C_NI][lane] = x.ig * tanh_deriv(x.ni);             // d_ni = this * ce
            coef[b][C_FG][lane] = logistic_deriv(x.fg) * x.c_earlier;  // d_fg = this * ce
            coef[b][C_IG][lane] = logistic_deriv(x.ig) * x.ni;         // d_ig = this * ce
            coef[b][C_E][lane] = x.e;
            coef[b][C_DOG][lane] = x.dog_old;
            coef[b][C_FGACT][lane] = x.fg;
            coef[b][C_DUMMY][lane] = ((t >= p.Tmin) && (x.pat == 0)) ? 1.0f : 0.0f;
        };
        StepIn in;
        const int sb = p.step_begin;
        {
            // the first two steps' inputs together: one trip to memory instead of two before the recursion starts
            StepIn first, second;
            load_step(sb, first); load_step(sb + 1, second);
            wait_all_vmem();
            put_coef(sb, first); put_coef(sb + 1, second);
        }
        load_step(sb + 2, in);
        const bool mtiming = p.phase_ticks != nullptr;
        long long mbusy = 0;
        lds_barrier();  // start of the recursion
        for (int step = sb; step < p.step_end; ++step) {
            const int t = slot_of(step), b = step & 1;
            lds_barrier();  // results of this step are in LDS; the cell wave is done with this parity's coefficients
            if (wait_failed) return;
            // This wave's loads and stores have a whole step to complete, but a compute unit returns its vector-memory
            // accesses in order over all of its waves: issued while the cell wave's poll for the next step is in flight
            // they hold that poll back.  The wave sleeps until the first poll is expected back (its coefficient
            // arithmetic then also stays off the SIMD of a product wave while the products run).
            for (int d = 0; d < p.mem_delay; ++d) __builtin_amdgcn_s_sleep(1);
            const long long tm0 = mtiming ? wall_clock64() : 0;
            wait_all_vmem();  // inputs requested a step ago are there, state stores of the step before are done
            put_coef(step + 2, in);
            load_step(step + 3, in);
            if (valid) {
                const size_t gi = (size_t)t * n + (size_t)s * H + j0 + ec;
                D.dni[gi] = dl[b][ej][0 * JB + ec]; D.dig[gi] = dl[b][ej][1 * JB + ec];
                D.dfg[gi] = dl[b][ej][2 * JB + ec]; D.dog[gi] = dl[b][ej][3 * JB + ec];
                D.cerr[gi] = res[b][1][lane];
                if (p.herr_out) p.herr_out[gi] = res[b][0][lane];
                else D.herr[gi] = res[b][0][lane];
            }
            if (step > 0) {
                // The words the cell wave consumed in this step (before the barrier) are empty again.  The slot is used
                // again three steps from now, so this hand-back can wait for this wave's turn instead of sitting in
                // front of the next poll in the compute unit's queue.
                const u32x4 empty = {kEmpty, kEmpty, kEmpty, kEmpty};
#pragma unroll
                for (int q = 0; q < RECV / 256; ++q)
                    __builtin_amdgcn_raw_buffer_store_b128(empty, mail, (int)((unsigned)((step - 1) % kMailSlots) * slot_words * 4u +
                                                           ((unsigned)me * RECV + (unsigned)(q * 64 + lane) * 4u) * 4u), 0, 0);
            }
            if (mtiming) mbusy += wall_clock64() - tm0;
        }
        if (mtiming && lane == 0) {
            p.phase_ticks[(size_t)blockIdx.x * 8 + 5] = mbusy;
        }
        return;
    }

    if (wave >= 1) {
        // ------------------------------------------------------------------ product waves
        const int pw = wave - 1;
        const int h = 64 * pw + lane;  // receiving cell whose weights this lane holds (MFMA A operand: lane = 4*block + row)
        float wreg[KW];
#pragma unroll
        for (int k = 0; k < KW; ++k) {
            const int g = k / JB, jj = k % JB;
            wreg[k] = D.w_int[(size_t)g * p.L * H + (size_t)(j0 + jj) * H + h];
        }
        // the accumulator's four rows of lane (block b, sequence j) are the receiving cells 64*pw + 4*b .. + 3
        const int bj = lane & 3, first_cell = 64 * pw + 4 * (lane >> 2);
        const unsigned pub_off = ((unsigned)(first_cell / JB) * RECV + (unsigned)me * PAIR + (unsigned)bj * JB +
                                  (unsigned)(first_cell % JB)) * 4u;
        wait_all_vmem();
        lds_barrier();  // start of the recursion
        const bool timing = p.phase_ticks != nullptr;
        long long busy = 0;
        for (int step = p.step_begin; step < p.step_end; ++step) {
            lds_barrier();  // the deltas of this step are in LDS
            // looked at only at the end of the step: the read is in flight behind the barrier together with the
            // deltas', and what a failed step publishes no longer matters
            // read through the LDS address space: a volatile read through a generic pointer becomes a flat load, which
            // takes the vector-memory path
            const int failed = *(__attribute__((address_space(3))) volatile int *)&wait_failed;
            if (tid == 64) trace_stamp(p, step, 3);
            const long long tp0 = timing ? wall_clock64() : 0;
            // everything this wave stored in the previous step (partial errors, resets) has reached the L2 before it
            // publishes again; those stores are a step old
            wait_all_vmem();
            if (step < T - 1) {
                f32x4 acc0 = {0, 0, 0, 0}, acc1 = {0, 0, 0, 0};
#pragma unroll
                for (int k4 = 0; k4 < KW; k4 += 4) {
                    const f32x4 dv = *reinterpret_cast<const f32x4 *>(&dl[step & 1][bj][k4]);  // B operand: lane = 4*block + sequence
                    acc0 = __builtin_amdgcn_mfma_f32_4x4x1f32(wreg[k4 + 0], dv[0], acc0, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_f32_4x4x1f32(wreg[k4 + 1], dv[1], acc1, 0, 0, 0);
                    acc0 = __builtin_amdgcn_mfma_f32_4x4x1f32(wreg[k4 + 2], dv[2], acc0, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_f32_4x4x1f32(wreg[k4 + 3], dv[3], acc1, 0, 0, 0);
                }
                u32x4 v = __builtin_bit_cast(u32x4, acc0 + acc1);
                // a NaN that happens to look like the empty marker is sent as the default NaN
                v.x = v.x == kEmpty ? 0x7FC00000u : v.x; v.y = v.y == kEmpty ? 0x7FC00000u : v.y;
                v.z = v.z == kEmpty ? 0x7FC00000u : v.z; v.w = v.w == kEmpty ? 0x7FC00000u : v.w;
                __builtin_amdgcn_raw_buffer_store_b128(v, mail, (int)((unsigned)(step % kMailSlots) * slot_words * 4u + pub_off), 0, 0);
            }
            if (tid == 64) trace_stamp(p, step, 4);
            if (failed) return;
            if (timing) {
                busy += wall_clock64() - tp0;
            }
        }
        if (timing && tid == 64) p.phase_ticks[(size_t)blockIdx.x * 8 + 2] = busy;
        return;
    }

    // ---------------------------------------------------------------------- cell wave
    // polling role: lane l reads 16 bytes at l*16 of the words senders i*SPW .. i*SPW + SPW-1 addressed to this
    // workgroup, i.e. chunk q = l % JB (four cells of one sequence) of sender i*SPW + l / JB
    const unsigned poll_off = ((unsigned)me * RECV + (unsigned)lane * 4u) * 4u;
    constexpr unsigned poll_stride = (unsigned)SPW * PAIR * 4u;
    // cell-update role: after the sum every lane holds its chunk's four totals; lane q + JB*r takes cell r of chunk q,
    // which is element e = q*4 + r = sequence*JB + cell
    const bool cell_lane = lane < EL;
    const int cr = cell_lane ? lane / JB : 0;
    const int e_id = cell_lane ? (lane % JB) * 4 + cr : 0;
    const int cj = e_id / JB, cc = e_id % JB;
    float p_ig = 0, p_fg = 0, p_og = 0;
    if (cell_lane) { p_ig = D.peep[0][j0 + cc]; p_fg = D.peep[1][j0 + cc]; p_og = D.peep[2][j0 + cc]; }
    float fg_later = 0, cerr_later = 0, dig_later = 0, dfg_later = 0;
    if (p.step_begin > 0 && cell_lane && cj < nseq) {
        // a launch that starts in the middle: what the step before carried over stands in the state arrays
        const size_t gi = (size_t)slot_of(p.step_begin - 1) * n + (size_t)(seq0 + cj) * H + j0 + cc;
        fg_later = D.fg[gi]; cerr_later = D.cerr[gi]; dig_later = D.dig[gi]; dfg_later = D.dfg[gi];
    }
    long long ph0 = 0, ph1 = 0, ph3 = 0, ph6 = 0, poll_rounds = 0;
    const bool timing = p.phase_ticks != nullptr;
    const long long tk_begin = timing ? wall_clock64() : 0;

    wait_all_vmem();  // peepholes are in registers before the recursion starts
    lds_barrier();    // start of the recursion: coefficients of steps 0 and 1 are in LDS

    for (int step = p.step_begin; step < p.step_end; ++step) {
        const long long tk0 = timing ? wall_clock64() : 0;
        const bool first = (step == 0), last = (step == T - 1);
        const int b = step & 1;
        if (tid == 0) trace_stamp(p, step, 0);
        // this step's coefficients: in LDS since before the previous barrier, fetched while the poll is in flight
        const float k_og = coef[b][C_OG][e_id], k_ce = coef[b][C_CE][e_id], k_ni = coef[b][C_NI][e_id];
        const float k_fg = coef[b][C_FG][e_id], k_ig = coef[b][C_IG][e_id], k_dog = coef[b][C_DOG][e_id];
        const float fg = coef[b][C_FGACT][e_id], dummy = coef[b][C_DUMMY][e_id];
        float e = coef[b][C_E][e_id];

        bool ok = true;
        if (!first) {
            const float *slot = mailbox + (size_t)((step - 1) % kMailSlots) * slot_words;
            u32x4 w[NL];
            unsigned spins = 0;
            for (int d = 0; d < p.poll_delay; ++d) __builtin_amdgcn_s_sleep(1);
            for (;;) {
                const long long tq0 = timing ? wall_clock64() : 0;
                poll_load<NL>(slot, poll_off, poll_stride, w);
                unsigned worst = 0;
#pragma unroll
                for (int i = 0; i < NL; ++i) worst = max(max(worst, w[i].x), max(max(w[i].y, w[i].z), w[i].w));
                if (timing) { ++poll_rounds; ph6 += wall_clock64() - tq0; }
                if (worst != kEmpty) break;
                if (++spins > p.spin_limit) { ok = false; break; }
                if ((spins & 255u) == 0u &&
                    __hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
                    ok = false;
                    break;
                }
                for (int d = 0; d < p.poll_gap; ++d) __builtin_amdgcn_s_sleep(1);
            }
            f32x4 sum = __builtin_bit_cast(f32x4, w[0]);
#pragma unroll
            for (int i = 1; i < NL; ++i) sum += __builtin_bit_cast(f32x4, w[i]);
            sum[0] = sender_sum<JB>(sum[0]); sum[1] = sender_sum<JB>(sum[1]);
            sum[2] = sender_sum<JB>(sum[2]); sum[3] = sender_sum<JB>(sum[3]);
            e += cr == 0 ? sum[0] : cr == 1 ? sum[1] : cr == 2 ? sum[2] : sum[3];
        }
        const long long tk1 = timing ? wall_clock64() : 0;
        if (tid == 0) trace_stamp(p, step, 1);
        if (cell_lane) {
            float s_ni = 0, s_ig = 0, s_fg = 0, s_og = 0, ce = 0;
            if (dummy == 0.0f) {
                const float d_og = (k_og * e) + k_dog;
                ce = k_ce * e + p_og * d_og;
                if (!first) ce += (fg_later * cerr_later + p_ig * dig_later + p_fg * dfg_later);
                const float d_ni = k_ni * ce;
                const float d_fg = last ? 0.0f : k_fg * ce;
                const float d_ig = k_ig * ce;
                s_ni = clip1(d_ni); s_ig = clip1(d_ig); s_fg = clip1(d_fg); s_og = clip1(d_og);
            }
            dl[b][cj][0 * JB + cc] = s_ni; dl[b][cj][1 * JB + cc] = s_ig;
            dl[b][cj][2 * JB + cc] = s_fg; dl[b][cj][3 * JB + cc] = s_og;
            res[b][0][e_id] = e; res[b][1][e_id] = ce;
            fg_later = fg; cerr_later = ce; dig_later = s_ig; dfg_later = s_fg;
        }
        if (tid == 0) trace_stamp(p, step, 2);
        wait_all_vmem();
        const bool failed = __builtin_amdgcn_ballot_w64(!ok) != 0;  // only this wave ever gives up
        if (failed) wait_failed = 1;
        lds_barrier();
        if (failed) {
            if (lane == 0) raise_abort(p);
            return;
        }
        if (timing) {
            const long long tk3 = wall_clock64();
            ph0 += tk1 - tk0; ph1 += tk3 - tk1;
        }
    }
    if (timing) ph3 = wall_clock64() - tk_begin;
    if (timing && tid == 0) {
        long long *o = p.phase_ticks + (size_t)blockIdx.x * 8;
        o[0] = ph0; o[1] = ph1; o[3] = ph3; o[4] = poll_rounds; o[6] = ph6;
        long long *tr = p.phase_ticks + kTraceBase + (size_t)blockIdx.x * kTraceStride;
        tr[0] = job; tr[1] = me; tr[2] = __builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20) & 15u;
        tr[3] = __builtin_amdgcn_s_getreg((31 << 11) | (0 << 6) | 4);  // HW_ID: cu_id [11:8], sh_id [12], se_id [15:13]
    }
}
