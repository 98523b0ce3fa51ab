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
// times the four sequences of the job).  Waves and roles as in the kernel above: H/64 receive waves poll and
// reduce, H/64 product waves multiply and publish, one memory wave does every other global access.
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

constexpr int local_threads(int H) { return (2 * (H / 64) + 1) * 64; }
constexpr size_t local_job_words(int H, int JB) {
    return (size_t)kMailSlots * (H / JB) * (H / JB) * kLocalSeqs * JB;
}

__device__ __forceinline__ unsigned ctl_load(const unsigned *p) {
    return __hip_atomic_load(p, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT);
}

// Role of this workgroup: job * 64 + member, or -1.  Called by one thread.
__device__ int local_claim_role(const ChainParams &p, int G) {
    const unsigned xcd = __builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20) & 15u;  // XCC_ID, bits 3:0
    if (xcd >= 8u) return -1;
    const unsigned ticket = __hip_atomic_fetch_add(p.ctl + kCtlTickets + xcd, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    const unsigned team = ticket / (unsigned)G, member = ticket % (unsigned)G;
    if (team >= (unsigned)kLocalTeams) return -1;
    unsigned *arrived = p.ctl + kCtlArrived + xcd * kLocalTeams + team;
    unsigned *team_job = p.ctl + kCtlTeamJob + xcd * kLocalTeams + team;
    unsigned *claimed = p.ctl + kCtlClaimed;
    const unsigned before = __hip_atomic_fetch_add(arrived, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    unsigned job = 0;  // 0: undecided, j + 1: job j, kNoJob: none
    if (before == (unsigned)G - 1u) {
        // this arrival completes the team
        if (team > 0) {
            // head start for the first teams of the other XCDs: about 20 us, or until every job is taken
            const long long t0 = wall_clock64();
            while (ctl_load(claimed) < (unsigned)p.njobs && wall_clock64() - t0 < 2000) __builtin_amdgcn_s_sleep(8);
        }
        const unsigned c = __hip_atomic_fetch_add(claimed, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        job = c < (unsigned)p.njobs ? c + 1u : kNoJob;
        __hip_atomic_store(team_job, job, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
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

// sum over groups of N neighbouring lanes (N = 4, 8 or 16, groups aligned); every lane ends up with its group's total
template <int N>
__device__ __forceinline__ float group_sum(float v) {
    static_assert(N == 4 || N == 8 || N == 16, "senders per receive wave");
    auto dpp = [](float x, auto ctrl) {
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), decltype(ctrl)::value, 0xF, 0xF, false));
    };
    v += dpp(v, std::integral_constant<int, 0xB1>{});   // quad_perm [1,0,3,2]
    v += dpp(v, std::integral_constant<int, 0x4E>{});   // quad_perm [2,3,0,1]: every lane holds its quad's sum
    if (N >= 8) v += dpp(v, std::integral_constant<int, 0x141>{});   // row_half_mirror: the other quad of the eight
    if (N >= 16) v += dpp(v, std::integral_constant<int, 0x140>{});  // row_mirror: the other half of the sixteen
    return v;
}

template <int H, int JB>
__global__ __launch_bounds__(local_threads(H)) void lstm_backward_local(const ChainParams p) {
    constexpr int G = H / JB;
    constexpr int NSQ = kLocalSeqs;
    constexpr int PW = H / 64;        // product waves, and receive waves
    constexpr int SPW = 64 / JB;      // senders whose words one receive wave polls
    constexpr int EL = NSQ * JB;      // (sequence, cell) elements of this workgroup: e = sequence * JB + cell
    constexpr int KW = 4 * JB;        // k extent of the product: (gate, own cell)
    constexpr int DP = KW + 4;        // pitch of a sequence's deltas in LDS (16-byte reads of four sequences: no bank shared)
    constexpr int PAIR = NSQ * JB;    // words of one (receiver, sender) pair
    constexpr int RECV = G * PAIR;    // words one receiver gets per step
    static_assert(JB % 4 == 0 && 64 % JB == 0 && EL <= 64 && G <= 64 && G % SPW == 0 && G / SPW == PW, "local recursion geometry");
    enum { C_OG = 0, C_CE, C_NI, C_FG, C_IG, C_E, C_DOG, C_FGACT, C_DUMMY, NCOEF };

    __shared__ __attribute__((aligned(16))) float psum[PW][EL];
    __shared__ __attribute__((aligned(16))) float dl[NSQ][DP];
    __shared__ float coef[NCOEF][EL];
    __shared__ float res[2][EL];  // summed output error, cell error
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

    if (wave == 2 * PW) {
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
            if (lane >= EL) return;
            const int t = slot_of(step);
            const float tc = tanh_act(x.c);
            coef[C_OG][lane] = logistic_deriv(x.og) * tc;           // d_og = this * e + dog_old
            coef[C_CE][lane] = x.og * tanh_deriv(tc);               // ce   = this * e + ...
            coef[C_NI][lane] = x.ig * tanh_deriv(x.ni);             // d_ni = this * ce
            coef[C_FG][lane] = logistic_deriv(x.fg) * x.c_earlier;  // d_fg = this * ce
            coef[C_IG][lane] = logistic_deriv(x.ig) * x.ni;         // d_ig = this * ce
            coef[C_E][lane] = x.e;
            coef[C_DOG][lane] = x.dog_old;
            coef[C_FGACT][lane] = x.fg;
            coef[C_DUMMY][lane] = ((t >= p.Tmin) && (x.pat == 0)) ? 1.0f : 0.0f;
        };
        auto run_step = [&](const int step, StepIn &far, const StepIn &near) __attribute__((always_inline)) -> bool {
            const int t = slot_of(step);
            if (step > 0) {
                lds_barrier();  // A: partial sums are in LDS
                if (wait_failed) return false;
            }
            wait_all_vmem();  // everything still in flight is at least a step old
            load_step(step + 2, far);
            lds_barrier();  // B: results of this step are in LDS
            if (step + 1 < T) put_coef(step + 1, near);
            if (valid) {
                const size_t gi = (size_t)t * n + (size_t)s * H + j0 + ec;
                D.dni[gi] = dl[ej][0 * JB + ec]; D.dig[gi] = dl[ej][1 * JB + ec];
                D.dfg[gi] = dl[ej][2 * JB + ec]; D.dog[gi] = dl[ej][3 * JB + ec];
                D.cerr[gi] = res[1][lane];
                if (p.herr_out) p.herr_out[gi] = res[0][lane];
                else D.herr[gi] = res[0][lane];
            }
            return true;
        };
        StepIn in_a, in_b;
        load_step(0, in_a);
        load_step(1, in_b);
        put_coef(0, in_a);
        lds_barrier();  // start of the recursion
        for (int step = 0; step < T; step += 2) {
            if (!run_step(step, in_a, in_b)) return;
            if (step + 1 < T && !run_step(step + 1, in_b, in_a)) return;
        }
        return;
    }

    if (wave >= PW) {
        // ------------------------------------------------------------------ product waves
        const int pw = wave - PW;
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
        // reset role: sixteen bytes of the block this workgroup's receive waves poll
        const unsigned reset_off = ((unsigned)me * RECV + (unsigned)(tid - PW * 64) * 4u) * 4u;
        wait_all_vmem();
        lds_barrier();  // start of the recursion
        const bool timing = p.phase_ticks != nullptr;
        long long busy = 0;
        for (int step = 0; step < T; ++step) {
            if (step > 0) {
                lds_barrier();  // A
                if (wait_failed) return;
                // everything this wave stored in the previous step (partial errors, resets) has reached the L2
                // before it publishes again; the wait hides behind the cell update
                wait_all_vmem();
            }
            lds_barrier();  // B: the deltas of this step are in LDS
            const long long tp0 = timing ? wall_clock64() : 0;
            if (step < T - 1) {
                f32x4 acc0 = {0, 0, 0, 0}, acc1 = {0, 0, 0, 0};
#pragma unroll
                for (int k4 = 0; k4 < KW; k4 += 4) {
                    const f32x4 dv = *reinterpret_cast<const f32x4 *>(&dl[bj][k4]);  // B operand: lane = 4*block + sequence
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
            if (step > 0) {
                // the words the receive waves consumed in this step (before barrier A) are empty again
                const u32x4 empty = {kEmpty, kEmpty, kEmpty, kEmpty};
                __builtin_amdgcn_raw_buffer_store_b128(empty, mail, (int)((unsigned)((step - 1) % kMailSlots) * slot_words * 4u + reset_off), 0, 0);
            }
            if (timing) busy += wall_clock64() - tp0;
        }
        if (timing && tid == PW * 64) p.phase_ticks[(size_t)blockIdx.x * 6 + 2] = busy;
        return;
    }

    // ---------------------------------------------------------------------- receive waves
    // polling role: 16-byte chunk q of the words sender g addressed to this workgroup
    const int q = lane / SPW, g = wave * SPW + lane % SPW;
    const unsigned poll_off = ((unsigned)me * RECV + (unsigned)g * PAIR + (unsigned)q * 4u) * 4u;
    // cell-update role (wave 0): element tid = sequence * JB + cell
    const bool cell_thread = tid < EL;
    const int cj = tid / JB, cc = tid % JB;
    float p_ig = 0, p_fg = 0, p_og = 0;
    if (cell_thread) { p_ig = D.peep[0][j0 + cc]; p_fg = D.peep[1][j0 + cc]; p_og = D.peep[2][j0 + cc]; }
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
            const float *slot = mailbox + (size_t)((step - 1) % kMailSlots) * slot_words;
            bool ok = true;
            u32x4 w[1];
            unsigned spins = 0;
            for (int d = 0; d < p.poll_delay; ++d) __builtin_amdgcn_s_sleep(1);
            for (;;) {
                poll_load<1>(slot, poll_off, 0u, w);
                if (timing) ++poll_rounds;
                if (max(max(w[0].x, w[0].y), max(w[0].z, w[0].w)) != kEmpty) break;
                if (++spins > p.spin_limit) { ok = false; break; }
                if ((spins & 255u) == 0u &&
                    __hip_atomic_load(p.abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) {
                    ok = false;
                    break;
                }
                for (int d = 0; d < p.poll_gap; ++d) __builtin_amdgcn_s_sleep(1);
            }
            f32x4 sum = __builtin_bit_cast(f32x4, w[0]);
            sum[0] = group_sum<SPW>(sum[0]); sum[1] = group_sum<SPW>(sum[1]);
            sum[2] = group_sum<SPW>(sum[2]); sum[3] = group_sum<SPW>(sum[3]);
            if (lane % SPW == 0) *reinterpret_cast<f32x4 *>(&psum[wave][q * 4]) = sum;  // any lane of the group would do
            wait_all_vmem();
            if (!ok) wait_failed = 1;
            lds_barrier();  // A
            if (wait_failed) {
                if (tid == 0) raise_abort(p);
                return;
            }
        }

        const long long tk1 = timing ? wall_clock64() : 0;
        if (cell_thread) {
            float e = coef[C_E][tid];
            if (!first) {
                float part[PW];
#pragma unroll
                for (int w2 = 0; w2 < PW; ++w2) part[w2] = psum[w2][tid];
                float acc = part[0];
#pragma unroll
                for (int w2 = 1; w2 < PW; ++w2) acc += part[w2];
                e += acc;
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
            dl[cj][0 * JB + cc] = s_ni; dl[cj][1 * JB + cc] = s_ig;
            dl[cj][2 * JB + cc] = s_fg; dl[cj][3 * JB + cc] = s_og;
            res[0][tid] = e; res[1][tid] = ce;
            fg_later = fg; cerr_later = ce; dig_later = s_ig; dfg_later = s_fg;
        }
        lds_barrier();  // B
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
