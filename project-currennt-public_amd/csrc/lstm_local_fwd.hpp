// XCD-local forward recursion (included by lstm.hip inside its anonymous namespace, after lstm_local.hpp).
//
// Same cut as the backward recursion: jobs = (direction, at most four sequences), a team of G = H/JB workgroups per
// job on one XCD, roles handed out at run time (local_claim_role).  The forward step is a GATHER -- every workgroup
// needs h[t-1] of all H cells -- and a team whose members all poll the same lines of one L2 waits 1.6-2.5 rounds per
// step for them.  Here every receiver has its own copy: a workgroup writes the h values of its JB cells G times, once
// into the private block of every member of the team (the same 4*JB*G words per step a backward workgroup
// publishes), so polls of different workgroups never meet on a line.
//
// Mailbox of a job: plain 4-byte words [slot][receiver][source cell / 4][sequence][source cell % 4], kEmpty = not
// written yet, four slots; a receiver hands the words of a slot back as empty in the step after it has read them.
//
// Waves and roles, one LDS-only barrier per step, every LDS buffer twice (step parity):
//   gather waves (H/64)  each takes 64 source cells for all of the workgroup's (gate, cell) rows: polls its quarter of
//                        the block (one 16-byte vector per lane), passes the words through its own corner of LDS into
//                        B operands of v_mfma_f32_4x4x1 (blocks = four rows x one residue of the cell index), leaves
//                        its share of the recurrent sums in LDS.  They issue no stores.
//   cell wave (1)        after the barrier: pre-activations = input projection + recurrent sums, gates, cell state,
//                        h[t]; publishes h[t] to every member's block and empties the block it read.
//   memory wave (1)      input projections two steps ahead; gate activations, cell states and outputs of the finished
//                        step to the state arrays.

template <int H, int JB>
__global__ __launch_bounds__(local_threads(H)) void lstm_forward_local(const ChainParams p) {
    constexpr int G = H / JB;
    constexpr int NSQ = kLocalSeqs;
    constexpr int PW = H / 64;           // gather waves
    constexpr int ROWS = 4 * JB;         // (gate, cell) rows of this workgroup: row = gate * JB + cell
    constexpr int NQ = H / 64;           // 16-byte vectors per polling lane: 16 blocks x NQ x 4 cells = H
    constexpr int EL = NSQ * JB;         // (sequence, cell) elements: e = sequence * JB + cell
    constexpr int PAIR = NSQ * JB;       // words one sender leaves in one receiver's block
    constexpr int CH = PAIR / 4;         // 16-byte chunks of those
    constexpr int RECV = G * PAIR;       // words of a receiver's block = NSQ * H
    constexpr int PUB = G / (64 / CH);   // publishing stores per lane
    static_assert(EL <= 64 && G % (64 / CH) == 0 && RECV == 64 * 4 * NQ, "local forward geometry");
    enum { R_NI = 0, R_IG, R_FG, R_OG, R_C, R_H, NRES };

    __shared__ float red[2][PW][ROWS][NSQ];   // recurrent sums of the step, one share per gather wave
    // a gather wave's 64 source cells per sequence, in cell order; the pitch keeps the four sequences' 16-byte reads
    // off each other's banks
    __shared__ __attribute__((aligned(16))) float hstage[PW][NSQ][64 + 4];
    __shared__ float pre[2][4][64];       // input projections of the step
    __shared__ int pre_dummy[2][64];
    __shared__ float res[2][NRES][64];    // results of the step
    __shared__ int res_flags[2][64];      // bit 0: gate activations to store, bit 1: cell state to store
    __shared__ __attribute__((aligned(16))) float hpub[NSQ][JB];
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
    float *const mailbox = p.flmail + (size_t)job * local_job_words(H, JB);
    constexpr unsigned slot_words = (unsigned)G * RECV;
    const __amdgpu_buffer_rsrc_t mail =
        __builtin_amdgcn_make_buffer_rsrc(mailbox, 0, (int)(local_job_words(H, JB) * sizeof(float)), 0x00020000);
    auto slot_of = [&](int step) { return dir ? (T - 1 - step) : step; };

    if (wave == PW + 1) {
        // ------------------------------------------------------------------ memory wave
        struct StepIn { float a[4]; char pat; };
        const int cs = lane / JB, cj = lane % JB;
        const bool valid = lane < EL && cs < nseq;
        const int s = seq0 + cs;
        auto load_step = [&](int step, StepIn &v) {
            v = StepIn{{0, 0, 0, 0}, 1};
            if (!valid || step >= T) return;
            const int t = slot_of(step);
            const size_t gi = (size_t)t * n + (size_t)s * H + j0 + cj;
            v.a[0] = D.ni[gi]; v.a[1] = D.ig[gi]; v.a[2] = D.fg[gi]; v.a[3] = D.og[gi];
            v.pat = p.pat[t * S + s];
        };
        auto put_pre = [&](int step, const StepIn &v) {
            const int t = slot_of(step);
#pragma unroll
            for (int g = 0; g < 4; ++g) pre[step & 1][g][lane] = v.a[g];
            pre_dummy[step & 1][lane] = ((t >= p.Tmin) && (v.pat == 0)) ? 1 : 0;
        };
        auto store_results = [&](int step) {
            if (!valid) return;
            const int t = slot_of(step), b = step & 1;
            const size_t gi = (size_t)t * n + (size_t)s * H + j0 + cj;
            const int flags = res_flags[b][lane];
            if (flags & 1) {
                D.ni[gi] = res[b][R_NI][lane]; D.ig[gi] = res[b][R_IG][lane];
                D.fg[gi] = res[b][R_FG][lane]; D.og[gi] = res[b][R_OG][lane];
            }
            if (flags & 2) D.c[gi] = res[b][R_C][lane];
            const float hval = res[b][R_H][lane];
            D.h[gi] = hval;
            if (p.out) p.out[((size_t)t * S + s) * p.L + dir * H + j0 + cj] = hval;
        };
        auto run_step = [&](const int step, StepIn &far, const StepIn &near) __attribute__((always_inline)) -> bool {
            lds_barrier();  // results of step-1 and the recurrent sums of this step are in LDS
            if (wait_failed) return false;
            wait_all_vmem();  // whatever is still in flight was issued a step ago
            load_step(step + 2, far);
            if (step + 1 < T) put_pre(step + 1, near);
            if (step > 0) store_results(step - 1);
            return true;
        };
        StepIn in_a, in_b;
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

    if (wave == PW) {
        // ------------------------------------------------------------------ cell wave
        const int cs = lane / JB, cj = lane % JB;
        const bool cell_lane = lane < EL;
        const bool cell_valid = cell_lane && cs < nseq;
        float b_ni = 0, b_ig = 0, b_fg = 0, b_og = 0, p_ig = 0, p_fg = 0, p_og = 0;
        if (cell_valid) {
            b_ni = p.bias * D.b[0][j0 + cj]; b_ig = p.bias * D.b[1][j0 + cj];
            b_fg = p.bias * D.b[2][j0 + cj]; b_og = p.bias * D.b[3][j0 + cj];
            p_ig = D.peep[0][j0 + cj]; p_fg = D.peep[1][j0 + cj]; p_og = D.peep[2][j0 + cj];
        }
        // publishing role: lane l writes chunk l % CH (cells 4*half .. + 3 of one sequence) into the blocks of the
        // receivers l / CH + (64 / CH) * i
        const int ch = lane % CH, ch_half = ch / NSQ, ch_seq = ch % NSQ;
        const unsigned pub_off = (((unsigned)(lane / CH)) * RECV + (unsigned)me * PAIR + (unsigned)ch * 4u) * 4u;
        constexpr unsigned pub_stride = (unsigned)(64 / CH) * RECV * 4u;
        const unsigned reset_off = ((unsigned)me * RECV + (unsigned)lane * 4u) * 4u;
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
            float hval = 0.0f;
            if (cell_lane) {
                float a_ni = pre[b][0][lane], a_ig = pre[b][1][lane], a_fg = pre[b][2][lane], a_og = pre[b][3][lane];
                if (!first) {
#pragma unroll
                    for (int w = 0; w < PW; ++w) {
                        a_ni += red[b][w][0 * JB + cj][cs]; a_ig += red[b][w][1 * JB + cj][cs];
                        a_fg += red[b][w][2 * JB + cj][cs]; a_og += red[b][w][3 * JB + cj][cs];
                    }
                }
                int flags;
                if (pre_dummy[b][lane]) {
                    // the reference leaves the summed pre-activations in place on padding slots, clears the cell only
                    // in the time-reversed direction and emits a zero output
                    res[b][R_NI][lane] = a_ni; res[b][R_IG][lane] = a_ig; res[b][R_FG][lane] = a_fg; res[b][R_OG][lane] = a_og;
                    res[b][R_C][lane] = 0.0f;
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
                    res[b][R_NI][lane] = ni; res[b][R_IG][lane] = ig; res[b][R_FG][lane] = fg; res[b][R_OG][lane] = og;
                    res[b][R_C][lane] = c;
                    flags = 3;
                    c_prev = c;
                }
                if (!cell_valid) hval = 0.0f;
                res[b][R_H][lane] = hval;
                res_flags[b][lane] = flags;
                hpub[cs][cj] = hval;
            }
            if (step + 1 < T) {
                // the wave's own LDS writes above are visible to all of its lanes
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                u32x4 v = *reinterpret_cast<const u32x4 *>(&hpub[ch_seq][4 * ch_half]);
                v.x = v.x == kEmpty ? 0x7FC00000u : v.x; v.y = v.y == kEmpty ? 0x7FC00000u : v.y;
                v.z = v.z == kEmpty ? 0x7FC00000u : v.z; v.w = v.w == kEmpty ? 0x7FC00000u : v.w;
#pragma unroll
                for (int i = 0; i < PUB; ++i)
                    __builtin_amdgcn_raw_buffer_store_b128(v, mail, (int)((unsigned)(step % kMailSlots) * slot_words * 4u + pub_off + (unsigned)i * pub_stride), 0, 0);
            }
            if (step > 0) {
                // the words the gather waves read for this step are empty again
                const u32x4 empty = {kEmpty, kEmpty, kEmpty, kEmpty};
#pragma unroll
                for (int q = 0; q < NQ; ++q)
                    __builtin_amdgcn_raw_buffer_store_b128(empty, mail, (int)((unsigned)((step - 1) % kMailSlots) * slot_words * 4u + reset_off + (unsigned)q * 1024u), 0, 0);
            }
        }
        lds_barrier();  // results of the last step are in LDS
        return;
    }

    // ---------------------------------------------------------------------- gather waves
    // Wave pw takes the source cells 64*pw .. 64*pw + 63 for ALL of the workgroup's rows.  MFMA blocks: block = kq * RG + rg
    // multiplies the four rows 4*rg .. + 3 with the kq-th run of NI source cells (cell = NI * kq + i in instruction i), so
    // the sum over a block's cells happens inside the accumulator and only the KQ runs meet across lanes afterwards.  A
    // lane's polled vector (four neighbouring cells of one sequence) goes to LDS as it is, and a lane's B operands are
    // NI neighbouring cells of its sequence: 16-byte LDS accesses on both sides.
    const int pw = wave;
    constexpr int RG = ROWS / 4;         // groups of four rows
    constexpr int KQ = 16 / RG;          // residues of the source cell index dealt to the blocks
    constexpr int NI = 64 / KQ;          // MFMA instructions per step
    static_assert(RG * KQ == 16 && (KQ == 2 || KQ == 4), "blocks of the recurrent product");
    const int blk = lane >> 2, sub = lane & 3;  // A operand: row sub of the block; B operand and accumulator: sequence sub
    const int rg = blk % RG, kq = blk / RG;
    float wreg[NI];
    {
        const int o = rg * 4 + sub, g = o / JB, jj = o % JB;
        const float *wg = D.w_int + (size_t)g * p.L * H + (size_t)(j0 + jj) * H + 64 * pw;
#pragma unroll
        for (int i = 0; i < NI; ++i) wreg[i] = wg[NI * kq + i];
    }
    // the wave's own staging buffer: [sequence][cell], written as the words arrive, read back as B operands
    float (*hb)[64 + 4] = hstage[pw];
    const unsigned poll_off = ((unsigned)me * RECV + (unsigned)(64 * pw + lane) * 4u) * 4u;
    long long ph0 = 0, ph1 = 0, ph2 = 0, ph3 = 0, poll_rounds = 0;
    const bool timing = p.phase_ticks != nullptr;
    const long long tk_begin = timing ? wall_clock64() : 0;
    wait_all_vmem();
    lds_barrier();  // start of the recursion
    lds_barrier();  // step 0 has nothing to gather

    for (int step = 1; step < T; ++step) {
        const long long tk0 = timing ? wall_clock64() : 0;
        const float *slot = mailbox + (size_t)((step - 1) % kMailSlots) * slot_words;
        bool ok = true;
        u32x4 w[1];
        unsigned spins = 0;
        for (int d = 0; d < p.poll_delay_fwd; ++d) __builtin_amdgcn_s_sleep(1);
        for (;;) {
            poll_load<1>(slot, poll_off, 0u, w);
            const unsigned worst = max(max(w[0].x, w[0].y), max(w[0].z, w[0].w));
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
        if (timing) ph1 += wall_clock64() - tk0;
        // this lane's vector: sequence sub, source cells 4*blk .. + 3 of the wave's 64
        *reinterpret_cast<f32x4 *>(&hb[sub][4 * blk]) = __builtin_bit_cast(f32x4, w[0]);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        f32x4 acc0 = {0, 0, 0, 0}, acc1 = {0, 0, 0, 0};
#pragma unroll
        for (int i4 = 0; i4 < NI; i4 += 4) {
            const f32x4 hv = *reinterpret_cast<const f32x4 *>(&hb[sub][NI * kq + i4]);
            acc0 = __builtin_amdgcn_mfma_f32_4x4x1f32(wreg[i4 + 0], hv[0], acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_4x4x1f32(wreg[i4 + 1], hv[1], acc1, 0, 0, 0);
            acc0 = __builtin_amdgcn_mfma_f32_4x4x1f32(wreg[i4 + 2], hv[2], acc0, 0, 0, 0);
            acc1 = __builtin_amdgcn_mfma_f32_4x4x1f32(wreg[i4 + 3], hv[3], acc1, 0, 0, 0);
        }
        f32x4 sum = acc0 + acc1;
        // the residues sit in lane bits 4 and 5 (KQ = 4) or in lane bit 5 (KQ = 2)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            float v = sum[r];
            if (KQ == 4) {
                const unsigned u = __builtin_bit_cast(unsigned, v);
                const auto x = __builtin_amdgcn_permlane16_swap(u, u, false, false);
                v = __builtin_bit_cast(float, (unsigned)x[0]) + __builtin_bit_cast(float, (unsigned)x[1]);
            }
            {
                const unsigned u = __builtin_bit_cast(unsigned, v);
                const auto x = __builtin_amdgcn_permlane32_swap(u, u, false, false);
                v = __builtin_bit_cast(float, (unsigned)x[0]) + __builtin_bit_cast(float, (unsigned)x[1]);
            }
            sum[r] = v;
        }
        if (kq == 0) {
#pragma unroll
            for (int r = 0; r < 4; ++r) red[step & 1][pw][rg * 4 + r][sub] = sum[r];
        }
        if (__builtin_amdgcn_ballot_w64(!ok) != 0) wait_failed = 1;
        const long long tk2 = timing ? wall_clock64() : 0;
        lds_barrier();
        if (timing) ph2 += wall_clock64() - tk2;
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
        o[0] = ph0; o[1] = ph1; o[2] = ph2; o[3] = ph3; o[4] = poll_rounds;
    }
}
