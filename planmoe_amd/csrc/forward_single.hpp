// The forward chain in ONE launch that reads x once (bf16, up to 16 experts, top_k <= 4).
//
// A work-group of 8 waves owns 16 * ROUNDS consecutive tokens and there is one work-group per
// compute unit, all resident together.  Phase 1 streams the tokens in rounds of 16 (one MFMA
// M-tile): gate GEMM split-K over the 8 waves, row min / max on the way, softmax / top-k of the
// round.  A row can be quantised as soon as its own min / max are known, so every round is turned
// into codes right away, while the loads of the next rounds are in flight: the codes of the first
// rounds are parked in LDS, those of the last two stay in registers.  Then the group publishes
// its expert histogram and waits until every group has done so (the slot of a second choice needs
// the first-choice counts of the whole batch); the last round is quantised during that wait.
// Phase 2 only stores: every parked row goes to its slots in full 4 KB rows from LDS (the register
// rounds pass through the same LDS rows), empty slots are zero-filled by all work-groups together.
//
// What the groups tell each other travels in 64-bit words that carry their own validity: the
// upper half is the launch's tag, the lower half four 8-bit counts (or one float of the score
// sums).  A word is written by one atomic store and read by one atomic load, so there is no
// ordering between words to enforce, no cache write-back or invalidation, and nothing to clear
// between launches: a word of an earlier launch, or whatever an uninitialised workspace holds,
// does not carry the tag.  The tag is the workspace's launch counter + 1, plus a salt the host
// draws once per process.  Launches on one workspace follow each other in stream order and each
// adds one to the counter, so no two of them share a tag, whatever mixture of eager calls and
// replays of a captured launch they are (a per-call number mixed in would break exactly that: two
// numbers that both grow by one can cancel).  Every work-group reads the counter first thing; the
// last group stores counter + 1 at its very end, by when every group has published, hence
// started, hence read the old value.  So the counter needs no initial value, and replays of a
// captured launch, whose arguments never change, still get a tag of their own each.
//
// Replaces gates/top.py:20-26 + moe_layer.py:230-256 + fast_dispatch.py:140-201 +
// Int8Compressor::compress (int8.cpp:7-44), like the two-launch chain.
#pragma once

namespace pm {

#ifdef PM_FS_TRACE
// measurement builds only: wall-clock stamps (100 MHz) of the phases, 16 per work-group
__device__ unsigned long long fs_trace[1024 * 16];
#define FS_STAMP(i) do { if (threadIdx.x == 0) fs_trace[blockIdx.x * 16 + (i)] = wall_clock64(); } while (0)
#else
#define FS_STAMP(i) do { } while (0)
#endif

constexpr int FS_WAVES = 8;
constexpr int FS_THREADS = FS_WAVES * WAVE;
constexpr int FS_MAX_GROUPS = 512;          // work-groups the published tables are sized for
constexpr int FS_ZERO_ROWS = 8;             // empty slots per ticket
constexpr int FS_SHARE = 8;                 // work-groups that share a ticket counter
constexpr int FS_COUNTER_STRIDE = 128;      // bytes between ticket counters (a cache line each)

// waits for LDS traffic only: loads and stores to global memory that are in flight stay in flight
// across the barrier (__syncthreads would drain them)
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// the one-launch kernel's part of the workspace: the launch counter at byte 0, from byte 256 the
// ticket counters of the empty slots, one per FS_SHARE work-groups (none of these needs an initial
// value), then the published words hist[groups][CAP] (4 planes x CAP experts, four counts per
// word), me[groups][CAP]
constexpr size_t FS_COUNTER_OFFSET = 256;
constexpr size_t FS_PUB_OFFSET = FS_COUNTER_OFFSET + (size_t)(FS_MAX_GROUPS / FS_SHARE) * FS_COUNTER_STRIDE;
__host__ __device__ inline size_t fs_pub_bytes(int groups) { return FS_PUB_OFFSET + (size_t)groups * (16 + 16) * 8; }
static_assert(FS_PUB_OFFSET + (size_t)FS_MAX_GROUPS * (16 + 16) * 8 <= FWD_TABLES_OFFSET,
              "the one-launch kernel's region ends where the tables of the other entry points begin");

template <int NMMA> struct FsGeom {
    static constexpr int M = 256 * NMMA;          // model_dim: every wave owns M / 8 elements of a row
    static constexpr int NV = M / 8;              // 16-byte vectors per row
    static constexpr int RS = M + 16;             // bytes per parked code row in LDS: lanes of different
                                                  // rows fall into different banks
    static constexpr int PIECES = M / 16;         // 16-byte pieces of a code row
    static constexpr int RV = (PIECES + WAVE - 1) / WAVE;          // ... per lane (a wave stores a whole row)
    // piece i of this lane exists (rows whose length is no multiple of 1024 end inside the last pass)
    static __device__ __forceinline__ bool piece(int i, int lane) { return PIECES % WAVE == 0 || i * WAVE + lane < PIECES; }
};

// four 8-bit counts -> four 16-bit fields (sums over up to 512 groups of counts up to 64 fit)
__device__ __forceinline__ unsigned long long fs_spread(uint32_t p)
{
    return (unsigned long long)(p & 0xffu) | ((unsigned long long)(p & 0xff00u) << 8) |
           ((unsigned long long)(p & 0xff0000u) << 16) | ((unsigned long long)(p >> 24) << 48);
}

template <int SDT, int CAP, int NMMA, int ROUNDS>
__global__ __launch_bounds__(FS_THREADS) void forward_single_kernel(
    const uint4 *__restrict__ x, const uint4 *__restrict__ wg, const float *__restrict__ logit_bias,
    int samples, int experts, int k, int normalize_gate, int capacity,
    int32_t *__restrict__ indices, int32_t *__restrict__ locations, void *__restrict__ gates, int64_t stride,
    void *__restrict__ logits_out, void *__restrict__ scores_out, float *__restrict__ l_aux,
    int32_t *__restrict__ counts_out, uint8_t *__restrict__ codes, void *__restrict__ bias_out,
    void *__restrict__ scale_out, void *__restrict__ workspace, unsigned long long salt, int spin_limit,
    int32_t *__restrict__ gave_up)
{
    using S = Elem<SDT>;
    using B16 = Elem<PLANMOE_BF16>;
    using G = FsGeom<NMMA>;
    static_assert(CAP == 8 || CAP == 16, "experts per token tile");
    static_assert(ROUNDS >= 1 && ROUNDS <= 4, "one lane per token in the ranking step");
    static_assert(NMMA >= 1 && NMMA <= 16, "a lane holds NMMA 16-byte vectors of each of its rows");
    constexpr int TOK = 16 * ROUNDS;
    constexpr int REG_ROUNDS = ROUNDS < 2 ? ROUNDS : 2;    // the last rounds keep their codes in registers
    constexpr int LDS_ROUNDS = ROUNDS - REG_ROUNDS;        // the first rounds park theirs in LDS
    constexpr int PARK_ROUNDS = LDS_ROUNDS > REG_ROUNDS ? LDS_ROUNDS : REG_ROUNDS;
    constexpr int HW = CAP;                                // published histogram words per group: 4 planes x CAP / 4
    __shared__ __align__(16) uint8_t park[PARK_ROUNDS * 16 * G::RS];
    __shared__ float part[2][FS_WAVES][16][CAP + 1];
    __shared__ int32_t pstat[2][FS_WAVES][16][3];
    __shared__ uint8_t s_best[4][TOK];
    __shared__ int32_t s_rank[4][TOK];
    __shared__ float s_mn[TOK], s_sc[TOK];
    __shared__ float s_logit[TOK][CAP + 1];
    constexpr int RPASSES = (TOK * CAP + FS_THREADS - 1) / FS_THREADS;       // routing passes of the 8 waves
    __shared__ float s_me[RPASSES * FS_WAVES][CAP];
    __shared__ int32_t s_hist[4][CAP];
    __shared__ unsigned long long s_before64[HW], s_full64[HW];
    __shared__ int32_t s_full[4][CAP], s_base[4][CAP], s_tot[CAP];
    __shared__ float s_mepart[FS_THREADS / CAP][CAP];
    __shared__ int s_vote[2][FS_WAVES];
    __shared__ int s_zdone;

    const int tid = threadIdx.x, w = tid >> 6, lane = lane_id(), m = lane & 15, g = lane >> 4;
    const int groups = gridDim.x, grp = blockIdx.x, t0 = grp * TOK;
    unsigned long long *launches = reinterpret_cast<unsigned long long *>(workspace);
    unsigned long long *pub_hist = reinterpret_cast<unsigned long long *>((char *)workspace + FS_PUB_OFFSET);
    unsigned long long *pub_me = pub_hist + (size_t)groups * HW;
    const unsigned long long launch = __hip_atomic_load(launches, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1;
    const uint32_t tag = (uint32_t)launch + (uint32_t)(salt ^ (salt >> 32));
    // tickets for the empty slots are drawn from a counter that only ever grows: what it holds now
    // is this launch's zero (no group draws before every group has published, i.e. has been here)
    // (32 bits, used modulo 2^32: only differences to the value read here matter)
    uint32_t *zero_tickets = reinterpret_cast<uint32_t *>((char *)workspace + FS_COUNTER_OFFSET +
                                                          (size_t)(grp / FS_SHARE) * FS_COUNTER_STRIDE);
    const uint32_t zero_base = __hip_atomic_load(zero_tickets, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const float eps = SDT == PLANMOE_F32 ? 1.1920928955078125e-07f : SDT == PLANMOE_BF16 ? 0.0078125f : 0.0009765625f;
    if (tid < HW) { s_before64[tid] = 0; s_full64[tid] = 0; }
    if (tid == 0) s_zdone = 0;

    // lane (m, g) of wave w holds, of row m of a round, the vectors  w * 4 NMMA + 4 i + g
    const int v0 = w * (4 * NMMA) + g;
    const uint4 *bp = wg + (int64_t)min(m, experts - 1) * G::NV + v0;
    auto row_ptr = [&](int r) { return x + (int64_t)min(t0 + 16 * r + m, samples - 1) * G::NV + v0; };
    uint8_t *my_park = park + m * G::RS + v0 * 8;          // this lane's 8 bytes of vector 0 in parked row m

    uint4 buf0[NMMA], buf1[NMMA];
    uint4 b[NMMA];                                         // this wave's K range of the gate weights, loaded once
    uint2 kept[REG_ROUNDS][NMMA];                          // codes of the last rounds (phase 2)

    // ---- one round: GEMM + row statistics of 16 tokens, their logits, the codes of the early rounds
    auto round = [&](auto rc, uint4 (&cur)[NMMA]) {
        constexpr int r = decltype(rc)::value;
        constexpr int par = r & 1;
        f32x4 acc = {0.f, 0.f, 0.f, 0.f};
        RowStats<PLANMOE_BF16, true> st;
        st.init();
#pragma unroll
        for (int i = 0; i < NMMA; ++i) {
            Mma<PLANMOE_BF16>::run(cur[i], b[i], acc);
            st.add(cur[i]);
        }
        {
            int a, bb, n;
            st.reduced(a, bb, n);
#pragma unroll
            for (int off = 16; off < 64; off <<= 1) {
                a = min(a, __shfl_xor(a, off, WAVE));
                bb = max(bb, __shfl_xor(bb, off, WAVE));
                n = max(n, __shfl_xor(n, off, WAVE));
            }
            if (g == 0) { pstat[par][w][m][0] = a; pstat[par][w][m][1] = bb; pstat[par][w][m][2] = n; }
        }
        if (m < CAP) {
#pragma unroll
            for (int i = 0; i < 4; ++i) part[par][w][4 * g + i][m] = acc[i];
        }
        if constexpr (r == 1) FS_STAMP(13);
        lds_barrier();
        if constexpr (r == 1) FS_STAMP(14);

        // min / max of this lane's row over the 8 K ranges
        float mn, mx;
        {
            int a = pstat[par][0][m][0], bb = pstat[par][0][m][1], n = pstat[par][0][m][2];
#pragma unroll
            for (int ww = 1; ww < FS_WAVES; ++ww) {
                a = min(a, pstat[par][ww][m][0]); bb = max(bb, pstat[par][ww][m][1]); n = max(n, pstat[par][ww][m][2]);
            }
            RowStats<PLANMOE_BF16, true>::decode(a, bb, n, mn, mx);
        }
        const float scale = B16::round(mx - mn);
        if (w == 0 && g == 0) { s_mn[16 * r + m] = mn; s_sc[16 * r + m] = scale; }

        // logits of the round: the 8 partial sums of every (token, expert), added in wave order
        if (tid < 16 * CAP) {
            const int tok16 = tid / CAP, e = tid % CAP;
            float v = part[par][0][tok16][e];
#pragma unroll
            for (int ww = 1; ww < FS_WAVES; ++ww) v += part[par][ww][tok16][e];
            s_logit[16 * r + tok16][e] = v;
        }

        // codes of the early rounds go to LDS, then their registers take the row two rounds ahead.
        // The last rounds stay in their registers as they are and are
        // coded in phase 2, under the stores.  The mode is a property of the row, i.e. of the lane
        // here: one branch for the wave.
        if constexpr (r < LDS_ROUNDS) {
            const RowEncoder<PLANMOE_BF16> enc(mn, scale);
            const uint4 *ahead = row_ptr(r + 2);
            auto body = [&](auto mode) {
#pragma unroll
                for (int i = 0; i < NMMA; ++i) {
                    uint32_t wd[2];
                    enc.template encode<decltype(mode)::value>(cur[i], wd);
                    *reinterpret_cast<uint2 *>(my_park + r * 16 * G::RS + 32 * i) = make_uint2(wd[0], wd[1]);
                }
                // (issuing these loads piecewise between the pieces of the encode costs registers
                // that the compiler then takes from the resident gate weights)
#pragma unroll
                for (int i = 0; i < NMMA; ++i) cur[i] = ahead[4 * i];
            };
            if (__ballot(!enc.rq.fast) == 0) body(std::true_type{}); else body(std::false_type{});
        }
    };

    FS_STAMP(0);
    {
        const uint4 *p0 = row_ptr(0), *p1 = row_ptr(ROUNDS > 1 ? 1 : 0);
#pragma unroll
        for (int i = 0; i < NMMA; ++i) buf0[i] = p0[4 * i];
#pragma unroll
        for (int i = 0; i < NMMA; ++i) b[i] = bp[4 * i];
        if constexpr (ROUNDS > 1) {
#pragma unroll
            for (int i = 0; i < NMMA; ++i) buf1[i] = p1[4 * i];
        }
    }
    round(std::integral_constant<int, 0>{}, buf0);
    FS_STAMP(1);
    if constexpr (ROUNDS > 1) round(std::integral_constant<int, 1>{}, buf1);
    FS_STAMP(2);
    if constexpr (ROUNDS > 2) round(std::integral_constant<int, 2>{}, buf0);
    FS_STAMP(3);
    if constexpr (ROUNDS > 3) round(std::integral_constant<int, 3>{}, buf1);
    lds_barrier();

    // ---- routing of the group's tokens by all waves at once: CAP lanes share a token, lane el
    // holds expert el; softmax and the k-fold arg-max are butterflies over those lanes
    {
        constexpr int LPT = CAP, TPP = WAVE / LPT;
        const int el = lane % LPT, tk = lane / LPT;
        auto token_reduce = [&](auto v, auto op) { return row_allreduce<LPT>(v, op); };
        const float lbias = (logit_bias && el < experts) ? logit_bias[el] : 0.f;    // (one round trip, not one per pass)
#pragma unroll
        for (int p = 0; p < RPASSES; ++p) {
            const int tok = min((p * FS_WAVES + w) * TPP + tk, TOK - 1), t = t0 + tok;
            const bool valid = (p * FS_WAVES + w) * TPP + tk < TOK && t < samples;
            float v = -INFINITY;
            if (el < experts) {
                v = S::round(s_logit[tok][el]);
                if (logits_out && valid) S::store(logits_out, (int64_t)t * experts + el, v);
                if (logit_bias) v = S::round(v + lbias);
            }
            const float mxl = token_reduce(v, [](float a, float c) { return fmaxf(a, c); });
            float sc = el < experts ? expf(v - mxl) : 0.f;
            const float sum = token_reduce(sc, [](float a, float c) { return a + c; });
            const float inv = 1.0f / sum;
            if (el < experts) {
                sc = S::round(sc * inv);
                if (scores_out && valid) S::store(scores_out, (int64_t)t * experts + el, sc);
            } else {
                sc = -INFINITY;
            }
            if (l_aux) {
                float c = (valid && el < experts) ? sc : 0.f;
#pragma unroll
                for (int off = LPT; off < WAVE; off <<= 1) c += __shfl_xor(c, off, WAVE);
                if (tk == 0) s_me[p * FS_WAVES + w][el] = c;
            }
            // k-fold arg-max, the lower expert id wins among equal scores
            bool taken = false;
            float denom = 0.f, my_gate = 0.f;
            int my_idx = 0;
            for (int j = 0; j < k; ++j) {
                float bv = -INFINITY; int bi = 0x7fffffff;
                if (!taken && el < experts) { bv = sc; bi = el; }
                auto merge = [&](float ov, int oi) {
                    const bool better = oi != 0x7fffffff && (bi == 0x7fffffff || ov > bv || (ov == bv && oi < bi));
                    if (better) { bv = ov; bi = oi; }
                };
                merge(row_partner<1>(bv), row_partner<1>(bi));
                merge(row_partner<2>(bv), row_partner<2>(bi));
                merge(row_partner<4>(bv), row_partner<4>(bi));
                if constexpr (LPT >= 16) merge(row_partner<8>(bv), row_partner<8>(bi));
                if (bi == el) taken = true;
                denom = (j == 0) ? bv : S::round(denom + bv);
                if (el == 0 && valid) s_best[j][tok] = (uint8_t)bi;
                if (el == j) { my_gate = bv; my_idx = bi; }
            }
            if (valid && el < k) {
                const bool norm = k > 1 && normalize_gate;
                const float d = fmaxf(denom, eps);
                indices[(int64_t)el * stride + t] = my_idx;
                S::store(gates, (int64_t)el * stride + t, norm ? my_gate / d : my_gate);
            }
        }
    }
    lds_barrier();
    FS_STAMP(4);

    // ---- the group's ranks and histogram, one lane per token: wave j takes choice plane j and
    // publishes that plane's words itself, wave 4 the score sums
    if (w < 4) {
        const int j = w;
        const bool valid = lane < TOK && t0 + lane < samples;
        const int best = (valid && j < k) ? (int)s_best[j][lane % TOK] : -1;
        int rank = 0;
#pragma unroll
        for (int e = 0; e < CAP; ++e) {
            const uint64_t mk = __ballot(best == e);
            if (best == e) rank = __popcll(mk & lanes_below());
            if (lane == e) s_hist[j][e] = __popcll(mk);
        }
        if (lane < TOK) s_rank[j][lane] = rank;
        __builtin_amdgcn_wave_barrier();
        if (lane < CAP / 4) {
            const int32_t *h = &s_hist[j][4 * lane];
            const uint32_t payload = (uint32_t)h[0] | ((uint32_t)h[1] << 8) | ((uint32_t)h[2] << 16) | ((uint32_t)h[3] << 24);
            __hip_atomic_store(pub_hist + (size_t)grp * HW + j * (CAP / 4) + lane, ((unsigned long long)tag << 32) | payload,
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    } else if (w == 4 && l_aux && lane < CAP) {
        float v = 0.f;
        if (lane < experts) {
            v = s_me[0][lane];
#pragma unroll
            for (int i = 1; i < RPASSES * FS_WAVES; ++i) v += s_me[i][lane];
        }
        __hip_atomic_store(pub_me + (size_t)grp * CAP + lane, ((unsigned long long)tag << 32) | __float_as_uint(v),
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    FS_STAMP(5);

    FS_STAMP(6);

    // ---- every group's histogram must be in before any slot is final.  Thread (gi, q) reads word q
    // of the groups gi, gi + GPP, ...; a word counts once its tag is the call's.  The wait is bounded.
    constexpr int GPP = FS_THREADS / HW;                   // groups per pass
    constexpr int PASSES = (FS_MAX_GROUPS + GPP - 1) / GPP;
    const int q = tid % HW, gi = tid / HW;
    const bool active = 4 * q < k * CAP;                   // words of planes past top_k hold no counts
    unsigned long long word[PASSES];
#pragma unroll
    for (int p = 0; p < PASSES; ++p) word[p] = (unsigned long long)tag << 32;
    bool all = false;
    for (int spin = 0; spin <= spin_limit; ++spin) {
        bool ok = true;
        if (active) {
#pragma unroll
            for (int p = 0; p < PASSES; ++p) {
                if (p * GPP < groups) {
                    const int gg = min(gi + p * GPP, groups - 1);
                    word[p] = __hip_atomic_load(pub_hist + (size_t)gg * HW + q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
            }
#pragma unroll
            for (int p = 0; p < PASSES; ++p) ok = ok && (uint32_t)(word[p] >> 32) == tag;
        }
        const int slot = spin & 1;
        const int wave_bad = __ballot(!ok) != 0;             // (taken by all lanes: a ballot sees active lanes only)
        if (lane == 0) s_vote[slot][w] = wave_bad;
        lds_barrier();
        int bad = 0;
#pragma unroll
        for (int ww = 0; ww < FS_WAVES; ++ww) bad |= s_vote[slot][ww];
        all = bad == 0;
        if (all) break;
        __builtin_amdgcn_s_sleep(8);
    }
    FS_STAMP(7);
    if (!all) {
        // not every group showed up in time: none of this group's rows is written.  So that a partial
        // result cannot pass for a whole one, the group's tokens are marked dropped (location =
        // capacity) and the loss becomes NaN; the flag is what the caller goes by
        if (tid == 0 && gave_up) __hip_atomic_store(gave_up, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        for (int i = tid; i < k * TOK; i += FS_THREADS) {
            const int j = i / TOK, t = t0 + i % TOK;
            if (t < samples) locations[(int64_t)j * stride + t] = capacity;
        }
        if (tid == 0 && l_aux) *l_aux = __uint_as_float(0x7fc00000u);
        if (tid == 0 && grp == groups - 1) __hip_atomic_store(launches, launch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return;
    }

    // entries of the groups before this one, and of all groups, for every (plane, expert)
    {
        unsigned long long before = 0, full = 0;
#pragma unroll
        for (int p = 0; p < PASSES; ++p) {
            const int gg = gi + p * GPP;
            const unsigned long long sp = fs_spread((uint32_t)word[p]);
            if (gg < groups) full += sp;
            if (gg < grp) before += sp;
        }
        // lanes q, q + HW, ... of a wave hold the same word index
#pragma unroll
        for (int off = HW; off < WAVE; off <<= 1) {
            before += __shfl_xor(before, off, WAVE);
            full += __shfl_xor(full, off, WAVE);
        }
        if (lane < HW) { atomicAdd(&s_before64[q], before); atomicAdd(&s_full64[q], full); }
    }
    lds_barrier();
    if (tid < CAP) {
        int taken = 0;                                   // all first choices of an expert precede its second choices
        for (int j = 0; j < 4; ++j) {
            const int idx = j * CAP + tid;
            const int bef = (int)((s_before64[idx / 4] >> (16 * (idx % 4))) & 0xffffu);
            const int ful = (int)((s_full64[idx / 4] >> (16 * (idx % 4))) & 0xffffu);
            s_base[j][tid] = taken + bef;
            s_full[j][tid] = ful;
            taken += ful;
        }
        s_tot[tid] = taken;
    }
    lds_barrier();
    FS_STAMP(8);

    // one parked row -> its slots (the k choices of a token hold the same codes: the all-ones gate)
    auto flush_row = [&](int prow, int tok) {
        const int t = t0 + tok;
        if (t >= samples) return;
        int slot = -1;
        if (lane < k) {
            const int e = s_best[lane][tok];
            const int l = s_rank[lane][tok] + s_base[lane][e];
            locations[(int64_t)lane * stride + t] = l;
            if (l < capacity) slot = e * capacity + l;
        }
        if (__ballot(slot >= 0) == 0) return;
        uint4 v[G::RV];
        const uint4 *src = reinterpret_cast<const uint4 *>(park + prow * G::RS) + lane;
#pragma unroll
        for (int i = 0; i < G::RV; ++i) v[i] = G::piece(i, lane) ? src[i * WAVE] : make_uint4(0u, 0u, 0u, 0u);
        if (slot >= 0) { B16::store(bias_out, slot, s_mn[tok]); B16::store(scale_out, slot, s_sc[tok]); }
        for (int j = 0; j < k; ++j) {
            const int s = rl_i(slot, j);
            if (s < 0) continue;
            uint4 *dst = reinterpret_cast<uint4 *>(codes + (int64_t)s * G::M) + lane;
#pragma unroll
            for (int i = 0; i < G::RV; ++i) if (G::piece(i, lane)) stream_store(dst + i * WAVE, v[i]);
        }
    };

    // codes of the rounds that stayed in registers
    auto encode_kept = [&]() {
#pragma unroll
        for (int rr = 0; rr < REG_ROUNDS; ++rr) {
            uint4 (&raw)[NMMA] = ((LDS_ROUNDS + rr) & 1) ? buf1 : buf0;
            const RowEncoder<PLANMOE_BF16> enc(s_mn[16 * (LDS_ROUNDS + rr) + m], s_sc[16 * (LDS_ROUNDS + rr) + m]);
            auto body = [&](auto mode) {
#pragma unroll
                for (int i = 0; i < NMMA; ++i) {
                    uint32_t wd[2];
                    enc.template encode<decltype(mode)::value>(raw[i], wd);
                    kept[rr][i] = make_uint2(wd[0], wd[1]);
                }
            };
            if (__ballot(!enc.rq.fast) == 0) body(std::true_type{}); else body(std::false_type{});
        }
    };
    // empty slots: zero rows.  Which compute units get their rows out first differs by several
    // microseconds, mostly from one XCD to the next, so the list of empty slots is dealt out by
    // tickets, FS_ZERO_ROWS rows each, to whoever is done with its own rows: FS_SHARE consecutive
    // work-groups (one per XCD) share a counter and a stretch of the list.  A ticket is drawn before
    // the rows of the one before are written; the first wave of a group that finds the stretch
    // exhausted tells the others, who then need not ask.  (One counter for the whole grid does not
    // do: a few thousand additions to one address take longer than the stores.)
    // The pointer is passed through a vector register: with an address it can prove uniform the
    // compiler rewrites the addition into its own one-lane form, which waits for the answer on the spot.
    typedef __attribute__((address_space(1))) uint32_t global_u32;
    global_u32 *zero_tickets_v = (global_u32 *)zero_tickets;
    asm volatile("" : "+v"(zero_tickets_v));
    auto draw = [&]() {
        uint32_t got = 0;
        if (lane == 0) got = __hip_atomic_fetch_add(zero_tickets_v, (uint32_t)FS_ZERO_ROWS, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return got;
    };
    // the answer to a draw is looked at only after the stores that follow it have been issued
    auto drawn = [&](uint32_t got) {
        asm volatile("" : "+v"(got) : : "memory");
        return (uint32_t)__builtin_amdgcn_readfirstlane((int)got) - zero_base;
    };
    auto zero_fill = [&]() {
        // the empty slots of all experts as one list, expert after expert: lane e < CAP of every wave holds
        // where expert e's stretch of the list begins and the first empty slot of e (a prefix over the
        // lanes; worked out here, off the path from the slot bases to the first stores)
        const int z_used = lane < experts && lane < CAP ? min(s_tot[min(lane, CAP - 1)], capacity) : capacity;
        int z_upto = capacity - z_used;                          // empty slots of the experts up to this lane's
#pragma unroll
        for (int off = 1; off < CAP; off <<= 1) {
            const int below = __shfl_up(z_upto, off, WAVE);
            if (lane >= off) z_upto += below;
        }
        const int z_beg = z_upto - (capacity - z_used);
        auto zero_row = [&](uint32_t idx) {
            const int e = __popcll(__ballot(lane >= 1 && lane < CAP && (uint32_t)z_beg <= idx));
            const int slot = e * capacity + __builtin_amdgcn_readlane(z_used, e) + (int)(idx - (uint32_t)__builtin_amdgcn_readlane(z_beg, e));
            uint4 *dst = reinterpret_cast<uint4 *>(codes + (int64_t)slot * G::M) + lane;
#pragma unroll
            for (int i = 0; i < G::RV; ++i) if (G::piece(i, lane)) stream_store(dst + i * WAVE, make_uint4(0u, 0u, 0u, 0u));
            if (lane == 0) { B16::store(bias_out, slot, 0.f); B16::store(scale_out, slot, 0.f); }
        };
        const uint32_t total = (uint32_t)__builtin_amdgcn_readlane(z_upto, CAP - 1);
        const uint32_t shares = (uint32_t)(groups + FS_SHARE - 1) / FS_SHARE, per = (total + shares - 1) / shares;
        const uint32_t lo = (uint32_t)(grp / FS_SHARE) * per, hi = min(lo + per, total);
        if (lo >= hi) return;
        uint32_t cur = lo + drawn(draw());
        while (cur < hi) {
            const bool ask = __hip_atomic_load(&s_zdone, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) == 0;
            uint32_t ticket = 0;
            if (ask) ticket = draw();
#pragma unroll
            for (int r = 0; r < FS_ZERO_ROWS; ++r) zero_row(min(cur + r, hi - 1));      // past the end: the last row once more
            cur = ask ? lo + drawn(ticket) : hi;
            if (cur >= hi && lane == 0) __hip_atomic_store(&s_zdone, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
    };

    // The two waves that share a SIMD (w and w + 4) take their steps in opposite order: one codes
    // while the other is held up by its stores, so the arithmetic of phase 2 hides under the stores.
    if (w < FS_WAVES / 2) {
        encode_kept();
        for (int tok = w; tok < 16 * LDS_ROUNDS; tok += FS_WAVES) flush_row(tok, tok);
    } else {
        for (int tok = w; tok < 16 * LDS_ROUNDS; tok += FS_WAVES) flush_row(tok, tok);
        encode_kept();
    }
    FS_STAMP(9);

    // those codes pass through the same LDS rows
    lds_barrier();
#pragma unroll
    for (int rr = 0; rr < REG_ROUNDS; ++rr)
#pragma unroll
        for (int i = 0; i < NMMA; ++i) *reinterpret_cast<uint2 *>(my_park + rr * 16 * G::RS + 32 * i) = kept[rr][i];
    lds_barrier();
    FS_STAMP(10);
    for (int i = w; i < 16 * REG_ROUNDS; i += FS_WAVES) flush_row(i, 16 * LDS_ROUNDS + i);
    FS_STAMP(11);
    zero_fill();
    FS_STAMP(12);

    // the last group closes the launch (every group has read the counter by now: all of them have
    // published) and finishes the GShard loss and the per-plane expert counts
    if (grp == groups - 1 && tid == 0) __hip_atomic_store(launches, launch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (grp == groups - 1 && (l_aux || counts_out)) {
        if (counts_out && tid < k * experts) counts_out[tid] = s_full[tid / experts][tid % experts];
        if (l_aux) {
            // score sums of all groups, added in a fixed order: thread (gi, e) over its groups, then
            // the partial sums one after the other
            constexpr int MG = FS_THREADS / CAP, MP = (FS_MAX_GROUPS + MG - 1) / MG;
            const int e = tid % CAP, mgi = tid / CAP;
            float acc = 0.f;
            bool in = false;
            for (int spin = 0; spin <= spin_limit && !in; ++spin) {
                unsigned long long mw[MP];
#pragma unroll
                for (int p = 0; p < MP; ++p)
                    mw[p] = __hip_atomic_load(pub_me + (size_t)min(mgi + p * MG, groups - 1) * CAP + e, __ATOMIC_RELAXED,
                                              __HIP_MEMORY_SCOPE_AGENT);
                in = true;
                acc = 0.f;
#pragma unroll
                for (int p = 0; p < MP; ++p) {
                    in = in && (uint32_t)(mw[p] >> 32) == tag;
                    if (mgi + p * MG < groups) acc += __uint_as_float((uint32_t)mw[p]);
                }
            }
            s_mepart[mgi][e] = in ? acc : __uint_as_float(0x7fc00000u);      // a sum that never came in shows as NaN
            lds_barrier();
            if (tid == 0) {
                float a = 0.f;
                for (int ee = 0; ee < experts; ++ee) {
                    float me = 0.f;
                    for (int i = 0; i < MG; ++i) me += s_mepart[i][ee];
                    a += me * ((float)s_full[0][ee] * ((float)experts / (float)samples));
                }
                // (a group that gave up has made the loss NaN: it stays NaN)
                const bool whole = !gave_up || __hip_atomic_load(gave_up, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0;
                *l_aux = whole ? a / (float)samples : __uint_as_float(0x7fc00000u);
            }
        }
    }
}

} // namespace pm
