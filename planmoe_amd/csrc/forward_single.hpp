// The forward chain in ONE launch that reads x once (bf16, up to 16 experts, top_k <= 4).
//
// A work-group of 8 waves owns 16 * ROUNDS consecutive tokens and there is one work-group per
// compute unit, all resident together.  Phase 1 streams the tokens in rounds of 16 (one MFMA
// M-tile): gate GEMM split-K over the 8 waves, row min / max on the way, softmax / top-k of the
// round.  A row can be quantised as soon as its own min / max are known, so the rows of the first
// rounds are turned into codes at once and parked in LDS; the last two rounds simply stay in the
// registers they were loaded into.  Then the group's expert histogram is published and the
// work-group waits until every group has done so (the slot of a second choice needs the number of
// first choices of the whole batch).  Phase 2 adds up the histogram columns it needs, once per
// work-group, and writes every parked row to its slots straight from LDS in full 4 KB rows, the
// register rounds being quantised (while the first stores drain) and passed through the same LDS
// rows; empty slots are zero-filled by all work-groups together.
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

// waits for LDS traffic only: loads and stores to global memory that are in flight stay in flight
// across the barrier (__syncthreads would drain them)
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// per-group tickets and the status word live behind the tables of the two-launch chain
struct FsSync {
    unsigned long long *flags;      // [groups]: the ticket of the call whose histogram row is complete
    uint32_t *status;               // [0]: ticket (low word) of a call that gave up waiting
};
__host__ __device__ inline FsSync fs_sync(const FwdWs &w, int samples)
{
    FsSync s;
    uintptr_t p = (uintptr_t)(w.row_max + samples);
    p = (p + 15) & ~(uintptr_t)15;
    s.status = (uint32_t *)p;
    s.flags = (unsigned long long *)(p + 16);
    return s;
}

template <int NMMA> struct FsGeom {
    static constexpr int M = 256 * NMMA;          // model_dim: every wave owns M / 8 elements of a row
    static constexpr int NV = M / 8;              // 16-byte vectors per row
    static constexpr int RS = M + 16;             // bytes per parked code row in LDS: lanes of different
                                                  // rows fall into different banks
    static constexpr int RV = M / 16 / WAVE;      // 16-byte pieces of a code row per lane
};

template <int SDT, int CAP, int NMMA, int ROUNDS>
__global__ __launch_bounds__(FS_THREADS) void forward_single_kernel(
    const uint4 *__restrict__ x, const uint4 *__restrict__ wg, const float *__restrict__ logit_bias,
    int samples, int experts, int k, int normalize_gate, int capacity,
    int32_t *__restrict__ indices, int32_t *__restrict__ locations, void *__restrict__ gates, int64_t stride,
    void *__restrict__ logits_out, void *__restrict__ scores_out, float *__restrict__ l_aux,
    int32_t *__restrict__ counts_out, uint8_t *__restrict__ codes, void *__restrict__ bias_out,
    void *__restrict__ scale_out, void *__restrict__ workspace, unsigned long long ticket, int spin_limit,
    int32_t *__restrict__ gave_up)
{
    using S = Elem<SDT>;
    using B16 = Elem<PLANMOE_BF16>;
    using G = FsGeom<NMMA>;
    static_assert(CAP == 8 || CAP == 16, "experts per token tile");
    static_assert(ROUNDS >= 1 && ROUNDS <= 4, "one lane per token in the ranking step");
    static_assert(NMMA % 4 == 0 && G::RV >= 1, "rows are dealt out in 16-byte pieces");
    constexpr int TOK = 16 * ROUNDS;
    constexpr int REG_ROUNDS = ROUNDS < 2 ? ROUNDS : 2;    // the last rounds stay raw in registers
    constexpr int LDS_ROUNDS = ROUNDS - REG_ROUNDS;        // the first rounds are parked as codes
    constexpr int PARK_ROUNDS = LDS_ROUNDS > REG_ROUNDS ? LDS_ROUNDS : REG_ROUNDS;
    __shared__ __align__(16) uint8_t park[PARK_ROUNDS * 16 * G::RS];
    __shared__ float part[2][FS_WAVES][16][CAP + 1];
    __shared__ int32_t pstat[2][FS_WAVES][16][3];
    __shared__ uint8_t s_best[4][TOK];
    __shared__ int32_t s_rank[4][TOK];
    __shared__ float s_mn[TOK], s_sc[TOK];
    __shared__ float s_me[ROUNDS][CAP];
    __shared__ int32_t s_hist[CAP];
    __shared__ int32_t s_part[4][CAP], s_full[4][CAP];     // histogram columns: groups before this one / all
    __shared__ int32_t s_base[4][CAP], s_tot[CAP];
    __shared__ float s_loss[CAP];
    __shared__ int s_fail;

    const int tid = threadIdx.x, w = tid >> 6, lane = lane_id(), m = lane & 15, g = lane >> 4;
    const int groups = gridDim.x, grp = blockIdx.x, t0 = grp * TOK;
    const FwdWs ws = fwd_ws(workspace, groups, k, experts, samples);
    const FsSync sync = fs_sync(ws, samples);
    const float eps = SDT == PLANMOE_F32 ? 1.1920928955078125e-07f : SDT == PLANMOE_BF16 ? 0.0078125f : 0.0009765625f;

    // lane (m, g) of wave w holds, of row m of a round, the vectors  w * 4 NMMA + 4 i + g
    const int v0 = w * (4 * NMMA) + g;
    const uint4 *bp = wg + (int64_t)min(m, experts - 1) * G::NV + v0;
    auto load_x = [&](uint4 (&a)[NMMA], int r) {
        const uint4 *p = x + (int64_t)min(t0 + 16 * r + m, samples - 1) * G::NV + v0;
#pragma unroll
        for (int i = 0; i < NMMA; ++i) a[i] = p[4 * i];
    };
    // codes of this lane's share of row `row` of the parking area
    auto encode_to_park = [&](const uint4 (&a)[NMMA], int row, float mn, float scale) {
        const RowEncoder<PLANMOE_BF16> enc(mn, scale);
        uint8_t *dst = park + row * G::RS + v0 * 8;
        auto body = [&](auto mode) {
#pragma unroll
            for (int i = 0; i < NMMA; ++i) {
                uint32_t wd[2];
                enc.template encode<decltype(mode)::value>(a[i], wd);
                *reinterpret_cast<uint2 *>(dst + 32 * i) = make_uint2(wd[0], wd[1]);
            }
        };
        // the mode is a property of the row, i.e. of the lane here: one branch for the wave
        if (__ballot(!enc.rq.fast) == 0) body(std::true_type{}); else body(std::false_type{});
    };

    uint4 buf0[NMMA], buf1[NMMA];
    float keep_mn[2] = {0.f, 0.f}, keep_sc[2] = {0.f, 0.f};       // row min / scale of the rows left in buf0 / buf1

    // ---- one round: GEMM + row statistics of 16 tokens, their routing, codes of the early rounds
    auto round = [&](auto rc, uint4 (&cur)[NMMA], uint4 (&nxt)[NMMA]) {
        constexpr int r = decltype(rc)::value;
        constexpr int par = r & 1;
        // gate weights of this wave's K range first, then the next round's rows: the MFMAs below
        // wait for the weights only, the rows stay in flight behind them
        uint4 b[NMMA];
#pragma unroll
        for (int i = 0; i < NMMA; ++i) b[i] = bp[4 * i];
        if constexpr (r + 1 < ROUNDS) load_x(nxt, r + 1);
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
        lds_barrier();

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

        // routing of the round's 16 tokens by one wave: CAP lanes share a token, lane el holds expert el
        if (w == (r + 1) % FS_WAVES) {
            constexpr int LPT = CAP, TPP = WAVE / LPT;
            const int el = lane % LPT, tk = lane / LPT;
            auto token_reduce = [&](auto v, auto op) { return row_allreduce<LPT>(v, op); };
            float me_acc = 0.f;
#pragma unroll
            for (int p = 0; p < 16 / TPP; ++p) {
                const int tok16 = p * TPP + tk, tok = 16 * r + tok16, t = t0 + tok;
                const bool valid = t < samples;
                float v = -INFINITY;
                if (el < experts) {
                    v = part[par][0][tok16][el];
#pragma unroll
                    for (int ww = 1; ww < FS_WAVES; ++ww) v += part[par][ww][tok16][el];
                    v = S::round(v);
                    if (logits_out && valid) S::store(logits_out, (int64_t)t * experts + el, v);
                    if (logit_bias) v = S::round(v + logit_bias[el]);
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
                    me_acc += c;
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
                    if (el == 0) s_best[j][tok] = (uint8_t)bi;
                    if (el == j) { my_gate = bv; my_idx = bi; }
                }
                if (valid && el < k) {
                    const bool norm = k > 1 && normalize_gate;
                    const float d = fmaxf(denom, eps);
                    indices[(int64_t)el * stride + t] = my_idx;
                    S::store(gates, (int64_t)el * stride + t, norm ? my_gate / d : my_gate);
                }
            }
            if (l_aux && tk == 0 && el < experts) s_me[r][el] = me_acc;
        }

        if constexpr (r < LDS_ROUNDS) {
            encode_to_park(cur, r * 16 + m, mn, scale);
        } else {
            keep_mn[par] = mn; keep_sc[par] = scale;
        }
    };

    FS_STAMP(0);
    load_x(buf0, 0);
    round(std::integral_constant<int, 0>{}, buf0, buf1);
    FS_STAMP(1);
    if constexpr (ROUNDS > 1) round(std::integral_constant<int, 1>{}, buf1, buf0);
    FS_STAMP(2);
    if constexpr (ROUNDS > 2) round(std::integral_constant<int, 2>{}, buf0, buf1);
    FS_STAMP(3);
    if constexpr (ROUNDS > 3) round(std::integral_constant<int, 3>{}, buf1, buf0);
    lds_barrier();
    FS_STAMP(4);

    // ---- the group's ranks and histogram (wave 0, one lane per token), then its ticket
    if (w == 0) {
        const bool valid = lane < TOK && t0 + lane < samples;
        for (int j = 0; j < k; ++j) {
            const int best = valid ? (int)s_best[j][lane % TOK] : -1;
            int rank = 0;
#pragma unroll
            for (int e = 0; e < CAP; ++e) {
                const uint64_t mk = __ballot(best == e);
                if (best == e) rank = __popcll(mk & lanes_below());
                if (lane == e) s_hist[e] = __popcll(mk);
            }
            if (lane < TOK) s_rank[j][lane] = rank;
            __builtin_amdgcn_wave_barrier();
            if (lane < experts) {
                int32_t *col = ws.hist_t + ((int64_t)j * experts + lane) * ws.gstride;
                col[grp] = s_hist[lane];
                if (grp == groups - 1)
                    for (int p = groups; p < ws.gstride; ++p) col[p] = 0;
            }
            __builtin_amdgcn_wave_barrier();
        }
        if (l_aux && lane < experts) {
            float v = s_me[0][lane];
#pragma unroll
            for (int r = 1; r < ROUNDS; ++r) v += s_me[r][lane];
            ws.me_t[(int64_t)lane * ws.gstride + grp] = v;
            if (grp == groups - 1)
                for (int p = groups; p < ws.gstride; ++p) ws.me_t[(int64_t)lane * ws.gstride + p] = 0.f;
        }
        __threadfence();
        FS_STAMP(5);
        if (lane == 0) __hip_atomic_store(sync.flags + grp, ticket, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);

        // every group's ticket must be in before any slot is final; the wait is bounded
        bool all = false;
        for (int spin = 0; spin <= spin_limit; ++spin) {
            bool ok = true;
            for (int i = lane; i < groups; i += WAVE)
                ok = ok && __hip_atomic_load(sync.flags + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == ticket;
            all = __ballot(!ok) == 0;
            if (all) break;
            __builtin_amdgcn_s_sleep(4);
        }
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        if (lane == 0) s_fail = all ? 0 : 1;
    }
    lds_barrier();
    FS_STAMP(6);
    if (s_fail) {
        // not every group showed up in time: none of this group's rows is written
        if (tid == 0) {
            __hip_atomic_store(sync.status, (uint32_t)ticket, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (gave_up) __hip_atomic_store(gave_up, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        return;
    }

    // ---- phase 2.  Histogram columns: entries of the groups before this one, and of all groups
    for (int item = w; item < k * experts; item += FS_WAVES) {
        const int32_t *col = ws.hist_t + (int64_t)item * ws.gstride;
        int before = 0, full = 0;
        for (int i = lane * 4; i < groups; i += 4 * WAVE) {
            const int4 v = *reinterpret_cast<const int4 *>(col + i);
            const int vv[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                if (i + c < groups) full += vv[c];
                if (i + c < grp) before += vv[c];
            }
        }
        before = wave_allreduce(before, [](int a, int c) { return a + c; });
        full = wave_allreduce(full, [](int a, int c) { return a + c; });
        if (lane == 0) { s_part[item / experts][item % experts] = before; s_full[item / experts][item % experts] = full; }
    }
    lds_barrier();
    if (tid < experts) {
        int taken = 0;                                   // all first choices of an expert precede its second choices
        for (int j = 0; j < k; ++j) { s_base[j][tid] = taken + s_part[j][tid]; taken += s_full[j][tid]; }
        s_tot[tid] = taken;
    }
    lds_barrier();

    FS_STAMP(7);
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
        for (int q = 0; q < G::RV; ++q) v[q] = src[q * WAVE];
        if (slot >= 0) { B16::store(bias_out, slot, s_mn[tok]); B16::store(scale_out, slot, s_sc[tok]); }
        for (int j = 0; j < k; ++j) {
            const int s = rl_i(slot, j);
            if (s < 0) continue;
            uint4 *dst = reinterpret_cast<uint4 *>(codes + (int64_t)s * G::M) + lane;
#pragma unroll
            for (int q = 0; q < G::RV; ++q) stream_store(dst + q * WAVE, v[q]);
        }
    };

    for (int tok = w; tok < 16 * LDS_ROUNDS; tok += FS_WAVES) flush_row(tok, tok);
    FS_STAMP(8);

    // empty slots: zero rows, dealt out over all waves of the grid
    {
        const int slots = experts * capacity, nwaves = groups * FS_WAVES;
        for (int s = grp * FS_WAVES + w; s < slots; s += nwaves) {
            const int e = s / capacity;
            if (s - e * capacity < s_tot[e]) continue;
            uint4 *dst = reinterpret_cast<uint4 *>(codes + (int64_t)s * G::M) + lane;
#pragma unroll
            for (int q = 0; q < G::RV; ++q) stream_store(dst + q * WAVE, make_uint4(0u, 0u, 0u, 0u));
            if (lane == 0) { B16::store(bias_out, s, 0.f); B16::store(scale_out, s, 0.f); }
        }
    }

    // the rounds that stayed in registers: quantised now, through the same LDS rows
    FS_STAMP(9);
    lds_barrier();
    FS_STAMP(10);
    if constexpr (REG_ROUNDS == 2) {
        constexpr int ra = ROUNDS - 2, rb = ROUNDS - 1;
        if constexpr ((ra & 1) == 0) {
            encode_to_park(buf0, m, keep_mn[0], keep_sc[0]);
            encode_to_park(buf1, 16 + m, keep_mn[1], keep_sc[1]);
        } else {
            encode_to_park(buf1, m, keep_mn[1], keep_sc[1]);
            encode_to_park(buf0, 16 + m, keep_mn[0], keep_sc[0]);
        }
        (void)rb;
    } else {
        encode_to_park(buf0, m, keep_mn[0], keep_sc[0]);
    }
    lds_barrier();
    FS_STAMP(11);
    for (int i = w; i < 16 * REG_ROUNDS; i += FS_WAVES) flush_row(i, 16 * LDS_ROUNDS + i);
    FS_STAMP(12);

    // the last group also finishes the GShard loss and the per-plane expert counts
    if (grp == groups - 1 && (l_aux || counts_out)) {
        if (counts_out && tid < k * experts) counts_out[tid] = s_full[tid / experts][tid % experts];
        if (l_aux) {
            for (int e = w; e < experts; e += FS_WAVES) {
                float me = column_partial(ws.me_t + (int64_t)e * ws.gstride, groups);
                me = wave_allreduce(me, [](float a, float c) { return a + c; });
                if (lane == 0) s_loss[e] = me * ((float)s_full[0][e] * ((float)experts / (float)samples));
            }
            lds_barrier();
            if (tid == 0) {
                float a = 0.f;
                for (int e = 0; e < experts; ++e) a += s_loss[e];
                *l_aux = a / (float)samples;
            }
        }
    }
}

} // namespace pm
