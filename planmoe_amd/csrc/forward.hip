// The forward chain in two launches (three when top_k > 4):
//
//   gate_route_kernel     x is read once: gate-logits GEMM on the matrix cores, then, for the
//                         work-group's 64 (or 32) tokens = one routing group, softmax, k-fold
//                         arg-max, gates, the rank of every token among the group's tokens with
//                         the same choice, and the group's expert histogram.
//   dispatch_int8_routed  slot = rank in group + entries of earlier groups and planes (all first
//                         choices of an expert precede its second choices), summed by every wave
//                         from the transposed histograms; token rows go to uint8 codes in their
//                         slots (x is read a second time), slots past an expert's fill are zero
//                         rows; one block finishes the GShard loss and the expert counts.
//   group_offsets_kernel  only for top_k > 4 and for planmoe_gate_route (routing without
//                         dispatch, finished by route_offsets_kernel): the prefix over groups as
//                         a launch of its own.
//
// This replaces gates/top.py:20-26 + moe_layer.py:230-256 + fast_dispatch.py:140-195 +
// fast_encode (fast_dispatch.py:197-201) + Int8Compressor::compress (int8.cpp:7-44).
//
// Workspace (32-bit words): hist_t[k][E][groups up to a multiple of 4], me_t[E][same] (fp32),
// totals[E], loss_part[64], hist[groups][k][E], offs[groups][k][E], me[groups][E] (fp32),
// rank[k][samples] (rank of a token inside its group), row_min[samples], row_max[samples]
// (fp32; bf16 inputs only: the gate kernel scans the rows it streams anyway).
#include "forward_shared.hpp"
#include <mutex>
#include <atomic>
#include <random>

namespace pm {

// tokens per work-group of the gate kernel = tokens per routing group (one lane each in the
// routing epilogue): 64, or 32 on the split-K path (up to 16 experts) when 64 would leave
// compute units without a work-group
inline int fwd_group_tokens(int experts, int samples)
{
    // measured at 8 experts: 16384 tokens (256 groups of 64) 39 us with 64, 44 us with 32;
    // 8192 tokens 32 us with 64, 28 us with 32
    return (experts <= 16 && samples < 64 * 256) ? 32 : 64;
}
constexpr int FWD_LOSS_PARTS = 64;
inline void *fwd_tables(void *workspace) { return (char *)workspace + FWD_TABLES_OFFSET; }

// hist_t / me_t are the transposes of hist / me with the group index running fastest (rows of
// gstride = groups rounded up to 4 entries, the padding zero): a column of the histogram, which
// is what a prefix over groups reads, is contiguous there.
struct FwdWs {
    int32_t *totals, *hist, *offs, *rank, *hist_t;
    float *loss_part, *me, *row_min, *row_max, *me_t;
    int gstride;
};
__host__ __device__ inline size_t fwd_pad4(size_t words) { return (words + 3) & ~(size_t)3; }
__host__ __device__ inline FwdWs fwd_ws(void *ws, int groups, int k, int experts, int samples)
{
    FwdWs w;
    w.gstride = (int)fwd_pad4((size_t)groups);
    w.hist_t = (int32_t *)ws;                                   // 16-byte aligned rows
    w.me_t = (float *)(w.hist_t + (size_t)k * experts * w.gstride);
    w.totals = (int32_t *)(w.me_t + (size_t)experts * w.gstride);
    w.loss_part = (float *)(w.totals + experts);
    w.hist = (int32_t *)(w.loss_part + FWD_LOSS_PARTS);
    w.offs = w.hist + (size_t)groups * k * experts;
    w.me = (float *)(w.offs + (size_t)groups * k * experts);
    w.rank = (int32_t *)(w.me + (size_t)groups * experts);
    w.row_min = (float *)(w.rank + (size_t)k * samples);
    w.row_max = w.row_min + samples;
    return w;
}

// This lane's share of the sum of col[0 .. limit): col is 16-byte aligned and readable up to the
// next multiple of 4 entries, limit is the same in every lane.  The wave reduction is left to the
// caller so that several columns can be loaded back to back and reduced together (one memory
// round trip and interleaved shuffle chains instead of one after the other).
__device__ __forceinline__ int column_partial(const int32_t *__restrict__ col, int limit)
{
    int s = 0;
    for (int i = lane_id() * 4; i < limit; i += 4 * WAVE) {
        const int4 v = *reinterpret_cast<const int4 *>(col + i);
        s += v.x + (i + 1 < limit ? v.y : 0) + (i + 2 < limit ? v.z : 0) + (i + 3 < limit ? v.w : 0);
    }
    return s;
}
__device__ __forceinline__ float column_partial(const float *__restrict__ col, int limit)
{
    float s = 0.f;
    for (int i = lane_id() * 4; i < limit; i += 4 * WAVE) {
        const float4 v = *reinterpret_cast<const float4 *>(col + i);
        s += (v.x + (i + 1 < limit ? v.y : 0.f)) + ((i + 2 < limit ? v.z : 0.f) + (i + 3 < limit ? v.w : 0.f));
    }
    return s;
}
// wave sums of N values at once
template <typename T, int N>
__device__ __forceinline__ void wave_sum_n(T (&v)[N])
{
#pragma unroll
    for (int i = 0; i < N; ++i) v[i] = wave_allreduce(v[i], [](T a, T b) { return a + b; });
}

// SDT: dtype of logits / scores / gates (F32 when fp32_gate, else the input dtype)
// CAP: compile-time bound of the expert count held in registers by the routing epilogue
// NT == 1: split-K over the 4 waves, weights straight from L2 (up to 16 experts);
// NT > 1: weights shared through LDS, a wave per 16 tokens.
// MODE 0: logits = x . wg^T computed here.  MODE 1 / 2: no GEMM; x holds the [samples, experts]
// logits / scores in the routing dtype (the stand-alone routing entry point) and only the
// epilogue runs, on 64-token groups.
template <int DT, int SDT, int NT, int CAP, bool SPLITK, int GROUP, int MODE = 0>
__global__ __launch_bounds__(256) void gate_route_kernel(
    const void *__restrict__ x, const void *__restrict__ wg, const float *__restrict__ logit_bias,
    int samples, int model_dim, int experts, int k, int normalize_gate,
    int32_t *__restrict__ indices, int32_t *__restrict__ locations, void *__restrict__ gates,
    int64_t stride, void *__restrict__ logits_out, void *__restrict__ scores_out,
    float *__restrict__ l_aux, int32_t *__restrict__ counts_out, void *__restrict__ workspace)
{
    using S = Elem<SDT>;
    static_assert(GROUP == 64 || (SPLITK && GROUP == 32), "the LDS-shared variant is built for 64 tokens");
    constexpr int COLS = 16 * NT + 1;
    // split-K: part[4][GROUP][COLS] floats; else the weight buffers / logits[GROUP][COLS]
    __shared__ uint4 smem[SPLITK ? (4 * GROUP * COLS + 3) / 4 : gate_lds_vectors<NT>()];
    __shared__ int32_t s_hist[CAP];
    float (*part)[GROUP][COLS] = reinterpret_cast<float (*)[GROUP][COLS]>(smem);

    const int tid = threadIdx.x, lane = lane_id();
    const int groups = gridDim.x;
    const FwdWs ws = fwd_ws(workspace, groups, k, experts, samples);
    const int t0 = blockIdx.x * GROUP;
    // the additive logit biases of this lane's experts, asked for before the GEMM: read where they are
    // used, their latency would stand in every pass of the epilogue (6.5 -> 2 us per group at 64 experts)
    constexpr int LPT_ = CAP < 16 ? CAP : 16, EPL_ = CAP / LPT_;
    float lbias[EPL_];
#pragma unroll
    for (int q = 0; q < EPL_; ++q) {
        const int e = q * LPT_ + lane % LPT_;
        lbias[q] = (MODE != 2 && logit_bias && e < experts) ? logit_bias[e] : 0.f;
    }
    constexpr bool STATS = DT == PLANMOE_BF16 && MODE == 0;
    static_assert(MODE == 0 || (!SPLITK && GROUP == 64), "routing from memory runs on 64-token groups");
    __shared__ int32_t pstat[SPLITK ? 4 : 1][GROUP][3];
    if constexpr (MODE != 0) {
        // the group's rows land where the GEMM would have left its logits: 8 loads in flight per
        // thread, at clamped indices so that they are straight-line loads
        const int n = min(GROUP, samples - t0) * experts;
        const int64_t base = (int64_t)t0 * experts;
        for (int i0 = tid; i0 < n; i0 += 8 * 256) {
            float v[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) v[q] = S::load(x, base + min(i0 + q * 256, n - 1));
#pragma unroll
            for (int q = 0; q < 8; ++q) {
                const int i = i0 + q * 256;
                if (i < n) {
                    const int tok = i / experts;
                    part[0][tok][i - tok * experts] = v[q];
                }
            }
        }
    } else if constexpr (SPLITK) {
        gate_tile_partials<DT, NT, GROUP / 16, 4, STATS>(x, wg, t0, samples, model_dim, experts, part, pstat);
    } else {
        gate_tile_lds<DT, NT, STATS>(x, wg, t0, samples, model_dim, experts, smem, pstat[0]);
    }
    __syncthreads();

    // ---- routing epilogue, part 1: all four waves, wave w owns GROUP / 4 consecutive tokens.
    // LPT lanes share a token, lane el holding the experts el, el + LPT, ...: softmax and the
    // k-fold arg-max are butterflies over those lanes instead of loops over the experts.
    constexpr int LPT = CAP < 16 ? CAP : 16;           // lanes per token
    constexpr int EPL = CAP / LPT;                     // experts per lane
    constexpr int TPW4 = GROUP / 4;                    // tokens per wave
    constexpr int TPP = WAVE / LPT < TPW4 ? WAVE / LPT : TPW4;   // tokens per pass of a wave
    __shared__ uint8_t s_best[64][GROUP];              // [plane][token] chosen expert
    __shared__ float s_me[4][CAP];
    const int wave = tid >> 6, el = lane % LPT, tk = lane / LPT;
    auto token_reduce = [&](auto v, auto op) { return row_allreduce<LPT>(v, op); };   // over the lanes of a token
    float me_acc[EPL];
#pragma unroll
    for (int q = 0; q < EPL; ++q) me_acc[q] = 0.f;
    const float eps = SDT == PLANMOE_F32 ? 1.1920928955078125e-07f
                    : SDT == PLANMOE_BF16 ? 0.0078125f : 0.0009765625f;

    for (int p = 0; p < TPW4 / TPP; ++p) {
        const int tok = wave * TPW4 + p * TPP + min(tk, TPP - 1);   // lanes past the pass repeat a token
        const int t = t0 + tok;
        const bool valid = t < samples && tk < TPP;
        float sc[EPL];
        float mx = -INFINITY;
#pragma unroll
        for (int q = 0; q < EPL; ++q) {
            const int e = q * LPT + el;
            float v = -INFINITY;
            if (e < experts) {
                if constexpr (SPLITK) v = ((part[0][tok][e] + part[1][tok][e]) + part[2][tok][e]) + part[3][tok][e];
                else v = part[0][tok][e];
                v = S::round(v);
                if constexpr (MODE != 2) {
                    if (logits_out && valid) S::store(logits_out, (int64_t)t * experts + e, v);
                    if (logit_bias) v = S::round(v + lbias[q]);
                }
            }
            sc[q] = v;                                    // MODE 2: the score itself (-inf past the experts)
            mx = fmaxf(mx, v);
        }
        if constexpr (MODE != 2) {
            mx = token_reduce(mx, [](float a, float b) { return fmaxf(a, b); });
            float sum = 0.f;
#pragma unroll
            for (int q = 0; q < EPL; ++q) {
                sc[q] = (q * LPT + el < experts) ? expf(sc[q] - mx) : 0.f;
                sum += sc[q];
            }
            sum = token_reduce(sum, [](float a, float b) { return a + b; });
            const float inv = 1.0f / sum;                 // scores are tolerance-level quantities
#pragma unroll
            for (int q = 0; q < EPL; ++q) {
                const int e = q * LPT + el;
                if (e < experts) {
                    sc[q] = S::round(sc[q] * inv);
                    if (scores_out && valid) S::store(scores_out, (int64_t)t * experts + e, sc[q]);
                } else {
                    sc[q] = -INFINITY;
                }
            }
        }
        // column sums of the wave's scores (GShard loss): over the tokens of the pass, then passes
        if (l_aux) {
#pragma unroll
            for (int q = 0; q < EPL; ++q) {
                float c = (valid && q * LPT + el < experts) ? sc[q] : 0.f;
#pragma unroll
                for (int off = LPT; off < WAVE; off <<= 1) c += __shfl_xor(c, off, WAVE);   // lanes past the pass hold 0
                me_acc[q] += c;
            }
        }
        // k-fold arg-max, the lower expert id wins among equal scores
        uint32_t taken = 0;
        float denom = 0.f, my_gate = 0.f;
        int my_idx = 0;
        for (int j = 0; j < k; ++j) {
            float bv = -INFINITY; int bi = 0x7fffffff;
#pragma unroll
            for (int q = 0; q < EPL; ++q) {
                const bool free_ = !((taken >> q) & 1u) && q * LPT + el < experts;
                if (free_ && (bi == 0x7fffffff || sc[q] > bv)) { bv = sc[q]; bi = q * LPT + el; }
            }
            auto merge = [&](float ov, int oi) {
                const bool better = oi != 0x7fffffff && (bi == 0x7fffffff || ov > bv || (ov == bv && oi < bi));
                if (better) { bv = ov; bi = oi; }
            };
            if constexpr (LPT >= 2) merge(row_partner<1>(bv), row_partner<1>(bi));
            if constexpr (LPT >= 4) merge(row_partner<2>(bv), row_partner<2>(bi));
            if constexpr (LPT >= 8) merge(row_partner<4>(bv), row_partner<4>(bi));
            if constexpr (LPT >= 16) merge(row_partner<8>(bv), row_partner<8>(bi));
#pragma unroll
            for (int q = 0; q < EPL; ++q) if (bi == q * LPT + el) taken |= 1u << q;
            denom = (j == 0) ? bv : S::round(denom + bv);
            if (el == 0 && tk < TPP) s_best[j][tok] = (uint8_t)bi;
            if (j < LPT) {
                if (el == j) { my_gate = bv; my_idx = bi; }
            } else if (valid && el == j % LPT) {
                // more planes than lanes per token: index and raw gate go out now, the gate is
                // normalised below
                indices[(int64_t)j * stride + t] = bi;
                S::store(gates, (int64_t)j * stride + t, bv);
            }
        }
        if (valid) {
            const bool norm = k > 1 && normalize_gate;
            const float d = fmaxf(denom, eps);
            if (el < k) {
                indices[(int64_t)el * stride + t] = my_idx;
                S::store(gates, (int64_t)el * stride + t, norm ? my_gate / d : my_gate);
            }
            if (norm) {
                for (int j = LPT + el; j < k; j += LPT) {
                    const float g = S::load(gates, (int64_t)j * stride + t);
                    S::store(gates, (int64_t)j * stride + t, g / d);
                }
            }
        }
    }
    if (l_aux && tk == 0) {
#pragma unroll
        for (int q = 0; q < EPL; ++q) if (q * LPT + el < experts) s_me[wave][q * LPT + el] = me_acc[q];
    }
    __syncthreads();

    // ---- part 2: wave 0, one lane per token: rank of every token among the group's tokens with
    // the same choice (wave ballots), the group's histograms, row min / max, score column sums
    if (tid < WAVE) {
        const int t = t0 + tid;
        const bool valid = tid < GROUP && t < samples;
        if constexpr (STATS) {
            if (valid) {
                // row min / max for the int8 codec of the dispatch launch
                int a = pstat[0][tid][0], b = pstat[0][tid][1], n = pstat[0][tid][2];
                if constexpr (SPLITK) {
#pragma unroll
                    for (int w = 1; w < 4; ++w) {
                        a = min(a, pstat[w][tid][0]); b = max(b, pstat[w][tid][1]); n = max(n, pstat[w][tid][2]);
                    }
                }
                float lo, hi;
                RowStats<PLANMOE_BF16, true>::decode(a, b, n, lo, hi);
                ws.row_min[t] = lo; ws.row_max[t] = hi;
            }
        }
        if (l_aux && lane < experts) {
            const float v = ((s_me[0][lane] + s_me[1][lane]) + s_me[2][lane]) + s_me[3][lane];
            ws.me[(int64_t)blockIdx.x * experts + lane] = v;
            ws.me_t[(int64_t)lane * ws.gstride + blockIdx.x] = v;
        }
        for (int j = 0; j < k; ++j) {
            const int best = valid ? (int)s_best[j][tid % GROUP] : -1;
            if (lane < CAP) s_hist[lane] = 0;
            __builtin_amdgcn_wave_barrier();
            int rank = 0;
            if constexpr (CAP <= 16) {
                // few experts: one ballot per expert, no serial dependence between them
#pragma unroll
                for (int e = 0; e < CAP; ++e) {
                    const uint64_t m = __ballot(best == e);
                    if (best == e) rank = __popcll(m & lanes_below());
                    if (lane == e) s_hist[e] = __popcll(m);
                }
            } else {
                uint64_t todo = __ballot(valid);
                while (todo) {
                    const int leader = __ffsll((unsigned long long)todo) - 1;
                    const int le = __builtin_amdgcn_readlane(best, leader);
                    const uint64_t m = __ballot(valid && best == le);
                    if (valid && best == le) rank = __popcll(m & lanes_below());
                    if (lane == leader) s_hist[le] = __popcll(m);
                    todo &= ~m;
                }
            }
            if (valid) ws.rank[(int64_t)j * samples + t] = rank;
            __builtin_amdgcn_wave_barrier();
            if (lane < experts) {
                ws.hist[((int64_t)blockIdx.x * k + j) * experts + lane] = s_hist[lane];
                int32_t *col = ws.hist_t + ((int64_t)j * experts + lane) * ws.gstride;
                col[blockIdx.x] = s_hist[lane];
                if ((int)blockIdx.x == groups - 1)             // the last group also clears the padding
                    for (int p = groups; p < ws.gstride; ++p) col[p] = 0;
            }
            __builtin_amdgcn_wave_barrier();
        }
    }
}

// locations += offset of the token's group (routing only, no dispatch)
__global__ __launch_bounds__(256) void route_offsets_kernel(const int32_t *__restrict__ indices,
                                                            int32_t *__restrict__ locations,
                                                            int64_t stride, int samples, int experts,
                                                            int k, const int32_t *__restrict__ hist,
                                                            const int32_t *__restrict__ rank, int group_tokens,
                                                            const float *__restrict__ loss_part,
                                                            int loss_parts, float *__restrict__ l_aux)
{
    finish_loss(loss_part, loss_parts, samples, l_aux);
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= samples * k) return;
    const int j = i / samples, t = i - j * samples;
    const int64_t o = (int64_t)j * stride + t;
    locations[o] = rank[i] + hist[((int64_t)(t / group_tokens) * k + j) * experts + indices[o]];
}

// ---- the prefix over the routing groups without a launch of its own (top_k <= 4): every wave
// sums the columns of the transposed histogram it needs.

// Lane j (< top_k) returns the slot of choice j of token t inside its expert: rank in the group +
// entries of the earlier planes + entries of the earlier groups of plane j.  e_l: its expert.
__device__ __forceinline__ int merged_location(const int32_t *__restrict__ indices, const int32_t *__restrict__ rank,
                                               const int32_t *__restrict__ hist_t, int64_t stride, int top_k,
                                               int samples, int experts, int t, int group_tokens, int groups,
                                               int gstride, int &e_l)
{
    const int lane = lane_id();
    int l = 0;
    e_l = 0;
    if (lane < top_k) {
        e_l = indices[(int64_t)lane * stride + t];
        l = rank[(int64_t)lane * samples + t];
    }
    const int g = t / group_tokens;
    // slots of expert e taken before this group's plane-j tokens: every entry of the planes
    // before j, and the groups before g in plane j
    int before[4] = {0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if (j < top_k) {
            const int e = rl_i(e_l, j);
            before[j] = column_partial(hist_t + ((int64_t)j * experts + e) * gstride, g);
            for (int jp = 0; jp < j; ++jp) before[j] += column_partial(hist_t + ((int64_t)jp * experts + e) * gstride, groups);
        }
    }
    wave_sum_n(before);
#pragma unroll
    for (int j = 0; j < 4; ++j) if (lane == j) l += before[j];
    return l;
}

// One work-group (4 waves) finishes the GShard loss and the per-plane expert counts.
// s_loss: 64 floats of LDS.
__device__ __forceinline__ void merged_stats(const int32_t *__restrict__ hist_t, const float *__restrict__ me_t,
                                             int groups, int gstride, int experts, int top_k, int samples,
                                             int32_t *__restrict__ counts_out, float *__restrict__ l_aux,
                                             float *s_loss)
{
    const int wave = threadIdx.x >> 6, lane = lane_id();
    // the one block that finishes the loss: l_aux = sum_e me[e] * ce[e] / T with
    // me[e] = column sum of the scores, ce[e] = first-choice count * E / T
    // four experts per pass and wave: the loads of a pass are in flight together
    for (int e0 = wave * 4; e0 < experts; e0 += 16) {
        int c0[4] = {0, 0, 0, 0};
        float m[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if (e0 + q < experts) {
                c0[q] = column_partial(hist_t + (int64_t)(e0 + q) * gstride, groups);
                if (l_aux) m[q] = column_partial(me_t + (int64_t)(e0 + q) * gstride, groups);
            }
        }
        wave_sum_n(c0);
        wave_sum_n(m);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            if (lane == 0 && e0 + q < experts) {
                if (counts_out) counts_out[e0 + q] = c0[q];
                s_loss[e0 + q] = m[q] * ((float)c0[q] * ((float)experts / (float)samples));
            }
        }
        if (counts_out) {
            for (int j = 1; j < top_k; ++j) {
                int c[4] = {0, 0, 0, 0};
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    if (e0 + q < experts) c[q] = column_partial(hist_t + ((int64_t)j * experts + e0 + q) * gstride, groups);
                wave_sum_n(c);
#pragma unroll
                for (int q = 0; q < 4; ++q) if (lane == 0 && e0 + q < experts) counts_out[j * experts + e0 + q] = c[q];
            }
        }
    }
    __syncthreads();
    if (l_aux && threadIdx.x == 0) {
        float a = 0.f;
        for (int e = 0; e < experts; ++e) a += s_loss[e];
        *l_aux = a / (float)samples;
    }
}

// locations of a stand-alone routing call (top_k <= 4): block 0 finishes the loss and the counts,
// the others take a token per wave
__global__ __launch_bounds__(256) void route_locations_merged_kernel(
    const int32_t *__restrict__ indices, int32_t *__restrict__ locations, int64_t stride, int top_k, int samples,
    int experts, const int32_t *__restrict__ rank, int group_tokens, const int32_t *__restrict__ hist_t,
    const float *__restrict__ me_t, int groups, int gstride, int32_t *__restrict__ counts_out,
    float *__restrict__ l_aux)
{
    __shared__ float s_loss[64];
    if (blockIdx.x == 0) {
        if (l_aux || counts_out)
            merged_stats(hist_t, me_t, groups, gstride, experts, top_k, samples, counts_out, l_aux, s_loss);
        return;
    }
    const int t = ((int)blockIdx.x - 1) * 4 + (int)(threadIdx.x >> 6);
    if (t >= samples) return;
    int e_l;
    const int l = merged_location(indices, rank, hist_t, stride, top_k, samples, experts, t, group_tokens, groups,
                                  gstride, e_l);
    if (lane_id() < top_k) locations[(int64_t)lane_id() * stride + t] = l;
}

// Dispatch + int8 with the slot offsets still to be added (see dispatch_int8_kernel for the
// stand-alone variant).  Only the all-ones gate helper (is_postscore) is fused here.
//
// MERGED: there was no group_offsets launch.  Every wave sums the histogram columns it needs
// itself (hist_t: one or two 16-byte loads per lane and column, k (k + 1) / 2 columns per token),
// the zero-fill blocks sum the expert totals, and one more block at the end of the grid finishes
// the GShard loss and the per-plane expert counts.  Used for top_k <= 4.
// SLOT_FIRST: a token's slots are worked out before its row is requested, and a token that keeps
// none of its choices leaves without reading its row.  Pays when many tokens are dropped (a
// capacity factor of 1 with skewed routing drops half of them); otherwise the row is requested
// first so that it travels while the slots are being worked out.
// PLAIN: no codec -- `codes` is the dispatched buffer in x's dtype and a kept row arrives there as
// 0 + x (what fast_encode's accumulation into zeros leaves: -0 becomes +0), an empty slot as zeros.
template <int DT, int CACHE, bool MERGED, bool SLOT_FIRST = false, bool PLAIN = false>
__global__ __launch_bounds__(256) void dispatch_int8_routed_kernel(
    const void *__restrict__ x, const int32_t *__restrict__ indices, int32_t *__restrict__ locations,
    int64_t stride, int top_k, int samples, int model_dim, int experts, int capacity,
    uint8_t *__restrict__ codes, void *__restrict__ bias_out, void *__restrict__ scale_out,
    const int32_t *__restrict__ hist, const int32_t *__restrict__ totals, const int32_t *__restrict__ rank,
    int group_tokens, int token_blocks, const float *__restrict__ loss_part, int loss_parts,
    float *__restrict__ l_aux, const float *__restrict__ row_min, const float *__restrict__ row_max,
    const int32_t *__restrict__ hist_t, const float *__restrict__ me_t, int groups, int gstride,
    int fill_blocks, int32_t *__restrict__ counts_out, int fill_first)
{
    using E = Elem<DT>;
    constexpr int V = E::VEC;
    const int wave = threadIdx.x >> 6, lane = lane_id();
    const int units = model_dim / V;
    __shared__ int32_t s_tot[64];
    __shared__ float s_loss[64];
    if constexpr (!MERGED) finish_loss(loss_part, loss_parts, samples, l_aux);

    // grid order: the block that finishes the loss (MERGED only; it starts with a few dependent
    // round trips over the histogram, which the streaming blocks behind it hide), then the token
    // blocks and the zero-fill blocks; the fill blocks go first when their own histogram pass is
    // long (many experts), last otherwise (measured both ways at 8 and at 64 experts).
    const int stat_blocks = (int)gridDim.x - fill_blocks - token_blocks;
    int bid = (int)blockIdx.x - stat_blocks;                              // < token_blocks: token block
    if (fill_first && bid >= 0) bid = bid < fill_blocks ? token_blocks + bid : bid - fill_blocks;
    if constexpr (MERGED) {
        if ((int)blockIdx.x < stat_blocks) {
            merged_stats(hist_t, me_t, groups, gstride, experts, top_k, samples, counts_out, l_aux, s_loss);
            return;
        }
    }

    if (bid >= token_blocks) {
        const int slots = experts * capacity;
        const int nwaves = fill_blocks * 4;
        const int fid = bid - token_blocks;
        if constexpr (MERGED) {
            // expert totals, four experts per pass and wave: the loads of a pass are in flight together
            for (int e0 = wave * 4; e0 < experts; e0 += 16) {
                int c[4] = {0, 0, 0, 0};
#pragma unroll
                for (int q = 0; q < 4; ++q)
                    if (e0 + q < experts)
                        for (int j = 0; j < top_k; ++j) c[q] += column_partial(hist_t + ((int64_t)j * experts + e0 + q) * gstride, groups);
                wave_sum_n(c);
#pragma unroll
                for (int q = 0; q < 4; ++q) if (lane == 0 && e0 + q < experts) s_tot[e0 + q] = c[q];
            }
            __syncthreads();
        }
        for (int s = fid * 4 + wave; s < slots; s += nwaves) {
            const int e = s / capacity;
            const int filled = MERGED ? s_tot[e] : totals[e];
            if (s - e * capacity < filled) continue;             // slot holds a token
            if constexpr (PLAIN) {
                uint4 *row = reinterpret_cast<uint4 *>(codes + (int64_t)s * units * 16);
                for (int u = lane; u < units; u += WAVE) stream_store(row + u, make_uint4(0u, 0u, 0u, 0u));
                continue;
            }
            uint8_t *row = codes + (int64_t)s * model_dim;
            for (int u = lane; u < units; u += WAVE) {
                if constexpr (V == 8) stream_store(reinterpret_cast<uint2 *>(row) + u, make_uint2(0u, 0u));
                else stream_store(reinterpret_cast<uint32_t *>(row) + u, 0u);
            }
            if (lane == 0) { E::store(bias_out, s, 0.f); E::store(scale_out, s, 0.f); }
        }
        return;
    }

    // tokens are walked from the last to the first: the rows the gate kernel read most recently
    // are the likeliest to still sit in cache
    const int t = samples - 1 - (bid * 4 + wave);
    if (t < 0) return;
    const uint4 *src = reinterpret_cast<const uint4 *>((const char *)x + (int64_t)t * model_dim * (int64_t)sizeof(typename E::store_t));
    uint4 cache[CACHE > 0 ? CACHE : 1];
    auto request_row = [&]() {
        if constexpr (CACHE > 0) {
#pragma unroll
            for (int c = 0; c < CACHE; ++c) {
                const int u = c * WAVE + lane;
                // (index clamped, not predicated: straight-line loads let the compiler wait for exactly these
                // loads; the re-read last vector is harmless for min / max and is never stored)
                cache[c] = src[min(u, units - 1)];
            }
        }
    };
    // lane j finalises choice j: slot = expert * capacity + rank in group + group offset
    auto find_slot = [&]() {
        int slot = -1;
        if constexpr (MERGED) {
            int e_l;
            const int l = merged_location(indices, rank, hist_t, stride, top_k, samples, experts, t, group_tokens, groups,
                                          gstride, e_l);
            if (lane < top_k) {
                locations[(int64_t)lane * stride + t] = l;
                if (l < capacity) slot = e_l * capacity + l;
            }
        } else if (lane < top_k) {
            const int64_t o = (int64_t)lane * stride + t;
            const int e = indices[o];
            const int l = rank[(int64_t)lane * samples + t] + hist[((int64_t)(t / group_tokens) * top_k + lane) * experts + e];
            locations[o] = l;
            if (l < capacity) slot = e * capacity + l;
        }
        return slot;
    };
    int slot;
    if constexpr (SLOT_FIRST) {
        slot = find_slot();
        if (__ballot(slot >= 0) == 0) return;
        request_row();
    } else {
        request_row();
        slot = find_slot();
        if (__ballot(slot >= 0) == 0) return;
    }

    if constexpr (PLAIN) {
        auto copy = [&](int u, const uint4 &raw) {
            float f[V];
            E::unpack(raw, f);
#pragma unroll
            for (int i = 0; i < V; ++i) f[i] = 0.f + f[i];
            const uint4 v = E::pack(f);
            for (int j = 0; j < top_k; ++j) {
                const int sl = rl_i(slot, j);
                if (sl >= 0) stream_store(reinterpret_cast<uint4 *>(codes + (int64_t)sl * units * 16) + u, v);
            }
        };
        if constexpr (CACHE > 0) {
#pragma unroll
            for (int c = 0; c < CACHE; ++c) if (c * WAVE + lane < units) copy(c * WAVE + lane, cache[c]);
        } else {
            for (int u = lane; u < units; u += WAVE) copy(u, src[u]);
        }
        return;
    }

    float mn, mx;
    if (row_min) {                                      // the gate kernel already scanned the row
        mn = row_min[t]; mx = row_max[t];
    } else {
        RowStats<DT, true> stats;
        stats.init();
        if constexpr (CACHE > 0) {
#pragma unroll
            for (int c = 0; c < CACHE; ++c) stats.add(cache[c]);
        } else {
            for (int u = lane; u < units; u += WAVE) stats.add(src[u]);
        }
        stats.finish(mn, mx);
    }
    const float scale = E::round(mx - mn);
    if (slot >= 0) { E::store(bias_out, slot, mn); E::store(scale_out, slot, scale); }
    const RowEncoder<DT> enc(mn, scale);

    auto body = [&](auto mode) {
        auto emit = [&](int u, const uint4 &raw) {
            uint32_t w[2];
            enc.template encode<decltype(mode)::value>(raw, w);
            for (int j = 0; j < top_k; ++j) {
                const int s = rl_i(slot, j);
                if (s < 0) continue;
                uint8_t *row = codes + (int64_t)s * model_dim;
                if constexpr (V == 8) stream_store(reinterpret_cast<uint2 *>(row) + u, make_uint2(w[0], w[1]));
                else stream_store(reinterpret_cast<uint32_t *>(row) + u, w[0]);
            }
        };
        if constexpr (CACHE > 0) {
#pragma unroll
            for (int c = 0; c < CACHE; ++c) if (c * WAVE + lane < units) emit(c * WAVE + lane, cache[c]);
        } else {
            for (int u = lane; u < units; u += WAVE) emit(u, src[u]);
        }
    };
    if (enc.fast()) body(std::true_type{}); else body(std::false_type{});
}

template <int DT, int SDT>
static void launch_gate_route(int experts, int groups, int group_tokens, hipStream_t st, const void *x, const void *wg,
                              const float *bias, int samples, int model_dim, int k, int normalize,
                              int32_t *indices, int32_t *locations, void *gates, int64_t stride,
                              void *logits_out, void *scores_out, float *l_aux, int32_t *counts, void *ws)
{
#define PM_GR_(NT, CAP, SPLITK, GROUP)                                                                   \
    gate_route_kernel<DT, SDT, NT, CAP, SPLITK, GROUP><<<groups, 256, 0, st>>>(x, wg, bias, samples, model_dim, experts, \
        k, normalize, indices, locations, gates, stride, logits_out, scores_out, l_aux, counts, ws)
#define PM_GR(NT, CAP, SPLITK) do { if (SPLITK && group_tokens == 32) PM_GR_(NT, CAP, SPLITK, (SPLITK ? 32 : 64)); \
                                    else PM_GR_(NT, CAP, SPLITK, 64); } while (0)
    // split-K measured faster than the LDS-shared variant up to 16 experts (30.7 vs 44.4 us at
    // 16384 x 4096 bf16, 8 experts), and the other way round above (168 -> 48 us at 64 experts)
    if (experts <= 8) PM_GR(1, 8, true);
    else if (experts <= 16) PM_GR(1, 16, true);
    else if (experts <= 32) PM_GR(2, 32, false);
    else PM_GR(4, 64, false);
#undef PM_GR
#undef PM_GR_
}

template <int DT>
static void launch_dispatch_routed(int per_lane, unsigned grid, hipStream_t st, const void *x,
                                   const int32_t *indices, int32_t *locations, int64_t stride, int top_k,
                                   int samples, int model_dim, int experts, int capacity, uint8_t *codes,
                                   void *bias, void *scale, const int32_t *offs, const int32_t *totals,
                                   const int32_t *rank, int group_tokens, int token_blocks,
                                   const float *loss_part, int loss_parts, float *l_aux,
                                   const float *row_min, const float *row_max, bool merged,
                                   const int32_t *hist_t, const float *me_t, int groups, int gstride,
                                   int fill_blocks, int32_t *counts, int fill_first, bool plain = false)
{
    // a capacity factor of at most 1: every imbalance of the routing drops tokens
    const bool slot_first = merged && (int64_t)experts * capacity <= (int64_t)top_k * samples;
#define PM_DR_(CACHE, MERGED, FIRST, PLAIN)                                                          \
    dispatch_int8_routed_kernel<DT, CACHE, MERGED, FIRST, PLAIN><<<grid, 256, 0, st>>>(x, indices, locations, stride, top_k, \
        samples, model_dim, experts, capacity, codes, bias, scale, offs, totals, rank, group_tokens,  \
        token_blocks, loss_part, loss_parts, l_aux, row_min, row_max, hist_t, me_t, groups, gstride,  \
        fill_blocks, counts, fill_first)
#define PM_DR(CACHE) do { if (plain) { if (slot_first) PM_DR_(CACHE, true, true, true); else if (merged) PM_DR_(CACHE, true, false, true); \
                                       else PM_DR_(CACHE, false, false, true); }                      \
                          else if (slot_first) PM_DR_(CACHE, true, true, false); else if (merged) PM_DR_(CACHE, true, false, false); \
                          else PM_DR_(CACHE, false, false, false); } while (0)
    if (per_lane <= 2) PM_DR(2);
    else if (per_lane <= 4) PM_DR(4);
    else if (per_lane <= 8) PM_DR(8);
    else if (per_lane <= 16) PM_DR(16);
    else PM_DR(0);
#undef PM_DR
#undef PM_DR_
}

static int fused_check(const char *who, const void *x, const void *wg, int dtype, int samples,
                       int model_dim, int experts, int top_k, int64_t stride)
{
    PM_REQUIRE(dtype_ok(dtype), "%s: bad dtype %d", who, dtype);
    PM_REQUIRE(samples >= 1 && model_dim >= 1 && experts >= 1 && top_k >= 1, "%s: bad shape", who);
    PM_REQUIRE(experts <= 64, "%s: the fused path supports up to 64 experts (got %d); use "
               "planmoe_gate_logits + planmoe_route_topk", who, experts);
    const int vec = dtype == PLANMOE_F32 ? 4 : 8;
    PM_REQUIRE(model_dim % vec == 0 && aligned16(x) && aligned16(wg),
               "%s: model_dim must be a multiple of %d and x / wg 16-byte aligned", who, vec);
    PM_REQUIRE(stride >= samples, "%s: plane_stride < samples", who);
    PM_REQUIRE(x && wg, "%s: NULL input", who);
    return 0;
}

struct FwdPlan {
    int k, groups, group_tokens, experts_per_block, blocks;
    bool merged;          // the dispatch launch does the prefix over groups itself
    FwdWs ws;
};
static void fwd_plan(FwdPlan &plan, void *workspace, int samples, int experts, int top_k)
{
    plan.k = top_k < experts ? top_k : experts;
    plan.group_tokens = fwd_group_tokens(experts, samples);
    plan.groups = (samples + plan.group_tokens - 1) / plan.group_tokens;
    plan.experts_per_block = go_experts_per_block(experts, plan.k);
    plan.blocks = (experts + plan.experts_per_block - 1) / plan.experts_per_block;
    plan.merged = plan.k <= 4;
    plan.ws = fwd_ws(workspace, plan.groups, plan.k, experts, samples);
}

// ranks in groups -> final slots (and the loss and the expert counts): one launch in which every
// wave sums the histogram columns it needs (top_k <= 4 and a small histogram), else the prefix
// over the groups and a launch that adds it
static void finish_routing(const FwdPlan &plan, const int32_t *indices, int32_t *locations, int64_t stride,
                           int samples, int experts, float *l_aux, int32_t *counts, hipStream_t st)
{
    // measured: 38.4 vs 39.7 us (256 groups x 8 experts), 58.6 vs 45.2 us (512 groups x 64 experts, where
    // nothing hides the one block that sums every column for the loss)
    if (plan.k <= 4 && (int64_t)plan.groups * experts <= 8192) {
        route_locations_merged_kernel<<<1 + (samples + 3) / 4, 256, 0, st>>>(
            indices, locations, stride, plan.k, samples, experts, plan.ws.rank, plan.group_tokens, plan.ws.hist_t,
            plan.ws.me_t, plan.groups, plan.ws.gstride, counts, l_aux);
        return;
    }
    group_offsets_kernel<<<plan.blocks, 256, 0, st>>>(plan.ws.hist, plan.ws.offs, plan.ws.me, plan.groups, plan.k, experts,
                                                      plan.experts_per_block, samples, plan.ws.totals, counts,
                                                      plan.ws.loss_part, l_aux != nullptr);
    route_offsets_kernel<<<(samples * plan.k + 255) / 256, 256, 0, st>>>(indices, locations, stride, samples, experts,
                                                                        plan.k, plan.ws.offs, plan.ws.rank,
                                                                        plan.group_tokens, plan.ws.loss_part, plan.blocks,
                                                                        l_aux);
}

// stand-alone routing from logits / scores in memory: the epilogue of gate_route_kernel on 64-token
// groups, then the prefix over the groups and the final slots
template <int SDT>
static void launch_route_groups(int experts, int groups, int mode, hipStream_t st, const void *input, const float *bias,
                                int samples, int k, int normalize, int32_t *indices, int32_t *locations, void *gates,
                                int64_t stride, void *scores_out, float *l_aux, int32_t *counts, void *ws)
{
#define PM_RG_(NT, CAP, MODE)                                                                              \
    gate_route_kernel<SDT, SDT, NT, CAP, false, 64, MODE><<<groups, 256, 0, st>>>(input, nullptr, bias, samples, 0, \
        experts, k, normalize, indices, locations, gates, stride, nullptr, scores_out, l_aux, counts, ws)
#define PM_RG(NT, CAP) do { if (mode == 1) PM_RG_(NT, CAP, 1); else PM_RG_(NT, CAP, 2); } while (0)
    if (experts <= 8) PM_RG(1, 8);
    else if (experts <= 16) PM_RG(1, 16);
    else if (experts <= 32) PM_RG(2, 32);
    else PM_RG(4, 64);
#undef PM_RG
#undef PM_RG_
}

int route_groups(const void *input, int dtype, int is_logits, const float *logit_bias, int samples, int experts,
                 int top_k, int normalize_gate, int32_t *indices, int32_t *locations, void *gates, int64_t stride,
                 void *scores_out, float *l_aux, int32_t *counts, void *workspace, hipStream_t st)
{
    FwdPlan plan;
    plan.k = top_k < experts ? top_k : experts;
    plan.group_tokens = 64;
    plan.groups = (samples + 63) / 64;
    plan.experts_per_block = go_experts_per_block(experts, plan.k);
    plan.blocks = (experts + plan.experts_per_block - 1) / plan.experts_per_block;
    plan.merged = false;
    workspace = fwd_tables(workspace);
    plan.ws = fwd_ws(workspace, plan.groups, plan.k, experts, samples);
    const int mode = is_logits ? 1 : 2;
    PM_DTYPE_SWITCH(dtype, SDT, (launch_route_groups<SDT>(experts, plan.groups, mode, st, input, is_logits ? logit_bias : nullptr,
                                                         samples, plan.k, normalize_gate, indices, locations, gates, stride,
                                                         is_logits ? scores_out : nullptr, l_aux, counts, workspace)));
    finish_routing(plan, indices, locations, stride, samples, experts, l_aux, counts, st);
    return 0;
}

// launches gate_route_kernel and, unless the dispatch launch will do that part, group_offsets_kernel
static int run_gate_route(const void *x, const void *wg, int dtype, int fp32_gate,
                          const float *logit_bias, int samples, int model_dim, int experts, int top_k,
                          int normalize_gate, int32_t *indices, int32_t *locations, void *gates,
                          int64_t stride, void *logits_out, void *scores_out, float *l_aux,
                          int32_t *counts, void *workspace, hipStream_t st, FwdPlan &plan,
                          bool offsets_follow)
{
    fwd_plan(plan, workspace, samples, experts, top_k);
    const int k = plan.k, groups = plan.groups;
    if (fp32_gate || dtype == PLANMOE_F32) {
        PM_DTYPE_SWITCH(dtype, DT, (launch_gate_route<DT, PLANMOE_F32>(
            experts, groups, plan.group_tokens, st, x, wg, logit_bias, samples, model_dim, k, normalize_gate, indices,
            locations, gates, stride, logits_out, scores_out, l_aux, counts, workspace)));
    } else if (dtype == PLANMOE_BF16) {
        launch_gate_route<PLANMOE_BF16, PLANMOE_BF16>(experts, groups, plan.group_tokens, st, x, wg, logit_bias, samples,
            model_dim, k, normalize_gate, indices, locations, gates, stride, logits_out, scores_out,
            l_aux, counts, workspace);
    } else {
        launch_gate_route<PLANMOE_F16, PLANMOE_F16>(experts, groups, plan.group_tokens, st, x, wg, logit_bias, samples,
            model_dim, k, normalize_gate, indices, locations, gates, stride, logits_out, scores_out,
            l_aux, counts, workspace);
    }
    if (offsets_follow)
        group_offsets_kernel<<<plan.blocks, 256, 0, st>>>(plan.ws.hist, plan.ws.offs, plan.ws.me, groups, k,
                                                          experts, plan.experts_per_block, samples,
                                                          plan.ws.totals, counts, plan.ws.loss_part,
                                                          l_aux != nullptr);
    return 0;
}

static int run_dispatch_routed(const void *x, int dtype, int samples, int model_dim, int experts,
                               int capacity, const int32_t *indices, int32_t *locations, int64_t stride,
                               float *l_aux, int32_t *counts, uint8_t *codes, void *bias, void *scale,
                               const FwdPlan &plan, hipStream_t st, bool plain = false)
{
    const int slots = experts * capacity;
    const int token_blocks = (samples + 3) / 4;
    int fill_blocks = min((slots + 3) / 4, 2048);
    if (plan.merged) {
        // every zero-fill block reads the whole transposed histogram once: keep that under ~32 MB
        const int64_t table = (int64_t)plan.k * experts * plan.ws.gstride * 4;
        fill_blocks = min(fill_blocks, (int)max((int64_t)64, ((int64_t)32 << 20) / table));
    }
    const int stat_blocks = plan.merged && (l_aux || counts) ? 1 : 0;
    const int vec = dtype == PLANMOE_F32 ? 4 : 8;
    const int per_lane = (model_dim / vec + WAVE - 1) / WAVE;
    PM_DTYPE_SWITCH(dtype, DT,
        launch_dispatch_routed<DT>(per_lane, (unsigned)(token_blocks + fill_blocks + stat_blocks), st, x, indices,
                                   locations, stride, plan.k, samples, model_dim, experts, capacity, codes, bias,
                                   scale, plan.ws.offs, plan.ws.totals, plan.ws.rank, plan.group_tokens, token_blocks,
                                   plan.ws.loss_part, plan.blocks, l_aux,
                                   dtype == PLANMOE_BF16 ? plan.ws.row_min : nullptr,
                                   dtype == PLANMOE_BF16 ? plan.ws.row_max : nullptr, plan.merged,
                                   plan.ws.hist_t, plan.ws.me_t, plan.groups, plan.ws.gstride, fill_blocks, counts,
                                   plan.merged && plan.k * experts > 32, plain));
    return 0;
}

} // namespace pm

#include "forward_single_launch.hpp"
#include "forward_ceiling.hpp"

namespace pm {

// a random number per process: the kernel adds it to the workspace's launch counter to form the tag
// of the words its work-groups publish, so that what an uninitialised workspace holds, or another
// process left behind, is unlikely to pass for a word of this launch
static unsigned long long process_salt()
{
    static const unsigned long long salt = [] {
        std::random_device rd;
        return ((unsigned long long)rd() << 32) | (unsigned long long)rd();
    }();
    return salt;
}

// Two one-launch kernels that run at the same time on one GPU can keep each other's work-groups
// from becoming resident, and then both wait until their bound.  So launches of the kernel on one
// device are put in a row on the host.  Launches on one stream follow each other anyway and cost
// nothing extra; when a launch comes in on another stream than the one before it, an event is
// recorded at the tail of that earlier stream (behind its launch, and behind whatever followed it
// there) and the new stream waits for it on the device.  (An event behind every launch would put a
// marker between back-to-back launches of one stream: 4 us each, measured.  A stream that is being
// captured into a graph is left alone: neither the wait nor the record belongs into the caller's
// graph; replays of such graphs are the caller's to keep apart.)
struct SingleOrder {
    std::mutex lock;
    hipEvent_t done = nullptr;
    hipStream_t last = nullptr;
    bool has_last = false;
};
static SingleOrder g_single_order[STATIC_SCRATCH_DEVICES_MAX];

static bool stream_is_capturing(hipStream_t st)
{
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(st, &status) != hipSuccess) { (void)hipGetLastError(); return false; }
    return status != hipStreamCaptureStatusNone;
}

// Call with order.lock held, before the launch on `st`.  0, or 1 with the error text set.
static int single_order_before(SingleOrder &order, hipStream_t st, bool ordered, const char *who)
{
    if (!ordered || !order.has_last || order.last == st || stream_is_capturing(order.last)) return 0;
    if (!order.done && hipEventCreateWithFlags(&order.done, hipEventDisableTiming) != hipSuccess)
        return fail("%s: cannot create an event", who);
    if (hipEventRecord(order.done, order.last) != hipSuccess) {
        (void)hipGetLastError();              // the earlier stream is gone: so is its work
        return 0;
    }
    if (hipStreamWaitEvent(st, order.done, 0) != hipSuccess)
        return fail("%s: cannot wait for the launch before this one", who);
    return 0;
}
static void single_order_after(SingleOrder &order, hipStream_t st, bool ordered)
{
    if (ordered) { order.last = st; order.has_last = true; }
}

#ifdef PM_FS_TRACE
// measurement build: the stamps of the one-launch kernel and of the ceiling kernels land in one array, so
// the kernel is instantiated in this translation unit, for rows of 4096 values only (what is measured)
PM_FS_DEFINE(16)
#define PM_FS_ABSENT(n) int fs_launch_m##n(const FsLaunch &) { return 2; }
PM_FS_ABSENT(1) PM_FS_ABSENT(2) PM_FS_ABSENT(3) PM_FS_ABSENT(4) PM_FS_ABSENT(5) PM_FS_ABSENT(6) PM_FS_ABSENT(7) PM_FS_ABSENT(8)
PM_FS_ABSENT(9) PM_FS_ABSENT(10) PM_FS_ABSENT(11) PM_FS_ABSENT(12) PM_FS_ABSENT(13) PM_FS_ABSENT(14) PM_FS_ABSENT(15)
#undef PM_FS_ABSENT
#endif

// 0: launched; 2: the shape is not served by the one-launch kernel (nothing was enqueued)
static int run_forward_single(const void *x, const void *wg, int dtype, int fp32_gate, const float *logit_bias,
                              int samples, int model_dim, int experts, int top_k, int normalize_gate, int capacity,
                              int32_t *indices, int32_t *locations, void *gates, int64_t stride, void *logits_out,
                              void *scores_out, float *l_aux, int32_t *counts, uint8_t *codes, void *bias,
                              void *scale, void *workspace, int spin_limit, int32_t *gave_up, hipStream_t st,
                              bool ask_only = false)
{
    const int k = top_k < experts ? top_k : experts;
    if (dtype != PLANMOE_BF16 || model_dim % 256 != 0 || model_dim < 256 || model_dim > 4096 || experts > 16 || k > 4 || samples < 1) return 2;
    if (!ask_only && !aligned16(codes) && capacity > 0) return 2;
    int cus = 0, dev = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 1) return 2;
    // as few tokens per work-group as it takes to put one work-group on every compute unit; beyond 64
    // tokens per compute unit, work-groups of 64 tokens, which short rows allow two of per compute unit
    // (the launch goes ahead only if the runtime says that all of them are resident at once)
    const int rounds = min((samples + 16 * cus - 1) / (16 * cus), 4);
    const int groups = (samples + 16 * rounds - 1) / (16 * rounds);
    if (groups > FS_MAX_GROUPS) return 2;
    const FsLaunch a{rounds, groups, st, x, wg, logit_bias, samples, experts, k, normalize_gate, capacity, indices,
                     locations, gates, stride, logits_out, scores_out, l_aux, counts, codes, bias, scale, workspace,
                     process_salt(), spin_limit, gave_up, fp32_gate, ask_only};
    // rows of 256 NMMA values: every wave owns an eighth of a row
    static int (*const launch[16])(const FsLaunch &) = {
        fs_launch_m1, fs_launch_m2, fs_launch_m3, fs_launch_m4, fs_launch_m5, fs_launch_m6, fs_launch_m7, fs_launch_m8,
        fs_launch_m9, fs_launch_m10, fs_launch_m11, fs_launch_m12, fs_launch_m13, fs_launch_m14, fs_launch_m15, fs_launch_m16};
    return launch[model_dim / 256 - 1](a);
}

} // namespace pm

using namespace pm;

extern "C" size_t planmoe_forward_workspace_bytes(int samples, int experts, int top_k)
{
    if (samples <= 0 || experts <= 0 || top_k <= 0) return FWD_TABLES_OFFSET + 256;
    const size_t k = (size_t)(top_k < experts ? top_k : experts);
    const size_t groups = ((size_t)samples + 15) / 16;      // upper bound over the group sizes
    const size_t tables = ((size_t)experts + FWD_LOSS_PARTS + 2 * groups * k * experts + groups * experts +
                           (k + 2) * (size_t)samples + (k + 1) * experts * fwd_pad4(groups)) * 4;
    // in front of the tables: the one-launch kernel's own region
    return FWD_TABLES_OFFSET + round_up(tables, 256);
}

extern "C" int planmoe_gate_route(const void *x, const void *wg, int dtype, int fp32_gate,
                                  const float *logit_bias, int samples, int model_dim, int experts,
                                  int top_k, int normalize_gate, int32_t *indices, int32_t *locations,
                                  void *gates, int64_t plane_stride, void *logits_out, void *scores_out,
                                  float *l_aux, int32_t *expert_counts, void *workspace,
                                  size_t workspace_bytes, void *stream)
{
    if (samples == 0) return 0;
    if (fused_check("planmoe_gate_route", x, wg, dtype, samples, model_dim, experts, top_k, plane_stride)) return 1;
    PM_REQUIRE(indices && locations && gates, "planmoe_gate_route: NULL output");
    PM_REQUIRE(workspace && workspace_bytes >= planmoe_forward_workspace_bytes(samples, experts, top_k),
               "planmoe_gate_route: workspace too small");
    workspace = fwd_tables(workspace);
    hipStream_t st = (hipStream_t)stream;
    FwdPlan plan;
    if (run_gate_route(x, wg, dtype, fp32_gate, logit_bias, samples, model_dim, experts, top_k,
                       normalize_gate, indices, locations, gates, plane_stride, logits_out, scores_out,
                       l_aux, expert_counts, workspace, st, plan, false)) return 1;
    finish_routing(plan, indices, locations, plane_stride, samples, experts, l_aux, expert_counts, st);
    PM_LAUNCH_CHECK("planmoe_gate_route");
    return 0;
}

extern "C" int planmoe_forward_int8(const void *x, const void *wg, int dtype, int fp32_gate,
                                    const float *logit_bias, int samples, int model_dim, int experts,
                                    int top_k, int normalize_gate, int capacity, int32_t *indices,
                                    int32_t *locations, void *gates, int64_t plane_stride,
                                    void *logits_out, void *scores_out, float *l_aux,
                                    int32_t *expert_counts, uint8_t *codes, void *bias, void *scale,
                                    void *workspace, size_t workspace_bytes, void *stream)
{
    PM_REQUIRE(capacity >= 0 && (int64_t)experts * capacity < (1ll << 31), "planmoe_forward_int8: bad capacity");
    if (fused_check("planmoe_forward_int8", x, wg, dtype, samples, model_dim, experts, top_k, plane_stride)) return 1;
    PM_REQUIRE(indices && locations && gates, "planmoe_forward_int8: NULL routing output");
    PM_REQUIRE((codes && bias && scale) || capacity == 0, "planmoe_forward_int8: NULL codec output");
    PM_REQUIRE((uintptr_t)codes % 8 == 0, "planmoe_forward_int8: codes must be 8-byte aligned");
    PM_REQUIRE(workspace && workspace_bytes >= planmoe_forward_workspace_bytes(samples, experts, top_k),
               "planmoe_forward_int8: workspace too small");
    workspace = fwd_tables(workspace);
    hipStream_t st = (hipStream_t)stream;
    FwdPlan plan;
    fwd_plan(plan, workspace, samples, experts, top_k);
    if (run_gate_route(x, wg, dtype, fp32_gate, logit_bias, samples, model_dim, experts, top_k,
                       normalize_gate, indices, locations, gates, plane_stride, logits_out, scores_out,
                       l_aux, expert_counts, workspace, st, plan, !plan.merged)) return 1;
    if (run_dispatch_routed(x, dtype, samples, model_dim, experts, capacity, indices, locations,
                            plane_stride, l_aux, expert_counts, codes, bias, scale, plan, st)) return 1;
    PM_LAUNCH_CHECK("planmoe_forward_int8");
    return 0;
}

extern "C" int planmoe_forward_plain(const void *x, const void *wg, int dtype, int fp32_gate,
                                     const float *logit_bias, int samples, int model_dim, int experts,
                                     int top_k, int normalize_gate, int capacity, int32_t *indices,
                                     int32_t *locations, void *gates, int64_t plane_stride,
                                     void *logits_out, void *scores_out, float *l_aux,
                                     int32_t *expert_counts, void *dispatched, void *workspace,
                                     size_t workspace_bytes, void *stream)
{
    PM_REQUIRE(capacity >= 0 && (int64_t)experts * capacity < (1ll << 31), "planmoe_forward_plain: bad capacity");
    if (fused_check("planmoe_forward_plain", x, wg, dtype, samples, model_dim, experts, top_k, plane_stride)) return 1;
    PM_REQUIRE(indices && locations && gates, "planmoe_forward_plain: NULL routing output");
    PM_REQUIRE(dispatched || capacity == 0, "planmoe_forward_plain: NULL output");
    PM_REQUIRE(aligned16(dispatched), "planmoe_forward_plain: the dispatched buffer must be 16-byte aligned");
    PM_REQUIRE(workspace && workspace_bytes >= planmoe_forward_workspace_bytes(samples, experts, top_k),
               "planmoe_forward_plain: workspace too small");
    workspace = fwd_tables(workspace);
    hipStream_t st = (hipStream_t)stream;
    FwdPlan plan;
    fwd_plan(plan, workspace, samples, experts, top_k);
    if (run_gate_route(x, wg, dtype, fp32_gate, logit_bias, samples, model_dim, experts, top_k,
                       normalize_gate, indices, locations, gates, plane_stride, logits_out, scores_out,
                       l_aux, expert_counts, workspace, st, plan, !plan.merged)) return 1;
    if (run_dispatch_routed(x, dtype, samples, model_dim, experts, capacity, indices, locations,
                            plane_stride, l_aux, expert_counts, (uint8_t *)dispatched, nullptr, nullptr, plan, st,
                            true)) return 1;
    PM_LAUNCH_CHECK("planmoe_forward_plain");
    return 0;
}

extern "C" int planmoe_forward_int8_single(const void *x, const void *wg, int dtype, int fp32_gate,
                                           const float *logit_bias, int samples, int model_dim, int experts,
                                           int top_k, int normalize_gate, int capacity, int32_t *indices,
                                           int32_t *locations, void *gates, int64_t plane_stride,
                                           void *logits_out, void *scores_out, float *l_aux,
                                           int32_t *expert_counts, uint8_t *codes, void *bias, void *scale,
                                           void *workspace, size_t workspace_bytes, int spin_limit,
                                           int32_t *gave_up, void *stream)
{
    PM_REQUIRE(capacity >= 0 && (int64_t)experts * capacity < (1ll << 31), "planmoe_forward_int8_single: bad capacity");
    if (fused_check("planmoe_forward_int8_single", x, wg, dtype, samples, model_dim, experts, top_k, plane_stride)) return 1;
    PM_REQUIRE(indices && locations && gates, "planmoe_forward_int8_single: NULL routing output");
    PM_REQUIRE((codes && bias && scale) || capacity == 0, "planmoe_forward_int8_single: NULL codec output");
    PM_REQUIRE(workspace && workspace_bytes >= planmoe_forward_workspace_bytes(samples, experts, top_k),
               "planmoe_forward_int8_single: workspace too small");
    PM_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 7u) == 0, "planmoe_forward_int8_single: workspace must be 8-byte aligned");
    PM_REQUIRE(spin_limit >= 0, "planmoe_forward_int8_single: spin_limit < 0");
    hipStream_t st = (hipStream_t)stream;
    int dev = 0;
    PM_REQUIRE(hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < STATIC_SCRATCH_DEVICES_MAX,
               "planmoe_forward_int8_single: no current device");
    SingleOrder &order = g_single_order[dev];
    const bool ordered = !stream_is_capturing(st);
    std::unique_lock<std::mutex> hold(order.lock);
    if (single_order_before(order, st, ordered, "planmoe_forward_int8_single")) return 1;
    const int rc = run_forward_single(x, wg, dtype, fp32_gate, logit_bias, samples, model_dim, experts, top_k,
                                      normalize_gate, capacity, indices, locations, gates, plane_stride, logits_out,
                                      scores_out, l_aux, expert_counts, codes, bias, scale, workspace,
                                      spin_limit > 0 ? spin_limit : (1 << 20), gave_up, st);
    if (rc == 0) single_order_after(order, st, ordered);
    hold.unlock();
    PM_REQUIRE(rc != 2, "planmoe_forward_int8_single: the one-launch kernel serves bf16 rows of 256 to 4096 values in steps of 256, up to 16 "
               "experts, top_k <= 4 and as many tokens as its work-groups of 64 hold while all resident at once "
               "(planmoe_forward_int8_single_serves tells); use planmoe_forward_int8");
    PM_LAUNCH_CHECK("planmoe_forward_int8_single");
    return rc;
}

extern "C" int planmoe_forward_int8_single_serves(int dtype, int fp32_gate, int samples, int model_dim, int experts, int top_k)
{
    if (samples < 1 || model_dim < 1 || experts < 1 || top_k < 1) return 0;
    return run_forward_single(nullptr, nullptr, dtype, fp32_gate, nullptr, samples, model_dim, experts, top_k, 1, 0,
                              nullptr, nullptr, nullptr, 0, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr,
                              nullptr, nullptr, 0, nullptr, nullptr, true) == 0;
}

extern "C" int planmoe_forward_int8_single_ceiling(const void *x, int samples, int model_dim, int experts, int top_k,
                                                   int capacity, uint8_t *codes, void *bias, void *scale,
                                                   int32_t *planes, void *workspace, size_t workspace_bytes,
                                                   int mode, int spin_limit, int32_t *gave_up, void *stream)
{
    PM_REQUIRE(x && codes && bias && scale && planes && workspace, "planmoe_forward_int8_single_ceiling: NULL argument");
    PM_REQUIRE(model_dim == 4096 && experts == 8 && top_k == 2 && samples >= 64 && samples % 128 == 0,
               "planmoe_forward_int8_single_ceiling: serves rows of 4096 bf16 values, 8 experts, top-2 and a multiple of "
               "128 tokens");
    const int groups = samples / 64;
    PM_REQUIRE(groups <= FS_MAX_GROUPS && capacity >= groups * 16 && (int64_t)experts * capacity < (1ll << 31),
               "planmoe_forward_int8_single_ceiling: needs a capacity of at least samples / 4");
    PM_REQUIRE(aligned16(x) && aligned16(codes) && (reinterpret_cast<uintptr_t>(workspace) & 7u) == 0,
               "planmoe_forward_int8_single_ceiling: bad alignment");
    PM_REQUIRE(workspace_bytes >= planmoe_forward_workspace_bytes(samples, experts, top_k),
               "planmoe_forward_int8_single_ceiling: workspace too small");
    PM_REQUIRE(mode >= 0 && mode <= 2, "planmoe_forward_int8_single_ceiling: mode is 0, 1 or 2");
    hipStream_t st = (hipStream_t)stream;
    int dev = 0, per_cu = 0, cus = 0;
    PM_REQUIRE(hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < STATIC_SCRATCH_DEVICES_MAX,
               "planmoe_forward_int8_single_ceiling: no current device");
    // like the kernel it stands in for: every work-group must be resident at once
    const void *fn = mode == 0 ? (const void *)forward_single_ceiling_kernel<0> : mode == 1 ? (const void *)forward_single_ceiling_kernel<1>
                               : (const void *)forward_single_ceiling_kernel<2>;
    PM_REQUIRE(hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, fn, FS_THREADS, 0) == hipSuccess &&
               hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess &&
               groups <= per_cu * cus, "planmoe_forward_int8_single_ceiling: more work-groups than fit on the GPU at once");
    SingleOrder &order = g_single_order[dev];
    const bool ordered = !stream_is_capturing(st);
    std::unique_lock<std::mutex> hold(order.lock);
    if (single_order_before(order, st, ordered, "planmoe_forward_int8_single_ceiling")) return 1;
    const int spins = spin_limit > 0 ? spin_limit : (1 << 20);
#define PM_CEIL(MODE_) forward_single_ceiling_kernel<MODE_><<<groups, FS_THREADS, 0, st>>>((const uint4 *)x, samples, capacity, \
            codes, (uint16_t *)bias, (uint16_t *)scale, planes, workspace, process_salt(), spins, gave_up)
    if (mode == 0) PM_CEIL(0); else if (mode == 1) PM_CEIL(1); else PM_CEIL(2);
#undef PM_CEIL
    single_order_after(order, st, ordered);
    hold.unlock();
    PM_LAUNCH_CHECK("planmoe_forward_int8_single_ceiling");
    return 0;
}

#ifdef PM_FS_TRACE
extern "C" int planmoe_debug_fs_trace(unsigned long long *out_host)
{
    return hipMemcpyFromSymbol(out_host, HIP_SYMBOL(pm::fs_trace), sizeof(unsigned long long) * 1024 * 16) != hipSuccess;
}
#endif

// ---- the same entry point for callers that can allocate nothing: its workspace is a file-scope
// array in device memory.  Host code must not hand `static_scratch` itself to a kernel (on the
// host the name is a stand-in, not a device address): the address is asked for once per device
// and kept.
constexpr size_t STATIC_SCRATCH_BYTES = (size_t)4 << 20;
constexpr int STATIC_SCRATCH_DEVICES = STATIC_SCRATCH_DEVICES_MAX;
static __device__ __align__(256) unsigned char static_scratch[STATIC_SCRATCH_BYTES];
static void *g_static_scratch[STATIC_SCRATCH_DEVICES];
static std::mutex g_static_scratch_lock;

// device address of this device's copy of the array (every GPU holds its own), NULL + error text on failure
static void *static_scratch_address()
{
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess || dev < 0 || dev >= STATIC_SCRATCH_DEVICES) {
        set_error("planmoe_forward_int8_static: no current device (%s)", hipGetErrorString(e));
        return nullptr;
    }
    std::lock_guard<std::mutex> hold(g_static_scratch_lock);
    if (!g_static_scratch[dev]) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(static_scratch));
        if (e != hipSuccess || !p) {
            set_error("planmoe_forward_int8_static: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
            return nullptr;
        }
        g_static_scratch[dev] = p;
    }
    return g_static_scratch[dev];
}

extern "C" int planmoe_forward_int8_static(const void *x, const void *wg, int dtype, int fp32_gate,
                                           const float *logit_bias, int samples, int model_dim, int experts,
                                           int top_k, int normalize_gate, int capacity, int32_t *indices,
                                           int32_t *locations, void *gates, int64_t plane_stride,
                                           void *logits_out, void *scores_out, float *l_aux,
                                           int32_t *expert_counts, uint8_t *codes, void *bias, void *scale,
                                           void *stream)
{
    const size_t need = planmoe_forward_workspace_bytes(samples, experts, top_k);
    PM_REQUIRE(need <= STATIC_SCRATCH_BYTES,
               "planmoe_forward_int8_static: %d tokens x %d experts x top-%d need %zu bytes of scratch, the "
               "built-in buffer holds %zu; use planmoe_forward_int8 with a workspace of the caller's",
               samples, experts, top_k, need, STATIC_SCRATCH_BYTES);
    void *ws = static_scratch_address();
    if (!ws) return 1;
    // nothing in the workspace has to start at zero: every word a launch reads was written by the
    // launch before it in the same call (the padding of the transposed histogram included)
    return planmoe_forward_int8(x, wg, dtype, fp32_gate, logit_bias, samples, model_dim, experts, top_k,
                                normalize_gate, capacity, indices, locations, gates, plane_stride, logits_out,
                                scores_out, l_aux, expert_counts, codes, bias, scale, ws, STATIC_SCRATCH_BYTES, stream);
}

extern "C" int planmoe_forward_int8_redispatch(const void *x, int dtype, int samples, int model_dim,
                                               int experts, int top_k, int capacity,
                                               const int32_t *indices, int32_t *locations,
                                               int64_t plane_stride, uint8_t *codes, void *bias,
                                               void *scale, void *workspace, size_t workspace_bytes,
                                               void *stream)
{
    PM_REQUIRE(dtype_ok(dtype) && samples >= 1 && experts >= 1 && experts <= 64 && top_k >= 1 && capacity >= 0,
               "planmoe_forward_int8_redispatch: bad arguments");
    PM_REQUIRE(x && indices && locations && workspace && ((codes && bias && scale) || capacity == 0),
               "planmoe_forward_int8_redispatch: NULL argument");
    PM_REQUIRE(workspace_bytes >= planmoe_forward_workspace_bytes(samples, experts, top_k),
               "planmoe_forward_int8_redispatch: workspace too small");
    const int vec = dtype == PLANMOE_F32 ? 4 : 8;
    PM_REQUIRE(model_dim % vec == 0 && aligned16(x) && (uintptr_t)codes % 8 == 0,
               "planmoe_forward_int8_redispatch: bad alignment");
    workspace = fwd_tables(workspace);
    FwdPlan plan;
    fwd_plan(plan, workspace, samples, experts, top_k);
    if (run_dispatch_routed(x, dtype, samples, model_dim, experts, capacity, indices, locations,
                            plane_stride, nullptr, nullptr, codes, bias, scale, plan, (hipStream_t)stream)) return 1;
    PM_LAUNCH_CHECK("planmoe_forward_int8_redispatch");
    return 0;
}
