// The forward chain in two launches:
//
//   gate_route_kernel     x is read once: gate-logits GEMM on the matrix cores, then, for the
//                         work-group's 32 tokens, softmax, k-fold arg-max, gates, the rank of
//                         every token among the group's tokens with the same choice, and the
//                         group's expert histogram.  The last work-group to finish turns the
//                         histograms into slot offsets (choice plane after choice plane) and
//                         computes the GShard loss.
//   dispatch_int8_routed  slot = rank in group + group offset; token rows go to uint8 codes in
//                         their slots (x read a second time, normally from cache), slots past an
//                         expert's fill are zero rows.  Or route_offsets_kernel when only the
//                         routing is wanted.
//
// This replaces gates/top.py:20-26 + moe_layer.py:230-256 + fast_dispatch.py:140-195 +
// fast_encode (fast_dispatch.py:197-201) + Int8Compressor::compress (int8.cpp:7-44).
//
// Workspace (int32 words): [0] finished-group counter (zero before the first use, restored to
// zero by every call), [1..15] unused, totals[E], hist[groups][k][E], me[groups][E] (fp32).
#include "gate_core.hpp"
#include "rows.hpp"
#include "int8_core.hpp"

namespace pm {

constexpr int FWD_TPW = 2;
constexpr int FWD_GROUP = 16 * FWD_TPW;      // tokens per work-group
constexpr int FWD_HEADER = 16;               // int32 words before totals

struct FwdWs {
    int32_t *counter, *totals, *hist;
    float *me;
};
__host__ __device__ inline FwdWs fwd_ws(void *ws, int groups, int k, int experts)
{
    FwdWs w;
    w.counter = (int32_t *)ws;
    w.totals = w.counter + FWD_HEADER;
    w.hist = w.totals + experts;
    w.me = (float *)(w.hist + (size_t)groups * k * experts);
    return w;
}

__device__ __forceinline__ uint64_t lanes_below() { return ((uint64_t)1 << lane_id()) - 1; }

// SDT: dtype of logits / scores / gates (F32 when fp32_gate, else the input dtype)
template <int DT, int SDT, int NT>
__global__ __launch_bounds__(256) void gate_route_kernel(
    const void *__restrict__ x, const void *__restrict__ wg, const float *__restrict__ logit_bias,
    int samples, int model_dim, int experts, int k, int normalize_gate,
    int32_t *__restrict__ indices, int32_t *__restrict__ locations, void *__restrict__ gates,
    int64_t stride, void *__restrict__ logits_out, void *__restrict__ scores_out,
    float *__restrict__ l_aux, int32_t *__restrict__ counts_out, void *__restrict__ workspace)
{
    using S = Elem<SDT>;
    constexpr int CAP = 16 * NT;
    __shared__ float part[4][FWD_GROUP][CAP + 1];
    __shared__ int32_t s_hist[CAP];
    __shared__ int32_t s_scan[256];
    __shared__ int s_last;

    const int tid = threadIdx.x, lane = lane_id();
    const int groups = gridDim.x;
    const FwdWs ws = fwd_ws(workspace, groups, k, experts);
    const int t0 = blockIdx.x * FWD_GROUP;
    gate_tile_partials<DT, NT, FWD_TPW>(x, wg, t0, samples, model_dim, experts, part);
    __syncthreads();

    if (tid < WAVE) {                                  // wave 0: one lane per token of the group
        const int t = t0 + tid;
        const bool valid = tid < FWD_GROUP && t < samples;
        float s[CAP];
        if (valid) {
            float mx = -INFINITY;
#pragma unroll
            for (int e = 0; e < CAP; ++e) {
                float v = -INFINITY;
                if (e < experts) {
                    v = ((part[0][tid][e] + part[1][tid][e]) + part[2][tid][e]) + part[3][tid][e];
                    v = S::round(v);
                    if (logits_out) S::store(logits_out, (int64_t)t * experts + e, v);
                    if (logit_bias) v = S::round(v + logit_bias[e]);
                }
                s[e] = v;
                mx = fmaxf(mx, v);
            }
            float sum = 0.f;
#pragma unroll
            for (int e = 0; e < CAP; ++e) if (e < experts) { s[e] = expf(s[e] - mx); sum += s[e]; }
#pragma unroll
            for (int e = 0; e < CAP; ++e) {
                if (e < experts) {
                    s[e] = S::round(s[e] / sum);
                    if (scores_out) S::store(scores_out, (int64_t)t * experts + e, s[e]);
                }
            }
        }
        // column sums of the group's scores (GShard loss)
        if (l_aux) {
#pragma unroll
            for (int e = 0; e < CAP; ++e) {
                if (e >= experts) break;
                const float v = wave_sum(valid ? s[e] : 0.f);
                if (lane == 0) ws.me[(int64_t)blockIdx.x * experts + e] = v;
            }
        }
        float denom = 0.f;
        uint64_t taken = 0;
        for (int j = 0; j < k; ++j) {
            int best = -1; float bv = -INFINITY;
            if (valid) {
#pragma unroll
                for (int e = 0; e < CAP; ++e) {
                    const bool free_ = !((taken >> e) & 1u) && e < experts;
                    if (free_ && (best < 0 || s[e] > bv)) { best = e; bv = s[e]; }
                }
                taken |= (uint64_t)1 << best;
                indices[(int64_t)j * stride + t] = best;
                S::store(gates, (int64_t)j * stride + t, bv);
                denom = (j == 0) ? bv : S::round(denom + bv);
            }
            __builtin_amdgcn_wave_barrier();
            if (lane < CAP) s_hist[lane] = 0;
            __builtin_amdgcn_wave_barrier();
            int rank = 0;
            uint64_t todo = __ballot(valid);
            while (todo) {
                const int leader = __ffsll((unsigned long long)todo) - 1;
                const int le = __builtin_amdgcn_readlane(best, leader);
                const uint64_t m = __ballot(valid && best == le);
                if (valid && best == le) rank = __popcll(m & lanes_below());
                if (lane == leader) s_hist[le] = __popcll(m);
                todo &= ~m;
            }
            if (valid) locations[(int64_t)j * stride + t] = rank;
            __builtin_amdgcn_wave_barrier();
            if (lane < experts) ws.hist[((int64_t)blockIdx.x * k + j) * experts + lane] = s_hist[lane];
        }
        if (valid && k > 1 && normalize_gate) {
            const float eps = SDT == PLANMOE_F32 ? 1.1920928955078125e-07f
                            : SDT == PLANMOE_BF16 ? 0.0078125f : 0.0009765625f;
            const float d = fmaxf(denom, eps);
            for (int j = 0; j < k; ++j) {
                const float g = S::load(gates, (int64_t)j * stride + t);
                S::store(gates, (int64_t)j * stride + t, g / d);
            }
        }
    }

    // ---- the last group to arrive scans the histograms of all groups
    __threadfence();
    __syncthreads();
    if (tid == 0) {
        const int ticket = atomicAdd(ws.counter, 1);
        s_last = (ticket == groups - 1);
    }
    __syncthreads();
    if (!s_last) return;
    __threadfence();

    int lanes_e = 1; while (lanes_e < experts) lanes_e <<= 1;      // experts <= 64
    const int chunks = 256 / lanes_e;
    const int e = tid % lanes_e, ch = tid / lanes_e;
    const bool live = e < experts;
    const int per = (groups + chunks - 1) / chunks;
    const int g0 = min(ch * per, groups), g1 = min(g0 + per, groups);
    int32_t carry = 0, count0 = 0;
    for (int j = 0; j < k; ++j) {
        int32_t sum = 0;
        if (live)
            for (int g = g0; g < g1; ++g) sum += ws.hist[((int64_t)g * k + j) * experts + e];
        s_scan[tid] = sum;
        __syncthreads();
        int32_t before = 0, total = 0;
        for (int c = 0; c < chunks; ++c) {
            const int32_t v = s_scan[c * lanes_e + e];
            before += (c < ch) ? v : 0;
            total += v;
        }
        if (live) {
            int32_t run = carry + before;
            for (int g = g0; g < g1; ++g) {
                const int64_t o = ((int64_t)g * k + j) * experts + e;
                const int32_t v = ws.hist[o];
                ws.hist[o] = run;
                run += v;
            }
            if (ch == 0 && counts_out) counts_out[j * experts + e] = total;
        }
        if (j == 0) count0 = total;
        carry += total;
        __syncthreads();
    }
    if (live && ch == 0) ws.totals[e] = carry;
    if (l_aux) {
        // l_aux = sum_e(me[e] * ce[e]) / T with ce[e] = count0[e] * (E / T)
        float mes = 0.f;
        if (live)
            for (int g = g0; g < g1; ++g) mes += ws.me[(int64_t)g * experts + e];
        float *f_scan = reinterpret_cast<float *>(s_scan);
        f_scan[tid] = mes;
        __syncthreads();
        if (tid < WAVE) {
            float acc = 0.f;
            if (tid < experts) {
                float me = 0.f;
                for (int c = 0; c < chunks; ++c) me += f_scan[c * lanes_e + tid];
                // count0 of expert `tid` lives in thread (ch 0, e = tid) == this thread
                acc = me * ((float)count0 * ((float)experts / (float)samples));
            }
            acc = wave_sum(acc);
            if (tid == 0) *l_aux = acc / (float)samples;
        }
    }
    if (tid == 0) *ws.counter = 0;                     // ready for the next call
}

// locations += offset of the token's group (routing only, no dispatch)
__global__ __launch_bounds__(256) void route_offsets_kernel(const int32_t *__restrict__ indices,
                                                            int32_t *__restrict__ locations,
                                                            int64_t stride, int samples, int experts,
                                                            int k, const int32_t *__restrict__ hist)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= samples * k) return;
    const int j = i / samples, t = i - j * samples;
    const int64_t o = (int64_t)j * stride + t;
    locations[o] += hist[((int64_t)(t / FWD_GROUP) * k + j) * experts + indices[o]];
}

// Dispatch + int8 with the slot offsets still to be added (see dispatch_int8_kernel for the
// stand-alone variant).  Only the all-ones gate helper (is_postscore) is fused here.
template <int DT, int CACHE>
__global__ __launch_bounds__(256) void dispatch_int8_routed_kernel(
    const void *__restrict__ x, const int32_t *__restrict__ indices, int32_t *__restrict__ locations,
    int64_t stride, int top_k, int samples, int model_dim, int experts, int capacity,
    uint8_t *__restrict__ codes, void *__restrict__ bias_out, void *__restrict__ scale_out,
    const int32_t *__restrict__ hist, const int32_t *__restrict__ totals, int token_blocks)
{
    using E = Elem<DT>;
    constexpr int V = E::VEC;
    const int wave = threadIdx.x >> 6, lane = lane_id();
    const int units = model_dim / V;

    if ((int)blockIdx.x >= token_blocks) {
        const int slots = experts * capacity;
        const int nwaves = (gridDim.x - token_blocks) * 4;
        for (int s = (blockIdx.x - token_blocks) * 4 + wave; s < slots; s += nwaves) {
            const int e = s / capacity;
            if (s - e * capacity < totals[e]) continue;          // slot holds a token
            uint8_t *row = codes + (int64_t)s * model_dim;
            for (int u = lane; u < units; u += WAVE) {
                if constexpr (V == 8) reinterpret_cast<uint2 *>(row)[u] = make_uint2(0u, 0u);
                else reinterpret_cast<uint32_t *>(row)[u] = 0u;
            }
            if (lane == 0) { E::store(bias_out, s, 0.f); E::store(scale_out, s, 0.f); }
        }
        return;
    }

    const int t = blockIdx.x * 4 + wave;
    if (t >= samples) return;
    const uint4 *src = reinterpret_cast<const uint4 *>((const char *)x + (int64_t)t * model_dim * (int64_t)sizeof(typename E::store_t));
    uint4 cache[CACHE > 0 ? CACHE : 1];
    if constexpr (CACHE > 0) {
#pragma unroll
        for (int c = 0; c < CACHE; ++c) {
            const int u = c * WAVE + lane;
            if (u < units) cache[c] = src[u];
        }
    }

    // lane j finalises choice j: slot = expert * capacity + rank in group + group offset
    int slot = -1;
    if (lane < top_k) {
        const int64_t o = (int64_t)lane * stride + t;
        const int e = indices[o];
        const int l = locations[o] + hist[((int64_t)(t / FWD_GROUP) * top_k + lane) * experts + e];
        locations[o] = l;
        if (l < capacity) slot = e * capacity + l;
    }
    if (__ballot(slot >= 0) == 0) return;

    float mn = INFINITY, mx = -INFINITY;
    auto visit = [&](const uint4 &raw) {
        float f[V];
        E::unpack(raw, f);
#pragma unroll
        for (int i = 0; i < V; ++i) { const float d = 0.f + f[i]; mn = nan_min(mn, d); mx = nan_max(mx, d); }
    };
    if constexpr (CACHE > 0) {
#pragma unroll
        for (int c = 0; c < CACHE; ++c) if (c * WAVE + lane < units) visit(cache[c]);
    } else {
        for (int u = lane; u < units; u += WAVE) visit(src[u]);
    }
    mn = wave_allreduce(mn, [](float a, float b) { return nan_min(a, b); });
    mx = wave_allreduce(mx, [](float a, float b) { return nan_max(a, b); });
    const float scale = E::round(mx - mn);
    if (slot >= 0) { E::store(bias_out, slot, mn); E::store(scale_out, slot, scale); }
    const RowQuant<DT> rq(mn, scale);

    auto emit = [&](int u, const uint4 &raw) {
        float f[V];
        E::unpack(raw, f);
        uint32_t w[2];
#pragma unroll
        for (int i = 0; i < V / 4; ++i)
            w[i] = rq(0.f + f[4 * i]) | (rq(0.f + f[4 * i + 1]) << 8) | (rq(0.f + f[4 * i + 2]) << 16) | (rq(0.f + f[4 * i + 3]) << 24);
        for (int j = 0; j < top_k; ++j) {
            const int s = rl_i(slot, j);
            if (s < 0) continue;
            uint8_t *row = codes + (int64_t)s * model_dim;
            if constexpr (V == 8) reinterpret_cast<uint2 *>(row)[u] = make_uint2(w[0], w[1]);
            else reinterpret_cast<uint32_t *>(row)[u] = w[0];
        }
    };
    if constexpr (CACHE > 0) {
#pragma unroll
        for (int c = 0; c < CACHE; ++c) if (c * WAVE + lane < units) emit(c * WAVE + lane, cache[c]);
    } else {
        for (int u = lane; u < units; u += WAVE) emit(u, src[u]);
    }
}

template <int DT, int SDT>
static void launch_gate_route(int experts, int groups, hipStream_t st, const void *x, const void *wg,
                              const float *bias, int samples, int model_dim, int k, int normalize,
                              int32_t *indices, int32_t *locations, void *gates, int64_t stride,
                              void *logits_out, void *scores_out, float *l_aux, int32_t *counts, void *ws)
{
#define PM_GR(NT)                                                                                   \
    gate_route_kernel<DT, SDT, NT><<<groups, 256, 0, st>>>(x, wg, bias, samples, model_dim, experts, \
        k, normalize, indices, locations, gates, stride, logits_out, scores_out, l_aux, counts, ws)
    if (experts <= 16) PM_GR(1);
    else if (experts <= 32) PM_GR(2);
    else PM_GR(4);
#undef PM_GR
}

template <int DT>
static void launch_dispatch_routed(int per_lane, unsigned grid, hipStream_t st, const void *x,
                                   const int32_t *indices, int32_t *locations, int64_t stride, int top_k,
                                   int samples, int model_dim, int experts, int capacity, uint8_t *codes,
                                   void *bias, void *scale, const int32_t *hist, const int32_t *totals,
                                   int token_blocks)
{
#define PM_DR(CACHE)                                                                                 \
    dispatch_int8_routed_kernel<DT, CACHE><<<grid, 256, 0, st>>>(x, indices, locations, stride, top_k, \
        samples, model_dim, experts, capacity, codes, bias, scale, hist, totals, token_blocks)
    if (per_lane <= 2) PM_DR(2);
    else if (per_lane <= 4) PM_DR(4);
    else if (per_lane <= 8) PM_DR(8);
    else if (per_lane <= 16) PM_DR(16);
    else PM_DR(0);
#undef PM_DR
}

static int fused_check(const char *who, const void *x, const void *wg, int dtype, int samples,
                       int model_dim, int experts, int top_k, int64_t stride)
{
    PM_REQUIRE(dtype_ok(dtype), "%s: bad dtype %d", who, dtype);
    PM_REQUIRE(samples >= 1 && model_dim >= 1 && experts >= 1 && top_k >= 1, "%s: bad shape", who);
    PM_REQUIRE(experts <= 64, "%s: the fused path supports up to 64 experts (got %d); use "
               "planmoe_gate_logits + planmoe_route_topk", who, experts);
    PM_REQUIRE(top_k <= 64, "%s: top_k must be <= 64", who);
    const int vec = dtype == PLANMOE_F32 ? 4 : 8;
    PM_REQUIRE(model_dim % vec == 0 && aligned16(x) && aligned16(wg),
               "%s: model_dim must be a multiple of %d and x / wg 16-byte aligned", who, vec);
    PM_REQUIRE(stride >= samples, "%s: plane_stride < samples", who);
    PM_REQUIRE(x && wg, "%s: NULL input", who);
    return 0;
}

} // namespace pm

using namespace pm;

extern "C" size_t planmoe_forward_workspace_bytes(int samples, int experts, int top_k)
{
    if (samples <= 0 || experts <= 0 || top_k <= 0) return 256;
    const size_t k = (size_t)(top_k < experts ? top_k : experts);
    const size_t groups = ((size_t)samples + FWD_GROUP - 1) / FWD_GROUP;
    return round_up((FWD_HEADER + (size_t)experts + groups * k * experts + groups * experts) * 4, 256);
}

extern "C" int planmoe_forward_workspace_init(void *workspace, size_t workspace_bytes, void *stream)
{
    PM_REQUIRE(workspace && workspace_bytes >= 256, "planmoe_forward_workspace_init: workspace too small");
    fill_u32((uint32_t *)workspace, FWD_HEADER, 0u, (hipStream_t)stream);
    PM_LAUNCH_CHECK("planmoe_forward_workspace_init");
    return 0;
}

static int run_gate_route(const char *who, const void *x, const void *wg, int dtype, int fp32_gate,
                          const float *logit_bias, int samples, int model_dim, int experts, int k,
                          int normalize_gate, int32_t *indices, int32_t *locations, void *gates,
                          int64_t stride, void *logits_out, void *scores_out, float *l_aux,
                          int32_t *counts, void *workspace, hipStream_t st)
{
    const int groups = (samples + FWD_GROUP - 1) / FWD_GROUP;
    if (fp32_gate || dtype == PLANMOE_F32) {
        PM_DTYPE_SWITCH(dtype, DT, (launch_gate_route<DT, PLANMOE_F32>(
            experts, groups, st, x, wg, logit_bias, samples, model_dim, k, normalize_gate, indices,
            locations, gates, stride, logits_out, scores_out, l_aux, counts, workspace)));
    } else if (dtype == PLANMOE_BF16) {
        launch_gate_route<PLANMOE_BF16, PLANMOE_BF16>(experts, groups, st, x, wg, logit_bias, samples,
            model_dim, k, normalize_gate, indices, locations, gates, stride, logits_out, scores_out,
            l_aux, counts, workspace);
    } else {
        launch_gate_route<PLANMOE_F16, PLANMOE_F16>(experts, groups, st, x, wg, logit_bias, samples,
            model_dim, k, normalize_gate, indices, locations, gates, stride, logits_out, scores_out,
            l_aux, counts, workspace);
    }
    (void)who;
    return 0;
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
    const int k = top_k < experts ? top_k : experts;
    hipStream_t st = (hipStream_t)stream;
    if (run_gate_route("planmoe_gate_route", x, wg, dtype, fp32_gate, logit_bias, samples, model_dim,
                       experts, k, normalize_gate, indices, locations, gates, plane_stride, logits_out,
                       scores_out, l_aux, expert_counts, workspace, st)) return 1;
    const int groups = (samples + FWD_GROUP - 1) / FWD_GROUP;
    const FwdWs ws = fwd_ws(workspace, groups, k, experts);
    route_offsets_kernel<<<(samples * k + 255) / 256, 256, 0, st>>>(indices, locations, plane_stride,
                                                                   samples, experts, k, ws.hist);
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
    PM_REQUIRE(codes && bias && scale, "planmoe_forward_int8: NULL codec output");
    PM_REQUIRE((uintptr_t)codes % 8 == 0, "planmoe_forward_int8: codes must be 8-byte aligned");
    PM_REQUIRE(workspace && workspace_bytes >= planmoe_forward_workspace_bytes(samples, experts, top_k),
               "planmoe_forward_int8: workspace too small");
    const int k = top_k < experts ? top_k : experts;
    hipStream_t st = (hipStream_t)stream;
    if (run_gate_route("planmoe_forward_int8", x, wg, dtype, fp32_gate, logit_bias, samples, model_dim,
                       experts, k, normalize_gate, indices, locations, gates, plane_stride, logits_out,
                       scores_out, l_aux, expert_counts, workspace, st)) return 1;
    const int groups = (samples + FWD_GROUP - 1) / FWD_GROUP;
    const FwdWs ws = fwd_ws(workspace, groups, k, experts);
    const int slots = experts * capacity;
    const int token_blocks = (samples + 3) / 4;
    const int fill_blocks = min((slots + 3) / 4, 2048);
    const int vec = dtype == PLANMOE_F32 ? 4 : 8;
    const int per_lane = (model_dim / vec + WAVE - 1) / WAVE;
    PM_DTYPE_SWITCH(dtype, DT,
        launch_dispatch_routed<DT>(per_lane, (unsigned)(token_blocks + fill_blocks), st, x, indices, locations,
                                   plane_stride, k, samples, model_dim, experts, capacity, codes, bias,
                                   scale, ws.hist, ws.totals, token_blocks));
    PM_LAUNCH_CHECK("planmoe_forward_int8");
    return 0;
}
