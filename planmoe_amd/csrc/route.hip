// Top-k routing with capacity-slot assignment, and the stand-alone capacity cumsum.
//
// planmoe_route_topk takes the place of extract_critical (impls/fast_dispatch.py:140-195):
// about 25 ATen launches over [samples, experts] one-hot matrices plus the E-block
// Blelloch scan of custom_kernel.cpp:339-376 become two or three launches that never build a
// one-hot matrix.  Up to 64 experts the work is done by the routing epilogue of the forward
// chain's first kernel (forward.hip, route_groups); above that by the kernels of this file:
//   route_tile_kernel   one thread per token, 256 tokens per tile: softmax (optional),
//                       k-fold arg-max, rank of the token among the tile's tokens that
//                       chose the same expert (wave ballots + an LDS table), per-tile
//                       expert histograms and per-tile column sums of the scores
//   group_offsets_kernel exclusive prefix of the histograms over tiles, choice plane after
//                       choice plane, so that all first choices precede all second choices
//   route_finish_kernel location = rank in tile + prefix; GShard loss
//
// Workspace layout (32-bit words): hist[tiles][k][E], offs[tiles][k][E], me[tiles][E] (fp32),
// loss_part[E] (fp32).
#include <algorithm>

#include "common.hpp"
#include "offsets.hpp"
#include "rows.hpp"

namespace pm {

#ifndef PM_ROUTE_TILE
#define PM_ROUTE_TILE 256
#endif
constexpr int TILE = PM_ROUTE_TILE;   // tokens per tile = threads per block
constexpr int TILE_WAVES = TILE / WAVE;
constexpr int ROUTE_MAX_E = 2048; // LDS table is 4 waves x experts counters

__device__ __forceinline__ uint64_t lanemask_lt()
{
    return ((uint64_t)1 << lane_id()) - 1;
}

template <int DT>
struct ScoreRow {
    using E = Elem<DT>;
    const void *in;
    const float *bias;
    int64_t base;
    int experts;
    bool logits;
    float mx, sum;

    __device__ __forceinline__ float logit(int e) const
    {
        float l = E::load(in, base + e);
        if (bias) l = E::round(l + bias[e]);
        return l;
    }
    __device__ void prepare()
    {
        if (!logits) return;
        mx = -INFINITY;
        for (int e = 0; e < experts; ++e) mx = fmaxf(mx, logit(e));
        sum = 0.f;
        for (int e = 0; e < experts; ++e) sum += expf(logit(e) - mx);
    }
    // score of expert e in the routing dtype
    __device__ __forceinline__ float score(int e) const
    {
        if (!logits) return E::load(in, base + e);
        return E::round(expf(logit(e) - mx) / sum);
    }
};

// CAP > 0: the row (<= CAP scores) lives in registers; CAP == 0: every pass recomputes
// the scores from memory.
template <int DT, int CAP>
__global__ __launch_bounds__(TILE) void route_tile_kernel(
    const void *__restrict__ input, int input_is_logits, const float *__restrict__ logit_bias,
    int samples, int experts, int k, int normalize_gate,
    int32_t *__restrict__ indices, int32_t *__restrict__ locations, void *__restrict__ gates,
    int64_t stride, void *__restrict__ scores_out, int32_t *__restrict__ hist,
    float *__restrict__ me_part)
{
    using E = Elem<DT>;
    extern __shared__ int32_t wave_cnt[];           // [TILE_WAVES][experts]
    const int tid = threadIdx.x, lane = lane_id(), wave = tid >> 6;
    const int t = blockIdx.x * TILE + tid;
    const bool valid = t < samples;

    ScoreRow<DT> row;
    row.in = input; row.bias = logit_bias; row.base = (int64_t)t * experts;
    row.experts = experts; row.logits = input_is_logits != 0;

    float s[CAP > 0 ? CAP : 1];
    if constexpr (CAP > 0) {
        // the tile's rows come in with coalesced loads, half a tile at a time, and every thread
        // picks its row out of LDS (row length + 1 keeps the banks apart)
        float *stage = reinterpret_cast<float *>(wave_cnt + TILE_WAVES * experts);       // [TILE / 2][experts + 1]
        const int64_t tile_base = (int64_t)blockIdx.x * TILE * experts;
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            const int r0 = half * (TILE / 2);
            const int nrows = max(0, min(TILE / 2, samples - (int)blockIdx.x * TILE - r0));
            // 8 loads in flight per thread (clamped index: straight-line loads, one wait per batch)
            const int n = nrows * experts;
            const int64_t half_base = tile_base + (int64_t)r0 * experts;
            for (int i0 = tid; i0 < n; i0 += 8 * TILE) {
                float v[8];
#pragma unroll
                for (int q = 0; q < 8; ++q) v[q] = E::load(input, half_base + min(i0 + q * TILE, n - 1));
#pragma unroll
                for (int q = 0; q < 8; ++q) {
                    const int i = i0 + q * TILE;
                    if (i < n) {
                        const int r = i / experts, e = i - r * experts;
                        stage[r * (experts + 1) + e] = v[q];
                    }
                }
            }
            __syncthreads();
            if (valid && tid / (TILE / 2) == half) {
#pragma unroll
                for (int e = 0; e < CAP; ++e)
                    s[e] = (e < experts) ? stage[(tid - r0) * (experts + 1) + e] : -INFINITY;
            }
            __syncthreads();
        }
        if (valid && row.logits) {
            float mx = -INFINITY;
#pragma unroll
            for (int e = 0; e < CAP; ++e) {
                if (e < experts) {
                    if (logit_bias) s[e] = E::round(s[e] + logit_bias[e]);
                    mx = fmaxf(mx, s[e]);
                }
            }
            float sum = 0.f;
#pragma unroll
            for (int e = 0; e < CAP; ++e) if (e < experts) { s[e] = expf(s[e] - mx); sum += s[e]; }
#pragma unroll
            for (int e = 0; e < CAP; ++e) if (e < experts) s[e] = E::round(s[e] / sum);
        }
    }
    if (valid) {
        if constexpr (CAP == 0) row.prepare();
        if (scores_out) {
            if constexpr (CAP > 0) {
#pragma unroll
                for (int e = 0; e < CAP; ++e) if (e < experts) E::store(scores_out, row.base + e, s[e]);
            } else {
                for (int e = 0; e < experts; ++e) E::store(scores_out, row.base + e, row.score(e));
            }
        }
    }

    // per-tile column sums of the scores (for the GShard loss), fixed reduction order
    if (me_part) {
        float *wsum = reinterpret_cast<float *>(wave_cnt);
        if constexpr (CAP > 0) {
#pragma unroll
            for (int e = 0; e < CAP; ++e) {
                if (e < experts) {
                    const float v = wave_sum(valid ? s[e] : 0.f);
                    if (lane == 0) wsum[wave * experts + e] = v;
                }
            }
        } else {
            for (int e = 0; e < experts; ++e) {
                const float v = wave_sum(valid ? row.score(e) : 0.f);
                if (lane == 0) wsum[wave * experts + e] = v;
            }
        }
        __syncthreads();
        for (int e = tid; e < experts; e += TILE)
        {
            float a = wsum[e];
            for (int w = 1; w < TILE_WAVES; ++w) a += wsum[w * experts + e];        // fixed order
            me_part[(int64_t)blockIdx.x * experts + e] = a;
        }
        __syncthreads();
    }

    // k-fold arg-max: lower expert id wins among equal scores
    float denom = 0.f;
    uint64_t taken_lo = 0;                       // experts < 64 already chosen (CAP path)
    for (int j = 0; j < k; ++j) {
        int best = -1; float bv = -INFINITY;
        if (valid) {
            if constexpr (CAP > 0) {
#pragma unroll
                for (int e = 0; e < CAP; ++e) {
                    const bool free_ = !((taken_lo >> e) & 1u) && e < experts;
                    if (free_ && (best < 0 || s[e] > bv)) { best = e; bv = s[e]; }
                }
                taken_lo |= (uint64_t)1 << best;
            } else {
                // chosen experts of earlier planes are re-read from the output planes
                for (int e = 0; e < experts; ++e) {
                    bool free_ = true;
                    for (int p = 0; p < j; ++p) free_ = free_ && (indices[(int64_t)p * stride + t] != e);
                    const float v = row.score(e);
                    if (free_ && (best < 0 || v > bv)) { best = e; bv = v; }
                }
            }
            indices[(int64_t)j * stride + t] = best;
            // raw gate now, normalised after the loop
            E::store(gates, (int64_t)j * stride + t, bv);
            denom = (j == 0) ? bv : E::round(denom + bv);
        }

        // rank of this token among the tile's tokens with the same j-th choice
        for (int e = tid; e < TILE_WAVES * experts; e += TILE) wave_cnt[e] = 0;
        __syncthreads();
        int rank = 0;
        uint64_t todo = __ballot(valid);
        while (todo) {
            const int leader = __ffsll((unsigned long long)todo) - 1;
            const int le = __builtin_amdgcn_readlane(best, leader);
            const uint64_t m = __ballot(valid && best == le);
            if (valid && best == le) rank = __popcll(m & lanemask_lt());
            if (lane == leader) wave_cnt[wave * experts + le] = __popcll(m);
            todo &= ~m;
        }
        __syncthreads();
        if (valid) {
            int before = 0;
            for (int w = 0; w < wave; ++w) before += wave_cnt[w * experts + best];
            locations[(int64_t)j * stride + t] = rank + before;
        }
        for (int e = tid; e < experts; e += TILE) {
            int32_t n = 0;
            for (int w = 0; w < TILE_WAVES; ++w) n += wave_cnt[w * experts + e];
            hist[((int64_t)blockIdx.x * k + j) * experts + e] = n;
        }
        __syncthreads();
    }

    if (valid && k > 1 && normalize_gate) {
        const float eps = DT == PLANMOE_F32 ? 1.1920928955078125e-07f
                        : DT == PLANMOE_BF16 ? 0.0078125f : 0.0009765625f;
        const float d = fmaxf(denom, eps);
        for (int j = 0; j < k; ++j) {
            const float g = E::load(gates, (int64_t)j * stride + t);
            E::store(gates, (int64_t)j * stride + t, g / d);
        }
    }
}

// Locations for routing decisions that already exist, with the tokens visited in a given order
// (batch-prioritised routing, fast_dispatch.py:135-138, 152-154: tokens sorted by importance take
// their slots first).  Thread p of a tile handles the token order[p] (or p): rank among the
// tile's tokens with the same choice + per-tile histograms, as in route_tile_kernel.
__global__ __launch_bounds__(TILE) void locate_tile_kernel(
    const int32_t *__restrict__ indices, const int32_t *__restrict__ order, int32_t *__restrict__ locations,
    int64_t stride, int samples, int experts, int k, int32_t *__restrict__ hist)
{
    extern __shared__ int32_t wave_cnt[];           // [TILE_WAVES][experts]
    const int tid = threadIdx.x, lane = lane_id(), wave = tid >> 6;
    const int p = blockIdx.x * TILE + tid;
    const bool valid = p < samples;
    const int t = valid ? (order ? order[p] : p) : 0;
    for (int j = 0; j < k; ++j) {
        int best = valid ? indices[(int64_t)j * stride + t] : -1;
        const bool live = valid && best >= 0 && best < experts;     // anything else takes no slot
        for (int e = tid; e < TILE_WAVES * experts; e += TILE) wave_cnt[e] = 0;
        __syncthreads();
        int rank = 0;
        uint64_t todo = __ballot(live);
        while (todo) {
            const int leader = __ffsll((unsigned long long)todo) - 1;
            const int le = __builtin_amdgcn_readlane(best, leader);
            const uint64_t m = __ballot(live && best == le);
            if (live && best == le) rank = __popcll(m & lanemask_lt());
            if (lane == leader) wave_cnt[wave * experts + le] = __popcll(m);
            todo &= ~m;
        }
        __syncthreads();
        if (live) {
            int before = 0;
            for (int w = 0; w < wave; ++w) before += wave_cnt[w * experts + best];
            locations[(int64_t)j * stride + t] = rank + before;
        } else if (valid) {
            locations[(int64_t)j * stride + t] = -1;
        }
        for (int e = tid; e < experts; e += TILE) {
            int32_t n = 0;
            for (int w = 0; w < TILE_WAVES; ++w) n += wave_cnt[w * experts + e];
            hist[((int64_t)blockIdx.x * k + j) * experts + e] = n;
        }
        __syncthreads();
    }
}

// location = rank in tile + offset of the tile; one thread of the launch finishes the loss
__global__ __launch_bounds__(TILE) void route_finish_kernel(
    const int32_t *__restrict__ indices, int32_t *__restrict__ locations, int64_t stride,
    int samples, int experts, int k, const int32_t *__restrict__ offs,
    const float *__restrict__ loss_part, int loss_parts, float *__restrict__ l_aux,
    const int32_t *__restrict__ order)
{
    finish_loss(loss_part, loss_parts, samples, l_aux);
    const int p = blockIdx.x * TILE + threadIdx.x;
    if (p >= samples) return;
    const int t = order ? order[p] : p;
    for (int j = 0; j < k; ++j) {
        const int64_t o = (int64_t)j * stride + t;
        const int e = indices[o];
        if (e >= 0 && e < experts) locations[o] += offs[((int64_t)blockIdx.x * k + j) * experts + e];
    }
}

// ------------------------------------------------------------------ routing backward
// Gradient of the gates (and of the GShard loss) with respect to the scores, optionally carried
// through the softmax to the logits.  One thread per token:
//   g_j = s_j / D, D = max(sum_i s_i, eps)  =>  ds_j = (dg_j - [sum >= eps] * sum_i dg_i g_i) / D
//   l_aux = sum_e me[e] ce[e] / T            =>  ds[t][e] += dl * ce[e] / T,  ce[e] = count0[e] * E / T
//   softmax: dlogit_e = s_e * (ds_e - sum_i ds_i s_i)
template <int DT>
__global__ __launch_bounds__(256) void route_bwd_kernel(
    const void *__restrict__ scores, const int32_t *__restrict__ indices, const void *__restrict__ dgates,
    int64_t stride, int samples, int experts, int k, int normalize_gate, const float *__restrict__ dl_aux,
    const int32_t *__restrict__ count0, int through_softmax, void *__restrict__ dscores)
{
    using E = Elem<DT>;
    const int t = blockIdx.x * 256 + threadIdx.x;
    if (t >= samples) return;
    const int64_t base = (int64_t)t * experts;
    const float dl = dl_aux ? dl_aux[0] : 0.f;
    const float lscale = dl * ((float)experts / (float)samples) / (float)samples;
    float sum = 0.f, dot = 0.f;
    for (int j = 0; j < k; ++j) {
        const float sj = E::load(scores, base + indices[(int64_t)j * stride + t]);
        sum = (j == 0) ? sj : E::round(sum + sj);
        dot += E::load(dgates, (int64_t)j * stride + t) * sj;
    }
    const float eps = DT == PLANMOE_F32 ? 1.1920928955078125e-07f : DT == PLANMOE_BF16 ? 0.0078125f : 0.0009765625f;
    const bool norm = k > 1 && normalize_gate;
    const float D = norm ? fmaxf(sum, eps) : 1.f;
    const float corr = (norm && sum >= eps) ? dot / (D * D) : 0.f;      // sum_i dg_i g_i / D
    auto ds_at = [&](int e) {
        float v = count0 ? lscale * (float)count0[e] : 0.f;
        for (int j = 0; j < k; ++j)
            if (indices[(int64_t)j * stride + t] == e) v += E::load(dgates, (int64_t)j * stride + t) / D - corr;
        return v;
    };
    if (!through_softmax) {
        for (int e = 0; e < experts; ++e) E::store(dscores, base + e, ds_at(e));
    } else {
        float inner = 0.f;
        for (int e = 0; e < experts; ++e) inner += ds_at(e) * E::load(scores, base + e);
        for (int e = 0; e < experts; ++e) {
            const float s = E::load(scores, base + e);
            E::store(dscores, base + e, s * (ds_at(e) - inner));
        }
    }
}

// ------------------------------------------------------------------ stand-alone cumsum
// out = cumsum(in, dim 0) - 1 over an int32 [samples, columns] matrix, three phases:
// per-tile column sums, prefix of the tile sums, per-tile rescan with the tile's offset.
// A block covers 64-column groups with 256 threads = column lanes x row lanes; a thread
// walks CS_ROWS consecutive rows of its column.
constexpr int CS_ROWS = 16;

struct CsGeom { int lanes_c, lanes_r, tile_rows; };
__host__ __device__ inline CsGeom cs_geom(int columns)
{
    CsGeom g;
    g.lanes_c = 1;
    while (g.lanes_c < columns && g.lanes_c < 64) g.lanes_c <<= 1;
    g.lanes_r = 256 / g.lanes_c;
    g.tile_rows = g.lanes_r * CS_ROWS;
    return g;
}

template <bool FINAL>
__global__ __launch_bounds__(256) void cumsum_tile_kernel(const int32_t *__restrict__ in,
                                                          int32_t *__restrict__ out, int samples,
                                                          int columns, int32_t *__restrict__ tile_sums)
{
    __shared__ int32_t part[256];
    const CsGeom g = cs_geom(columns);
    const int cl = threadIdx.x % g.lanes_c, rl = threadIdx.x / g.lanes_c;
    const int c = blockIdx.y * 64 + cl;
    const bool live = c < columns;
    const int r0 = blockIdx.x * g.tile_rows + rl * CS_ROWS;
    int32_t v[CS_ROWS];
    int32_t s = 0;
#pragma unroll
    for (int i = 0; i < CS_ROWS; ++i) {
        const int r = r0 + i;
        v[i] = (live && r < samples) ? in[(int64_t)r * columns + c] : 0;
        s += v[i];
    }
    part[threadIdx.x] = s;
    __syncthreads();
    int32_t before = 0, total = 0;
    for (int q = 0; q < g.lanes_r; ++q) {
        const int32_t p = part[q * g.lanes_c + cl];
        before += (q < rl) ? p : 0;
        total += p;
    }
    if constexpr (!FINAL) {
        if (live && rl == 0) tile_sums[(int64_t)blockIdx.x * columns + c] = total;
    } else {
        if (!live) return;
        int32_t run = tile_sums[(int64_t)blockIdx.x * columns + c] + before - 1;
#pragma unroll
        for (int i = 0; i < CS_ROWS; ++i) {
            const int r = r0 + i;
            run += v[i];
            if (r < samples) out[(int64_t)r * columns + c] = run;
        }
    }
}

} // namespace pm

using namespace pm;

extern "C" size_t planmoe_cumsum_workspace_bytes(int samples, int columns)
{
    if (samples <= 0 || columns <= 0) return 16;
    const CsGeom g = cs_geom(columns);
    const size_t tiles = ((size_t)samples + g.tile_rows - 1) / g.tile_rows;
    return round_up(2 * tiles * (size_t)columns * sizeof(int32_t), 256);     // tile sums + their prefix
}

extern "C" int planmoe_cumsum_sub_one(const int32_t *in, int32_t *out, int samples, int columns,
                                      void *workspace, size_t workspace_bytes, void *stream)
{
    PM_REQUIRE(samples >= 0 && columns >= 0, "planmoe_cumsum_sub_one: bad shape");
    if (samples == 0 || columns == 0) return 0;
    PM_REQUIRE(in && out, "planmoe_cumsum_sub_one: NULL argument");
    PM_REQUIRE(workspace && workspace_bytes >= planmoe_cumsum_workspace_bytes(samples, columns),
               "planmoe_cumsum_sub_one: workspace too small");
    const CsGeom g = cs_geom(columns);
    const int tiles = (samples + g.tile_rows - 1) / g.tile_rows;
    const int cgroups = (columns + 63) / 64;
    PM_REQUIRE(cgroups <= 65535, "planmoe_cumsum_sub_one: too many columns");
    hipStream_t st = (hipStream_t)stream;
    int32_t *sums = (int32_t *)workspace;
    int32_t *prefix = sums + (size_t)tiles * columns;
    cumsum_tile_kernel<false><<<dim3(tiles, cgroups), 256, 0, st>>>(in, out, samples, columns, sums);
    const int epb = go_experts_per_block(columns, 1);
    group_offsets_kernel<<<(columns + epb - 1) / epb, 256, 0, st>>>(sums, prefix, nullptr, tiles, 1, columns, epb,
                                                                   samples, nullptr, nullptr, nullptr, 0);
    cumsum_tile_kernel<true><<<dim3(tiles, cgroups), 256, 0, st>>>(in, out, samples, columns, prefix);
    PM_LAUNCH_CHECK("planmoe_cumsum_sub_one");
    return 0;
}

extern "C" int planmoe_route_bwd(const void *scores, int dtype, const int32_t *indices, const void *grad_gates,
                                 int64_t plane_stride, int samples, int experts, int top_k, int normalize_gate,
                                 const float *grad_l_aux, const int32_t *first_choice_counts,
                                 int through_softmax, void *grad_scores, void *stream)
{
    PM_REQUIRE(dtype_ok(dtype), "planmoe_route_bwd: bad dtype %d", dtype);
    PM_REQUIRE(samples >= 0 && experts >= 1 && top_k >= 1, "planmoe_route_bwd: bad shape");
    PM_REQUIRE(plane_stride >= samples, "planmoe_route_bwd: plane_stride < samples");
    PM_REQUIRE(!grad_l_aux || first_choice_counts, "planmoe_route_bwd: grad_l_aux needs first_choice_counts");
    if (samples == 0) return 0;
    PM_REQUIRE(scores && indices && grad_gates && grad_scores, "planmoe_route_bwd: NULL argument");
    const int k = top_k < experts ? top_k : experts;
    PM_DTYPE_SWITCH(dtype, DT,
        (route_bwd_kernel<DT><<<(samples + 255) / 256, 256, 0, (hipStream_t)stream>>>(
            scores, indices, grad_gates, plane_stride, samples, experts, k, normalize_gate, grad_l_aux,
            grad_l_aux ? first_choice_counts : nullptr, through_softmax, grad_scores)));
    PM_LAUNCH_CHECK("planmoe_route_bwd");
    return 0;
}

static inline size_t route_tiles(int samples) { return ((size_t)samples + TILE - 1) / TILE; }

extern "C" size_t planmoe_route_workspace_bytes(int samples, int experts, int top_k)
{
    if (samples <= 0 || experts <= 0 || top_k <= 0) return 16;
    const size_t k = (size_t)(top_k < experts ? top_k : experts);
    const size_t tiles = route_tiles(samples);
    // hist[tiles][k][E] + offs[tiles][k][E] + me[tiles][E] + loss_part[E]; up to 64 experts the
    // routing runs on the forward chain's groups and takes that chain's workspace
    const size_t own = round_up((2 * tiles * k * experts + tiles * experts + (size_t)experts) * 4, 256);
    return experts <= 64 ? std::max(own, planmoe_forward_workspace_bytes(samples, experts, top_k)) : own;
}

template <int DT>
static int launch_route_tile(int cap, dim3 grid, size_t lds, hipStream_t st, const void *input,
                             int is_logits, const float *bias, int samples, int experts, int k,
                             int normalize, int32_t *indices, int32_t *locations, void *gates,
                             int64_t stride, void *scores_out, int32_t *hist, float *me)
{
#define PM_ROUTE_LAUNCH(CAP)                                                                  \
    route_tile_kernel<DT, CAP><<<grid, TILE, lds, st>>>(input, is_logits, bias, samples,      \
        experts, k, normalize, indices, locations, gates, stride, scores_out, hist, me)
    if (cap <= 8) PM_ROUTE_LAUNCH(8);
    else if (cap <= 16) PM_ROUTE_LAUNCH(16);
    else if (cap <= 64) PM_ROUTE_LAUNCH(64);
    else PM_ROUTE_LAUNCH(0);
#undef PM_ROUTE_LAUNCH
    return 0;
}

extern "C" int planmoe_route_topk(const void *input, int dtype, int input_is_logits,
                                  const float *logit_bias, int samples, int experts, int top_k,
                                  int normalize_gate, int32_t *indices, int32_t *locations,
                                  void *gates, int64_t plane_stride, void *scores_out, float *l_aux,
                                  int32_t *expert_counts, void *workspace, size_t workspace_bytes,
                                  void *stream)
{
    PM_REQUIRE(dtype == PLANMOE_F32 || dtype == PLANMOE_BF16 || dtype == PLANMOE_F16,
               "planmoe_route_topk: bad dtype %d", dtype);
    PM_REQUIRE(samples >= 0 && experts >= 1 && top_k >= 1, "planmoe_route_topk: bad shape");
    PM_REQUIRE(experts <= ROUTE_MAX_E, "planmoe_route_topk: experts %d > supported %d", experts, ROUTE_MAX_E);
    PM_REQUIRE(plane_stride >= samples, "planmoe_route_topk: plane_stride < samples");
    PM_REQUIRE(!logit_bias || input_is_logits, "planmoe_route_topk: logit_bias needs input_is_logits");
    const int k = top_k < experts ? top_k : experts;
    hipStream_t st = (hipStream_t)stream;
    if (samples == 0) {
        if (expert_counts) fill_u32((uint32_t *)expert_counts, (size_t)k * experts, 0u, st);
        // the loss of an empty batch is 0/0 in the reference; leave l_aux untouched
        return 0;
    }
    PM_REQUIRE(input && indices && locations && gates, "planmoe_route_topk: NULL argument");
    PM_REQUIRE(workspace && workspace_bytes >= planmoe_route_workspace_bytes(samples, experts, top_k),
               "planmoe_route_topk: workspace too small (%zu < %zu)", workspace_bytes,
               planmoe_route_workspace_bytes(samples, experts, top_k));
    if (experts <= 64) {
        // lanes share a token and the experts of a row (softmax and arg-max as butterflies), 64-token
        // groups: several times the parallelism of the thread-per-token tiles below
        if (route_groups(input, dtype, input_is_logits, logit_bias, samples, experts, top_k, normalize_gate, indices,
                         locations, gates, plane_stride, scores_out, l_aux, expert_counts, workspace, st)) return 1;
        PM_LAUNCH_CHECK("planmoe_route_topk");
        return 0;
    }
    const int tiles = (int)route_tiles(samples);
    int32_t *hist = (int32_t *)workspace;
    int32_t *offs = hist + (size_t)tiles * k * experts;
    float *me = (float *)(offs + (size_t)tiles * k * experts);
    float *loss_part = me + (size_t)tiles * experts;
    // TILE_WAVES x experts counters, and for rows held in registers the staging area of half a tile
    const size_t lds = 4 * (TILE_WAVES * (size_t)experts + (experts <= 64 ? (size_t)(TILE / 2) * (experts + 1) : 0));

    PM_DTYPE_SWITCH(dtype, DT,
        launch_route_tile<DT>(experts, dim3(tiles), lds, st, input, input_is_logits, logit_bias,
                              samples, experts, k, normalize_gate, indices, locations, gates,
                              plane_stride, scores_out, hist, l_aux ? me : nullptr));
    const int epb = go_experts_per_block(experts, k);
    const int blocks = (experts + epb - 1) / epb;
    group_offsets_kernel<<<blocks, 256, 0, st>>>(hist, offs, me, tiles, k, experts, epb, samples, nullptr,
                                                 expert_counts, loss_part, l_aux != nullptr);
    route_finish_kernel<<<tiles, TILE, 0, st>>>(indices, locations, plane_stride, samples, experts, k, offs,
                                               loss_part, blocks, l_aux, nullptr);
    PM_LAUNCH_CHECK("planmoe_route_topk");
    return 0;
}

extern "C" int planmoe_route_locations(const int32_t *indices, int64_t plane_stride, int samples,
                                       int experts, int top_k, const int32_t *order,
                                       int32_t *locations, int32_t *expert_counts, void *workspace,
                                       size_t workspace_bytes, void *stream)
{
    PM_REQUIRE(samples >= 0 && experts >= 1 && top_k >= 1, "planmoe_route_locations: bad shape");
    PM_REQUIRE(experts <= ROUTE_MAX_E, "planmoe_route_locations: experts %d > supported %d", experts, ROUTE_MAX_E);
    PM_REQUIRE(plane_stride >= samples, "planmoe_route_locations: plane_stride < samples");
    // the workspace query sizes its tables with min(top_k, experts) planes; the planes given here
    // are used as they are, so more planes than experts would run past it
    PM_REQUIRE(top_k <= experts, "planmoe_route_locations: top_k %d > experts %d", top_k, experts);
    hipStream_t st = (hipStream_t)stream;
    if (samples == 0) {
        if (expert_counts) fill_u32((uint32_t *)expert_counts, (size_t)top_k * experts, 0u, st);
        return 0;
    }
    PM_REQUIRE(indices && locations, "planmoe_route_locations: NULL argument");
    PM_REQUIRE(workspace && workspace_bytes >= planmoe_route_workspace_bytes(samples, experts, top_k),
               "planmoe_route_locations: workspace too small");
    const int k = top_k;
    const int tiles = (int)route_tiles(samples);
    int32_t *hist = (int32_t *)workspace;
    int32_t *offs = hist + (size_t)tiles * k * experts;
    locate_tile_kernel<<<tiles, TILE, sizeof(int32_t) * TILE_WAVES * (size_t)experts, st>>>(
        indices, order, locations, plane_stride, samples, experts, k, hist);
    const int epb = go_experts_per_block(experts, k);
    group_offsets_kernel<<<(experts + epb - 1) / epb, 256, 0, st>>>(hist, offs, nullptr, tiles, k, experts, epb,
                                                                   samples, nullptr, expert_counts, nullptr, 0);
    route_finish_kernel<<<tiles, TILE, 0, st>>>(indices, locations, plane_stride, samples, experts, k, offs,
                                               nullptr, 0, nullptr, order);
    PM_LAUNCH_CHECK("planmoe_route_locations");
    return 0;
}
