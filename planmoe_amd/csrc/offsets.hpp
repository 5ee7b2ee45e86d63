// Prefix of per-group expert histograms: the step between "rank of a token inside its group"
// and "slot of the token inside its expert".  Shared by the stand-alone routing, the fused
// forward chain and the stand-alone cumsum.
#pragma once
#include "common.hpp"

namespace pm {

// 256 threads = 16 column lanes x 16 row lanes.  A block owns `experts_per_block` experts and
// walks the k choice planes in chunks of (16 / experts_per_block) planes; a column is one
// (plane, expert) pair, the row lanes split the groups.  Every thread loads its rows in batches
// so that the loads of a batch are in flight together.
//   offs[g][j][e] = slots of expert e taken before group g of plane j
//                 = all entries of planes < j  +  entries of groups < g in plane j
//   totals[e]     = sum over all planes and groups (optional)
//   counts_out[j][e] = entries of plane j (optional)
//   loss_part[block] = this block's share of sum_e(me[e] * ce[e]), ce[e] = count0[e] * E / T,
//                      me[e] = sum over groups of me[g][e] (optional, with want_loss)
constexpr int GO_COLS = 16, GO_ROWS = 16, GO_BATCH = 16;

inline int go_experts_per_block(int experts, int k)
{
    int epb = k >= GO_COLS ? 1 : GO_COLS / k;
    return epb > experts ? experts : epb;
}

static __global__ __launch_bounds__(256) void group_offsets_kernel(
    const int32_t *__restrict__ hist, int32_t *__restrict__ offs, const float *__restrict__ me,
    int groups, int k, int experts, int experts_per_block, int samples,
    int32_t *__restrict__ totals, int32_t *__restrict__ counts_out, float *__restrict__ loss_part,
    int want_loss)
{
    __shared__ int32_t s_sum[GO_ROWS][GO_COLS];
    __shared__ int32_t s_tot[GO_COLS];
    __shared__ int32_t s_base[GO_COLS];                 // per expert: entries of the planes done so far
    __shared__ int32_t s_cnt0[GO_COLS];
    __shared__ float s_me[GO_ROWS][GO_COLS];
    const int cl = threadIdx.x % GO_COLS, rl = threadIdx.x / GO_COLS;
    const int e0 = blockIdx.x * experts_per_block;
    const int ne = min(experts_per_block, experts - e0);
    const int planes_per_chunk = GO_COLS / experts_per_block;
    const int jc = cl / experts_per_block, el = cl - jc * experts_per_block;
    const int e = e0 + el;
    const int per = (groups + GO_ROWS - 1) / GO_ROWS;
    const int g0 = min(rl * per, groups), g1 = min(g0 + per, groups);
    if (threadIdx.x < GO_COLS) s_base[threadIdx.x] = 0;

    // column sums of the scores first: their loads overlap those of the histograms
    float mes = 0.f;
    if (want_loss && jc == 0 && el < ne) {
        for (int g = g0; g < g1; g += GO_BATCH) {
            float v[GO_BATCH];
#pragma unroll
            for (int i = 0; i < GO_BATCH; ++i) v[i] = (g + i < g1) ? me[(int64_t)(g + i) * experts + e] : 0.f;
#pragma unroll
            for (int i = 0; i < GO_BATCH; ++i) mes += v[i];
        }
    }

    for (int j0 = 0; j0 < k; j0 += planes_per_chunk) {
        const int j = j0 + jc;
        const bool live = jc < planes_per_chunk && j < k && el < ne;
        int32_t sum = 0;
        int32_t keep[GO_BATCH];                          // first batch stays in registers for pass 2
#pragma unroll
        for (int i = 0; i < GO_BATCH; ++i) keep[i] = 0;
        if (live) {
#pragma unroll
            for (int i = 0; i < GO_BATCH; ++i)
                if (g0 + i < g1) keep[i] = hist[((int64_t)(g0 + i) * k + j) * experts + e];
#pragma unroll
            for (int i = 0; i < GO_BATCH; ++i) sum += keep[i];
            for (int g = g0 + GO_BATCH; g < g1; g += GO_BATCH) {
                int32_t v[GO_BATCH];
#pragma unroll
                for (int i = 0; i < GO_BATCH; ++i)
                    v[i] = (g + i < g1) ? hist[((int64_t)(g + i) * k + j) * experts + e] : 0;
#pragma unroll
                for (int i = 0; i < GO_BATCH; ++i) sum += v[i];
            }
        }
        __syncthreads();                                 // s_base of the previous chunk is final
        s_sum[rl][cl] = sum;
        __syncthreads();
        int32_t before = 0, total = 0;
#pragma unroll
        for (int r = 0; r < GO_ROWS; ++r) {
            const int32_t v = s_sum[r][cl];
            before += (r < rl) ? v : 0;
            total += v;
        }
        if (rl == 0) s_tot[cl] = live ? total : 0;
        __syncthreads();
        int32_t base = s_base[el];                       // planes of earlier chunks
        for (int p = 0; p < jc; ++p) base += s_tot[p * experts_per_block + el];
        if (live) {
            int32_t run = base + before;
#pragma unroll
            for (int i = 0; i < GO_BATCH; ++i) {
                if (g0 + i < g1) offs[((int64_t)(g0 + i) * k + j) * experts + e] = run;
                run += keep[i];
            }
            for (int g = g0 + GO_BATCH; g < g1; g += GO_BATCH) {
                int32_t v[GO_BATCH];
#pragma unroll
                for (int i = 0; i < GO_BATCH; ++i)
                    v[i] = (g + i < g1) ? hist[((int64_t)(g + i) * k + j) * experts + e] : 0;
#pragma unroll
                for (int i = 0; i < GO_BATCH; ++i) {
                    if (g + i < g1) offs[((int64_t)(g + i) * k + j) * experts + e] = run;
                    run += v[i];
                }
            }
            if (rl == 0) {
                if (counts_out) counts_out[j * experts + e] = total;
                if (j == 0) s_cnt0[el] = total;
            }
        }
        __syncthreads();
        if ((int)threadIdx.x < experts_per_block) {
            int32_t add = 0;
            for (int p = 0; p < planes_per_chunk; ++p) add += s_tot[p * experts_per_block + threadIdx.x];
            s_base[threadIdx.x] += add;
        }
    }
    __syncthreads();
    if (totals && (int)threadIdx.x < ne) totals[e0 + threadIdx.x] = s_base[threadIdx.x];

    if (want_loss) {
        s_me[rl][cl] = mes;
        __syncthreads();
        if (threadIdx.x < WAVE) {
            float acc = 0.f;
            if ((int)threadIdx.x < ne) {
                float m = 0.f;
#pragma unroll
                for (int r = 0; r < GO_ROWS; ++r) m += s_me[r][threadIdx.x];
                acc = m * ((float)s_cnt0[threadIdx.x] * ((float)experts / (float)samples));
            }
            acc = wave_sum(acc);
            if (threadIdx.x == 0) loss_part[blockIdx.x] = acc;
        }
    }
}

// l_aux = (sum of the per-block shares) / T, written by one thread of the launch
__device__ __forceinline__ void finish_loss(const float *loss_part, int loss_parts, int samples, float *l_aux)
{
    if (l_aux && blockIdx.x == 0 && threadIdx.x == 0) {
        float a = 0.f;
        for (int b = 0; b < loss_parts; ++b) a += loss_part[b];
        *l_aux = a / (float)samples;
    }
}

} // namespace pm
