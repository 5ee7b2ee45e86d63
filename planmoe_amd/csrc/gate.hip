// Gate logits: logits[T, E] = x[T, M] . wg[E, M]^T  (gates/top.py:20-26).
//
// The GEMM is skinny (E is 2..128) and bound by reading x once from HBM; the matrix cores
// (MFMA 16x16 tiles, fp32 accumulation) keep the arithmetic off the critical path.
// Up to 16 experts: a work-group of 4 waves owns 16*TPW tokens; the K axis is dealt to the 4
// waves in 16-vector steps (round robin, so the group streams 1 KB of every token row at a
// time) and the 4 partial tiles meet in LDS, summed in a fixed order.  Both MFMA operands use
// the same lane -> k mapping.  17..128 experts: the gate weights are staged through LDS once per
// work-group of 64 tokens and every wave runs the whole K axis for its 16 tokens.
#include "gate_core.hpp"

namespace pm {

template <int DT, int NT, int TPW, int NW>
__global__ __launch_bounds__(64 * NW) void gate_logits_kernel(
    const void *__restrict__ x, const void *__restrict__ wg, void *__restrict__ logits, int out_dt,
    int samples, int model_dim, int experts)
{
    __shared__ float part[NW][16 * TPW][16 * NT + 1];
    const int t0 = blockIdx.x * 16 * TPW;
    gate_tile_partials<DT, NT, TPW, NW>(x, wg, t0, samples, model_dim, experts, part);
    __syncthreads();
    for (int i = threadIdx.x; i < 16 * TPW * experts; i += 64 * NW) {
        const int r = i / experts, e = i - r * experts;
        const int t = t0 + r;
        if (t >= samples) continue;
        float v = part[0][r][e];
#pragma unroll
        for (int w = 1; w < NW; ++w) v += part[w][r][e];
        const int64_t o = (int64_t)t * experts + e;
        if (out_dt == PLANMOE_F32) ((float *)logits)[o] = v;
        else if (out_dt == PLANMOE_BF16) ((uint16_t *)logits)[o] = (uint16_t)f32_to_bf16(v);
        else ((uint16_t *)logits)[o] = (uint16_t)f32_to_f16(v);
    }
}

// more than 16 experts: gate weights shared through LDS, 64 tokens per work-group
template <int DT, int NT>
__global__ __launch_bounds__(256) void gate_logits_lds_kernel(
    const void *__restrict__ x, const void *__restrict__ wg, void *__restrict__ logits, int out_dt,
    int samples, int model_dim, int experts)
{
    __shared__ uint4 smem[gate_lds_vectors<NT>()];
    const int t0 = blockIdx.x * 64;
    gate_tile_lds<DT, NT>(x, wg, t0, samples, model_dim, experts, smem);
    __syncthreads();
    const float (*tile)[16 * NT + 1] = reinterpret_cast<const float (*)[16 * NT + 1]>(smem);
    const int rows = min(64, samples - t0);
    for (int i = threadIdx.x; i < rows * experts; i += 256) {
        const int r = i / experts, e = i - r * experts;
        const float v = tile[r][e];
        const int64_t o = (int64_t)t0 * experts + i;
        if (out_dt == PLANMOE_F32) ((float *)logits)[o] = v;
        else if (out_dt == PLANMOE_BF16) ((uint16_t *)logits)[o] = (uint16_t)f32_to_bf16(v);
        else ((uint16_t *)logits)[o] = (uint16_t)f32_to_f16(v);
    }
}

// any shape / alignment: one thread per logit
template <int DT>
__global__ __launch_bounds__(256) void gate_logits_naive_kernel(
    const void *__restrict__ x, const void *__restrict__ wg, void *__restrict__ logits, int out_dt,
    int samples, int model_dim, int experts)
{
    using E = Elem<DT>;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= (int64_t)samples * experts) return;
    const int64_t t = i / experts; const int e = (int)(i - t * experts);
    float acc = 0.f;
    for (int m = 0; m < model_dim; ++m)
        acc = fmaf(E::load(x, t * model_dim + m), E::load(wg, (int64_t)e * model_dim + m), acc);
    if (out_dt == PLANMOE_F32) ((float *)logits)[i] = acc;
    else if (out_dt == PLANMOE_BF16) ((uint16_t *)logits)[i] = (uint16_t)f32_to_bf16(acc);
    else ((uint16_t *)logits)[i] = (uint16_t)f32_to_f16(acc);
}

template <int DT>
static void launch_gate_logits(const void *x, const void *wg, void *logits, int out_dt, int samples,
                               int model_dim, int experts, bool mfma, hipStream_t st)
{
    if (!mfma) {
        const int64_t n = (int64_t)samples * experts;
        gate_logits_naive_kernel<DT><<<(unsigned)((n + 255) / 256), 256, 0, st>>>(x, wg, logits, out_dt,
                                                                                 samples, model_dim, experts);
        return;
    }
#define PM_GATE(NT, TPW, NW)                                                                      \
    gate_logits_kernel<DT, NT, TPW, NW><<<(samples + 16 * TPW - 1) / (16 * TPW), 64 * NW, 0, st>>>(  \
        x, wg, logits, out_dt, samples, model_dim, experts)
#define PM_GATE_LDS(NT)                                                                           \
    gate_logits_lds_kernel<DT, NT><<<(samples + 63) / 64, 256, 0, st>>>(x, wg, logits, out_dt, samples, \
                                                                        model_dim, experts)
    if (experts <= 16) PM_GATE(1, 4, 4);
    else if (experts <= 32) PM_GATE_LDS(2);
    else if (experts <= 64) PM_GATE_LDS(4);
    else PM_GATE_LDS(8);
#undef PM_GATE_LDS
#undef PM_GATE
}

// dx[t, :] += sum_e g[t, e] * wg[e, :] -- the gate's share of the gradient of x (the backward of
// logits = x wg^T) added onto the gradient that came through the dispatched rows.  With a handful of
// experts (up to 8: measured 64 -> 48 us at 16384 x 4096 x 8 bf16; at 16 a library GEMM wins) this
// is a streaming read-modify-write of dx, not a GEMM worth a library call: a lane owns
// one 16-byte unit of columns and keeps the EP weight rows of those columns in registers, a work-group
// owns 256 units and walks a chunk of the token rows.  g is rounded to dx's dtype first (as the cast
// before a library GEMM would), products and the sum are fp32, one rounding at the end.
template <int DT, int EP>
__global__ __launch_bounds__(256) void gate_dx_accumulate_kernel(void *__restrict__ dx, const float *__restrict__ g,
                                                                const void *__restrict__ wg, int samples,
                                                                int model_dim, int experts, int rows_per_block)
{
    using E = Elem<DT>;
    constexpr int V = E::VEC;
    const int units = model_dim / V;
    const int u = blockIdx.x * 256 + threadIdx.x;
    const int uc = min(u, units - 1);                               // clamped: straight-line loads; stores are guarded
    float w[EP][V];
#pragma unroll
    for (int e = 0; e < EP; ++e) {
        if (e < experts) {
            E::unpack(reinterpret_cast<const uint4 *>((const char *)wg + (int64_t)e * model_dim * sizeof(typename E::store_t))[uc], w[e]);
        } else {
#pragma unroll
            for (int i = 0; i < V; ++i) w[e][i] = 0.f;
        }
    }
    const int t0 = blockIdx.y * rows_per_block, t1 = min(t0 + rows_per_block, samples);
    constexpr int R = 4;                                            // rows in flight per thread
    const int64_t row_bytes = (int64_t)model_dim * sizeof(typename E::store_t);
    for (int tb = t0; tb < t1; tb += R) {
        uint4 raw[R];
#pragma unroll
        for (int r = 0; r < R; ++r)                                 // clamped rows: straight-line loads
            raw[r] = reinterpret_cast<const uint4 *>((const char *)dx + (int64_t)min(tb + r, t1 - 1) * row_bytes)[uc];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int t = min(tb + r, t1 - 1);
            float acc[V];
            E::unpack(raw[r], acc);
#pragma unroll
            for (int e = 0; e < EP; ++e) {
                const float ge = e < experts ? E::round(g[(int64_t)t * experts + e]) : 0.f;   // uniform: scalar loads
#pragma unroll
                for (int i = 0; i < V; ++i) acc[i] = fmaf(ge, w[e][i], acc[i]);
            }
            if (u < units && tb + r < t1)
                reinterpret_cast<uint4 *>((char *)dx + (int64_t)t * row_bytes)[u] = E::pack(acc);
        }
    }
}

} // namespace pm

using namespace pm;

extern "C" int planmoe_gate_dx_accumulate(void *dx, int dtype, const float *grad_logits, const void *wg,
                                          int samples, int model_dim, int experts, void *stream)
{
    const char *who = "planmoe_gate_dx_accumulate";
    PM_REQUIRE(dtype_ok(dtype), "%s: bad dtype %d", who, dtype);
    PM_REQUIRE(samples >= 0 && model_dim >= 1, "%s: bad shape", who);
    PM_REQUIRE(experts >= 1 && experts <= 8, "%s: built for up to 8 experts (got %d); a GEMM is faster above that", who, experts);
    const int vec = dtype == PLANMOE_F32 ? 4 : 8;
    PM_REQUIRE(model_dim % vec == 0, "%s: model_dim must be a multiple of %d", who, vec);
    if (samples == 0) return 0;
    PM_REQUIRE(dx && grad_logits && wg && aligned16(dx) && aligned16(wg), "%s: NULL or unaligned argument", who);
    const int units = model_dim / vec;
    const unsigned gx = (unsigned)((units + 255) / 256);
    // enough work-groups to fill the GPU, rows in chunks of at least 16
    int rows_per_block = (int)(((int64_t)samples * gx + 2047) / 2048);
    if (rows_per_block < 16) rows_per_block = 16;
    const unsigned gy = (unsigned)((samples + rows_per_block - 1) / rows_per_block);
    PM_REQUIRE(gy < 65536u, "%s: too many row chunks", who);
    const dim3 grid(gx, gy);
    hipStream_t st = (hipStream_t)stream;
#define PM_GDX(EP) PM_DTYPE_SWITCH(dtype, DT, (gate_dx_accumulate_kernel<DT, EP><<<grid, 256, 0, st>>>( \
        dx, grad_logits, wg, samples, model_dim, experts, rows_per_block)))
    if (experts <= 2) { PM_GDX(2); }
    else if (experts <= 4) { PM_GDX(4); }
    else { PM_GDX(8); }
#undef PM_GDX
    PM_LAUNCH_CHECK(who);
    return 0;
}

extern "C" int planmoe_gate_logits(const void *x, const void *wg, int dtype, void *logits,
                                   int out_dtype, int samples, int model_dim, int experts,
                                   void *stream)
{
    PM_REQUIRE(dtype_ok(dtype) && dtype_ok(out_dtype), "planmoe_gate_logits: bad dtype");
    PM_REQUIRE(out_dtype == PLANMOE_F32 || out_dtype == dtype,
               "planmoe_gate_logits: out_dtype must be F32 or the input dtype");
    PM_REQUIRE(samples >= 0 && model_dim >= 1 && experts >= 1, "planmoe_gate_logits: bad shape");
    if (samples == 0) return 0;
    PM_REQUIRE(x && wg && logits, "planmoe_gate_logits: NULL argument");
    const int vec = dtype == PLANMOE_F32 ? 4 : 8;
    const bool mfma = experts <= 128 && model_dim % vec == 0 && aligned16(x) && aligned16(wg);
    PM_DTYPE_SWITCH(dtype, DT, launch_gate_logits<DT>(x, wg, logits, out_dtype, samples, model_dim,
                                                      experts, mfma, (hipStream_t)stream));
    PM_LAUNCH_CHECK("planmoe_gate_logits");
    return 0;
}
