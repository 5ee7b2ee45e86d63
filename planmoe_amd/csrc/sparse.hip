// Dispatch / combine / gate-gradient kernels: the token <-> capacity-slot row movers.
//
// They take the place of the three JIT-compiled CUDA kernels of the reference
// (jit_kernels/sparse.py:17-134) and of the per-choice launch loops around them
// (impls/fast_dispatch.py:16-79).  Layout: x / out are [samples, model_dim] rows,
// dispatched is [experts * capacity, model_dim] rows; one wavefront owns one token row and
// moves it with 16-byte accesses, all k choices of the token in the same pass.
#include "rows.hpp"

namespace pm {

// ------------------------------------------------------------------ slot occupancy flags
__global__ __launch_bounds__(256) void slot_flags_clear(uint32_t *flags, int slots)
{
    int i = blockIdx.x * 256 + threadIdx.x;
    if (i < slots) flags[i] = 0u;
}

__global__ __launch_bounds__(256) void slot_flags_mark(uint32_t *flags, const int32_t *indices,
                                                       const int32_t *locations, int64_t stride,
                                                       int top_k, int samples, int experts,
                                                       int capacity)
{
    int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= samples * top_k) return;
    int j = i / samples, t = i - j * samples;
    int64_t o = (int64_t)j * stride + t;
    int e = indices[o], l = locations[o];
    if (e >= 0 && e < experts && l >= 0 && l < capacity) flags[e * capacity + l] = 1u;
}

// ------------------------------------------------------------------ dispatch (scatter rows)
// Blocks [0, token_blocks) move token rows: dispatched[slot] = 0 + gate * x[t].
// Blocks [token_blocks, gridDim.x) write zero rows into the slots no live pair addresses.
template <int DT, bool VECTOR>
__global__ __launch_bounds__(256) void dispatch_kernel(
    const void *__restrict__ x, const float *__restrict__ gates,
    const int32_t *__restrict__ indices, const int32_t *__restrict__ locations, int64_t stride,
    int top_k, int samples, int model_dim, int experts, int capacity,
    void *__restrict__ dispatched, const uint32_t *__restrict__ flags, int token_blocks)
{
    using IO = RowIO<DT, VECTOR>;
    const int wave = threadIdx.x >> 6, lane = lane_id();
    const int units = model_dim / IO::U;
    const int64_t row_bytes = (int64_t)model_dim * sizeof(typename Elem<DT>::store_t);

    if ((int)blockIdx.x >= token_blocks) {
        const int slots = experts * capacity;
        const int nwaves = (gridDim.x - token_blocks) * 4;
        for (int s = (blockIdx.x - token_blocks) * 4 + wave; s < slots; s += nwaves) {
            if (flags[s]) continue;
            char *row = (char *)dispatched + (int64_t)s * row_bytes;
            for (int u = lane; u < units; u += WAVE) IO::store_zero(row, u);
        }
        return;
    }

    const int t = blockIdx.x * 4 + wave;
    if (t >= samples) return;
    const char *src = (const char *)x + (int64_t)t * row_bytes;

    for (int j0 = 0; j0 < top_k; j0 += WAVE) {
        const int np = min(top_k - j0, WAVE);
        int slot; float gate;
        fetch_planes(gates, indices, locations, stride, t, j0, np, experts, capacity, slot, gate);
        if (__ballot(slot >= 0) == 0) continue;          // every choice of this pass dropped: the row is not read
        for (int u = lane; u < units; u += WAVE) {
            float v[IO::U];
            IO::load(src, u, v);
            for (int j = 0; j < np; ++j) {
                const int s = rl_i(slot, j);
                if (s < 0) continue;
                const float g = rl_f(gate, j);
                float o[IO::U];
#pragma unroll
                for (int i = 0; i < IO::U; ++i) o[i] = 0.f + g * v[i];
                IO::store((char *)dispatched + (int64_t)s * row_bytes, u, o);
            }
        }
    }
}

// ------------------------------------------------------------------ combine (gather rows)
// out[t] = sum_j (live_j ? gate_j * dispatched[slot_j] : 0), planes added left to right.
template <int DT, bool VECTOR>
__global__ __launch_bounds__(256) void combine_kernel(
    const void *__restrict__ dispatched, const float *__restrict__ gates,
    const int32_t *__restrict__ indices, const int32_t *__restrict__ locations, int64_t stride,
    int top_k, int samples, int model_dim, int capacity, void *__restrict__ out)
{
    using IO = RowIO<DT, VECTOR>;
    const int wave = threadIdx.x >> 6, lane = lane_id();
    const int units = model_dim / IO::U;
    const int64_t row_bytes = (int64_t)model_dim * sizeof(typename Elem<DT>::store_t);
    const int t = blockIdx.x * 4 + wave;
    if (t >= samples) return;
    char *dst = (char *)out + (int64_t)t * row_bytes;

    if (top_k <= WAVE) {
        int slot; float gate;
        fetch_planes(gates, indices, locations, stride, t, 0, top_k, 0x7fffffff, capacity, slot, gate);
        // four units of a row per lane and pass, fetched with straight-line loads at clamped
        // addresses (a dropped choice reads slot 0 and contributes zeros): four loads in flight
        // per choice instead of one load, one wait
        constexpr int B = 4;
        for (int u0 = lane; u0 < units; u0 += B * WAVE) {
            float acc[B][IO::U];
            for (int j = 0; j < top_k; ++j) {
                const int s = rl_i(slot, j);
                const float g = rl_f(gate, j);
                const char *row = (const char *)dispatched + (int64_t)max(s, 0) * row_bytes;
                float term[B][IO::U];
#pragma unroll
                for (int b = 0; b < B; ++b) IO::load(row, min(u0 + b * WAVE, units - 1), term[b]);
#pragma unroll
                for (int b = 0; b < B; ++b) {
#pragma unroll
                    for (int i = 0; i < IO::U; ++i) {
                        const float v = s >= 0 ? g * term[b][i] : 0.f;
                        acc[b][i] = (j == 0) ? v : acc[b][i] + v;
                    }
                }
            }
#pragma unroll
            for (int b = 0; b < B; ++b)
                if (u0 + b * WAVE < units) IO::store(dst, u0 + b * WAVE, acc[b]);
        }
    } else {
        // more planes than lanes: walk the planes straight from memory
        for (int u = lane; u < units; u += WAVE) {
            float acc[IO::U];
            for (int j = 0; j < top_k; ++j) {
                const int64_t o = (int64_t)j * stride + t;
                const int e = indices[o], l = locations[o];
                const float g = gates ? gates[o] : 1.f;
                float term[IO::U];
                if (e >= 0 && l >= 0 && l < capacity) {
                    IO::load((const char *)dispatched + ((int64_t)e * capacity + l) * row_bytes, u, term);
#pragma unroll
                    for (int i = 0; i < IO::U; ++i) term[i] = g * term[i];
                } else {
#pragma unroll
                    for (int i = 0; i < IO::U; ++i) term[i] = 0.f;
                }
#pragma unroll
                for (int i = 0; i < IO::U; ++i) acc[i] = (j == 0) ? term[i] : acc[i] + term[i];
            }
            IO::store(dst, u, acc);
        }
    }
}

template <int DT, bool VECTOR>
__global__ __launch_bounds__(256) void zero_rows_kernel(void *__restrict__ out, int samples, int model_dim)
{
    using IO = RowIO<DT, VECTOR>;
    const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= samples) return;
    char *dst = (char *)out + (int64_t)t * model_dim * (int64_t)sizeof(typename Elem<DT>::store_t);
    for (int u = lane_id(); u < model_dim / IO::U; u += WAVE) IO::store_zero(dst, u);
}

// ------------------------------------------------------------------ gate gradient
// grad_gates[j][t] = <dispatched[slot_j], x[t]> (0 for a dropped pair).  One wave per token;
// planes are taken four at a time so the token row is read once per group.
template <int DT, bool VECTOR>
__global__ __launch_bounds__(256) void bwd_gate_kernel(
    const void *__restrict__ x, const void *__restrict__ dispatched,
    const int32_t *__restrict__ indices, const int32_t *__restrict__ locations, int64_t stride,
    int top_k, int samples, int model_dim, int capacity, float *__restrict__ grad_gates)
{
    using IO = RowIO<DT, VECTOR>;
    constexpr int G = 4;
    const int wave = threadIdx.x >> 6, lane = lane_id();
    const int units = model_dim / IO::U;
    const int64_t row_bytes = (int64_t)model_dim * sizeof(typename Elem<DT>::store_t);
    const int t = blockIdx.x * 4 + wave;
    if (t >= samples) return;
    const char *xr = (const char *)x + (int64_t)t * row_bytes;

    for (int j0 = 0; j0 < top_k; j0 += G) {
        const int np = min(G, top_k - j0);
        int slot; float gate;
        fetch_planes(nullptr, indices, locations, stride, t, j0, np, 0x7fffffff, capacity, slot, gate);
        int s[G];
#pragma unroll
        for (int j = 0; j < G; ++j) s[j] = (j < np) ? rl_i(slot, j) : -1;
        float acc[G] = {0.f, 0.f, 0.f, 0.f};
        // two units of the row per lane and pass; the slot rows of all choices are requested with
        // straight-line loads at clamped addresses (a dropped choice reads slot 0 and is left out
        // of the sum; the caller guarantees a slot 0 to read: capacity >= 1)
        constexpr int B = 2;
        for (int u0 = lane; u0 < units; u0 += B * WAVE) {
            float a[B][IO::U];
#pragma unroll
            for (int b = 0; b < B; ++b) IO::load_stream(xr, min(u0 + b * WAVE, units - 1), a[b]);
#pragma unroll
            for (int j = 0; j < G; ++j) {
                if (j < np) {
                    const char *row = (const char *)dispatched + (int64_t)max(s[j], 0) * row_bytes;
                    float d[B][IO::U];
#pragma unroll
                    for (int b = 0; b < B; ++b) IO::load_stream(row, min(u0 + b * WAVE, units - 1), d[b]);
#pragma unroll
                    for (int b = 0; b < B; ++b) {
                        const bool live = s[j] >= 0 && u0 + b * WAVE < units;
#pragma unroll
                        for (int i = 0; i < IO::U; ++i) acc[j] = live ? fmaf(d[b][i], a[b][i], acc[j]) : acc[j];
                    }
                }
            }
        }
#pragma unroll
        for (int j = 0; j < G; ++j) {
            if (j >= np) break;
            const float r = wave_sum(acc[j]);
            if (lane == 0) grad_gates[(int64_t)(j0 + j) * stride + t] = r;
        }
    }
}

void launch_slot_flags(uint32_t *flags, const int32_t *indices, const int32_t *locations,
                       int64_t stride, int top_k, int samples, int experts, int capacity,
                       hipStream_t st)
{
    const int slots = experts * capacity;
    slot_flags_clear<<<(slots + 255) / 256, 256, 0, st>>>(flags, slots);
    if (samples > 0)
        slot_flags_mark<<<(samples * top_k + 255) / 256, 256, 0, st>>>(flags, indices, locations, stride,
                                                                      top_k, samples, experts, capacity);
}

int check_planes(const char *who, const int32_t *indices, const int32_t *locations,
                        int64_t stride, int top_k, int samples)
{
    PM_REQUIRE(indices && locations, "%s: indices/locations must not be NULL", who);
    PM_REQUIRE(top_k >= 1, "%s: top_k must be >= 1 (got %d)", who, top_k);
    PM_REQUIRE(samples >= 0, "%s: samples must be >= 0", who);
    PM_REQUIRE(stride >= samples, "%s: plane_stride %lld < samples %d", who, (long long)stride, samples);
    return 0;
}

} // namespace pm

using namespace pm;

extern "C" size_t planmoe_dispatch_workspace_bytes(int experts, int capacity)
{
    if (experts <= 0 || capacity <= 0) return 16;
    return round_up((size_t)experts * (size_t)capacity * sizeof(uint32_t), 256);
}

extern "C" int planmoe_dispatch_fwd(const void *x, int dtype, const float *gates,
                                    const int32_t *indices, const int32_t *locations,
                                    int64_t plane_stride, int top_k, int samples, int model_dim,
                                    int experts, int capacity, void *dispatched, void *workspace,
                                    size_t workspace_bytes, void *stream)
{
    if (check_planes("planmoe_dispatch_fwd", indices, locations, plane_stride, top_k, samples)) return 1;
    PM_REQUIRE(dtype_ok(dtype), "planmoe_dispatch_fwd: bad dtype %d", dtype);
    PM_REQUIRE(model_dim >= 1 && experts >= 1 && capacity >= 0, "planmoe_dispatch_fwd: bad shape");
    PM_REQUIRE((int64_t)experts * capacity < (1ll << 31), "planmoe_dispatch_fwd: experts*capacity overflows int32");
    PM_REQUIRE((int64_t)samples * top_k < (1ll << 31), "planmoe_dispatch_fwd: samples*top_k overflows int32");
    const int slots = experts * capacity;
    if (slots == 0) return 0;
    PM_REQUIRE(x || samples == 0, "planmoe_dispatch_fwd: x is NULL");
    PM_REQUIRE(dispatched, "planmoe_dispatch_fwd: dispatched is NULL");
    PM_REQUIRE(workspace && workspace_bytes >= planmoe_dispatch_workspace_bytes(experts, capacity),
               "planmoe_dispatch_fwd: workspace too small (%zu < %zu)", workspace_bytes,
               planmoe_dispatch_workspace_bytes(experts, capacity));
    hipStream_t st = (hipStream_t)stream;
    uint32_t *flags = (uint32_t *)workspace;

    launch_slot_flags(flags, indices, locations, plane_stride, top_k, samples, experts, capacity, st);
    const int token_blocks = (samples + 3) / 4;
    const int fill_blocks = min((slots + 3) / 4, 2048);
    const int vec = dtype == PLANMOE_F32 ? 4 : 8;
    const bool vector = (model_dim % vec == 0) && aligned16(x) && aligned16(dispatched);
    PM_DTYPE_SWITCH(dtype, DT, {
        if (vector)
            dispatch_kernel<DT, true><<<token_blocks + fill_blocks, 256, 0, st>>>(
                x, gates, indices, locations, plane_stride, top_k, samples, model_dim, experts,
                capacity, dispatched, flags, token_blocks);
        else
            dispatch_kernel<DT, false><<<token_blocks + fill_blocks, 256, 0, st>>>(
                x, gates, indices, locations, plane_stride, top_k, samples, model_dim, experts,
                capacity, dispatched, flags, token_blocks);
    });
    PM_LAUNCH_CHECK("planmoe_dispatch_fwd");
    return 0;
}

extern "C" int planmoe_combine_fwd(const void *dispatched, int dtype, const float *gates,
                                   const int32_t *indices, const int32_t *locations,
                                   int64_t plane_stride, int top_k, int samples, int model_dim,
                                   int capacity, void *out, void *stream)
{
    if (check_planes("planmoe_combine_fwd", indices, locations, plane_stride, top_k, samples)) return 1;
    PM_REQUIRE(dtype_ok(dtype), "planmoe_combine_fwd: bad dtype %d", dtype);
    PM_REQUIRE(model_dim >= 1 && capacity >= 0, "planmoe_combine_fwd: bad shape");
    if (samples == 0) return 0;
    PM_REQUIRE(out, "planmoe_combine_fwd: out is NULL");
    PM_REQUIRE(dispatched || capacity == 0, "planmoe_combine_fwd: dispatched is NULL");
    hipStream_t st = (hipStream_t)stream;
    const int vec = dtype == PLANMOE_F32 ? 4 : 8;
    const bool vector = (model_dim % vec == 0) && aligned16(out) && aligned16(dispatched);
    const int blocks = (samples + 3) / 4;
    if (capacity == 0) {
        // no slot exists, every choice is dropped: zero rows.  (combine_kernel fetches rows with
        // unconditional loads at clamped slots and must not run without a row to read.)
        PM_DTYPE_SWITCH(dtype, DT, {
            if (vector) zero_rows_kernel<DT, true><<<blocks, 256, 0, st>>>(out, samples, model_dim);
            else zero_rows_kernel<DT, false><<<blocks, 256, 0, st>>>(out, samples, model_dim);
        });
        PM_LAUNCH_CHECK("planmoe_combine_fwd");
        return 0;
    }
    PM_DTYPE_SWITCH(dtype, DT, {
        if (vector)
            combine_kernel<DT, true><<<blocks, 256, 0, st>>>(dispatched, gates, indices, locations,
                                                            plane_stride, top_k, samples, model_dim,
                                                            capacity, out);
        else
            combine_kernel<DT, false><<<blocks, 256, 0, st>>>(dispatched, gates, indices, locations,
                                                             plane_stride, top_k, samples, model_dim,
                                                             capacity, out);
    });
    PM_LAUNCH_CHECK("planmoe_combine_fwd");
    return 0;
}

extern "C" int planmoe_bwd_gate(const void *x, const void *dispatched, int dtype,
                                const int32_t *indices, const int32_t *locations,
                                int64_t plane_stride, int top_k, int samples, int model_dim,
                                int capacity, float *grad_gates, void *stream)
{
    if (check_planes("planmoe_bwd_gate", indices, locations, plane_stride, top_k, samples)) return 1;
    PM_REQUIRE(dtype_ok(dtype), "planmoe_bwd_gate: bad dtype %d", dtype);
    PM_REQUIRE(model_dim >= 1 && capacity >= 0, "planmoe_bwd_gate: bad shape");
    if (samples == 0) return 0;
    PM_REQUIRE(x && grad_gates, "planmoe_bwd_gate: NULL argument");
    PM_REQUIRE(dispatched || capacity == 0, "planmoe_bwd_gate: dispatched is NULL");
    hipStream_t st = (hipStream_t)stream;
    if (capacity == 0) {                               // no slot, no row to read: every gradient is zero
        for (int j = 0; j < top_k; ++j) fill_u32((uint32_t *)(grad_gates + (int64_t)j * plane_stride), (size_t)samples, 0u, st);
        PM_LAUNCH_CHECK("planmoe_bwd_gate");
        return 0;
    }
    const int vec = dtype == PLANMOE_F32 ? 4 : 8;
    const bool vector = (model_dim % vec == 0) && aligned16(x) && aligned16(dispatched);
    const int blocks = (samples + 3) / 4;
    PM_DTYPE_SWITCH(dtype, DT, {
        if (vector)
            bwd_gate_kernel<DT, true><<<blocks, 256, 0, st>>>(x, dispatched, indices, locations,
                                                             plane_stride, top_k, samples,
                                                             model_dim, capacity, grad_gates);
        else
            bwd_gate_kernel<DT, false><<<blocks, 256, 0, st>>>(x, dispatched, indices, locations,
                                                              plane_stride, top_k, samples,
                                                              model_dim, capacity, grad_gates);
    });
    PM_LAUNCH_CHECK("planmoe_bwd_gate");
    return 0;
}
