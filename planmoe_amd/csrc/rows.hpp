// Row access helpers shared by the kernels that move token rows to and from capacity slots.
#pragma once
#include "common.hpp"

namespace pm {

template <int DT, bool VECTOR>
struct RowIO {
    using E = Elem<DT>;
    static constexpr int U = VECTOR ? E::VEC : 1;      // elements per lane access
    __device__ static __forceinline__ void load(const void *row, int unit, float *f)
    {
        if constexpr (VECTOR) E::unpack(reinterpret_cast<const uint4 *>(row)[unit], f);
        else f[0] = E::load(row, unit);
    }
    // for launches that store nothing in bulk (measured: streaming loads next to streaming
    // stores slow the dispatch / combine kernels down, alone they help)
    __device__ static __forceinline__ void load_stream(const void *row, int unit, float *f)
    {
        if constexpr (VECTOR) E::unpack(stream_load(reinterpret_cast<const uint4 *>(row) + unit), f);
        else f[0] = E::load(row, unit);
    }
    __device__ static __forceinline__ void store(void *row, int unit, const float *f)
    {
        if constexpr (VECTOR) stream_store(reinterpret_cast<uint4 *>(row) + unit, E::pack(f));
        else E::store(row, unit, f[0]);
    }
    __device__ static __forceinline__ void store_zero(void *row, int unit)
    {
        if constexpr (VECTOR) stream_store(reinterpret_cast<uint4 *>(row) + unit, make_uint4(0, 0, 0, 0));
        else E::store(row, unit, 0.f);
    }
};

__device__ __forceinline__ int   rl_i(int v, int lane)   { return __builtin_amdgcn_readlane(v, lane); }
__device__ __forceinline__ float rl_f(float v, int lane) { return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane)); }

// Lane j (< nplanes) of the calling wave fetches plane j0+j of token t: its slot row
// (-1 when the pair is not live) and its gate.
__device__ __forceinline__ void fetch_planes(const float *gates, const int32_t *indices,
                                             const int32_t *locations, int64_t stride, int t,
                                             int j0, int nplanes, int experts, int capacity,
                                             int &slot, float &gate)
{
    slot = -1; gate = 1.f;
    const int lane = lane_id();
    if (lane < nplanes) {
        const int64_t o = (int64_t)(j0 + lane) * stride + t;
        const int e = indices[o], l = locations[o];
        if (e >= 0 && e < experts && l >= 0 && l < capacity) slot = e * capacity + l;
        if (gates) gate = gates[o];
    }
}

// occupancy flags of the experts*capacity slots (1 = some live pair addresses the slot)
void launch_slot_flags(uint32_t *flags, const int32_t *indices, const int32_t *locations,
                       int64_t stride, int top_k, int samples, int experts, int capacity,
                       hipStream_t st);
int check_planes(const char *who, const int32_t *indices, const int32_t *locations,
                 int64_t stride, int top_k, int samples);
// routing of up to 64 experts from [samples, experts] logits / scores with the forward chain's
// epilogue; workspace of planmoe_forward_workspace_bytes(samples, experts, top_k)
int route_groups(const void *input, int dtype, int is_logits, const float *logit_bias, int samples, int experts,
                 int top_k, int normalize_gate, int32_t *indices, int32_t *locations, void *gates, int64_t stride,
                 void *scores_out, float *l_aux, int32_t *counts, void *workspace, hipStream_t st);

} // namespace pm
