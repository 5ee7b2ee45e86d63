// MFMA core of the gate-logits GEMM, shared by the stand-alone and the fused gate kernels.
#pragma once
#include "common.hpp"

namespace pm {

typedef float    f32x4  __attribute__((ext_vector_type(4)));
typedef __bf16   bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8  __attribute__((ext_vector_type(8)));

// One 16-byte vector per lane of each operand -> one 16x16 tile update.
// Lane l carries row (l % 16) of its operand and the k-slice selected by (l / 16); both
// operands use the same k-slice, so any assignment of k values to (l / 16, element) is valid.
template <int DT> struct Mma;

template <> struct Mma<PLANMOE_BF16> {
    __device__ static __forceinline__ void run(const uint4 &a, const uint4 &b, f32x4 &c)
    {
        c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                    __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
};
template <> struct Mma<PLANMOE_F16> {
    __device__ static __forceinline__ void run(const uint4 &a, const uint4 &b, f32x4 &c)
    {
        c = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                   __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
};
template <> struct Mma<PLANMOE_F32> {
    __device__ static __forceinline__ void run(const uint4 &a, const uint4 &b, f32x4 &c)
    {
        c = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(a.x), __uint_as_float(b.x), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(a.y), __uint_as_float(b.y), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(a.z), __uint_as_float(b.z), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_16x16x4f32(__uint_as_float(a.w), __uint_as_float(b.w), c, 0, 0, 0);
    }
};

// Partial logits of tokens [t0, t0 + 16*TPW) against experts [0, 16*NT): wave w accumulates
// the K steps w, w+4, ... and leaves its tiles in part[w][token][expert].
// Requires model_dim % VEC == 0 and 16-byte aligned x / wg.  Call with all 256 threads.
template <int DT, int NT, int TPW>
__device__ __forceinline__ void gate_tile_partials(const void *__restrict__ x,
                                                   const void *__restrict__ wg, int t0, int samples,
                                                   int model_dim, int experts,
                                                   float (*part)[16 * TPW][16 * NT + 1])
{
    constexpr int V = Elem<DT>::VEC;
    const int w = threadIdx.x >> 6, l = lane_id();
    const int m = l & 15, g = l >> 4;
    const int nv = model_dim / V;                    // 16-byte vectors per row
    const int steps = (nv + 15) / 16;
    const int64_t row_vecs = nv;

    const uint4 *arow[TPW];
    const uint4 *brow[NT];
#pragma unroll
    for (int tp = 0; tp < TPW; ++tp) {
        const int t = t0 + tp * 16 + m;
        arow[tp] = t < samples ? reinterpret_cast<const uint4 *>(x) + (int64_t)t * row_vecs : nullptr;
    }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int e = nt * 16 + m;
        brow[nt] = e < experts ? reinterpret_cast<const uint4 *>(wg) + (int64_t)e * row_vecs : nullptr;
    }

    f32x4 acc[TPW][NT];
#pragma unroll
    for (int tp = 0; tp < TPW; ++tp)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[tp][nt] = f32x4{0.f, 0.f, 0.f, 0.f};

    const uint4 zero = make_uint4(0, 0, 0, 0);
    for (int step = w; step < steps; step += 4) {
        const int v0 = step * 16 + g * 4;
        uint4 a[TPW][4], b[NT][4];
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const bool in = v0 + s < nv;
#pragma unroll
            for (int tp = 0; tp < TPW; ++tp) a[tp][s] = (in && arow[tp]) ? arow[tp][v0 + s] : zero;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) b[nt][s] = (in && brow[nt]) ? brow[nt][v0 + s] : zero;
        }
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int tp = 0; tp < TPW; ++tp)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) Mma<DT>::run(a[tp][s], b[nt][s], acc[tp][nt]);
    }

#pragma unroll
    for (int tp = 0; tp < TPW; ++tp)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 4; ++i) part[w][tp * 16 + 4 * g + i][nt * 16 + m] = acc[tp][nt][i];
}

} // namespace pm
