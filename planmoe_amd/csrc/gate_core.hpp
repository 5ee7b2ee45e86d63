// MFMA core of the gate-logits GEMM, shared by the stand-alone and the fused gate kernels.
#pragma once
#include "common.hpp"
#include "int8_core.hpp"

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

template <int NT, int TPW>
struct GateFrag {
    uint4 a[TPW][4];
    uint4 b[NT][4];
};

// Partial logits of tokens [t0, t0 + 16*TPW) against experts [0, 16*NT): wave w of the NW waves
// of the work-group accumulates the K steps w, w+NW, ... (a step is 16 vectors = 256 bytes of
// every row) and leaves its tiles in part[w][token][expert].  Rows past the end of x / wg are clamped to the last valid
// row: their products land in tile entries nobody reads.  Loads of the next step are issued
// before the MFMAs of the current one.
// With STATS (bf16 only) the wave also keeps the running min / max / NaN scan of every token row
// it streams (the VALU is idle while the loads are in flight) and leaves, per wave, the three
// 32-bit words of RowStats<bf16>::reduced() in pstat[w][token][0..2].
// Requires model_dim % VEC == 0 and 16-byte aligned x / wg.  Call with all 64*NW threads.
template <int DT, int NT, int TPW, int NW = 4, bool STATS = false>
__device__ __forceinline__ void gate_tile_partials(const void *__restrict__ x,
                                                   const void *__restrict__ wg, int t0, int samples,
                                                   int model_dim, int experts,
                                                   float (*part)[16 * TPW][16 * NT + 1],
                                                   int32_t (*pstat)[16 * TPW][3] = nullptr)
{
    static_assert(!STATS || DT == PLANMOE_BF16, "row statistics ride along for bf16 only");
    RowStats<PLANMOE_BF16, true> st[TPW];
    if constexpr (STATS) {
#pragma unroll
        for (int tp = 0; tp < TPW; ++tp) st[tp].init();
    }
    constexpr int V = Elem<DT>::VEC;
    const int w = threadIdx.x >> 6, l = lane_id();
    const int m = l & 15, g = l >> 4;
    const int nv = model_dim / V;                    // 16-byte vectors per row
    const int full = nv / 16, rem = nv % 16;

    const uint4 *ap[TPW];
    const uint4 *bp[NT];
    bool bv[NT];                                     // lane holds a real gate-weight row
#pragma unroll
    for (int tp = 0; tp < TPW; ++tp)
        ap[tp] = reinterpret_cast<const uint4 *>(x) + (int64_t)min(t0 + tp * 16 + m, samples - 1) * nv + g * 4;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
    {
        bv[nt] = nt * 16 + m < experts;
        bp[nt] = reinterpret_cast<const uint4 *>(wg) + (int64_t)min(nt * 16 + m, experts - 1) * nv + g * 4;
    }

    f32x4 acc[TPW][NT];
#pragma unroll
    for (int tp = 0; tp < TPW; ++tp)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[tp][nt] = f32x4{0.f, 0.f, 0.f, 0.f};

    auto load = [&](GateFrag<NT, TPW> &f, int step) {
        const int o = step * 16;
#pragma unroll
        for (int tp = 0; tp < TPW; ++tp)
#pragma unroll
            for (int s = 0; s < 4; ++s) f.a[tp][s] = ap[tp][o + s];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            // lanes past the last expert skip the load: whatever their registers hold only
            // reaches tile columns nobody reads
            if (bv[nt]) {
#pragma unroll
                for (int s = 0; s < 4; ++s) f.b[nt][s] = bp[nt][o + s];
            }
        }
    };
    auto mma = [&](const GateFrag<NT, TPW> &f) {
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int tp = 0; tp < TPW; ++tp) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) Mma<DT>::run(f.a[tp][s], f.b[nt][s], acc[tp][nt]);
                if constexpr (STATS) st[tp].add(f.a[tp][s]);
            }
    };

    GateFrag<NT, TPW> f0, f1;
    int step = w;
    if (step < full) load(f0, step);
    while (step < full) {
        const bool more1 = step + NW < full;
        if (more1) load(f1, step + NW);
        mma(f0);
        if (!more1) break;
        const bool more2 = step + 2 * NW < full;
        if (more2) load(f0, step + 2 * NW);
        mma(f1);
        step += 2 * NW;
        if (!more2) break;
    }

    if (rem && (full % NW) == w) {
        // last, partial step: vectors past the row end are read from a clamped index and zeroed
        GateFrag<NT, TPW> f;
        const int o = full * 16;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const bool in = g * 4 + s < rem;
            const int off = in ? o + s : o - g * 4;   // out of range: re-read vector `o` of the row, then zero it
#pragma unroll
            for (int tp = 0; tp < TPW; ++tp) {
                uint4 v = ap[tp][off];
                f.a[tp][s] = in ? v : make_uint4(0, 0, 0, 0);
                // vector `o` read again in place of a vector past the row end: harmless for min / max
                if constexpr (STATS) st[tp].add(v);
            }
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                uint4 v = bp[nt][off];
                f.b[nt][s] = in ? v : make_uint4(0, 0, 0, 0);
            }
        }
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int tp = 0; tp < TPW; ++tp)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) Mma<DT>::run(f.a[tp][s], f.b[nt][s], acc[tp][nt]);
    }

    if constexpr (STATS) {
        // the 4 lanes (l % 16 == m) of a row hold its k-slices: combine them, lane g == 0 writes
#pragma unroll
        for (int tp = 0; tp < TPW; ++tp) {
            int a, b, n;
            st[tp].reduced(a, b, n);
#pragma unroll
            for (int off = 16; off < 64; off <<= 1) {
                a = min(a, __shfl_xor(a, off, WAVE));
                b = max(b, __shfl_xor(b, off, WAVE));
                n = max(n, __shfl_xor(n, off, WAVE));
            }
            if (g == 0) { pstat[w][tp * 16 + m][0] = a; pstat[w][tp * 16 + m][1] = b; pstat[w][tp * 16 + m][2] = n; }
        }
    }

#pragma unroll
    for (int tp = 0; tp < TPW; ++tp)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int i = 0; i < 4; ++i) part[w][tp * 16 + 4 * g + i][nt * 16 + m] = acc[tp][nt][i];
}

} // namespace pm
