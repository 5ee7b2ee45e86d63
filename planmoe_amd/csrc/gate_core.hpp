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
// Here vector s of lane (m, g) is vector 4 s + g of the step: the four lanes of a row read 64
// contiguous bytes with one load instruction, which keeps the number of cache lines an
// instruction touches at 16.
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
#pragma unroll
    for (int tp = 0; tp < TPW; ++tp)
        ap[tp] = reinterpret_cast<const uint4 *>(x) + (int64_t)min(t0 + tp * 16 + m, samples - 1) * nv + g;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
        bp[nt] = reinterpret_cast<const uint4 *>(wg) + (int64_t)min(nt * 16 + m, experts - 1) * nv + g;

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
            for (int s = 0; s < 4; ++s) f.a[tp][s] = ap[tp][o + s * 4];
        // lanes past the last expert re-read the last gate-weight row (clamped above): their
        // products only reach tile columns nobody reads.  No predicate here, and no branch around
        // a prefetch below: the compiler counts outstanding loads per basic block, and a load
        // that may or may not have been issued makes it wait for everything.
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
            for (int s = 0; s < 4; ++s) f.b[nt][s] = bp[nt][o + s * 4];
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
    if (w < full) {
        const int nsteps = (full - w + NW - 1) / NW;     // steps of this wave: w, w + NW, ...
        const int last = w + (nsteps - 1) * NW;
        int step = w;
        if (nsteps & 1) { load(f0, step); mma(f0); step += NW; }
        if (step <= last) {
            // pairs of steps, one straight-line body: each buffer is re-filled while the MFMAs of
            // the other run.  The last prefetch re-reads the wave's last step (a cache hit).
            load(f0, step);
            for (; step <= last; step += 2 * NW) {
                load(f1, step + NW);
                mma(f0);
                load(f0, min(step + 2 * NW, last));
                mma(f1);
            }
        }
    }

    if (rem && (full % NW) == w) {
        // last, partial step: vectors past the row end are read from a clamped index and zeroed
        GateFrag<NT, TPW> f;
        const int o = full * 16;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const bool in = s * 4 + g < rem;
            const int off = in ? o + s * 4 : o - g;   // out of range: re-read vector `o` of the row, then zero it
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

// ---------------------------------------------------------------------------------------------
// Variant for more than 16 experts: the gate weights are the larger operand per token tile, so
// the work-group shares them through LDS instead of every wave streaming them from L2.
//   * a work-group of 4 waves owns 64 tokens, wave w the tokens [16 w, 16 w + 16) over the
//     whole K axis (no split-K: the accumulators of a token stay in one wave);
//   * K is walked in chunks of 16 vectors (256 bytes of every row).  The chunk of all 16*NT
//     gate-weight rows is copied global -> registers -> LDS by the 256 threads with fully
//     coalesced 16-byte loads, double buffered, one barrier per chunk;
//   * inside LDS a row's 16 vectors are stored at (vector ^ (row % 16)): the 16 lanes of an
//     MFMA fragment read (different rows, same logical vector) hit 16 different vector slots,
//     i.e. all 64 banks once;
//   * token fragments go straight from global memory to registers, one chunk ahead.
// Result: logits[token][expert] (fp32) in LDS.  `smem` must hold gate_lds_vectors<NT>() uint4;
// the logits alias the weight buffers (a barrier separates the two uses).
// With STATS the wave leaves the words of RowStats<bf16>::reduced() of its rows in pstat[token].
template <int NT> __host__ __device__ constexpr int gate_lds_vectors()
{
    // 2 buffers x (16 NT rows x 16 vectors)  vs  64 x (16 NT + 1) floats
    return (2 * 16 * NT * 16) > ((64 * (16 * NT + 1) + 3) / 4) ? (2 * 16 * NT * 16) : ((64 * (16 * NT + 1) + 3) / 4);
}

template <int DT, int NT, bool STATS = false>
__device__ __forceinline__ void gate_tile_lds(const void *__restrict__ x, const void *__restrict__ wg,
                                              int t0, int samples, int model_dim, int experts,
                                              uint4 *smem, int32_t (*pstat)[3] = nullptr)
{
    static_assert(!STATS || DT == PLANMOE_BF16, "row statistics ride along for bf16 only");
    static_assert(NT == 1 || NT == 2 || NT == 4 || NT == 8, "16 NT rows are dealt to 256 threads, 16 per row");
    constexpr int V = Elem<DT>::VEC;
    constexpr int ROWS = 16 * NT;
    constexpr int BV = ROWS / 16;                    // weight vectors per thread and chunk
    const int tid = threadIdx.x, w = tid >> 6, l = lane_id();
    const int m = l & 15, g = l >> 4;
    const int nv = model_dim / V;                    // 16-byte vectors per row

    RowStats<PLANMOE_BF16, true> st;
    if constexpr (STATS) st.init();

    const uint4 *ap = reinterpret_cast<const uint4 *>(x) + (int64_t)min(t0 + w * 16 + m, samples - 1) * nv;
    const int bvec = tid & 15;                       // thread's vector inside the chunk
    const uint4 *bp[BV];
    int bdst[BV];
#pragma unroll
    for (int i = 0; i < BV; ++i) {
        const int row = i * 16 + (tid >> 4);
        bp[i] = reinterpret_cast<const uint4 *>(wg) + (int64_t)min(row, experts - 1) * nv + bvec;
        bdst[i] = row * 16 + (bvec ^ (row & 15));
    }

    f32x4 acc[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[nt] = f32x4{0.f, 0.f, 0.f, 0.f};

    const int full = nv / 16, rem = nv % 16;
    // full chunks: straight-line loads (no predicate, no branch around a prefetch, so that the
    // compiler can count the loads in flight and wait for the older buffer only)
    auto load_a = [&](uint4 (&a)[4], int c) {
        const int o = c * 16 + g;
#pragma unroll
        for (int s = 0; s < 4; ++s) a[s] = ap[o + 4 * s];
    };
    auto load_b = [&](uint4 (&b)[BV], int c) {
#pragma unroll
        for (int i = 0; i < BV; ++i) b[i] = bp[i][c * 16];
    };
    auto store_b = [&](const uint4 (&b)[BV], int buf) {
#pragma unroll
        for (int i = 0; i < BV; ++i) smem[buf * ROWS * 16 + bdst[i]] = b[i];
    };
    auto compute = [&](const uint4 (&a)[4], int buf) {
        const uint4 *bb = smem + buf * ROWS * 16 + m * 16;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            uint4 bf[NT];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) bf[nt] = bb[nt * 256 + ((4 * s + g) ^ m)];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) Mma<DT>::run(a[s], bf[nt], acc[nt]);
        }
    };
    auto scan = [&](const uint4 (&a)[4]) {
        if constexpr (STATS) {
#pragma unroll
            for (int s = 0; s < 4; ++s) st.add(a[s]);
        }
    };

    uint4 a0[4], a1[4], bs[BV];
    if (full > 0) {
        load_a(a0, 0);
        load_b(bs, 0);
        store_b(bs, 0);
        __syncthreads();
        int c = 0;
        while (true) {
            if (c + 1 >= full) { scan(a0); compute(a0, 0); __syncthreads(); break; }
            load_a(a1, c + 1); load_b(bs, c + 1);
            scan(a0); compute(a0, 0);
            store_b(bs, 1);
            __syncthreads();
            ++c;
            if (c + 1 >= full) { scan(a1); compute(a1, 1); __syncthreads(); break; }
            load_a(a0, c + 1); load_b(bs, c + 1);
            scan(a1); compute(a1, 1);
            store_b(bs, 0);
            __syncthreads();
            ++c;
        }
    }
    if (rem) {
        // last, partial chunk: vectors past the row end are read from a clamped index (valid
        // memory, harmless for the min / max scan) and enter the products as zero in BOTH operands
        const int o = full * 16;
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const int v = 4 * s + g;
            a0[s] = ap[o + min(v, rem - 1)];
        }
        scan(a0);
#pragma unroll
        for (int s = 0; s < 4; ++s) if (4 * s + g >= rem) a0[s] = make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < BV; ++i) {
            bs[i] = bp[i][o + min(bvec, rem - 1) - bvec];
            if (bvec >= rem) bs[i] = make_uint4(0, 0, 0, 0);
        }
        store_b(bs, 0);                                  // every wave is past the barrier of the loop
        __syncthreads();
        compute(a0, 0);
        __syncthreads();
    }

    if constexpr (STATS) {
        int a, b, n;
        st.reduced(a, b, n);
#pragma unroll
        for (int off = 16; off < 64; off <<= 1) {
            a = min(a, __shfl_xor(a, off, WAVE));
            b = max(b, __shfl_xor(b, off, WAVE));
            n = max(n, __shfl_xor(n, off, WAVE));
        }
        if (g == 0) { pstat[w * 16 + m][0] = a; pstat[w * 16 + m][1] = b; pstat[w * 16 + m][2] = n; }
    }

    // every wave is past its last read of the weight buffers (barrier above): reuse them
    float (*logits)[ROWS + 1] = reinterpret_cast<float (*)[ROWS + 1]>(smem);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int i = 0; i < 4; ++i) logits[w * 16 + 4 * g + i][nt * 16 + m] = acc[nt][i];
}

} // namespace pm
