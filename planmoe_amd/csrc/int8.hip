// "int8" codec: per-row min/max affine quantisation to uint8 and its inverse.
//
// Takes the place of the ATen op chains of Int8Compressor (custom/compressor/int8.cpp:10-24
// and :47-58): seven elementwise/reduction launches plus a copy become one pass.  One
// wavefront owns one row; the row stays in registers between the min/max reduction and the
// quantisation when it fits (up to CACHE 16-byte vectors per lane), otherwise it is read a
// second time (from cache).  The three roundings of (x - bias) / scale * 255 are kept
// separate and in the tensor's dtype so the codes equal the reference's bit for bit.
#include "int8_core.hpp"

namespace pm {

// VECTOR: row_len % VEC == 0 and 16-byte aligned rows; CACHE = vectors per lane kept in registers
// WIDE (16-bit types, row_len % 16 == 0, 16-byte aligned code rows): a lane takes two adjacent
// vectors (32 bytes of the row) so that its 16 codes leave as one 16-byte store
template <int DT, int CACHE, bool WIDE>
__global__ __launch_bounds__(256) void int8_compress_vec_kernel(
    const void *__restrict__ x, int64_t rows, int row_len, uint8_t *__restrict__ codes,
    void *__restrict__ bias_out, void *__restrict__ scale_out)
{
    using E = Elem<DT>;
    constexpr int V = E::VEC;
    const int lane = lane_id();
    const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= rows) return;
    const int units = row_len / V;
    const uint4 *src = reinterpret_cast<const uint4 *>((const char *)x + r * row_len * (int64_t)sizeof(typename E::store_t));

    static_assert(!WIDE || (V == 8 && CACHE > 0 && CACHE % 2 == 0), "wide stores pair up cached vectors");
    auto unit_of = [&](int c) { return WIDE ? (c >> 1) * (2 * WAVE) + 2 * lane + (c & 1) : c * WAVE + lane; };
    uint4 cache[CACHE > 0 ? CACHE : 1];
    RowStats<DT, false> stats;
    stats.init();
    if constexpr (CACHE > 0) {
#pragma unroll
        for (int c = 0; c < CACHE; ++c) {
            const int u = unit_of(c);
            // (index clamped, not predicated: straight-line loads let the compiler wait for exactly these
            // loads; the re-read last vector is harmless for min / max and is never stored)
            cache[c] = stream_load(src + min(u, units - 1));
        }
#pragma unroll
        for (int c = 0; c < CACHE; ++c)
            stats.add(cache[c]);
    } else {
        for (int u = lane; u < units; u += WAVE) stats.add(src[u]);
    }
    float mn, mx;
    stats.finish(mn, mx);
    const float scale = E::round(mx - mn);
    if (lane == 0) { E::store(bias_out, r, mn); E::store(scale_out, r, scale); }

    uint8_t *dst = codes + r * row_len;
    // A scale of 0 (constant row: an empty capacity slot), infinity or NaN turns every quotient into
    // 0 or NaN, and both encode to 0: such rows are written as zeros without going through the
    // quantiser (which would take the IEEE division for them).
    if (!(scale > 0.f && scale < INFINITY)) {
        for (int u = lane; u < units; u += WAVE) {
            if constexpr (V == 8) stream_store(reinterpret_cast<uint2 *>(dst) + u, make_uint2(0u, 0u));
            else stream_store(reinterpret_cast<uint32_t *>(dst) + u, 0u);
        }
        return;
    }
    const RowEncoder<DT> enc(mn, scale);
    auto body = [&](auto mode) {
        constexpr bool FAST = decltype(mode)::value;
        auto emit = [&](int u, const uint4 &raw) {
            uint32_t w[2];
            enc.template encode<FAST>(raw, w);
            if constexpr (V == 8) stream_store(reinterpret_cast<uint2 *>(dst) + u, make_uint2(w[0], w[1]));
            else stream_store(reinterpret_cast<uint32_t *>(dst) + u, w[0]);
        };
        if constexpr (WIDE) {
#pragma unroll
            for (int c = 0; c < CACHE; c += 2) {
                const int u = unit_of(c);             // even, and units is even: u + 1 < units as well
                if (u < units) {
                    uint32_t w[4];
                    enc.template encode<FAST>(cache[c], w);
                    enc.template encode<FAST>(cache[c + 1], w + 2);
                    stream_store(reinterpret_cast<uint4 *>(dst) + (u >> 1), make_uint4(w[0], w[1], w[2], w[3]));
                }
            }
        } else if constexpr (CACHE > 0) {
#pragma unroll
            for (int c = 0; c < CACHE; ++c) {
                const int u = c * WAVE + lane;
                if (u < units) emit(u, cache[c]);
            }
        } else {
            for (int u = lane; u < units; u += WAVE) emit(u, src[u]);
        }
    };
    if (enc.fast()) body(std::true_type{}); else body(std::false_type{});
}

// any row length / alignment: one element per lane access
template <int DT>
__global__ __launch_bounds__(256) void int8_compress_scalar_kernel(
    const void *__restrict__ x, int64_t rows, int row_len, uint8_t *__restrict__ codes,
    void *__restrict__ bias_out, void *__restrict__ scale_out)
{
    using E = Elem<DT>;
    const int lane = lane_id();
    const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= rows) return;
    const int64_t base = r * row_len;
    float mn = INFINITY, mx = -INFINITY;
    for (int j = lane; j < row_len; j += WAVE) {
        const float v = E::load(x, base + j);
        mn = nan_min(mn, v); mx = nan_max(mx, v);
    }
    mn = wave_allreduce(mn, [](float a, float b) { return nan_min(a, b); });
    mx = wave_allreduce(mx, [](float a, float b) { return nan_max(a, b); });
    const float scale = E::round(mx - mn);
    if (lane == 0) { E::store(bias_out, r, mn); E::store(scale_out, r, scale); }
    for (int j = lane; j < row_len; j += WAVE)
        codes[base + j] = (uint8_t)quantise<DT>(E::load(x, base + j), mn, scale);
}

template <int DT>
__global__ __launch_bounds__(256) void int8_decompress_vec_kernel(
    const uint8_t *__restrict__ codes, const void *__restrict__ bias_in,
    const void *__restrict__ scale_in, int64_t rows, int row_len, void *__restrict__ out)
{
    using E = Elem<DT>;
    constexpr int V = E::VEC;
    const int lane = lane_id();
    const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= rows) return;
    const RowDequant<DT> dq(E::load(bias_in, r), E::load(scale_in, r));
    const int units = row_len / V;
    const uint8_t *src = codes + r * row_len;
    uint4 *dst = reinterpret_cast<uint4 *>((char *)out + r * row_len * (int64_t)sizeof(typename E::store_t));
    // the 256 values of this row, worked out once (4 per lane) into the wave's own table
    __shared__ float s_tab[4][256];
    float *tab = s_tab[threadIdx.x >> 6];
#pragma unroll
    for (int q = 0; q < 4; ++q) tab[q * WAVE + lane] = dq((uint32_t)(q * WAVE + lane));
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    for (int u = lane; u < units; u += WAVE) {
        uint32_t w[2];
        if constexpr (V == 8) { const uint2 c = reinterpret_cast<const uint2 *>(src)[u]; w[0] = c.x; w[1] = c.y; }
        else { w[0] = reinterpret_cast<const uint32_t *>(src)[u]; w[1] = 0; }
        float f[V];
#pragma unroll
        for (int i = 0; i < V; ++i) f[i] = tab[(w[i / 4] >> (8 * (i % 4))) & 0xffu];
        stream_store(dst + u, E::pack(f));
    }
}

template <int DT>
__global__ __launch_bounds__(256) void int8_decompress_scalar_kernel(
    const uint8_t *__restrict__ codes, const void *__restrict__ bias_in,
    const void *__restrict__ scale_in, int64_t rows, int row_len, void *__restrict__ out)
{
    using E = Elem<DT>;
    const int lane = lane_id();
    const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= rows) return;
    const float bias = E::load(bias_in, r), scale = E::load(scale_in, r);
    const int64_t base = r * row_len;
    for (int j = lane; j < row_len; j += WAVE)
        E::store(out, base + j, dequantise<DT>(codes[base + j], bias, scale));
}

template <int DT>
static void launch_compress(const void *x, int64_t rows, int row_len, uint8_t *codes, void *bias,
                            void *scale, bool vector, hipStream_t st)
{
    const unsigned blocks = (unsigned)((rows + 3) / 4);
    if (!vector) {
        int8_compress_scalar_kernel<DT><<<blocks, 256, 0, st>>>(x, rows, row_len, codes, bias, scale);
        return;
    }
    const int per_lane = (row_len / Elem<DT>::VEC + WAVE - 1) / WAVE;
#define PM_I8C(CACHE, WIDE) \
    int8_compress_vec_kernel<DT, CACHE, WIDE><<<blocks, 256, 0, st>>>(x, rows, row_len, codes, bias, scale)
    if constexpr (Elem<DT>::VEC == 8) {
        if (row_len % 16 == 0 && aligned16(codes) && per_lane <= 16) {
            if (per_lane <= 2) PM_I8C(2, true);
            else if (per_lane <= 4) PM_I8C(4, true);
            else if (per_lane <= 8) PM_I8C(8, true);
            else PM_I8C(16, true);
            return;
        }
    }
    if (per_lane <= 2) PM_I8C(2, false);
    else if (per_lane <= 4) PM_I8C(4, false);
    else if (per_lane <= 8) PM_I8C(8, false);
    else if (per_lane <= 16) PM_I8C(16, false);
    else PM_I8C(0, false);
#undef PM_I8C
}

} // namespace pm

using namespace pm;

extern "C" int planmoe_int8_compress(const void *x, int dtype, int64_t rows, int row_len,
                                     uint8_t *codes, void *bias, void *scale, void *stream)
{
    PM_REQUIRE(dtype_ok(dtype), "planmoe_int8_compress: bad dtype %d", dtype);
    PM_REQUIRE(rows >= 0 && row_len >= 1, "planmoe_int8_compress: bad shape rows=%lld row_len=%d",
               (long long)rows, row_len);
    PM_REQUIRE((rows + 3) / 4 < (1ll << 31), "planmoe_int8_compress: too many rows");
    if (rows == 0) return 0;
    PM_REQUIRE(x && codes && bias && scale, "planmoe_int8_compress: NULL argument");
    const int vec = dtype == PLANMOE_F32 ? 4 : 8;
    const bool vector = (row_len % vec == 0) && aligned16(x) && ((uintptr_t)codes % 8 == 0);
    PM_DTYPE_SWITCH(dtype, DT, launch_compress<DT>(x, rows, row_len, codes, bias, scale, vector,
                                                   (hipStream_t)stream));
    PM_LAUNCH_CHECK("planmoe_int8_compress");
    return 0;
}

extern "C" int planmoe_int8_decompress(const uint8_t *codes, const void *bias, const void *scale,
                                       int dtype, int64_t rows, int row_len, void *out, void *stream)
{
    PM_REQUIRE(dtype_ok(dtype), "planmoe_int8_decompress: bad dtype %d", dtype);
    PM_REQUIRE(rows >= 0 && row_len >= 1, "planmoe_int8_decompress: bad shape");
    PM_REQUIRE((rows + 3) / 4 < (1ll << 31), "planmoe_int8_decompress: too many rows");
    if (rows == 0) return 0;
    PM_REQUIRE(codes && bias && scale && out, "planmoe_int8_decompress: NULL argument");
    const int vec = dtype == PLANMOE_F32 ? 4 : 8;
    const bool vector = (row_len % vec == 0) && aligned16(out) && ((uintptr_t)codes % 8 == 0);
    const unsigned blocks = (unsigned)((rows + 3) / 4);
    hipStream_t st = (hipStream_t)stream;
    PM_DTYPE_SWITCH(dtype, DT, {
        if (vector) int8_decompress_vec_kernel<DT><<<blocks, 256, 0, st>>>(codes, bias, scale, rows, row_len, out);
        else int8_decompress_scalar_kernel<DT><<<blocks, 256, 0, st>>>(codes, bias, scale, rows, row_len, out);
    });
    PM_LAUNCH_CHECK("planmoe_int8_decompress");
    return 0;
}
