// Element-level arithmetic of the "int8" codec, shared by the stand-alone and fused kernels.
#pragma once
#include "common.hpp"
#include <type_traits>

namespace pm {

template <int DT>
__device__ __forceinline__ uint32_t quantise(float v, float bias, float scale)
{
    using E = Elem<DT>;
    const float d = E::round(v - bias);
    const float q = E::round(d / scale);
    const float m = E::round(q * 255.0f);
    // NaN (0/0 on a constant row) and anything below 1 encode to 0; m never exceeds 255
    return (m >= 1.0f) ? (uint32_t)fminf(m, 255.0f) : 0u;
}

// Per-row quantiser.  For bf16 the quotient (x - bias) / scale is a ratio a / b of two 8-bit
// significands.  It is never a bf16 rounding boundary (a 9-bit midpoint m / 2^9 with m odd would
// need a = m * b / 2^k >= 257), and it is at least 1 / (512 b) > 2^-17 (relative) away from
// every boundary, while d * fl(1 / scale) is within 2^-23 of it.  So the reciprocal multiply
// rounds to the same bf16 value as the IEEE division followed by the bf16 rounding.  Scales
// outside [2^-100, 2^100] and the other dtypes take the IEEE division.
template <int DT>
struct RowQuant {
    float bias, scale, inv;
    bool fast;
    __device__ __forceinline__ RowQuant(float b, float s) : bias(b), scale(s), inv(0.f), fast(false)
    {
        if constexpr (DT == PLANMOE_BF16) {
            fast = s >= 7.888609052210118e-31f && s <= 1.2676506002282294e30f;
            inv = fast ? 1.0f / s : 0.f;
        }
    }
    __device__ __forceinline__ uint32_t operator()(float v) const
    {
        if constexpr (DT == PLANMOE_BF16) {
            if (fast) {
                using E = Elem<DT>;
                const float d = E::round(v - bias);
                const float q = E::round(d * inv);
                const float m = E::round(q * 255.0f);
                return (m >= 1.0f) ? (uint32_t)fminf(m, 255.0f) : 0u;
            }
        }
        return quantise<DT>(v, bias, scale);
    }
};

template <int DT>
__device__ __forceinline__ float dequantise(uint32_t code, float bias, float scale)
{
    using E = Elem<DT>;
    float v = (float)code;                 // <= 255: exact in every dtype here
    v = E::round(v / 255.0f);
    v = E::round(v * scale);
    return E::round(v + bias);
}

// Per-row dequantiser.  code / 255 is again a ratio of two 8-bit integers, so the bf16 path
// can use the reciprocal multiply (see RowQuant).
template <int DT>
struct RowDequant {
    float bias, scale;
    __device__ __forceinline__ RowDequant(float b, float s) : bias(b), scale(s) {}
    __device__ __forceinline__ float operator()(uint32_t code) const
    {
        if constexpr (DT == PLANMOE_BF16) {
            using E = Elem<DT>;
            const float c = (float)code;
            constexpr float inv = 1.0f / 255.0f;
            float v = E::round(c * inv);
            v = E::round(v * scale);
            return E::round(v + bias);
        } else {
            return dequantise<DT>(code, bias, scale);
        }
    }
};

// Decoder of one row for callers that consume the values as fp32 right away (combine fused with
// the decode): four codes of a 32-bit word -> four values, each rounded to the dtype after every
// step exactly as RowDequant does.  bf16 works on pairs, so that every rounding is one packed
// conversion for two values.
template <int DT>
struct RowDecoder {
    RowDequant<DT> dq;
    __device__ __forceinline__ RowDecoder(float b, float s) : dq(b, s) {}
    __device__ __forceinline__ void word(uint32_t w, float *f) const
    {
#pragma unroll
        for (int i = 0; i < 4; ++i) f[i] = dq((w >> (8 * i)) & 0xffu);
    }
};
template <>
struct RowDecoder<PLANMOE_BF16> {
    float bias, scale;
    __device__ __forceinline__ RowDecoder(float b, float s) : bias(b), scale(s) {}
    __device__ __forceinline__ void pair(float c0, float c1, float &o0, float &o1) const
    {
        constexpr float inv = 1.0f / 255.0f;
        uint32_t pk = f32x2_to_bf16x2(c0 * inv, c1 * inv);
        pk = f32x2_to_bf16x2(__uint_as_float(pk << 16) * scale, __uint_as_float(pk & 0xffff0000u) * scale);
        pk = f32x2_to_bf16x2(__uint_as_float(pk << 16) + bias, __uint_as_float(pk & 0xffff0000u) + bias);
        o0 = __uint_as_float(pk << 16); o1 = __uint_as_float(pk & 0xffff0000u);
    }
    __device__ __forceinline__ void word(uint32_t w, float *f) const
    {
        pair((float)(w & 0xffu), (float)((w >> 8) & 0xffu), f[0], f[1]);
        pair((float)((w >> 16) & 0xffu), (float)(w >> 24), f[2], f[3]);
    }
};

// ---------------------------------------------------------------- row-level building blocks
// RowStats<DT, CANON>: running min / max of a row, NaN-propagating like torch.min / torch.max.
// CANON: the row as the dispatcher would store it (0 + x, so -0 reads as +0).  RowEncoder<DT>: one 16-byte vector of
// the row -> VEC codes packed four per 32-bit word.
template <int DT, bool CANON>
struct RowStats {
    using E = Elem<DT>;
    float mn, mx;
    __device__ __forceinline__ void init() { mn = INFINITY; mx = -INFINITY; }
    __device__ __forceinline__ void add(const uint4 &raw)
    {
        float f[E::VEC];
        E::unpack(raw, f);
#pragma unroll
        for (int i = 0; i < E::VEC; ++i) { const float d = CANON ? 0.f + f[i] : f[i]; mn = nan_min(mn, d); mx = nan_max(mx, d); }
    }
    // reduce over the wavefront
    __device__ __forceinline__ void finish(float &lo, float &hi) const
    {
        lo = wave_allreduce(mn, [](float a, float b) { return nan_min(a, b); });
        hi = wave_allreduce(mx, [](float a, float b) { return nan_max(a, b); });
    }
};

template <int DT>
struct RowEncoder {
    using E = Elem<DT>;
    RowQuant<DT> rq;
    __device__ __forceinline__ RowEncoder(float bias, float scale) : rq(bias, scale) {}
    // no reciprocal path for this dtype: both modes are the IEEE division
    __device__ __forceinline__ constexpr bool fast() const { return false; }
    template <bool FAST>
    __device__ __forceinline__ void encode(const uint4 &raw, uint32_t *w) const
    {
        float f[E::VEC];
        E::unpack(raw, f);
#pragma unroll
        for (int i = 0; i < E::VEC / 4; ++i)
            w[i] = rq(0.f + f[4 * i]) | (rq(0.f + f[4 * i + 1]) << 8) | (rq(0.f + f[4 * i + 2]) << 16) | (rq(0.f + f[4 * i + 3]) << 24);
    }
    // the row scaled by its gate first, as the dispatcher stores it: round(0 + g * x)
    template <bool FAST>
    __device__ __forceinline__ void encode_gated(const uint4 &raw, float g, uint32_t *w) const
    {
        float f[E::VEC];
        E::unpack(raw, f);
#pragma unroll
        for (int i = 0; i < E::VEC; ++i) f[i] = E::round(0.f + g * f[i]);
#pragma unroll
        for (int i = 0; i < E::VEC / 4; ++i)
            w[i] = rq(f[4 * i]) | (rq(f[4 * i + 1]) << 8) | (rq(f[4 * i + 2]) << 16) | (rq(f[4 * i + 3]) << 24);
    }
};

// bf16: two elements per 32-bit word all the way, three packed integer operations per word and no
// key to compute.  Read as signed 16-bit integers the non-negative values are in order, read as
// unsigned ones every negative value lies above every non-negative one and a larger pattern is a
// more negative value.  So with  b = max as signed,  a = min as unsigned,  n = max as unsigned:
//   row max = b if the row has a value >= +0 (b >= 0), else a (the least negative);
//   row min = n if the row has a negative value (n >= 0x8000), else a (the least positive);
//   a NaN shows as b > 0x7f80 (positive) or n > 0xff80 (negative).
// Shares of a row merge with min / max / max.
typedef short          s16x2_t __attribute__((ext_vector_type(2)));
typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));

template <bool CANON>
struct RowStats<PLANMOE_BF16, CANON> {
    s16x2_t mxs;
    u16x2_t mnu, mxu;
    __device__ __forceinline__ void init()
    {
        mxs = s16x2_t{(short)0x8000, (short)0x8000};
        mnu = u16x2_t{0xffff, 0xffff};
        mxu = u16x2_t{0, 0};
    }
    __device__ __forceinline__ void add_word(uint32_t w)
    {
        mxs = __builtin_elementwise_max(mxs, __builtin_bit_cast(s16x2_t, w));
        mnu = __builtin_elementwise_min(mnu, __builtin_bit_cast(u16x2_t, w));
        mxu = __builtin_elementwise_max(mxu, __builtin_bit_cast(u16x2_t, w));
    }
    __device__ __forceinline__ void add(const uint4 &raw)
    {
        add_word(raw.x); add_word(raw.y); add_word(raw.z); add_word(raw.w);
    }
    __device__ static __forceinline__ float bits_to_f32(int pattern)
    {
        uint32_t bits = (uint32_t)pattern & 0xffffu;
        if (CANON && bits == 0x8000u) bits = 0u;         // 0 + (-0) = +0
        return bf16_to_f32(bits);
    }
    // this lane's share as three plain integers (merge with min / max / max)
    __device__ __forceinline__ void reduced(int &a, int &b, int &n) const
    {
        a = min((int)mnu.x, (int)mnu.y);
        b = max((int)mxs.x, (int)mxs.y);
        n = max((int)mxu.x, (int)mxu.y);
    }
    // min / max of the row from combined integers
    __device__ static __forceinline__ void decode(int a, int b, int n, float &lo, float &hi)
    {
        hi = bits_to_f32(b >= 0 ? b : a);
        lo = bits_to_f32(n >= 0x8000 ? n : a);
        if (b > 0x7f80 || n > 0xff80) { lo = __uint_as_float(0x7fc00000u); hi = lo; }
    }
    __device__ __forceinline__ void finish(float &lo, float &hi) const
    {
        int a, b, n;
        reduced(a, b, n);
        a = wave_allreduce(a, [](int p, int q) { return min(p, q); });
        b = wave_allreduce(b, [](int p, int q) { return max(p, q); });
        n = wave_allreduce(n, [](int p, int q) { return max(p, q); });
        decode(a, b, n, lo, hi);
    }
};

template <>
struct RowEncoder<PLANMOE_BF16> {
    RowQuant<PLANMOE_BF16> rq;
    __device__ __forceinline__ RowEncoder(float bias, float scale) : rq(bias, scale) {}
    // The mode is a property of the row, hence of the whole wave: callers branch on it once
    // (a scalar branch) and run one of two straight-line encoders.
    __device__ __forceinline__ bool fast() const { return __builtin_amdgcn_readfirstlane((int)rq.fast) != 0; }
    // two bf16 in w -> code0 | code1 << 8
    template <bool FAST>
    __device__ __forceinline__ uint32_t pair(uint32_t w) const
    {
        return pair_values<FAST>(__uint_as_float(w << 16), __uint_as_float(w & 0xffff0000u));
    }
    // two values that are bf16 already -> code0 | code1 << 8
    template <bool FAST>
    __device__ __forceinline__ uint32_t pair_values(float f0, float f1) const
    {
        if constexpr (!FAST) return quantise<PLANMOE_BF16>(0.f + f0, rq.bias, rq.scale) | (quantise<PLANMOE_BF16>(0.f + f1, rq.bias, rq.scale) << 8);
        // (each difference rounded on its own, into the upper half of a word with zeros below: the
        // rounded value is a float right away, one conversion per value instead of one per pair
        // and an unpacking of both)
        const float d0 = __uint_as_float(f32x2_to_bf16x2(0.f, f0 - rq.bias)), d1 = __uint_as_float(f32x2_to_bf16x2(0.f, f1 - rq.bias));
        uint32_t pk = f32x2_to_bf16x2(d0 * rq.inv, d1 * rq.inv);
        // bf16(255 q) without multiplying: for q = a 2^e with an 8-bit a in [128, 255] the product
        // 255 a = 256 a - a has 16 bits and rounds to a - 1 (its fraction a / 256 lies strictly between
        // 1/2 and 1) for a >= 129, and is 255 2^7 for a = 128: in both cases the bit pattern of
        // q plus 8 exponent steps minus one, i.e. 256 times the bf16 value just below q.  A zero
        // or denormal q lands on a value below 2^-100 and a NaN q (0 / 0 rows) on a negative one:
        // the truncation below makes 0 of both, as it does of their true products.
        pk += 0x03ff03ffu;
        // (the upper value keeps the lower one's bits below its own: less than one bf16 step on top
        // of a value below 256, whose steps are 1 / 2^k, so no integer lies in between and the
        // truncation does not see them)
        const float m0 = __uint_as_float(pk << 16), m1 = __uint_as_float(pk);
        // truncation; the conversion saturates NaN (0/0 rows) and negatives to 0, m <= 255
        return __float2uint_rz(m0) | (__float2uint_rz(m1) << 8);
    }
    template <bool FAST>
    __device__ __forceinline__ void encode(const uint4 &raw, uint32_t *w) const
    {
        w[0] = pair<FAST>(raw.x) | (pair<FAST>(raw.y) << 16);
        w[1] = pair<FAST>(raw.z) | (pair<FAST>(raw.w) << 16);
    }
    // the row scaled by its gate first, as the dispatcher stores it: round(0 + g * x)
    template <bool FAST>
    __device__ __forceinline__ uint32_t pair_gated(uint32_t w, float g) const
    {
        const float x0 = __uint_as_float(w << 16), x1 = __uint_as_float(w & 0xffff0000u);
        const uint32_t pk = f32x2_to_bf16x2(0.f + g * x0, 0.f + g * x1);
        return pair_values<FAST>(__uint_as_float(pk << 16), __uint_as_float(pk & 0xffff0000u));
    }
    template <bool FAST>
    __device__ __forceinline__ void encode_gated(const uint4 &raw, float g, uint32_t *w) const
    {
        w[0] = pair_gated<FAST>(raw.x, g) | (pair_gated<FAST>(raw.y, g) << 16);
        w[1] = pair_gated<FAST>(raw.z, g) | (pair_gated<FAST>(raw.w, g) << 16);
    }
};

} // namespace pm
