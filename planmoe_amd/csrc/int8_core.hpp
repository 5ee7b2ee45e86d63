// Element-level arithmetic of the "int8" codec, shared by the stand-alone and fused kernels.
#pragma once
#include "common.hpp"

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

// Per-row quantiser.  For bf16 the quotient (x - bias) / scale is a ratio of two 8-bit
// significands: it can only sit on a bf16 rounding boundary when it is exactly representable,
// and every other quotient is more than 2^-17 (relative) away from one.  So a reciprocal
// multiply with one residual correction -- exact whenever the quotient is representable, within
// a few 2^-24 otherwise -- rounds to the same bf16 value as the IEEE division.  Scales outside
// [2^-100, 2^100] and the other dtypes take the IEEE division.
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
                float t = d * inv;
                const float r = fmaf(-t, scale, d);
                t = fmaf(r, inv, t);
                const float q = E::round(t);
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
// can use the corrected reciprocal multiply (see RowQuant).
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
            float t = c * inv;
            const float r = fmaf(-t, 255.0f, c);
            t = fmaf(r, inv, t);
            float v = E::round(t);
            v = E::round(v * scale);
            return E::round(v + bias);
        } else {
            return dequantise<DT>(code, bias, scale);
        }
    }
};

} // namespace pm
