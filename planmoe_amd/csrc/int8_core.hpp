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

template <int DT>
__device__ __forceinline__ float dequantise(uint32_t code, float bias, float scale)
{
    using E = Elem<DT>;
    float v = (float)code;                 // <= 255: exact in every dtype here
    v = E::round(v / 255.0f);
    v = E::round(v * scale);
    return E::round(v + bias);
}

} // namespace pm
