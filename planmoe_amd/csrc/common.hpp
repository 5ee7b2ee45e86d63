// Shared device/host helpers for the gfx950 kernels of libplanmoe_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include <string>
#include <cstdio>
#include <cstdarg>

#include "../../include/planmoe_hip.h"

namespace pm {

constexpr int WAVE = 64;

// ---------------------------------------------------------------- host-side error state
void set_error(const char *fmt, ...);
int  fail(const char *fmt, ...);          // sets the error text, returns 1

#define PM_REQUIRE(cond, ...)                                                   \
    do { if (!(cond)) return ::pm::fail(__VA_ARGS__); } while (0)

#define PM_LAUNCH_CHECK(what)                                                   \
    do { hipError_t e_ = hipGetLastError();                                     \
         if (e_ != hipSuccess) return ::pm::fail("%s: launch failed: %s", what, \
                                                 hipGetErrorString(e_)); } while (0)

// device fill with a kernel (safe to record into a HIP graph, unlike a memset node)
void fill_u32(uint32_t *p, size_t n, uint32_t value, hipStream_t stream);

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline size_t round_up(size_t v, size_t a) { return (v + a - 1) / a * a; }
inline int dtype_bytes(int dt) { return dt == PLANMOE_F32 ? 4 : 2; }
inline bool dtype_ok(int dt) { return dt == PLANMOE_F32 || dt == PLANMOE_BF16 || dt == PLANMOE_F16; }

// ---------------------------------------------------------------- scalar conversions
__device__ __forceinline__ float bf16_to_f32(uint32_t bits) { return __uint_as_float(bits << 16); }

// round-to-nearest-even float -> bf16 (the rounding torch applies after each bf16 op), done by
// the gfx950 conversion instruction
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float  f32x2_t  __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t f32_to_bf16(float f)
{
    const __bf16 h = (__bf16)f;
    return (uint32_t)__builtin_bit_cast(uint16_t, h);
}
// two values at once: lo in bits 0..15, hi in bits 16..31
__device__ __forceinline__ uint32_t f32x2_to_bf16x2(float lo, float hi)
{
    const f32x2_t p = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(p, bf16x2_t));
}

__device__ __forceinline__ float f16_to_f32(uint32_t bits)
{
    union { uint16_t u; _Float16 h; } c; c.u = (uint16_t)bits; return (float)c.h;
}
__device__ __forceinline__ uint32_t f32_to_f16(float f)
{
    union { uint16_t u; _Float16 h; } c; c.h = (_Float16)f; return c.u;
}

// Element traits: VEC elements per 16-byte vector, conversion to and from fp32, and
// round(): fp32 value rounded to the storage precision (what one ATen op in that dtype keeps).
// Bulk outputs are written once and not read again by the same launch: streaming (non-temporal)
// stores keep them from displacing the inputs in L2.
typedef uint32_t pm_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t pm_u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void stream_store(uint4 *p, const uint4 &v)
{
    __builtin_nontemporal_store(pm_u32x4{v.x, v.y, v.z, v.w}, reinterpret_cast<pm_u32x4 *>(p));
}
__device__ __forceinline__ void stream_store(uint2 *p, const uint2 &v)
{
    __builtin_nontemporal_store(pm_u32x2{v.x, v.y}, reinterpret_cast<pm_u32x2 *>(p));
}
__device__ __forceinline__ void stream_store(uint32_t *p, uint32_t v)
{
    __builtin_nontemporal_store(v, p);
}

// Streaming loads for inputs read exactly once; used where measurement showed a gain.
__device__ __forceinline__ uint4 stream_load(const uint4 *p)
{
    const pm_u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const pm_u32x4 *>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 stream_load(const uint2 *p)
{
    const pm_u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const pm_u32x2 *>(p));
    return make_uint2(v.x, v.y);
}

template <int DT> struct Elem;

template <> struct Elem<PLANMOE_F32> {
    using store_t = float;
    static constexpr int VEC = 4;
    __device__ static __forceinline__ void unpack(const uint4 &v, float *f)
    {
        f[0] = __uint_as_float(v.x); f[1] = __uint_as_float(v.y);
        f[2] = __uint_as_float(v.z); f[3] = __uint_as_float(v.w);
    }
    __device__ static __forceinline__ uint4 pack(const float *f)
    {
        return make_uint4(__float_as_uint(f[0]), __float_as_uint(f[1]),
                          __float_as_uint(f[2]), __float_as_uint(f[3]));
    }
    __device__ static __forceinline__ float load(const void *p, int64_t i) { return ((const float *)p)[i]; }
    __device__ static __forceinline__ void store(void *p, int64_t i, float v) { ((float *)p)[i] = v; }
    __device__ static __forceinline__ float round(float v) { return v; }
};

template <> struct Elem<PLANMOE_BF16> {
    using store_t = uint16_t;
    static constexpr int VEC = 8;
    __device__ static __forceinline__ void unpack(const uint4 &v, float *f)
    {
        f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
        f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
        f[4] = __uint_as_float(v.z << 16); f[5] = __uint_as_float(v.z & 0xffff0000u);
        f[6] = __uint_as_float(v.w << 16); f[7] = __uint_as_float(v.w & 0xffff0000u);
    }
    __device__ static __forceinline__ uint4 pack(const float *f)
    {
        return make_uint4(f32x2_to_bf16x2(f[0], f[1]), f32x2_to_bf16x2(f[2], f[3]),
                          f32x2_to_bf16x2(f[4], f[5]), f32x2_to_bf16x2(f[6], f[7]));
    }
    __device__ static __forceinline__ float load(const void *p, int64_t i) { return bf16_to_f32(((const uint16_t *)p)[i]); }
    __device__ static __forceinline__ void store(void *p, int64_t i, float v) { ((uint16_t *)p)[i] = (uint16_t)f32_to_bf16(v); }
    __device__ static __forceinline__ float round(float v) { return bf16_to_f32(f32_to_bf16(v)); }
};

template <> struct Elem<PLANMOE_F16> {
    using store_t = uint16_t;
    static constexpr int VEC = 8;
    __device__ static __forceinline__ void unpack(const uint4 &v, float *f)
    {
        f[0] = f16_to_f32(v.x & 0xffffu); f[1] = f16_to_f32(v.x >> 16);
        f[2] = f16_to_f32(v.y & 0xffffu); f[3] = f16_to_f32(v.y >> 16);
        f[4] = f16_to_f32(v.z & 0xffffu); f[5] = f16_to_f32(v.z >> 16);
        f[6] = f16_to_f32(v.w & 0xffffu); f[7] = f16_to_f32(v.w >> 16);
    }
    __device__ static __forceinline__ uint4 pack(const float *f)
    {
        return make_uint4(f32_to_f16(f[0]) | (f32_to_f16(f[1]) << 16),
                          f32_to_f16(f[2]) | (f32_to_f16(f[3]) << 16),
                          f32_to_f16(f[4]) | (f32_to_f16(f[5]) << 16),
                          f32_to_f16(f[6]) | (f32_to_f16(f[7]) << 16));
    }
    __device__ static __forceinline__ float load(const void *p, int64_t i) { return f16_to_f32(((const uint16_t *)p)[i]); }
    __device__ static __forceinline__ void store(void *p, int64_t i, float v) { ((uint16_t *)p)[i] = (uint16_t)f32_to_f16(v); }
    __device__ static __forceinline__ float round(float v) { return f16_to_f32(f32_to_f16(v)); }
};

// ---------------------------------------------------------------- wavefront helpers (wave64)
__device__ __forceinline__ int lane_id() { return (int)(threadIdx.x & (WAVE - 1)); }

// Partner exchange for reductions inside a row of 16 lanes with DPP modifiers (register-file
// speed; a __shfl is an LDS round trip).  STEP 1, 2: lane ^ 1, lane ^ 2 (quad permutes);
// STEP 4: lane <-> 7 - lane inside each group of 8; STEP 8: lane <-> 15 - lane inside the row.
// After steps 1, 2, .., N / 2 every lane holds the reduction over its aligned group of N lanes,
// provided the operation is commutative and associative.
template <int STEP, typename T>
__device__ __forceinline__ T row_partner(T v)
{
    static_assert(sizeof(T) == 4, "32-bit values");
    constexpr int ctrl = STEP == 1 ? 0xB1 : STEP == 2 ? 0x4E : STEP == 4 ? 0x141 : 0x140;
    const int x = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(T, __builtin_amdgcn_update_dpp(x, x, ctrl, 0xf, 0xf, false));
}

// reduction over aligned groups of N <= 16 lanes, result in every lane of the group
template <int N, typename T, typename Op>
__device__ __forceinline__ T row_allreduce(T v, Op op)
{
    if constexpr (N >= 2) v = op(v, row_partner<1>(v));
    if constexpr (N >= 4) v = op(v, row_partner<2>(v));
    if constexpr (N >= 8) v = op(v, row_partner<4>(v));
    if constexpr (N >= 16) v = op(v, row_partner<8>(v));
    return v;
}

template <typename T, typename Op>
__device__ __forceinline__ T wave_allreduce(T v, Op op)
{
    v = row_allreduce<16>(v, op);
    // the four rows meet through scalar registers
    const int x = __builtin_bit_cast(int, v);
    const T r0 = __builtin_bit_cast(T, __builtin_amdgcn_readlane(x, 0));
    const T r1 = __builtin_bit_cast(T, __builtin_amdgcn_readlane(x, 16));
    const T r2 = __builtin_bit_cast(T, __builtin_amdgcn_readlane(x, 32));
    const T r3 = __builtin_bit_cast(T, __builtin_amdgcn_readlane(x, 48));
    return op(op(r0, r1), op(r2, r3));
}

__device__ __forceinline__ float wave_sum(float v)
{
    return wave_allreduce(v, [](float a, float b) { return a + b; });
}

// min / max that keep a NaN once seen, like torch.min / torch.max
__device__ __forceinline__ float nan_min(float a, float b) { return (b < a || b != b) ? b : a; }
__device__ __forceinline__ float nan_max(float a, float b) { return (b > a || b != b) ? b : a; }

// Dispatch a dtype tag to a template parameter.
#define PM_DTYPE_SWITCH(dt, DT, ...)                                            \
    switch (dt) {                                                               \
    case PLANMOE_F32:  { constexpr int DT = PLANMOE_F32;  __VA_ARGS__; break; } \
    case PLANMOE_BF16: { constexpr int DT = PLANMOE_BF16; __VA_ARGS__; break; } \
    case PLANMOE_F16:  { constexpr int DT = PLANMOE_F16;  __VA_ARGS__; break; } \
    default: return ::pm::fail("unsupported dtype tag %d", (int)(dt));          \
    }

} // namespace pm
