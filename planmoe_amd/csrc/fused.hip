// Dispatch fused with the "int8" codec: token rows go straight to uint8 codes in their
// capacity slots, so the [experts*capacity, model_dim] tensor that fast_encode would hand to
// Compress.apply (impls/moe_layer.py:265, impls/overlap.py:12-16, int8.cpp:10-24) never
// exists in memory.  One wavefront owns one token: the row is read once into registers,
// reduced to min/max across lanes, quantised, and the codes are written to every live slot
// of the token.  With the all-ones gate helper every choice shares one set of codes.
#include "rows.hpp"
#include <type_traits>

#include "int8_core.hpp"

namespace pm {

// CACHE = 16-byte vectors per lane held in registers (0: re-read the row from cache)
// GATED: rows are scaled by their gate first (one code row per choice); GRAD: the gate gradient
// <x[t], other[slot]> rides along (GATED only)
// CODED: `other` is given as int8 codes + per-row bias / scale (what the decompressor would have
// turned into the rows of `other`); the rows are decoded on the fly, same values, half the bytes
template <int DT, int CACHE, bool GATED, bool GRAD, bool CODED = false>
__global__ __launch_bounds__(256) void dispatch_int8_kernel(
    const void *__restrict__ x, const float *__restrict__ gates,
    const int32_t *__restrict__ indices, const int32_t *__restrict__ locations, int64_t stride,
    int top_k, int samples, int model_dim, int experts, int capacity,
    uint8_t *__restrict__ codes, void *__restrict__ bias_out, void *__restrict__ scale_out,
    const uint32_t *__restrict__ flags, int token_blocks,
    const void *__restrict__ other, float *__restrict__ grad_gates,
    const void *__restrict__ other_bias, const void *__restrict__ other_scale)
{
    using E = Elem<DT>;
    constexpr int V = E::VEC;
    const int wave = threadIdx.x >> 6, lane = lane_id();
    const int units = model_dim / V;
    __shared__ float s_dtab[CODED ? 4 : 1][CODED ? 256 : 1];         // [wave][code]: decoded values of one row

    if ((int)blockIdx.x >= token_blocks) {
        // slots no live pair addresses: all-zero row -> codes 0, bias 0, scale 0
        const int slots = experts * capacity;
        const int nwaves = (gridDim.x - token_blocks) * 4;
        for (int s = (blockIdx.x - token_blocks) * 4 + wave; s < slots; s += nwaves) {
            if (flags[s]) continue;
            uint8_t *row = codes + (int64_t)s * model_dim;
            for (int u = lane; u < units; u += WAVE) {
                if constexpr (V == 8) stream_store(reinterpret_cast<uint2 *>(row) + u, make_uint2(0u, 0u));
                else stream_store(reinterpret_cast<uint32_t *>(row) + u, 0u);
            }
            if (lane == 0) { E::store(bias_out, s, 0.f); E::store(scale_out, s, 0.f); }
        }
        return;
    }

    const int t = blockIdx.x * 4 + wave;
    if (t >= samples) return;
    const uint4 *src = reinterpret_cast<const uint4 *>((const char *)x + (int64_t)t * model_dim * (int64_t)sizeof(typename E::store_t));

    uint4 cache[CACHE > 0 ? CACHE : 1];
    if constexpr (CACHE > 0) {
#pragma unroll
        for (int c = 0; c < CACHE; ++c) {
            const int u = c * WAVE + lane;
            // (index clamped, not predicated: straight-line loads let the compiler wait for exactly these
            // loads; the re-read last vector is harmless for min / max and is never stored)
            cache[c] = src[min(u, units - 1)];
        }
    }
    auto cache_ref = [&](int c) -> const uint4 & { return cache[c]; };

    // gate gradient of one choice: <x[t], other[slot]> (GatingDecoder.backward, fast_dispatch.py:73-78)
    auto dot_with = [&](int s) {
        float acc = 0.f;
        if constexpr (CODED) {
            // V codes per unit: one or two 32-bit words
            using cword_t = typename std::conditional<V == 8, uint2, uint32_t>::type;
            const cword_t *crow = reinterpret_cast<const cword_t *>((const uint8_t *)other + (int64_t)s * model_dim);
            // the 256 values a code of this row can stand for, worked out once (4 per lane, the
            // decompressor's arithmetic) and looked up per element; the table is the wave's own
            const RowDequant<DT> dq(E::load(other_bias, s), E::load(other_scale, s));
            float *tab = s_dtab[wave];
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
#pragma unroll
            for (int q = 0; q < 4; ++q) tab[q * WAVE + lane] = dq((uint32_t)(q * WAVE + lane));
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            auto visit = [&](const uint4 &a, const cword_t &cw) {
                float fa[V], fb[V];
                E::unpack(a, fa);
                if constexpr (V == 8) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) { fb[i] = tab[(cw.x >> (8 * i)) & 0xffu]; fb[4 + i] = tab[(cw.y >> (8 * i)) & 0xffu]; }
                } else {
#pragma unroll
                    for (int i = 0; i < 4; ++i) fb[i] = tab[(cw >> (8 * i)) & 0xffu];
                }
#pragma unroll
                for (int i = 0; i < V; ++i) acc = fmaf(fb[i], fa[i], acc);
            };
            if constexpr (CACHE > 0) {
                cword_t o[CACHE];
#pragma unroll
                for (int c = 0; c < CACHE; ++c) o[c] = crow[min(c * WAVE + lane, units - 1)];
#pragma unroll
                for (int c = 0; c < CACHE; ++c) if (c * WAVE + lane < units) visit(cache_ref(c), o[c]);
            } else {
                for (int u = lane; u < units; u += WAVE) visit(src[u], crow[u]);
            }
        } else {
            const uint4 *orow = reinterpret_cast<const uint4 *>((const char *)other + (int64_t)s * model_dim * (int64_t)sizeof(typename E::store_t));
            auto visit = [&](const uint4 &a, const uint4 &b) {
                float fa[V], fb[V];
                E::unpack(a, fa); E::unpack(b, fb);
#pragma unroll
                for (int i = 0; i < V; ++i) acc = fmaf(fb[i], fa[i], acc);
            };
            if constexpr (CACHE > 0) {
                uint4 o[CACHE];
#pragma unroll
                for (int c = 0; c < CACHE; ++c) if (c * WAVE + lane < units) o[c] = orow[c * WAVE + lane];
#pragma unroll
                for (int c = 0; c < CACHE; ++c) if (c * WAVE + lane < units) visit(cache_ref(c), o[c]);
            } else {
                for (int u = lane; u < units; u += WAVE) visit(src[u], orow[u]);
            }
        }
        return wave_sum(acc);
    };

    // the row as the dispatcher would store it for gate g: round(0 + g * x)
    auto reduce = [&](float g, float &mn, float &mx) {
        mn = INFINITY; mx = -INFINITY;
        auto visit = [&](const uint4 &raw) {
            float f[V];
            E::unpack(raw, f);
#pragma unroll
            for (int i = 0; i < V; ++i) {
                const float d = E::round(0.f + g * f[i]);
                mn = nan_min(mn, d); mx = nan_max(mx, d);
            }
        };
        if constexpr (CACHE > 0) {
#pragma unroll
            for (int c = 0; c < CACHE; ++c) if (c * WAVE + lane < units) visit(cache[c]);
        } else {
            for (int u = lane; u < units; u += WAVE) visit(src[u]);
        }
        mn = wave_allreduce(mn, [](float a, float b) { return nan_min(a, b); });
        mx = wave_allreduce(mx, [](float a, float b) { return nan_max(a, b); });
    };
    auto put = [&](int s, int u, const uint32_t *w) {
        uint8_t *row = codes + (int64_t)s * model_dim;
        if constexpr (V == 8) stream_store(reinterpret_cast<uint2 *>(row) + u, make_uint2(w[0], w[1]));
        else stream_store(reinterpret_cast<uint32_t *>(row) + u, w[0]);
    };

    for (int j0 = 0; j0 < top_k; j0 += WAVE) {
        const int np = min(top_k - j0, WAVE);
        int slot; float gate;
        fetch_planes(gates, indices, locations, stride, t, j0, np, experts, capacity, slot, gate);
        if (GRAD && lane < np && slot < 0) grad_gates[(int64_t)(j0 + lane) * stride + t] = 0.f;
        if (__ballot(slot >= 0) == 0) continue;

        if constexpr (!GATED) {
            // one code row shared by all live choices; 0 + 1 * x needs no rounding
            RowStats<DT, true> stats;
            stats.init();
            if constexpr (CACHE > 0) {
#pragma unroll
                for (int c = 0; c < CACHE; ++c) stats.add(cache[c]);
            } else {
                for (int u = lane; u < units; u += WAVE) stats.add(src[u]);
            }
            float mn, mx;
            stats.finish(mn, mx);
            const float scale = E::round(mx - mn);
            if (lane < np && slot >= 0) { E::store(bias_out, slot, mn); E::store(scale_out, slot, scale); }
            const RowEncoder<DT> enc(mn, scale);
            auto body = [&](auto mode) {
                auto emit = [&](int u, const uint4 &raw) {
                    uint32_t w[2];
                    enc.template encode<decltype(mode)::value>(raw, w);
                    for (int j = 0; j < np; ++j) {
                        const int s = rl_i(slot, j);
                        if (s >= 0) put(s, u, w);
                    }
                };
                if constexpr (CACHE > 0) {
#pragma unroll
                    for (int c = 0; c < CACHE; ++c) if (c * WAVE + lane < units) emit(c * WAVE + lane, cache[c]);
                } else {
                    for (int u = lane; u < units; u += WAVE) emit(u, src[u]);
                }
            };
            if (enc.fast()) body(std::true_type{}); else body(std::false_type{});
        } else {
            // min / max of the unscaled row once: rounding and scaling by a finite non-zero gate
            // are monotonic, so the extremes of round(0 + g * x) are the images of the extremes
            RowStats<DT, true> stats;
            stats.init();
            if constexpr (CACHE > 0) {
#pragma unroll
                for (int c = 0; c < CACHE; ++c) stats.add(cache[c]);
            } else {
                for (int u = lane; u < units; u += WAVE) stats.add(src[u]);
            }
            float xmn, xmx;
            stats.finish(xmn, xmx);
            for (int j = 0; j < np; ++j) {
                const int s = rl_i(slot, j);
                if (s < 0) continue;
                const float g = rl_f(gate, j);
                if constexpr (GRAD) {
                    const float gg = dot_with(s);
                    if (lane == 0) grad_gates[(int64_t)(j0 + j) * stride + t] = gg;
                }
                float mn, mx;
                if (g != 0.f && fabsf(g) < INFINITY && xmn == xmn) {
                    mn = E::round(0.f + g * (g > 0.f ? xmn : xmx));
                    mx = E::round(0.f + g * (g > 0.f ? xmx : xmn));
                } else {
                    reduce(g, mn, mx);           // 0 * inf, NaN rows and the like: element by element
                }
                const float scale = E::round(mx - mn);
                if (lane == 0) { E::store(bias_out, s, mn); E::store(scale_out, s, scale); }
                const RowEncoder<DT> enc(mn, scale);
                auto body = [&](auto mode) {
                    auto emit = [&](int u, const uint4 &raw) {
                        uint32_t w[2];
                        enc.template encode_gated<decltype(mode)::value>(raw, g, w);
                        put(s, u, w);
                    };
                    if constexpr (CACHE > 0) {
#pragma unroll
                        for (int c = 0; c < CACHE; ++c) if (c * WAVE + lane < units) emit(c * WAVE + lane, cache[c]);
                    } else {
                        for (int u = lane; u < units; u += WAVE) emit(u, src[u]);
                    }
                };
                if (enc.fast()) body(std::true_type{}); else body(std::false_type{});
            }
        }
    }
}

// Combine fused with the "int8" decode (the receive side: Int8Compressor::decompress,
// int8.cpp:46-60, followed by fast_decode, fast_dispatch.py:203-207): the token row is the
// gate-weighted sum of its slots' rows, decoded from the codes on the fly, so the
// [experts*capacity, model_dim] tensor never exists in memory.  One wavefront owns one token and
// all its planes; every decoded value is rounded to the tensor's dtype exactly as the stand-alone
// decoder stores it before it enters the fp32 sum (planes left to right, one rounding at the end).
template <int DT>
__global__ __launch_bounds__(256) void combine_int8_kernel(
    const uint8_t *__restrict__ codes, const void *__restrict__ bias_in, const void *__restrict__ scale_in,
    const float *__restrict__ gates, const int32_t *__restrict__ indices,
    const int32_t *__restrict__ locations, int64_t stride, int top_k, int samples, int model_dim,
    int capacity, void *__restrict__ out)
{
    using E = Elem<DT>;
    constexpr int V = E::VEC;
    const int wave = threadIdx.x >> 6, lane = lane_id();
    const int units = model_dim / V;
    const int t = blockIdx.x * 4 + wave;
    if (t >= samples) return;
    uint4 *dst = reinterpret_cast<uint4 *>((char *)out + (int64_t)t * model_dim * (int64_t)sizeof(typename E::store_t));

    auto load_codes = [&](int s, int u, uint32_t *w) {
        const uint8_t *row = codes + (int64_t)s * model_dim;
        if constexpr (V == 8) { const uint2 c = reinterpret_cast<const uint2 *>(row)[u]; w[0] = c.x; w[1] = c.y; }
        else { w[0] = reinterpret_cast<const uint32_t *>(row)[u]; w[1] = 0; }
    };
    __shared__ float s_tab[4][4][256];                               // [wave][plane][code]
    if (top_k <= 4) {
        // the usual case: all planes of four units are requested before any is decoded
        constexpr int UB = 4;
        int slot; float gate;
        fetch_planes(gates, indices, locations, stride, t, 0, top_k, 0x7fffffff, capacity, slot, gate);
        float b_l = 0.f, s_l = 0.f;
        if (lane < top_k && slot >= 0) { b_l = E::load(bias_in, slot); s_l = E::load(scale_in, slot); }
        // A row has 256 possible values: gate * decoded(code), worked out once per row (4 entries per
        // lane and plane, the same arithmetic as the decoder) and looked up per element.
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (j < top_k && rl_i(slot, j) >= 0) {
                const RowDequant<DT> dq(rl_f(b_l, j), rl_f(s_l, j));
                const float g = rl_f(gate, j);
#pragma unroll
                for (int q = 0; q < 4; ++q) s_tab[wave][j][q * WAVE + lane] = g * dq((uint32_t)(q * WAVE + lane));
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");       // the wave's own table: no work-group barrier
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        for (int u0 = 0; u0 < units; u0 += UB * WAVE) {
            uint32_t cw[4][UB][2];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int s = j < top_k ? rl_i(slot, j) : -1;
#pragma unroll
                for (int b = 0; b < UB; ++b) {
                    cw[j][b][0] = cw[j][b][1] = 0u;
                    // clamped, not predicated: straight-line loads (dead planes read slot 0)
                    load_codes(max(s, 0), min(u0 + b * WAVE + lane, units - 1), cw[j][b]);
                }
            }
#pragma unroll
            for (int b = 0; b < UB; ++b) {
                const int u = u0 + b * WAVE + lane;
                float acc[V];
#pragma unroll
                for (int i = 0; i < V; ++i) acc[i] = 0.f;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (j < top_k) {
                        const int s = rl_i(slot, j);
                        float term[V];
                        if (s >= 0) {
                            const float *tab = s_tab[wave][j];
#pragma unroll
                            for (int i = 0; i < V; ++i) term[i] = tab[(cw[j][b][i / 4] >> (8 * (i % 4))) & 0xffu];
                        } else {
#pragma unroll
                            for (int i = 0; i < V; ++i) term[i] = 0.f;
                        }
#pragma unroll
                        for (int i = 0; i < V; ++i) acc[i] = (j == 0) ? term[i] : acc[i] + term[i];
                    }
                }
                if (u < units) stream_store(dst + u, E::pack(acc));
            }
        }
        return;
    }
    for (int u0 = 0; u0 < units; u0 += WAVE) {
        const int u = u0 + lane;
        float acc[V];
#pragma unroll
        for (int i = 0; i < V; ++i) acc[i] = 0.f;
        for (int j0 = 0; j0 < top_k; j0 += WAVE) {
            const int np = min(top_k - j0, WAVE);
            int slot; float gate;
            fetch_planes(gates, indices, locations, stride, t, j0, np, 0x7fffffff, capacity, slot, gate);
            // bias and scale of the lane's own plane, broadcast below
            float b_l = 0.f, s_l = 0.f;
            if (lane < np && slot >= 0) { b_l = E::load(bias_in, slot); s_l = E::load(scale_in, slot); }
            for (int j = 0; j < np; ++j) {
                const int s = rl_i(slot, j);
                const float g = rl_f(gate, j);
                float term[V];
                if (s >= 0 && u < units) {
                    const RowDecoder<DT> dec(rl_f(b_l, j), rl_f(s_l, j));
                    uint32_t w[2];
                    load_codes(s, u, w);
#pragma unroll
                    for (int q = 0; q < V / 4; ++q) dec.word(w[q], term + 4 * q);
#pragma unroll
                    for (int i = 0; i < V; ++i) term[i] = g * term[i];
                } else {
#pragma unroll
                    for (int i = 0; i < V; ++i) term[i] = 0.f;
                }
#pragma unroll
                for (int i = 0; i < V; ++i) acc[i] = (j0 + j == 0) ? term[i] : acc[i] + term[i];
            }
        }
        if (u < units) stream_store(dst + u, E::pack(acc));
    }
}

template <int DT>
static void launch_dispatch_int8(int per_lane, unsigned grid, hipStream_t st, const void *x,
                                 const float *gates, const int32_t *indices, const int32_t *locations,
                                 int64_t stride, int top_k, int samples, int model_dim, int experts,
                                 int capacity, uint8_t *codes, void *bias, void *scale,
                                 const uint32_t *flags, int token_blocks, const void *other,
                                 float *grad_gates, const void *other_bias, const void *other_scale)
{
#define PM_DI8_(CACHE, GATED, GRAD, CODED)                                                       \
    dispatch_int8_kernel<DT, CACHE, GATED, GRAD, CODED><<<grid, 256, 0, st>>>(x, gates, indices, locations, stride, \
        top_k, samples, model_dim, experts, capacity, codes, bias, scale, flags, token_blocks,   \
        other, grad_gates, other_bias, other_scale)
#define PM_DI8(CACHE)                                                                            \
    do {                                                                                         \
        if (!gates) PM_DI8_(CACHE, false, false, false);                                         \
        else if (!grad_gates) PM_DI8_(CACHE, true, false, false);                                \
        else if (!other_bias) PM_DI8_(CACHE, true, true, false);                                 \
        else PM_DI8_(CACHE, true, true, true);                                                   \
    } while (0)
    if (per_lane <= 2) PM_DI8(2);
    else if (per_lane <= 4) PM_DI8(4);
    else if (per_lane <= 8) PM_DI8(8);
    else if (per_lane <= 16) PM_DI8(16);
    else PM_DI8(0);
#undef PM_DI8
#undef PM_DI8_
}

} // namespace pm

using namespace pm;

static int run_dispatch_int8(const char *who, const void *x, int dtype, const float *gates,
                             const int32_t *indices, const int32_t *locations, int64_t plane_stride,
                             int top_k, int samples, int model_dim, int experts, int capacity,
                             uint8_t *codes, void *bias, void *scale, void *workspace,
                             size_t workspace_bytes, const void *other, float *grad_gates, void *stream,
                             const void *other_bias = nullptr, const void *other_scale = nullptr)
{
    if (check_planes(who, indices, locations, plane_stride, top_k, samples)) return 1;
    PM_REQUIRE(dtype_ok(dtype), "%s: bad dtype %d", who, dtype);
    PM_REQUIRE(model_dim >= 1 && experts >= 1 && capacity >= 0, "%s: bad shape", who);
    PM_REQUIRE((int64_t)experts * capacity < (1ll << 31), "%s: experts*capacity overflows int32", who);
    PM_REQUIRE((int64_t)samples * top_k < (1ll << 31), "%s: samples*top_k overflows int32", who);
    const int slots = experts * capacity;
    if (slots == 0) {
        // every token is dropped: nothing to encode, and no gate receives a gradient
        if (grad_gates && samples > 0) {
            fill_u32((uint32_t *)grad_gates, (size_t)(top_k - 1) * plane_stride + samples, 0u, (hipStream_t)stream);
            PM_LAUNCH_CHECK(who);
        }
        return 0;
    }
    PM_REQUIRE(x || samples == 0, "%s: x is NULL", who);
    PM_REQUIRE(codes && bias && scale, "%s: NULL output", who);
    PM_REQUIRE(workspace && workspace_bytes >= planmoe_dispatch_workspace_bytes(experts, capacity),
               "%s: workspace too small", who);
    const int vec = dtype == PLANMOE_F32 ? 4 : 8;
    PM_REQUIRE(model_dim % vec == 0 && aligned16(x) && ((uintptr_t)codes % 8 == 0) &&
               (!other || (other_bias ? (uintptr_t)other % 8 == 0 : aligned16(other))),
               "%s: model_dim must be a multiple of %d and buffers 16-byte aligned; "
               "use the unfused entry points otherwise", who, vec);
    hipStream_t st = (hipStream_t)stream;
    uint32_t *flags = (uint32_t *)workspace;
    launch_slot_flags(flags, indices, locations, plane_stride, top_k, samples, experts, capacity, st);
    const int token_blocks = (samples + 3) / 4;
    const int fill_blocks = min((slots + 3) / 4, 2048);
    const int per_lane = (model_dim / vec + WAVE - 1) / WAVE;
    PM_DTYPE_SWITCH(dtype, DT,
        launch_dispatch_int8<DT>(per_lane, (unsigned)(token_blocks + fill_blocks), st, x, gates, indices,
                                 locations, plane_stride, top_k, samples, model_dim, experts, capacity,
                                 codes, bias, scale, flags, token_blocks, other, grad_gates, other_bias, other_scale));
    PM_LAUNCH_CHECK(who);
    return 0;
}

extern "C" int planmoe_dispatch_int8(const void *x, int dtype, const float *gates,
                                     const int32_t *indices, const int32_t *locations,
                                     int64_t plane_stride, int top_k, int samples, int model_dim,
                                     int experts, int capacity, uint8_t *codes, void *bias,
                                     void *scale, void *workspace, size_t workspace_bytes,
                                     void *stream)
{
    return run_dispatch_int8("planmoe_dispatch_int8", x, dtype, gates, indices, locations, plane_stride,
                             top_k, samples, model_dim, experts, capacity, codes, bias, scale, workspace,
                             workspace_bytes, nullptr, nullptr, stream);
}

extern "C" int planmoe_combine_bwd_int8(const void *grad_out, const void *expert_out, int dtype,
                                        const float *gates, const int32_t *indices,
                                        const int32_t *locations, int64_t plane_stride, int top_k,
                                        int samples, int model_dim, int experts, int capacity,
                                        uint8_t *codes, void *bias, void *scale, float *grad_gates,
                                        void *workspace, size_t workspace_bytes, void *stream)
{
    PM_REQUIRE(gates && grad_gates && (expert_out || (int64_t)experts * capacity == 0),
               "planmoe_combine_bwd_int8: gates, expert_out and grad_gates must not be NULL");
    return run_dispatch_int8("planmoe_combine_bwd_int8", grad_out, dtype, gates, indices, locations,
                             plane_stride, top_k, samples, model_dim, experts, capacity, codes, bias, scale,
                             workspace, workspace_bytes, expert_out, grad_gates, stream);
}

extern "C" int planmoe_combine_bwd_int8_coded(const void *grad_out, const uint8_t *expert_codes,
                                              const void *expert_bias, const void *expert_scale, int dtype,
                                              const float *gates, const int32_t *indices,
                                              const int32_t *locations, int64_t plane_stride, int top_k,
                                              int samples, int model_dim, int experts, int capacity,
                                              uint8_t *codes, void *bias, void *scale, float *grad_gates,
                                              void *workspace, size_t workspace_bytes, void *stream)
{
    PM_REQUIRE(gates && grad_gates && ((expert_codes && expert_bias && expert_scale) || (int64_t)experts * capacity == 0),
               "planmoe_combine_bwd_int8_coded: gates, the coded expert output and grad_gates must not be NULL");
    return run_dispatch_int8("planmoe_combine_bwd_int8_coded", grad_out, dtype, gates, indices, locations,
                             plane_stride, top_k, samples, model_dim, experts, capacity, codes, bias, scale,
                             workspace, workspace_bytes, expert_codes, grad_gates, stream, expert_bias, expert_scale);
}

extern "C" int planmoe_combine_int8(const uint8_t *codes, const void *bias, const void *scale, int dtype,
                                    const float *gates, const int32_t *indices, const int32_t *locations,
                                    int64_t plane_stride, int top_k, int samples, int model_dim,
                                    int capacity, void *out, void *stream)
{
    if (check_planes("planmoe_combine_int8", indices, locations, plane_stride, top_k, samples)) return 1;
    PM_REQUIRE(dtype_ok(dtype), "planmoe_combine_int8: bad dtype %d", dtype);
    PM_REQUIRE(model_dim >= 1 && capacity >= 0, "planmoe_combine_int8: bad shape");
    if (samples == 0) return 0;
    PM_REQUIRE(out, "planmoe_combine_int8: out is NULL");
    PM_REQUIRE((codes && bias && scale) || capacity == 0, "planmoe_combine_int8: NULL codec input");
    const int vec = dtype == PLANMOE_F32 ? 4 : 8;
    PM_REQUIRE(model_dim % vec == 0 && aligned16(out) && (uintptr_t)codes % 8 == 0,
               "planmoe_combine_int8: model_dim must be a multiple of %d, out 16-byte and codes 8-byte aligned "
               "(use planmoe_int8_decompress + planmoe_combine_fwd otherwise)", vec);
    if (capacity == 0) {
        // no slot can be live: every token row is zero
        fill_u32((uint32_t *)out, (size_t)samples * model_dim * (dtype == PLANMOE_F32 ? 4 : 2) / 4, 0u, (hipStream_t)stream);
        PM_LAUNCH_CHECK("planmoe_combine_int8");
        return 0;
    }
    const int blocks = (samples + 3) / 4;
    PM_DTYPE_SWITCH(dtype, DT, (combine_int8_kernel<DT><<<blocks, 256, 0, (hipStream_t)stream>>>(
        codes, bias, scale, gates, indices, locations, plane_stride, top_k, samples, model_dim, capacity, out)));
    PM_LAUNCH_CHECK("planmoe_combine_int8");
    return 0;
}
