// A measuring stick for forward_single_kernel, not a product path: a kernel with that kernel's
// grid, its loads of x (same addresses, same two rounds in flight), one exchange of tagged words
// between all work-groups, and its streaming stores (every slot row of the [experts * capacity,
// 4096] code buffer once, bias / scale and the routing planes), but none of its arithmetic: no
// GEMM, no row statistics, no quantiser, no routing.  What it takes is what this way of moving the
// bytes costs on the GPU at hand; forward_single_kernel cannot be faster than that.
// MODE 0: the structure of forward_single_kernel (read everything, exchange, store everything).
// MODE 1: the same without the wait at the exchange (words are published, nobody waits for them):
//         what the traffic alone costs when every work-group may store as soon as it has read,
//         i.e. the floor under ANY arrangement of this kernel's loads and stores.  The difference
//         to MODE 0 is the price of the dependency (a second choice's slot needs every first
//         choice of the batch).
// MODE 2: tokens dealt in two halves; the first-choice rows of the first half leave while the
//         second half is read (their slots need the first half's counts only), one more exchange.
// Serves exactly the shape the roofline is quoted on: 64 tokens per work-group, rows of 4096 bf16
// values, 2 choices per token, 8 experts with every slot written once.
#pragma once

namespace pm {

template <int MODE>
__global__ __launch_bounds__(FS_THREADS) void forward_single_ceiling_kernel(
    const uint4 *__restrict__ x, int samples, int capacity, uint8_t *__restrict__ codes, uint16_t *__restrict__ bias_out,
    uint16_t *__restrict__ scale_out, int32_t *__restrict__ planes, void *__restrict__ workspace, unsigned long long salt,
    int spin_limit, int32_t *__restrict__ gave_up)
{
    using G = FsGeom<16>;
    constexpr int NMMA = 16, TOK = 64, E = 8, K = 2;
    __shared__ __align__(16) uint8_t park[2 * 16 * G::RS];
    __shared__ int s_vote[2][FS_WAVES];
    const int tid = threadIdx.x, w = tid >> 6, lane = lane_id(), m = lane & 15, g = lane >> 4;
    const int groups = gridDim.x, grp = blockIdx.x;
    unsigned long long *launches = reinterpret_cast<unsigned long long *>(workspace);
    unsigned long long *pub = reinterpret_cast<unsigned long long *>((char *)workspace + FS_PUB_OFFSET);
    const unsigned long long launch = __hip_atomic_load(launches, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1;
    const uint32_t tag = (uint32_t)launch + (uint32_t)(salt ^ (salt >> 32));
    const int v0 = w * (4 * NMMA) + g;
    auto token_of = [&](int r, int row) {
        if constexpr (MODE != 2) return grp * TOK + 16 * r + row;
        return (r < 2 ? 0 : samples / 2) + grp * (TOK / 2) + 16 * (r & 1) + row;
    };
    auto row_ptr = [&](int r) { return x + (int64_t)min(token_of(r, m), samples - 1) * G::NV + v0; };
    uint8_t *my_park = park + m * G::RS + v0 * 8;
    uint4 buf0[NMMA], buf1[NMMA];
    uint32_t fold = 0;

    auto round = [&](auto rc, uint4 (&cur)[NMMA]) {
        constexpr int r = decltype(rc)::value;
#pragma unroll
        for (int i = 0; i < NMMA; ++i) fold ^= cur[i].x ^ cur[i].y ^ cur[i].z ^ cur[i].w;
        lds_barrier();
        if constexpr (r < 2) {
            const uint4 *ahead = row_ptr(r + 2);
#pragma unroll
            for (int i = 0; i < NMMA; ++i)
                *reinterpret_cast<uint2 *>(my_park + r * 16 * G::RS + 32 * i) = make_uint2(cur[i].x ^ cur[i].y, cur[i].z ^ cur[i].w);
#pragma unroll
            for (int i = 0; i < NMMA; ++i) cur[i] = ahead[4 * i];
        }
    };
    // slot of pair p = 2 * token + choice of this group: expert p % 8, the group's own stretch of 16
    auto slot_of = [&](int p) { return (p % E) * capacity + grp * (TOK * K / E) + p / E; };
    auto store_row = [&](const uint4 (&v)[G::RV], int slot, bool meta) {
        uint4 *dst = reinterpret_cast<uint4 *>(codes + (int64_t)slot * G::M) + lane;
#pragma unroll
        for (int i = 0; i < G::RV; ++i) stream_store(dst + i * WAVE, v[i]);
        if (meta && lane == 0) { bias_out[slot] = (uint16_t)fold; scale_out[slot] = (uint16_t)(fold >> 16); }
    };
    // parked row `prow` holds token `tok` of the group; which = 1: first choice, 2: second, 3: both
    auto flush_row = [&](int prow, int tok, int which) {
        uint4 v[G::RV];
        const uint4 *src = reinterpret_cast<const uint4 *>(park + prow * G::RS) + lane;
#pragma unroll
        for (int i = 0; i < G::RV; ++i) v[i] = src[i * WAVE];
        if (which & 1) store_row(v, slot_of(2 * tok), true);
        if (which & 2) store_row(v, slot_of(2 * tok + 1), true);
    };
    auto publish = [&](int word) {
        if (tid == 0) {
            __hip_atomic_store(pub + (size_t)grp * 16 + word, ((unsigned long long)tag << 32) | fold, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        }
    };
    // true when this wave saw the word of every group (no waiting)
    auto wave_sees_all = [&](int word) {
        bool ok = true;
        for (int gg = lane; gg < groups; gg += WAVE) {
            const unsigned long long wd = __hip_atomic_load(pub + (size_t)gg * 16 + word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            ok = ok && (uint32_t)(wd >> 32) == tag;
            fold ^= (uint32_t)wd & 1u;
        }
        return __ballot(!ok) == 0;
    };

    FS_STAMP(0);
    {
        const uint4 *p0 = row_ptr(0), *p1 = row_ptr(1);
#pragma unroll
        for (int i = 0; i < NMMA; ++i) buf0[i] = p0[4 * i];
#pragma unroll
        for (int i = 0; i < NMMA; ++i) buf1[i] = p1[4 * i];
    }
    bool early = false;
    round(std::integral_constant<int, 0>{}, buf0);
    FS_STAMP(1);
    round(std::integral_constant<int, 1>{}, buf1);
    FS_STAMP(2);
    if constexpr (MODE == 2) {
        lds_barrier();
        publish(1);
    }
    round(std::integral_constant<int, 2>{}, buf0);
    if constexpr (MODE == 2) {
        if (wave_sees_all(1)) {
            early = true;
            for (int tok = w; tok < 32; tok += FS_WAVES) flush_row(tok, tok, 1);
        }
    }
    FS_STAMP(3);
    round(std::integral_constant<int, 3>{}, buf1);
    lds_barrier();
    FS_STAMP(4);
    // the routing planes: 3 x [2][samples] words
    if (tid < TOK * K) {
        const int tok = tid % TOK, j = tid / TOK;
        const int t = token_of(tok / 16, tok % 16);
        if (t < samples) {
            planes[(int64_t)(0 * K + j) * samples + t] = (2 * tok + j) % E;
            planes[(int64_t)(1 * K + j) * samples + t] = grp * (TOK * K / E) + (2 * tok + j) / E;
            planes[(int64_t)(2 * K + j) * samples + t] = (int)fold;
        }
    }
    publish(0);
    FS_STAMP(5);

    bool all = MODE == 1;
    for (int spin = 0; spin <= spin_limit && MODE != 1; ++spin) {
        const bool ok = wave_sees_all(0);
        const int slot = spin & 1;
        if (lane == 0) s_vote[slot][w] = !ok;
        lds_barrier();
        int bad = 0;
#pragma unroll
        for (int ww = 0; ww < FS_WAVES; ++ww) bad |= s_vote[slot][ww];
        all = bad == 0;
        if (all) break;
        __builtin_amdgcn_s_sleep(8);
    }
    if (!all) {
        if (tid == 0 && gave_up) __hip_atomic_store(gave_up, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (tid == 0 && grp == groups - 1) __hip_atomic_store(launches, launch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        return;
    }

    FS_STAMP(7);
    FS_STAMP(8);
    // phase 2: the parked rows, then the register rounds through the same LDS rows, then the zero rows
    for (int tok = w; tok < 32; tok += FS_WAVES) flush_row(tok, tok, early ? 2 : 3);
    FS_STAMP(9);
    lds_barrier();
#pragma unroll
    for (int i = 0; i < NMMA; ++i) {
        *reinterpret_cast<uint2 *>(my_park + 32 * i) = make_uint2(buf0[i].x ^ buf0[i].y, buf0[i].z ^ buf0[i].w);
        *reinterpret_cast<uint2 *>(my_park + 16 * G::RS + 32 * i) = make_uint2(buf1[i].x ^ buf1[i].y, buf1[i].z ^ buf1[i].w);
    }
    lds_barrier();
    FS_STAMP(10);
    for (int i = w; i < 32; i += FS_WAVES) flush_row(i, 32 + i, 3);
    FS_STAMP(11);
    {
        // empty slots: 32 per group, 4 per wave, behind the 4096 used slots of every expert
        const uint4 z[G::RV] = {};
        const int used = groups * (TOK * K / E), per = capacity - used;      // empty slots per expert
        for (int i = w; i < per * E / groups + 1; i += FS_WAVES) {
            const int zi = grp + i * groups;                                 // one list over all experts
            if (zi < per * E) {
                const int slot = (zi / per) * capacity + used + zi % per;
                uint4 *dst = reinterpret_cast<uint4 *>(codes + (int64_t)slot * G::M) + lane;
#pragma unroll
                for (int q = 0; q < G::RV; ++q) stream_store(dst + q * WAVE, z[q]);
                if (lane == 0) { bias_out[slot] = 0; scale_out[slot] = 0; }
            }
        }
    }
    FS_STAMP(12);
    if (grp == groups - 1 && tid == 0) __hip_atomic_store(launches, launch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

} // namespace pm
