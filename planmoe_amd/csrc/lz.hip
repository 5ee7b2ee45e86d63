// GPULZ ("lz") lossless codec for gfx950: byte-identical streams to the reference's
// lz_compress / lz_decompress (custom/compressor/gpulz.cu), built differently.
//
// One wavefront codes one block of 512 symbols (2048 bytes), lane l owning the 8 consecutive
// symbols 8l .. 8l+7:
//   match   every lane keeps the 39 symbols before its last one in registers and tests its 8
//           symbols against their 32-symbol windows (256 compares, no memory traffic).  A
//           position has a match exactly when its symbol occurs in its window, so only the
//           positions that pass run the reference's matcher (gpulz.cu:46-85) through LDS.
//   parse   the greedy token walk (gpulz.cu:98-127, one thread there) advances a whole run of
//           literals or one match per step with ballots and scalar bit scans.
//   pack    token ranks and byte offsets come from one packed wave scan; flags and token bytes
//           are put together in LDS.
//   place   a work-group publishes the sizes of its blocks and takes the sum over all earlier
//           work-groups from their published words (single pass; work-groups are numbered by
//           a ticket, so a group only ever waits for groups that already run), then copies its
//           bytes to their final place.  The reference stages every block at a fixed stride,
//           scans the sizes with a library call and copies everything once more
//           (gpulz.cu:148-211, 460-494, 220-258).
// A second launch zeroes what lies beyond the totals (the reference allocates zeroed buffers).
#include "common.hpp"

namespace pm {
namespace {

constexpr int LZ_SYMS = 512;             // symbols per block (gpulz.cu:6 / sizeof(float))
constexpr int LZ_WINDOW = 32;            // gpulz.cu:12
constexpr int LZ_BLOCK_BYTES = 2048;
constexpr int LZ_WAVES = 8;              // blocks per work-group
constexpr uint32_t NAN_WINDOW = 0x7f800002u;   // key of a NaN seen as a window symbol ...
constexpr uint32_t NAN_AHEAD = 0x7f800001u;    // ... and as a look-ahead symbol: never equal

// status word of a work-group: state in bits 62..63, flag bytes in 31..57, token bytes in 0..30
constexpr uint64_t ST_AGGREGATE = 1ull << 62, ST_INCLUSIVE = 2ull << 62, ST_MASK = 3ull << 62;
constexpr int LOOKBACK_SPINS = 1 << 22;

__device__ __forceinline__ uint64_t st_pack(uint32_t flag_bytes, uint32_t data_bytes)
{
    return ((uint64_t)flag_bytes << 31) | data_bytes;
}
__device__ __forceinline__ uint32_t st_flags(uint64_t v) { return (uint32_t)((v & ~ST_MASK) >> 31); }
__device__ __forceinline__ uint32_t st_data(uint64_t v) { return (uint32_t)(v & 0x7fffffffu); }

// float equality on bit patterns: both zeros share a key, NaNs get a key per role
__device__ __forceinline__ uint32_t window_key(uint32_t bits)
{
    if ((bits << 1) == 0) return 0;
    if ((bits & 0x7fffffffu) > 0x7f800000u) return NAN_WINDOW;
    return bits;
}
__device__ __forceinline__ uint32_t ahead_key(uint32_t wkey) { return wkey == NAN_WINDOW ? NAN_AHEAD : wkey; }

// LDS written by some lanes of a wavefront and read by others of the same wavefront
__device__ __forceinline__ void wave_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__device__ __forceinline__ uint32_t wave_exclusive_sum(uint32_t v, uint32_t &total)
{
    uint32_t inc = v;
#pragma unroll
    for (int d = 1; d < WAVE; d <<= 1) {
        const uint32_t o = __shfl_up(inc, d, WAVE);
        if (lane_id() >= d) inc += o;
    }
    total = __builtin_amdgcn_readlane(inc, WAVE - 1);
    return inc - v;
}

struct LzShared {
    uint32_t keys[LZ_WAVES][LZ_WINDOW + LZ_SYMS];   // window keys, 32 never-matching entries in front
    uint16_t stage[LZ_WAVES][LZ_BLOCK_BYTES / 2];   // token bytes of the block
    uint32_t flagw[LZ_WAVES][16];                   // flag bits of the block
    uint32_t sizes[LZ_WAVES][2];                    // flag bytes, token bytes per block
    uint32_t base[2];                               // sums over all earlier work-groups
    uint32_t ticket;
};

__global__ __launch_bounds__(LZ_WAVES * WAVE) void lz_compress_kernel(
    const uint32_t *__restrict__ in, int64_t nsym, int64_t blocks, int32_t *__restrict__ flag_off,
    int32_t *__restrict__ data_off, uint8_t *__restrict__ flags, uint8_t *__restrict__ data,
    uint32_t *__restrict__ ws)
{
    __shared__ LzShared sh;
    uint32_t *ticket = ws;
    uint32_t *error = ws + 1;
    uint64_t *status = reinterpret_cast<uint64_t *>(ws + 2);

    const int lane = lane_id();
    const int wave = (int)(threadIdx.x >> 6);
    if (threadIdx.x == 0) sh.ticket = atomicAdd(ticket, 1u);
    __syncthreads();
    const int64_t group = sh.ticket;                  // groups are numbered in the order they start
    const int64_t block = group * LZ_WAVES + wave;
    const bool live = block < blocks;                 // wave-uniform

    uint32_t raw[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    uint32_t lens_lo = 0, lens_hi = 0, offs_lo = 0, offs_hi = 0;   // one byte per owned position
    uint32_t match_mask = 0, start_mask = 0;
    uint32_t tok_base = 0, byte_base = 0, flag_bytes = 0, data_bytes = 0;

    if (live) {
        // ---- load: 8 consecutive symbols per lane, zero beyond the end of the input
        const int64_t s0 = block * LZ_SYMS + 8 * lane;
        if (s0 + 8 <= nsym) {
            const uint4 a = *reinterpret_cast<const uint4 *>(in + s0);
            const uint4 b = *reinterpret_cast<const uint4 *>(in + s0 + 4);
            raw[0] = a.x; raw[1] = a.y; raw[2] = a.z; raw[3] = a.w;
            raw[4] = b.x; raw[5] = b.y; raw[6] = b.z; raw[7] = b.w;
        } else {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                if (s0 + i < nsym) raw[i] = in[s0 + i];
        }
        uint32_t *keys = sh.keys[wave];
        uint32_t own[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) own[i] = window_key(raw[i]);
        if (lane < LZ_WINDOW / 4)
            *reinterpret_cast<uint4 *>(keys + 4 * lane) = make_uint4(NAN_WINDOW, NAN_WINDOW, NAN_WINDOW, NAN_WINDOW);
        *reinterpret_cast<uint4 *>(keys + LZ_WINDOW + 8 * lane) = make_uint4(own[0], own[1], own[2], own[3]);
        *reinterpret_cast<uint4 *>(keys + LZ_WINDOW + 8 * lane + 4) = make_uint4(own[4], own[5], own[6], own[7]);
        wave_sync();

        // ---- which positions see their symbol in their window
        uint32_t win[40];                               // keys[8l .. 8l+39] = positions 8l-32 .. 8l+7
#pragma unroll
        for (int q = 0; q < 10; ++q) {
            const uint4 v = *reinterpret_cast<const uint4 *>(keys + 8 * lane + 4 * q);
            win[4 * q] = v.x; win[4 * q + 1] = v.y; win[4 * q + 2] = v.z; win[4 * q + 3] = v.w;
        }
        uint32_t any = 0;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const uint32_t k = ahead_key(own[i]);
            bool hit = false;
#pragma unroll
            for (int j = 0; j < LZ_WINDOW; ++j) hit |= (k == win[i + j]);
            any |= (uint32_t)hit << i;
        }

        // ---- the reference's matcher for those positions (gpulz.cu:46-85): one pass over the
        // window; a failed comparison drops the run and still consumes the window symbol
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if (__ballot((any >> i) & 1) == 0) continue;
            uint32_t len = 0, off = 0;
            if ((any >> i) & 1) {
                const int p = 8 * lane + i;
                int ahead = p;
                uint32_t run = 0, run_off = 0;
                for (int j = 0; j < LZ_WINDOW; ++j) {          // window symbol p - 32 + j
                    if (ahead < LZ_SYMS) {
                        const uint32_t a = ahead_key(keys[LZ_WINDOW + ahead]);
                        const uint32_t b = keys[p + j];
                        if (a == b) {
                            if (run == 0) run_off = (uint32_t)(ahead - p + LZ_WINDOW - j);
                            ++run;
                            ++ahead;
                        } else {
                            if (run > len) { len = run; off = run_off; }
                            run = 0;
                            ahead = p;
                        }
                    }
                }
                if (run > len) { len = run; off = run_off; }
            }
            if (i < 4) { lens_lo |= len << (8 * i); offs_lo |= off << (8 * i); }
            else       { lens_hi |= len << (8 * (i - 4)); offs_hi |= off << (8 * (i - 4)); }
            match_mask |= (uint32_t)(len != 0) << i;
        }

        // ---- greedy parse: [cur, nxt) is a run of literals, nxt the next position with a match
        int cur = 0;
        while (cur < LZ_SYMS) {
            const int rel = cur - 8 * lane;
            const uint32_t mm = rel >= 8 ? 0u : (rel <= 0 ? match_mask : (match_mask & (0xffu << rel)));
            const uint64_t bal = __ballot(mm != 0);
            int nxt = LZ_SYMS, step = 0;
            if (bal != 0) {
                const int owner = __builtin_ctzll(bal);
                const uint32_t m = __builtin_amdgcn_readlane(mm, owner);
                const int bit = __builtin_ctz(m);
                nxt = 8 * owner + bit;
                const uint32_t lo = __builtin_amdgcn_readlane(lens_lo, owner);
                const uint32_t hi = __builtin_amdgcn_readlane(lens_hi, owner);
                step = (int)(((bit < 4 ? lo : hi) >> (8 * (bit & 3))) & 0xffu);
            }
            // the literals and, when there is one, the match token at nxt all start a token
            const int last = bal != 0 ? nxt + 1 : nxt;
            const int lo_b = min(max(cur - 8 * lane, 0), 8);
            const int hi_b = min(max(last - 8 * lane, 0), 8);
            start_mask |= ((1u << hi_b) - 1u) & ~((1u << lo_b) - 1u);
            cur = nxt + step;                          // step >= 1 whenever nxt < 512
        }

        // ---- sizes: tokens and token bytes before this lane, totals of the block
        const uint32_t ntok = __popc(start_mask);
        const uint32_t nmatch = __popc(start_mask & match_mask);
        uint32_t total;
        const uint32_t before = wave_exclusive_sum(ntok | ((4u * ntok - 2u * nmatch) << 16), total);
        tok_base = before & 0xffffu;
        byte_base = before >> 16;
        flag_bytes = ((total & 0xffffu) + 7u) >> 3;
        data_bytes = total >> 16;

        // ---- token bytes and flag bits of the block, in LDS
        uint16_t *stage = sh.stage[wave];
        uint32_t *flagw = sh.flagw[wave];
        if (lane < 16) flagw[lane] = 0;
        wave_sync();
        uint32_t bits = 0, nb = 0, at = byte_base >> 1;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if ((start_mask >> i) & 1) {
                if ((match_mask >> i) & 1) {
                    const uint32_t l = ((i < 4 ? lens_lo : lens_hi) >> (8 * (i & 3))) & 0xffu;
                    const uint32_t o = ((i < 4 ? offs_lo : offs_hi) >> (8 * (i & 3))) & 0xffu;
                    stage[at] = (uint16_t)(l | (o << 8));
                    at += 1;
                    bits |= 1u << nb;
                } else {
                    stage[at] = (uint16_t)raw[i];
                    stage[at + 1] = (uint16_t)(raw[i] >> 16);
                    at += 2;
                }
                ++nb;
            }
        }
        if (bits) {
            const uint64_t wide = (uint64_t)bits << (tok_base & 31u);
            atomicOr(&flagw[tok_base >> 5], (uint32_t)wide);
            if ((uint32_t)(wide >> 32)) atomicOr(&flagw[(tok_base >> 5) + 1], (uint32_t)(wide >> 32));
        }
    }
    if (lane == 0) { sh.sizes[wave][0] = flag_bytes; sh.sizes[wave][1] = data_bytes; }
    __syncthreads();

    // ---- place: publish the group's sizes, sum the groups before it
    if (wave == 0) {
        uint32_t gf = 0, gd = 0;
#pragma unroll
        for (int w = 0; w < LZ_WAVES; ++w) { gf += sh.sizes[w][0]; gd += sh.sizes[w][1]; }
        if (lane == 0)
            __hip_atomic_store(&status[group], (group == 0 ? ST_INCLUSIVE : ST_AGGREGATE) | st_pack(gf, gd),
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        uint32_t pf = 0, pd = 0;
        int64_t nearest = group - 1;                   // lane 0 looks at it, lane j at nearest - j
        int spins = 0;
        while (nearest >= 0) {
            const int64_t mine = nearest - lane;
            uint64_t v = ST_INCLUSIVE;                 // before the first group: nothing
            if (mine >= 0) v = __hip_atomic_load(&status[mine], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const uint64_t inclusive = __ballot((v & ST_MASK) == ST_INCLUSIVE);
            const uint64_t empty = __ballot((v & ST_MASK) == 0);
            const int stop = inclusive ? __builtin_ctzll(inclusive) : WAVE;   // first word that sums everything before it
            const uint64_t needed = stop >= WAVE - 1 ? ~0ull : ((2ull << stop) - 1ull);
            if (empty & needed) {                      // a group in reach has not published yet
                if (++spins > LOOKBACK_SPINS) {        // cannot happen while earlier groups run; never spin for ever
                    if (lane == 0) atomicOr(error, 1u);
                    break;
                }
                __builtin_amdgcn_s_sleep(2);
                continue;
            }
            const bool take = lane <= stop;
            pf += wave_allreduce(take ? st_flags(v) : 0u, [](uint32_t a, uint32_t b) { return a + b; });
            pd += wave_allreduce(take ? st_data(v) : 0u, [](uint32_t a, uint32_t b) { return a + b; });
            if (stop < WAVE) break;
            nearest -= WAVE;
        }
        // never let a wrong sum move a write out of the buffers
        pf = min(pf, (uint32_t)(group * LZ_WAVES * (LZ_SYMS / 8)));
        pd = min(pd, (uint32_t)(group * LZ_WAVES * LZ_BLOCK_BYTES));
        if (lane == 0) {
            if (group != 0)
                __hip_atomic_store(&status[group], ST_INCLUSIVE | st_pack(pf + gf, pd + gd),
                                   __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            sh.base[0] = pf;
            sh.base[1] = pd;
        }
    }
    __syncthreads();
    if (!live) return;

    uint32_t fbase = sh.base[0], dbase = sh.base[1];
    for (int w = 0; w < wave; ++w) { fbase += sh.sizes[w][0]; dbase += sh.sizes[w][1]; }
    if (lane == 0) {
        flag_off[block] = (int32_t)fbase;
        data_off[block] = (int32_t)dbase;
        if (block == blocks - 1) {
            flag_off[blocks] = (int32_t)(fbase + flag_bytes);
            data_off[blocks] = (int32_t)(dbase + data_bytes);
        }
    }
    if ((uint32_t)lane < flag_bytes)
        flags[(size_t)fbase + lane] = (uint8_t)(sh.flagw[wave][lane >> 2] >> (8 * (lane & 3)));

    // token bytes: dbase is even; 2 bytes up to a 4-byte boundary, whole words, 2 bytes at the end
    const uint16_t *stage = sh.stage[wave];
    uint8_t *dst = data + dbase;
    const uint32_t head = (reinterpret_cast<uintptr_t>(dst) & 2u) ? 2u : 0u;
    if (head && lane == 0) *reinterpret_cast<uint16_t *>(dst) = stage[0];
    const uint32_t words = (data_bytes - head) >> 2;
    uint32_t *dw = reinterpret_cast<uint32_t *>(dst + head);
    for (uint32_t k = lane; k < words; k += WAVE) {
        const uint32_t h = (head >> 1) + 2 * k;
        stream_store(dw + k, (uint32_t)stage[h] | ((uint32_t)stage[h + 1] << 16));
    }
    if (((data_bytes - head) & 2u) && lane == 0)
        *reinterpret_cast<uint16_t *>(dst + data_bytes - 2) = stage[data_bytes / 2 - 1];
}

// zero flags[flag_off[blocks] ..) and data[data_off[blocks] ..): 64 bytes per thread
__global__ __launch_bounds__(256) void lz_clear_slack_kernel(const int32_t *__restrict__ flag_off,
                                                            const int32_t *__restrict__ data_off,
                                                            int64_t blocks, uint8_t *__restrict__ flags,
                                                            uint8_t *__restrict__ data, int64_t flag_chunks)
{
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const bool is_flags = t < flag_chunks;
    uint8_t *buf = is_flags ? flags : data;
    const int64_t size = is_flags ? blocks * (LZ_SYMS / 8) : blocks * LZ_BLOCK_BYTES;
    const int64_t used = is_flags ? flag_off[blocks] : data_off[blocks];
    const int64_t lo = (is_flags ? t : t - flag_chunks) * 64;
    if (lo >= size || lo + 64 <= used) return;
    if (lo >= used) {
        uint4 *p = reinterpret_cast<uint4 *>(buf + lo);      // both sizes are multiples of 64
        const uint4 z = make_uint4(0, 0, 0, 0);
        p[0] = z; p[1] = z; p[2] = z; p[3] = z;
    } else {
        for (int64_t b = used; b < lo + 64; ++b) buf[b] = 0;
    }
}

struct LzDecodeShared {
    uint32_t bytes[LZ_WAVES][LZ_BLOCK_BYTES / 4 + 1];  // token bytes of the block (one spare word)
    uint32_t out[LZ_WAVES][LZ_SYMS];
};

__device__ __forceinline__ uint32_t lds_u16(const uint32_t *words, uint32_t byte_at)   // byte_at even
{
    return (words[byte_at >> 2] >> (8 * (byte_at & 2u))) & 0xffffu;
}

__global__ __launch_bounds__(LZ_WAVES * WAVE) void lz_decompress_kernel(
    uint32_t *__restrict__ out, int64_t nsym, int64_t blocks, const int32_t *__restrict__ flag_off,
    const int32_t *__restrict__ data_off, const uint8_t *__restrict__ flags,
    const uint8_t *__restrict__ data)
{
    __shared__ LzDecodeShared sh;
    const int lane = lane_id();
    const int wave = (int)(threadIdx.x >> 6);
    const int64_t block = (int64_t)blockIdx.x * LZ_WAVES + wave;
    if (block >= blocks) return;                       // no work-group barrier below
    uint32_t *bytes = sh.bytes[wave];
    uint32_t *sym = sh.out[wave];

    // offsets of a stream of this coder ascend and stay inside the buffers; clamp all the same
    const int64_t fcap = blocks * (LZ_SYMS / 8), dcap = blocks * LZ_BLOCK_BYTES;
    const int64_t f0 = min(max((int64_t)flag_off[block], (int64_t)0), fcap);
    const int64_t f1 = min(max((int64_t)flag_off[block + 1], f0), min(f0 + LZ_SYMS / 8, fcap));
    const int64_t d0 = min(max((int64_t)data_off[block], (int64_t)0), dcap) & ~(int64_t)1;
    const int64_t d1 = min(max((int64_t)data_off[block + 1], d0), min(d0 + LZ_BLOCK_BYTES, dcap));
    const uint32_t nflag = (uint32_t)(f1 - f0), nbytes = (uint32_t)(d1 - d0);

    // ---- stage the token bytes (source is 2-byte aligned), clear the output block
    {
        const uint8_t *src = data + d0;
        const uint32_t head = (reinterpret_cast<uintptr_t>(src) & 2u) ? 2u : 0u;    // bytes before a word boundary
        // word k of the staged block = source bytes 4k .. 4k+3
        for (uint32_t k = lane; k < LZ_BLOCK_BYTES / 4 + 1; k += WAVE) {
            uint32_t v = 0;
            if (4 * k < nbytes) {
                if (head == 0) {
                    // may run 2 bytes past nbytes; never past the buffer, whose size is a multiple of 4
                    v = *reinterpret_cast<const uint32_t *>(src + 4 * k);
                } else {
                    const uint32_t lo = *reinterpret_cast<const uint16_t *>(src + 4 * k);
                    const uint32_t hi = 4 * k + 2 < nbytes ? *reinterpret_cast<const uint16_t *>(src + 4 * k + 2) : 0u;
                    v = lo | (hi << 16);
                }
            }
            bytes[k] = v;
        }
        for (uint32_t k = lane; k < LZ_SYMS; k += WAVE) sym[k] = 0;
    }
    const uint32_t fb = (uint32_t)lane < nflag ? flags[f0 + lane] : 0u;   // lane l: tokens 8l .. 8l+7
    wave_sync();

    // ---- where each token's bytes and symbols start
    const uint32_t ntok_lane = (uint32_t)lane < nflag ? 8u : 0u;
    const uint32_t nm = __popc(fb);
    uint32_t total;
    uint32_t at = wave_exclusive_sum(4u * ntok_lane - 2u * nm, total);    // byte offset of the lane's first token
    uint32_t tok[8];                                   // match: pos | len << 10 | off << 18 | 1 << 31
    uint32_t nsyms = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        uint32_t t = 0;
        if ((uint32_t)lane < nflag) {
            if ((fb >> i) & 1) {
                const uint32_t lo = at < nbytes ? lds_u16(bytes, at) : 0u;
                t = ((lo & 0xffu) << 10) | ((lo >> 8) << 18) | (1u << 31);
                nsyms += lo & 0xffu;
                at += 2;
            } else {
                t = at << 10;                          // literal: remember where its bytes are
                nsyms += 1;
                at += 4;
            }
        }
        tok[i] = t;
    }
    uint32_t pos = wave_exclusive_sum(nsyms, total);
    uint32_t has_match = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        if ((uint32_t)lane < nflag && pos < (uint32_t)LZ_SYMS) {
            if (tok[i] >> 31) {
                const uint32_t len = (tok[i] >> 10) & 0xffu, off = (tok[i] >> 18) & 0xffu;
                // a match of this coder lies inside the block and copies from before its start
                if (len != 0 && off >= len && off <= pos && pos + len <= (uint32_t)LZ_SYMS) {
                    tok[i] |= pos;
                    has_match |= 1u << i;
                }
                pos += len;
            } else {
                const uint32_t where = tok[i] >> 10;
                if (where + 4 <= nbytes)
                    sym[pos] = lds_u16(bytes, where) | (lds_u16(bytes, where + 2) << 16);
                pos += 1;
            }
        }
    }
    wave_sync();

    // ---- matches in token order: each copies symbols that are complete by then
    uint64_t pending = __ballot(has_match != 0);
    while (pending) {
        const int owner = __builtin_ctzll(pending);
        pending &= pending - 1;
        const uint32_t which = __builtin_amdgcn_readlane(has_match, owner);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if (!((which >> i) & 1)) continue;
            const uint32_t t = __builtin_amdgcn_readlane(tok[i], owner);
            const uint32_t p = t & 0x3ffu, len = (t >> 10) & 0xffu, off = (t >> 18) & 0xffu;
            if ((uint32_t)lane < len) sym[p + lane] = sym[p - off + lane];
            wave_sync();
        }
    }

    // ---- write the block
    const int64_t s0 = block * LZ_SYMS + 8 * lane;
    const uint4 a = *reinterpret_cast<const uint4 *>(sym + 8 * lane);
    const uint4 b = *reinterpret_cast<const uint4 *>(sym + 8 * lane + 4);
    if (s0 + 8 <= nsym) {
        stream_store(reinterpret_cast<uint4 *>(out + s0), a);
        stream_store(reinterpret_cast<uint4 *>(out + s0 + 4), b);
    } else {
        const uint32_t v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (s0 + i < nsym) out[s0 + i] = v[i];
    }
}

int lz_check(const char *who, int64_t nbytes)
{
    PM_REQUIRE(nbytes >= 0 && nbytes % 4 == 0, "%s: nbytes must be a non-negative multiple of 4 (got %lld)", who,
               (long long)nbytes);
    PM_REQUIRE(nbytes + LZ_BLOCK_BYTES <= (1ll << 31), "%s: nbytes too large for int32 offsets (%lld)", who,
               (long long)nbytes);
    return 0;
}

} // namespace
} // namespace pm

using namespace pm;

extern "C" int64_t planmoe_lz_blocks(int64_t nbytes)
{
    return nbytes <= 0 ? 0 : (nbytes + LZ_BLOCK_BYTES - 1) / LZ_BLOCK_BYTES;
}

extern "C" size_t planmoe_lz_workspace_bytes(int64_t nbytes)
{
    const int64_t groups = (planmoe_lz_blocks(nbytes) + LZ_WAVES - 1) / LZ_WAVES;
    return round_up(8 + 8 * (size_t)groups, 256);
}

extern "C" int planmoe_lz_compress(const void *input, int64_t nbytes, int32_t *flag_offsets,
                                   int32_t *data_offsets, uint8_t *flags, uint8_t *data, void *workspace,
                                   size_t workspace_bytes, void *stream)
{
    if (lz_check("planmoe_lz_compress", nbytes)) return 1;
    PM_REQUIRE(flag_offsets && data_offsets, "planmoe_lz_compress: offset tables must not be NULL");
    hipStream_t st = (hipStream_t)stream;
    const int64_t blocks = planmoe_lz_blocks(nbytes);
    if (blocks == 0) {
        fill_u32((uint32_t *)flag_offsets, 1, 0u, st);
        fill_u32((uint32_t *)data_offsets, 1, 0u, st);
        PM_LAUNCH_CHECK("planmoe_lz_compress");
        return 0;
    }
    PM_REQUIRE(input && flags && data, "planmoe_lz_compress: NULL argument");
    PM_REQUIRE(aligned16(input) && aligned16(flags) && aligned16(data),
               "planmoe_lz_compress: input, flags and data must be 16-byte aligned");
    PM_REQUIRE(workspace && workspace_bytes >= planmoe_lz_workspace_bytes(nbytes) &&
               (reinterpret_cast<uintptr_t>(workspace) & 7u) == 0,
               "planmoe_lz_compress: workspace too small or not 8-byte aligned");
    const int64_t groups = (blocks + LZ_WAVES - 1) / LZ_WAVES;
    fill_u32((uint32_t *)workspace, 2 + 2 * (size_t)groups, 0u, st);
    lz_compress_kernel<<<(unsigned)groups, LZ_WAVES * WAVE, 0, st>>>(
        (const uint32_t *)input, nbytes / 4, blocks, flag_offsets, data_offsets, flags, data, (uint32_t *)workspace);
    const int64_t flag_chunks = blocks * (LZ_SYMS / 8) / 64, data_chunks = blocks * LZ_BLOCK_BYTES / 64;
    lz_clear_slack_kernel<<<(unsigned)((flag_chunks + data_chunks + 255) / 256), 256, 0, st>>>(
        flag_offsets, data_offsets, blocks, flags, data, flag_chunks);
    PM_LAUNCH_CHECK("planmoe_lz_compress");
    return 0;
}

extern "C" int planmoe_lz_decompress(void *output, int64_t nbytes, const int32_t *flag_offsets,
                                     const int32_t *data_offsets, const uint8_t *flags, const uint8_t *data,
                                     void *stream)
{
    if (lz_check("planmoe_lz_decompress", nbytes)) return 1;
    const int64_t blocks = planmoe_lz_blocks(nbytes);
    if (blocks == 0) return 0;
    PM_REQUIRE(output && flag_offsets && data_offsets && flags && data, "planmoe_lz_decompress: NULL argument");
    PM_REQUIRE(aligned16(output) && (reinterpret_cast<uintptr_t>(data) & 3u) == 0,
               "planmoe_lz_decompress: output must be 16-byte and data 4-byte aligned");
    const int64_t groups = (blocks + LZ_WAVES - 1) / LZ_WAVES;
    lz_decompress_kernel<<<(unsigned)groups, LZ_WAVES * WAVE, 0, (hipStream_t)stream>>>(
        (uint32_t *)output, nbytes / 4, blocks, flag_offsets, data_offsets, flags, data);
    PM_LAUNCH_CHECK("planmoe_lz_decompress");
    return 0;
}
