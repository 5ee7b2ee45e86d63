// GPULZ ("lz") lossless codec for gfx950: byte-identical streams to the reference's
// lz_compress / lz_decompress (custom/compressor/gpulz.cu), built differently.
//
// One wavefront codes one block of 512 symbols (2048 bytes), lane l owning the 8 consecutive
// symbols 8l .. 8l+7:
//   match   every lane keeps the 39 symbols before its last one in registers and tests its 8
//           symbols against their 32-symbol windows (256 compares, no memory traffic).  A
//           position has a match exactly when its symbol occurs in its window; a block where
//           none does is stored as it is.  Otherwise the comparisons are kept as one 32-bit hit
//           mask per position, and the reference's matcher (gpulz.cu:46-85) walks those masks
//           instead of the symbols: a run grows while the next positions hit at the same
//           distance, 8 positions per step.  A block of one repeated value (an empty capacity
//           slot) has a closed form and is not analysed at all.
//   parse   the greedy token walk (gpulz.cu:98-127, one thread there) advances a whole run of
//           literals or one match per step with ballots and scalar bit scans.
//   pack    token ranks and byte offsets come from one packed wave scan; flags and token bytes
//           are put together in LDS and copied out with aligned word stores.
// The launches: sizes of every block (match + parse, nothing written but two integers and a
// class byte per block), an in-place exclusive scan of the sizes (chunks, then chunk totals),
// placement (stored blocks are copied straight through, the others analysed again and packed at
// their final offset), and a launch that zeroes what lies beyond the totals.  The reference
// stages every block at a fixed stride in a buffer as large as the input, scans with a library
// call and copies everything once more (gpulz.cu:148-211, 460-494, 220-258); here no
// full-size temporary exists and no work-group ever waits for another.
#include "common.hpp"

namespace pm {
namespace {

constexpr int LZ_SYMS = 512;             // symbols per block (gpulz.cu:6 / sizeof(float))
constexpr int LZ_WINDOW = 32;            // gpulz.cu:12
constexpr int LZ_BLOCK_BYTES = 2048;
constexpr int LZ_WAVES = 8;              // blocks per work-group
constexpr int LZ_SCAN_CHUNK = 8192;      // table entries scanned by one work-group
constexpr int LZ_MAX_CHUNKS = 256;       // (2^31 / 2048 + 1) / 8192 rounded up to the scan's width
constexpr uint32_t NAN_WINDOW = 0x7f800002u;   // key of a NaN seen as a window symbol ...
constexpr uint32_t NAN_AHEAD = 0x7f800001u;    // ... and as a look-ahead symbol: never equal
enum : uint8_t { LZ_STORED = 0, LZ_CONSTANT = 1, LZ_GENERAL = 2 };

// float equality on bit patterns: both zeros share a key, NaNs get a key per role
__device__ __forceinline__ uint32_t window_key(uint32_t bits)
{
    const float f = __uint_as_float(bits);
    const bool is_nan = __builtin_amdgcn_classf(f, 0x003);          // signalling or quiet NaN
    const bool is_zero = __builtin_amdgcn_classf(f, 0x060);         // -0 or +0
    return is_nan ? NAN_WINDOW : (is_zero ? 0u : bits);
}
__device__ __forceinline__ uint32_t ahead_key(uint32_t wkey) { return wkey == NAN_WINDOW ? NAN_AHEAD : wkey; }

// m = 2 * m + (a == b): the comparison lands in the carry, the add-with-carry shifts it in.
// (Written out so that the compiler does not keep these comparisons and the ones of the quick
// any-hit test as one set of 256 live lane masks.)
__device__ __forceinline__ uint32_t shift_in_equal(uint32_t m, uint32_t a, uint32_t b)
{
    // gfx950 wants two wait states between a VALU write of VCC and a VALU read of it
    asm("v_cmp_eq_u32 vcc, %1, %2\n\ts_nop 1\n\tv_addc_co_u32 %0, vcc, %0, %0, vcc"
        : "+v"(m) : "v"(a), "v"(b) : "vcc");
    return m;
}

// 16 bytes at an even address: token bytes start wherever the blocks before them end.  Global
// memory takes such accesses as they are.
typedef pm_u32x4 __attribute__((aligned(2))) lz_u32x4_a2;

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

// what a wavefront knows about its block after the analysis
struct LzBlock {
    uint32_t lens_lo, lens_hi, offs_lo, offs_hi;   // best match per owned position, one byte each
    uint32_t match_mask, start_mask;               // owned positions with a match / that start a token
    uint32_t tok_base, byte_base;                  // tokens and token bytes before this lane
    uint32_t flag_bytes, data_bytes;               // sizes of the block
};

// 8 consecutive symbols per lane, zero beyond the end of the input
__device__ __forceinline__ void lz_load(const uint32_t *__restrict__ in, int64_t nsym, int64_t block, int lane,
                                        uint32_t (&raw)[8])
{
    const int64_t s0 = block * LZ_SYMS + 8 * lane;
    if (s0 + 8 <= nsym) {
        const uint4 a = *reinterpret_cast<const uint4 *>(in + s0);
        const uint4 b = *reinterpret_cast<const uint4 *>(in + s0 + 4);
        raw[0] = a.x; raw[1] = a.y; raw[2] = a.z; raw[3] = a.w;
        raw[4] = b.x; raw[5] = b.y; raw[6] = b.z; raw[7] = b.w;
    } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) raw[i] = s0 + i < nsym ? in[s0 + i] : 0u;
    }
}

// Class of the block and, for LZ_GENERAL, everything in `b`.  keys: 544 words of LDS owned by
// the wavefront.  All lanes of the wavefront call it together.
__device__ __forceinline__ int lz_analyse(const uint32_t (&raw)[8], uint32_t *keys, int lane, LzBlock &b)
{
    keys = static_cast<uint32_t *>(__builtin_assume_aligned(keys, 16));
    uint32_t own[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) own[i] = window_key(raw[i]);

    // ---- one repeated value: tokens L (1,1) (2,2) (4,4) (8,8) (16,16) and (32,32) to the end
    const uint32_t first = __builtin_amdgcn_readfirstlane(own[0]);
    uint64_t differ = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) differ |= __ballot(own[i] != first);
    if (first != NAN_WINDOW && differ == 0) {
        b.flag_bytes = 3;
        b.data_bytes = 44;
        return LZ_CONSTANT;
    }

    if (lane < LZ_WINDOW / 4)
        *reinterpret_cast<uint4 *>(keys + 4 * lane) = make_uint4(NAN_WINDOW, NAN_WINDOW, NAN_WINDOW, NAN_WINDOW);
    *reinterpret_cast<uint4 *>(keys + LZ_WINDOW + 8 * lane) = make_uint4(own[0], own[1], own[2], own[3]);
    *reinterpret_cast<uint4 *>(keys + LZ_WINDOW + 8 * lane + 4) = make_uint4(own[4], own[5], own[6], own[7]);
    wave_sync();

    // ---- which positions see their symbol in their window
    uint32_t win[40];                                   // keys[8l .. 8l+39] = positions 8l-32 .. 8l+7
#pragma unroll
    for (int q = 0; q < 10; ++q) {
        const uint4 v = *reinterpret_cast<const uint4 *>(keys + 8 * lane + 4 * q);
        win[4 * q] = v.x; win[4 * q + 1] = v.y; win[4 * q + 2] = v.z; win[4 * q + 3] = v.w;
    }
    uint64_t hit[8], some = 0;                          // lane masks, kept in scalar registers
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t k = ahead_key(own[i]);
        hit[i] = 0;
#pragma unroll
        for (int j = 0; j < LZ_WINDOW; ++j) hit[i] |= __ballot(k == win[i + j]);
        some |= hit[i];
    }
    if (some == 0) {                                    // 512 literals, 64 zero flag bytes
        wave_sync();                                    // the keys may be overwritten by the next block
        b.flag_bytes = LZ_SYMS / 8;
        b.data_bytes = LZ_BLOCK_BYTES;
        return LZ_STORED;
    }
    uint32_t any = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) any |= (uint32_t)((hit[i] >> lane) & 1u) << i;

    // ---- hit masks: bit j of hits[i] = symbol 8l+i equals window symbol 8l+i-32+j.
    // They hold all the matcher needs: while symbol p+r still equals window symbol w+r, bit
    // (w - p + 32) of the mask of position p+r is set.
    uint32_t hits[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        hits[i] = 0;
        if (hit[i] == 0) continue;
        const uint32_t k = ahead_key(own[i]);
        uint32_t m = 0;
#pragma unroll
        for (int j = LZ_WINDOW - 1; j >= 0; --j) m = shift_in_equal(m, k, win[i + j]);
        hits[i] = m;
    }
    uint32_t *hmask = keys;                             // the keys are all in registers by now
    wave_sync();
    *reinterpret_cast<uint4 *>(hmask + 8 * lane) = make_uint4(hits[0], hits[1], hits[2], hits[3]);
    *reinterpret_cast<uint4 *>(hmask + 8 * lane + 4) = make_uint4(hits[4], hits[5], hits[6], hits[7]);
    wave_sync();

    // ---- the reference's matcher (gpulz.cu:46-85) on the masks: a run starts at the next hit,
    // grows while the following positions hit at the same distance, and the window symbol after
    // a run is consumed by the comparison that ended it
    b.lens_lo = b.lens_hi = b.offs_lo = b.offs_hi = b.match_mask = 0;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        if (hit[i] == 0) continue;
        uint32_t len = 0, off = 0;
        if ((any >> i) & 1) {
            const int p = 8 * lane + i;
            const uint32_t room = (uint32_t)(LZ_SYMS - p);              // symbols left in the block
            uint32_t j = 0;
            while (j < (uint32_t)LZ_WINDOW) {
                const uint32_t rest = hits[i] & (0xffffffffu << j);
                if (rest == 0) break;
                const uint32_t j0 = __builtin_ctz(rest);
                // the run ends with the window (32 - j0 symbols from its start) or the block
                const uint32_t limit = min((uint32_t)LZ_WINDOW - j0, room);
                uint32_t r = 1;
                while (r < limit) {                     // 8 positions per step; words past the block are cut off by limit
                    uint32_t ones = 0;
#pragma unroll
                    for (int t = 0; t < 8; ++t) ones |= ((hmask[p + r + t] >> j0) & 1u) << t;
                    const uint32_t cnt = __builtin_ctz(~ones);
                    r += cnt;
                    if (cnt < 8) break;
                }
                r = min(r, limit);
                if (r > len) { len = r; off = LZ_WINDOW - j0; }
                if (r >= room) break;                   // the look-ahead reached the end of the block
                j = j0 + r + 1;
            }
        }
        if (i < 4) { b.lens_lo |= len << (8 * i); b.offs_lo |= off << (8 * i); }
        else       { b.lens_hi |= len << (8 * (i - 4)); b.offs_hi |= off << (8 * (i - 4)); }
        b.match_mask |= (uint32_t)(len != 0) << i;
    }
    wave_sync();                                        // hmask is the key area of the next block

    // ---- greedy parse: [cur, nxt) is a run of literals, nxt the next position with a match
    b.start_mask = 0;
    int cur = 0;
    while (cur < LZ_SYMS) {
        const int rel = cur - 8 * lane;
        const uint32_t mm = rel >= 8 ? 0u : (rel <= 0 ? b.match_mask : (b.match_mask & (0xffu << rel)));
        const uint64_t bal = __ballot(mm != 0);
        int nxt = LZ_SYMS, step = 0;
        if (bal != 0) {
            const int owner = __builtin_ctzll(bal);
            const uint32_t m = __builtin_amdgcn_readlane(mm, owner);
            const int bit = __builtin_ctz(m);
            nxt = 8 * owner + bit;
            const uint32_t lo = __builtin_amdgcn_readlane(b.lens_lo, owner);
            const uint32_t hi = __builtin_amdgcn_readlane(b.lens_hi, owner);
            step = (int)(((bit < 4 ? lo : hi) >> (8 * (bit & 3))) & 0xffu);
        }
        // the literals and, when there is one, the match token at nxt all start a token
        const int last = bal != 0 ? nxt + 1 : nxt;
        const int lo_b = min(max(cur - 8 * lane, 0), 8);
        const int hi_b = min(max(last - 8 * lane, 0), 8);
        b.start_mask |= ((1u << hi_b) - 1u) & ~((1u << lo_b) - 1u);
        cur = nxt + step;                              // step >= 1 whenever nxt < 512
    }

    // ---- sizes: tokens and token bytes before this lane, totals of the block
    const uint32_t ntok = __popc(b.start_mask);
    const uint32_t nmatch = __popc(b.start_mask & b.match_mask);
    uint32_t total;
    const uint32_t before = wave_exclusive_sum(ntok | ((4u * ntok - 2u * nmatch) << 16), total);
    b.tok_base = before & 0xffffu;
    b.byte_base = before >> 16;
    b.flag_bytes = ((total & 0xffffu) + 7u) >> 3;
    b.data_bytes = total >> 16;
    return LZ_GENERAL;
}

// ---- launch 1: sizes and class of every block
__global__ __launch_bounds__(LZ_WAVES * WAVE) void lz_sizes_kernel(
    const uint32_t *__restrict__ in, int64_t nsym, int64_t blocks, int32_t *__restrict__ flag_off,
    int32_t *__restrict__ data_off, uint8_t *__restrict__ cls)
{
    __shared__ __attribute__((aligned(16))) uint32_t keys[LZ_WAVES][LZ_WINDOW + LZ_SYMS];
    const int lane = lane_id();
    const int wave = (int)(threadIdx.x >> 6);
    const int64_t block = (int64_t)blockIdx.x * LZ_WAVES + wave;
    if (block >= blocks) return;                       // no work-group barrier below
    uint32_t raw[8];
    lz_load(in, nsym, block, lane, raw);
    LzBlock b;
    const int c = lz_analyse(raw, keys[wave], lane, b);
    if (lane == 0) {
        flag_off[block] = (int32_t)b.flag_bytes;
        data_off[block] = (int32_t)b.data_bytes;
        cls[block] = (uint8_t)c;
        if (block == blocks - 1) { flag_off[blocks] = 0; data_off[blocks] = 0; }
    }
}

// ---- launch 2: both tables, in place: exclusive sums inside chunks of 8192 entries, chunk totals
__global__ __launch_bounds__(256) void lz_scan_chunks_kernel(int32_t *__restrict__ flag_off,
                                                            int32_t *__restrict__ data_off, int64_t entries,
                                                            uint32_t *__restrict__ totals)
{
    __shared__ uint32_t wave_tot[4];
    constexpr int PER = LZ_SCAN_CHUNK / 256;            // 32 entries per thread, contiguous
    const int lane = lane_id(), wave = (int)(threadIdx.x >> 6);
    const int64_t e0 = (int64_t)blockIdx.x * LZ_SCAN_CHUNK + (int64_t)threadIdx.x * PER;
    const bool whole = e0 + PER <= entries;
    for (int a = 0; a < 2; ++a) {
        int32_t *t = a ? data_off : flag_off;
        uint32_t v[PER];
        if (whole) {
#pragma unroll
            for (int q = 0; q < PER / 4; ++q) {
                const int4 w = *reinterpret_cast<const int4 *>(t + e0 + 4 * q);
                v[4 * q] = (uint32_t)w.x; v[4 * q + 1] = (uint32_t)w.y; v[4 * q + 2] = (uint32_t)w.z; v[4 * q + 3] = (uint32_t)w.w;
            }
        } else {
#pragma unroll
            for (int q = 0; q < PER; ++q) v[q] = e0 + q < entries ? (uint32_t)t[e0 + q] : 0u;
        }
        uint32_t sum = 0;
#pragma unroll
        for (int q = 0; q < PER; ++q) sum += v[q];
        uint32_t total;
        uint32_t run = wave_exclusive_sum(sum, total);
        __syncthreads();                                // the totals of the other table have been read
        if (lane == 0) wave_tot[wave] = total;
        __syncthreads();
        for (int w = 0; w < wave; ++w) run += wave_tot[w];
#pragma unroll
        for (int q = 0; q < PER; ++q) { const uint32_t x = v[q]; v[q] = run; run += x; }
        if (whole) {
#pragma unroll
            for (int q = 0; q < PER / 4; ++q)
                *reinterpret_cast<int4 *>(t + e0 + 4 * q) =
                    make_int4((int)v[4 * q], (int)v[4 * q + 1], (int)v[4 * q + 2], (int)v[4 * q + 3]);
        } else {
#pragma unroll
            for (int q = 0; q < PER; ++q)
                if (e0 + q < entries) t[e0 + q] = (int32_t)v[q];
        }
        if (threadIdx.x == 255) totals[2 * blockIdx.x + a] = run;   // the last thread ends with the chunk's sum
    }
}

// ---- launch 3: chunk totals -> sums over all earlier chunks (one work-group)
__global__ __launch_bounds__(LZ_MAX_CHUNKS) void lz_scan_totals_kernel(const uint32_t *__restrict__ totals,
                                                                      int chunks, uint32_t *__restrict__ bases)
{
    __shared__ uint32_t wave_tot[2][LZ_MAX_CHUNKS / WAVE];
    const int lane = lane_id(), wave = (int)(threadIdx.x >> 6);
    uint32_t before[2];
#pragma unroll
    for (int a = 0; a < 2; ++a) {
        const uint32_t v = (int)threadIdx.x < chunks ? totals[2 * threadIdx.x + a] : 0u;
        uint32_t total;
        before[a] = wave_exclusive_sum(v, total);
        if (lane == 0) wave_tot[a][wave] = total;
    }
    __syncthreads();
    if ((int)threadIdx.x < chunks) {
#pragma unroll
        for (int a = 0; a < 2; ++a) {
            uint32_t run = before[a];
            for (int w = 0; w < wave; ++w) run += wave_tot[a][w];
            bases[2 * threadIdx.x + a] = run;
        }
    }
}

struct __attribute__((aligned(16))) LzPlaceShared {
    uint32_t keys[LZ_WAVES][LZ_WINDOW + LZ_SYMS];
    uint16_t stage[LZ_WAVES][LZ_BLOCK_BYTES / 2];   // token bytes of the block
    uint32_t flagw[LZ_WAVES][16];                   // flag bits of the block
};

// ---- launch 4: every block to its final place
__global__ __launch_bounds__(LZ_WAVES * WAVE) void lz_place_kernel(
    const uint32_t *__restrict__ in, int64_t nsym, int64_t blocks, int32_t *__restrict__ flag_off,
    int32_t *__restrict__ data_off, const uint8_t *__restrict__ cls, const uint32_t *__restrict__ bases,
    uint8_t *__restrict__ flags, uint8_t *__restrict__ data)
{
    __shared__ LzPlaceShared sh;
    const int lane = lane_id();
    const int wave = (int)(threadIdx.x >> 6);
    const int64_t block = (int64_t)blockIdx.x * LZ_WAVES + wave;
    if (block >= blocks) return;                       // no work-group barrier below

    uint32_t raw[8];
    lz_load(in, nsym, block, lane, raw);
    const int64_t chunk = block / LZ_SCAN_CHUNK;
    const uint32_t fbase = (uint32_t)flag_off[block] + bases[2 * chunk];
    const uint32_t dbase = (uint32_t)data_off[block] + bases[2 * chunk + 1];
    int c = cls[block];
    c = __builtin_amdgcn_readfirstlane(c);
    // never let a wrong table move a write out of the buffers
    const uint32_t fb = min(fbase, (uint32_t)(block * (LZ_SYMS / 8)));
    const uint32_t db = min(dbase, (uint32_t)(block * LZ_BLOCK_BYTES)) & ~1u;
    if (lane == 0) {
        flag_off[block] = (int32_t)fbase;
        data_off[block] = (int32_t)dbase;
        if (block == blocks - 1) {                     // the totals sit in the entry after the last block
            const int64_t ce = blocks / LZ_SCAN_CHUNK;
            flag_off[blocks] = (int32_t)((uint32_t)flag_off[blocks] + bases[2 * ce]);
            data_off[blocks] = (int32_t)((uint32_t)data_off[blocks] + bases[2 * ce + 1]);
        }
    }
    uint8_t *dst = data + db;
    uint16_t *stage = sh.stage[wave];
    uint32_t *flagw = sh.flagw[wave];
    uint32_t flag_bytes, data_bytes;

    if (c == LZ_STORED) {                              // 512 literals: the block itself, at an even address
        flags[(size_t)fb + lane] = 0;
        lz_u32x4_a2 *to = reinterpret_cast<lz_u32x4_a2 *>(dst);
        __builtin_nontemporal_store(pm_u32x4{raw[0], raw[1], raw[2], raw[3]}, to + 2 * lane);
        __builtin_nontemporal_store(pm_u32x4{raw[4], raw[5], raw[6], raw[7]}, to + 2 * lane + 1);
        return;
    } else if (c == LZ_CONSTANT) {
        flag_bytes = 3;
        data_bytes = 44;
        const uint32_t sym0 = __builtin_amdgcn_readfirstlane(raw[0]);
        if (lane < 22) {
            const uint32_t n = lane < 7 ? 1u << (lane - 2) : 32u;          // lanes 2..21: the 20 matches
            stage[lane] = (uint16_t)(lane == 0 ? sym0 : lane == 1 ? sym0 >> 16 : n | (n << 8));
        }
        if (lane == 0) flagw[0] = 0x001ffffeu;
    } else {
        LzBlock b;
        if (lz_analyse(raw, sh.keys[wave], lane, b) != LZ_GENERAL) return;   // the input changed between the launches
        flag_bytes = b.flag_bytes;
        data_bytes = b.data_bytes;
        if (lane < 16) flagw[lane] = 0;
        wave_sync();
        uint32_t bits = 0, nb = 0, at = b.byte_base >> 1;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if ((b.start_mask >> i) & 1) {
                if ((b.match_mask >> i) & 1) {
                    const uint32_t l = ((i < 4 ? b.lens_lo : b.lens_hi) >> (8 * (i & 3))) & 0xffu;
                    const uint32_t o = ((i < 4 ? b.offs_lo : b.offs_hi) >> (8 * (i & 3))) & 0xffu;
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
            const uint64_t wide = (uint64_t)bits << (b.tok_base & 31u);
            atomicOr(&flagw[b.tok_base >> 5], (uint32_t)wide);
            if ((uint32_t)(wide >> 32)) atomicOr(&flagw[(b.tok_base >> 5) + 1], (uint32_t)(wide >> 32));
        }
    }
    wave_sync();
    if ((uint32_t)lane < flag_bytes)
        flags[(size_t)fb + lane] = (uint8_t)(flagw[lane >> 2] >> (8 * (lane & 3)));

    // token bytes: the offset is even; 2 bytes up to a 4-byte boundary, whole words, 2 bytes at the end
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

// ---- launch 5: zero flags[flag_off[blocks] ..) and data[data_off[blocks] ..): 16 bytes per lane and step,
// neighbouring lanes at neighbouring addresses (the piece the used part ends in byte by byte)
__global__ __launch_bounds__(256) void lz_clear_slack_kernel(const int32_t *__restrict__ flag_off,
                                                            const int32_t *__restrict__ data_off,
                                                            int64_t blocks, uint8_t *__restrict__ flags,
                                                            uint8_t *__restrict__ data)
{
    const int64_t tid = (int64_t)blockIdx.x * 256 + threadIdx.x, nthreads = (int64_t)gridDim.x * 256;
#pragma unroll
    for (int a = 0; a < 2; ++a) {
        uint8_t *buf = a ? data : flags;
        const int64_t size = a ? blocks * LZ_BLOCK_BYTES : blocks * (LZ_SYMS / 8);     // multiples of 64
        const int64_t used = min(max((int64_t)(a ? data_off[blocks] : flag_off[blocks]), (int64_t)0), size);
        for (int64_t lo = (used / 16 + tid) * 16; lo < size; lo += nthreads * 16) {
            if (lo >= used) {
                *reinterpret_cast<uint4 *>(buf + lo) = make_uint4(0, 0, 0, 0);
            } else {
                for (int64_t q = used; q < lo + 16; ++q) buf[q] = 0;
            }
        }
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

// A block with matches (or at an odd address): tokens are laid out with two wave scans, literals
// land in parallel, matches follow in token order.  bytes / sym: LDS of the wavefront.
__device__ __forceinline__ void lz_decode_block(uint32_t *__restrict__ out, int64_t nsym, int64_t block, int lane,
                                                uint32_t fb, uint32_t nflag, int64_t d0, uint32_t nbytes,
                                                const uint8_t *__restrict__ data, uint32_t *bytes, uint32_t *sym)
{
    const int64_t s0 = block * LZ_SYMS + 8 * lane;
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

constexpr int LZ_DEC_PER = 4;            // blocks per wavefront: their loads are in flight together

__global__ __launch_bounds__(LZ_WAVES * WAVE) void lz_decompress_kernel(
    uint32_t *__restrict__ out, int64_t nsym, int64_t blocks, const int32_t *__restrict__ flag_off,
    const int32_t *__restrict__ data_off, const uint8_t *__restrict__ flags,
    const uint8_t *__restrict__ data)
{
    __shared__ LzDecodeShared sh;
    const int lane = lane_id();
    const int wave = (int)(threadIdx.x >> 6);
    const int64_t first = ((int64_t)blockIdx.x * LZ_WAVES + wave) * LZ_DEC_PER;
    if (first >= blocks) return;                       // no work-group barrier below

    // All loads below are unconditional, at clamped addresses: a load under a branch would make
    // every later wait drain the whole queue, and the blocks would be fetched one after the other.
    const int64_t fcap = blocks * (LZ_SYMS / 8), dcap = blocks * LZ_BLOCK_BYTES;
    int32_t fo[LZ_DEC_PER + 1], dofs[LZ_DEC_PER + 1];
#pragma unroll
    for (int u = 0; u <= LZ_DEC_PER; ++u) {
        const int64_t e = min(first + u, blocks);
        fo[u] = flag_off[e];
        dofs[u] = data_off[e];
    }
    // offsets of a stream of this coder ascend and stay inside the buffers; clamp all the same
    int64_t f0[LZ_DEC_PER], d0[LZ_DEC_PER];
    uint32_t nflag[LZ_DEC_PER], nbytes[LZ_DEC_PER], fb[LZ_DEC_PER];
    bool direct[LZ_DEC_PER];
    pm_u32x4 va[LZ_DEC_PER], vb[LZ_DEC_PER];
#pragma unroll
    for (int u = 0; u < LZ_DEC_PER; ++u) {
        const int64_t block = min(first + u, blocks - 1);
        f0[u] = min(max((int64_t)fo[u], (int64_t)0), fcap);
        const int64_t f1 = min(max((int64_t)fo[u + 1], f0[u]), min(f0[u] + LZ_SYMS / 8, fcap));
        d0[u] = min(max((int64_t)dofs[u], (int64_t)0), dcap) & ~(int64_t)1;
        const int64_t d1 = min(max((int64_t)dofs[u + 1], d0[u]), min(d0[u] + LZ_BLOCK_BYTES, dcap));
        nflag[u] = (uint32_t)(f1 - f0[u]);
        nbytes[u] = (uint32_t)(d1 - d0[u]);
        // a stored block (512 literals) is its own bytes: fetch them before the flags are known
        direct[u] = nflag[u] == LZ_SYMS / 8 && nbytes[u] == LZ_BLOCK_BYTES && block * LZ_SYMS + LZ_SYMS <= nsym;
    }
#pragma unroll
    for (int u = 0; u < LZ_DEC_PER; ++u) {
        fb[u] = flags[min(f0[u] + lane, fcap - 1)];                        // lane l: tokens 8l .. 8l+7
        const lz_u32x4_a2 *src = reinterpret_cast<const lz_u32x4_a2 *>(data + (direct[u] ? d0[u] : 0));
        va[u] = src[lane];                             // 1 KB per instruction
        vb[u] = src[lane + WAVE];
    }
#pragma unroll
    for (int u = 0; u < LZ_DEC_PER; ++u) {
        const int64_t block = first + u;
        if (block >= blocks) break;
        const uint32_t mine = (uint32_t)lane < nflag[u] ? fb[u] : 0u;
        if (direct[u] && __ballot(mine != 0) == 0) {
            pm_u32x4 *dst = reinterpret_cast<pm_u32x4 *>(out + block * LZ_SYMS);
            __builtin_nontemporal_store(va[u], dst + lane);
            __builtin_nontemporal_store(vb[u], dst + lane + WAVE);
        } else {
            lz_decode_block(out, nsym, block, lane, mine, nflag[u], d0[u], nbytes[u], data, sh.bytes[wave], sh.out[wave]);
            wave_sync();                               // the LDS of the wavefront serves the next block
        }
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

// workspace: class byte per block | chunk totals | chunk bases
static size_t lz_class_bytes(int64_t blocks) { return round_up((size_t)blocks, 256); }

extern "C" size_t planmoe_lz_workspace_bytes(int64_t nbytes)
{
    return lz_class_bytes(planmoe_lz_blocks(nbytes)) + 2 * (2 * LZ_MAX_CHUNKS * sizeof(uint32_t));
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
    PM_REQUIRE(aligned16(input) && aligned16(flags) && aligned16(data) && aligned16(flag_offsets) &&
               aligned16(data_offsets),
               "planmoe_lz_compress: input, flags, data and the offset tables must be 16-byte aligned");
    PM_REQUIRE(workspace && workspace_bytes >= planmoe_lz_workspace_bytes(nbytes) &&
               (reinterpret_cast<uintptr_t>(workspace) & 3u) == 0,
               "planmoe_lz_compress: workspace too small or not 4-byte aligned");
    uint8_t *cls = (uint8_t *)workspace;
    uint32_t *totals = (uint32_t *)(cls + lz_class_bytes(blocks));
    uint32_t *bases = totals + 2 * LZ_MAX_CHUNKS;
    const int64_t groups = (blocks + LZ_WAVES - 1) / LZ_WAVES;
    const int64_t entries = blocks + 1;
    const int chunks = (int)((entries + LZ_SCAN_CHUNK - 1) / LZ_SCAN_CHUNK);      // <= 128 below 2^31 bytes
    lz_sizes_kernel<<<(unsigned)groups, LZ_WAVES * WAVE, 0, st>>>((const uint32_t *)input, nbytes / 4, blocks,
                                                                flag_offsets, data_offsets, cls);
    lz_scan_chunks_kernel<<<chunks, 256, 0, st>>>(flag_offsets, data_offsets, entries, totals);
    lz_scan_totals_kernel<<<1, LZ_MAX_CHUNKS, 0, st>>>(totals, chunks, bases);
    lz_place_kernel<<<(unsigned)groups, LZ_WAVES * WAVE, 0, st>>>((const uint32_t *)input, nbytes / 4, blocks,
                                                                flag_offsets, data_offsets, cls, bases, flags, data);
    const int64_t slack_chunks = (blocks * LZ_BLOCK_BYTES / 16 + 255) / 256;          // enough for all of data
    lz_clear_slack_kernel<<<(unsigned)min(slack_chunks, (int64_t)4096), 256, 0, st>>>(flag_offsets, data_offsets,
                                                                                   blocks, flags, data);
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
    const int64_t groups = (blocks + LZ_WAVES * LZ_DEC_PER - 1) / (LZ_WAVES * LZ_DEC_PER);
    lz_decompress_kernel<<<(unsigned)groups, LZ_WAVES * WAVE, 0, (hipStream_t)stream>>>(
        (uint32_t *)output, nbytes / 4, blocks, flag_offsets, data_offsets, flags, data);
    PM_LAUNCH_CHECK("planmoe_lz_decompress");
    return 0;
}
