// zfp fixed-rate float codec (stream-compatible with stock zfp 0.5.5), 1-D and 2-D.
//
// Takes the place of zfp_compress / zfp_decompress with the CUDA execution policy as called
// by ZfpCompressor (custom/compressor/zfpc.cpp:31-51, 66-84).  One thread owns one block
// (4 or 4x4 values): block-floating-point cast, lifting transform, negabinary reorder and the
// embedded bit-plane coder all run in registers; a block's bits leave the thread as NW
// 32-bit words (2-D rate 8: exactly one 16-byte store).  Loads are 16 bytes per lane per
// row, consecutive lanes taking consecutive blocks along the fastest axis.
#include "common.hpp"
#include <cmath>

namespace pm {

// The words of a block's bit stream are parked in LDS while the block is coded (word i of thread
// t at lds[i * 256 + t]): a register array would need a select per word on every flush, since
// the word index differs from lane to lane.
template <int NW>
struct BitWriter {
    uint32_t *slot;
    uint64_t acc;
    int fill;
    __device__ __forceinline__ void init(uint32_t *lds)
    {
        slot = lds + threadIdx.x;
#pragma unroll
        for (int i = 0; i < NW; ++i) slot[i * 256] = 0u;
        acc = 0; fill = 0;
    }
    // append the low n (<= 32) bits of v; bits of v above n must be zero
    __device__ __forceinline__ void put(uint32_t v, int n)
    {
        acc |= (uint64_t)v << fill;
        fill += n;
        if (fill >= 32) { *slot = (uint32_t)acc; slot += 256; acc >>= 32; fill -= 32; }
    }
    __device__ __forceinline__ void finish() { if (fill > 0) *slot = (uint32_t)acc; }
    __device__ __forceinline__ void words(uint32_t *lds, uint32_t *w) const
    {
#pragma unroll
        for (int i = 0; i < NW; ++i) w[i] = lds[i * 256 + threadIdx.x];
    }
};

// The decoder looks at the stream by bit position: the block's words sit in LDS (NW words per
// thread and three zero words behind them: an odd stride) and a look is neighbouring words
// funnel-shifted, so there is no refill state to carry and no branch in the reader.  A bit plane
// takes one look of 64 bits (a plane never uses more than 48) and is then parsed in registers: the
// group tests of a 2-D block eight stream bits at a time by table (gt16_step), except the plane the
// block's budget ends in, which is walked bit by bit.
// Streams of one or two words stay in a register pair that is shifted as bits are consumed.
template <int NW>
struct BitReader {
    static constexpr int STRIDE = NW + 3;
    const uint32_t *words;      // this thread's NW + 3 words in LDS
    int pos;
    uint64_t small;             // NW <= 2: the whole stream in a register pair instead
    __device__ __forceinline__ void init(uint32_t *lds, const uint32_t *w)
    {
        pos = 0;
        if constexpr (NW <= 2) {
            small = w[0];
            if constexpr (NW == 2) small |= (uint64_t)w[1] << 32;
            words = nullptr;
        } else {
            uint32_t *mine = lds + threadIdx.x * STRIDE;
#pragma unroll
            for (int i = 0; i < NW; ++i) mine[i] = w[i];
            mine[NW] = 0u;
            mine[NW + 1] = 0u;
            mine[NW + 2] = 0u;
            words = mine;
            small = 0;
        }
    }
    // the next 32 bits of the stream (zeros past its end)
    __device__ __forceinline__ uint32_t peek() const
    {
        if constexpr (NW <= 2) {
            return (uint32_t)small;                 // skip() keeps the register pair shifted
        } else {
            const int i = pos >> 5;
            return __builtin_amdgcn_alignbit(words[i + 1], words[i], pos & 31);
        }
    }
    // the next 64 bits
    __device__ __forceinline__ uint64_t peek64() const
    {
        if constexpr (NW <= 2) {
            return small;
        } else {
            const int i = pos >> 5, sh = pos & 31;
            const uint32_t w0 = words[i], w1 = words[i + 1], w2 = words[i + 2];
            return (uint64_t)__builtin_amdgcn_alignbit(w1, w0, sh) | ((uint64_t)__builtin_amdgcn_alignbit(w2, w1, sh) << 32);
        }
    }
    __device__ __forceinline__ void skip(int n)      // n <= 32 (NW <= 2), any n otherwise
    {
        if constexpr (NW <= 2) small >>= n;
        else pos += n;
    }
    __device__ __forceinline__ uint32_t get(int n)   // n <= 31
    {
        const uint32_t v = peek() & ((1u << n) - 1u);
        skip(n);
        return v;
    }
};

__device__ __forceinline__ void fwd_lift(int32_t &x, int32_t &y, int32_t &z, int32_t &w)
{
    x += w; x >>= 1; w -= x;
    z += y; z >>= 1; y -= z;
    x += z; x >>= 1; z -= x;
    w += y; w >>= 1; y -= w;
    w += y >> 1; y -= w >> 1;
}

__device__ __forceinline__ void inv_lift(int32_t &x, int32_t &y, int32_t &z, int32_t &w)
{
    y += w >> 1; w -= y >> 1;
    y += w; w = (int32_t)((uint32_t)w << 1); w -= y;
    z += x; x = (int32_t)((uint32_t)x << 1); x -= z;
    y += z; z = (int32_t)((uint32_t)z << 1); z -= y;
    w += x; x = (int32_t)((uint32_t)x << 1); x -= w;
}

__device__ __forceinline__ uint32_t to_negabinary(int32_t v) { return ((uint32_t)v + 0xaaaaaaaau) ^ 0xaaaaaaaau; }
__device__ __forceinline__ int32_t from_negabinary(uint32_t v) { return (int32_t)((v ^ 0xaaaaaaaau) - 0xaaaaaaaau); }

// 16 x 16 bit matrix transpose.  w[j] holds row 2j in its low and row 2j+1 in its high half;
// afterwards bit i of row k is what bit k of row i was.  Used to turn the upper halves of the 16
// coefficients of a 2-D block into their 16 upper bit planes (and back) in about 100
// instructions instead of 32 per plane.
__device__ __forceinline__ void transpose16(uint32_t (&w)[8])
{
    auto swap_blocks = [](uint32_t &a, uint32_t &b, int s, uint32_t m) {
        const uint32_t t = ((a >> s) ^ b) & m;
        b ^= t; a ^= t << s;
    };
#pragma unroll
    for (int j = 0; j < 4; ++j) swap_blocks(w[j], w[j + 4], 8, 0x00ff00ffu);
    swap_blocks(w[0], w[2], 4, 0x0f0f0f0fu); swap_blocks(w[1], w[3], 4, 0x0f0f0f0fu);
    swap_blocks(w[4], w[6], 4, 0x0f0f0f0fu); swap_blocks(w[5], w[7], 4, 0x0f0f0f0fu);
#pragma unroll
    for (int j = 0; j < 8; j += 2) swap_blocks(w[j], w[j + 1], 2, 0x33333333u);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const uint32_t t = ((w[j] >> 15) ^ w[j]) & 0x0000aaaau;
        w[j] ^= t | (t << 15);
    }
}

// sequency order of the 4x4 coefficients (index into the i + 4j block layout)
__device__ constexpr int perm2(int i)
{
    constexpr int P[16] = {0, 1, 4, 5, 2, 8, 6, 9, 3, 12, 10, 7, 13, 11, 14, 15};
    return P[i];
}

// Group-test code of one bit plane without a data-dependent loop.
// For the not yet significant part r of a plane (bit p = value nsig + p) zfp emits, segment by
// segment, a test bit '1', the zeros below the next one bit and that one bit; i.e. the bits of r
// up to its highest one with a '1' put in front of bit 0 and of every bit that follows a one.
// The table holds that expansion for 8 bits of r at a time: entry [prev][byte] = code in the low
// 16 bits, its length (8 + prev + ones among the low 7 bits) above.  What follows the highest
// one (a single '0' test bit, or nothing at the block end) and the implicit last one are a
// matter of the total length, see encode_block.
__device__ inline uint32_t group_code_entry(int prev, int byte)
{
    uint32_t code = 0; int len = 0;
    for (int p = 0; p < 8; ++p) {
        const int bit = (byte >> p) & 1;
        if (prev) { code |= 1u << len; ++len; }
        code |= (uint32_t)bit << len; ++len;
        prev = bit;
    }
    return code | ((uint32_t)len << 16);
}
// all 256 threads of the work-group; tab has 512 entries
__device__ __forceinline__ void group_code_table(uint32_t *tab)
{
    tab[threadIdx.x] = group_code_entry(0, threadIdx.x);
    tab[256 + threadIdx.x] = group_code_entry(1, threadIdx.x);
    __syncthreads();
}
__device__ __forceinline__ uint32_t low_bits(int n) { return (uint32_t)(((uint64_t)1 << n) - 1u); }   // n in 0..32

// N = values per block (4 or 16).  f is consumed; the block's maxbits = 32*NW bits land in bw.
template <int N, int NW>
__device__ __forceinline__ void encode_block(const float *f, BitWriter<NW> &bw, uint32_t *lds,
                                             const uint32_t *tab)
{
    bw.init(lds);
    float m = 0.f;
#pragma unroll
    for (int i = 0; i < N; ++i) m = fmaxf(m, fabsf(f[i]));
    if (!(m > 0.f)) return;                       // all-zero block: '0' flag and zero padding
    // frexp exponent clamped at 1 - 127, i.e. exponent field - 126 (a denormal maximum reads 0)
    const int field = (int)((__float_as_uint(m) >> 23) & 0xffu);
    const int emax = field - 126;
    bw.put(2u * (uint32_t)(emax + 127) + 1u, 9);

    // block-floating-point cast: q = (int32)(f * 2^(30 - emax)), x86 conversion on overflow
    const int se = 30 - emax;
    const float s = se > 127 ? INFINITY : __uint_as_float((uint32_t)(se + 127) << 23);
    int32_t q[N];
#pragma unroll
    for (int i = 0; i < N; ++i) {
        const float v = f[i] * s;
        // -2^31 itself converts to INT_MIN either way
        q[i] = fabsf(v) < 2147483648.0f ? (int32_t)v : (int32_t)0x80000000;
    }
    uint32_t u[N];
    if constexpr (N == 4) {
        fwd_lift(q[0], q[1], q[2], q[3]);
#pragma unroll
        for (int i = 0; i < 4; ++i) u[i] = to_negabinary(q[i]);
    } else {
#pragma unroll
        for (int y = 0; y < 4; ++y) fwd_lift(q[4 * y], q[4 * y + 1], q[4 * y + 2], q[4 * y + 3]);
#pragma unroll
        for (int x = 0; x < 4; ++x) fwd_lift(q[x], q[x + 4], q[x + 8], q[x + 12]);
#pragma unroll
        for (int i = 0; i < 16; ++i) u[i] = to_negabinary(q[perm2(i)]);
    }

    // embedded coding: bit planes from the top, group-tested, until the budget is spent
    int bits = 32 * NW - 9;
    int nsig = 0;
    auto code_plane = [&](uint32_t x) __attribute__((always_inline)) {
        const int mm = min(nsig, bits);
        bits -= mm;
        bw.put(x & ((1u << mm) - 1u), mm);
        if (nsig < N && bits > 0) {
            const uint32_t r = x >> mm;                   // mm == nsig here
            // r == 0 runs through the same formulas: top = -1, no code bits, length 1 (the '0')
            const int top = 31 - __clz((int)r), ones = __builtin_popcount(r);
            const uint32_t e0 = tab[256 + (r & 0xffu)];
            uint32_t code = e0 & 0xffffu;
            if constexpr (N > 8) {
                const uint32_t e1 = tab[((r >> 7) & 1u) * 256 + (r >> 8)];
                code |= (e1 & 0xffffu) << (e0 >> 16);
            }
            // cut after the highest one bit (not emitted when it is the block's last value),
            // then one more '0' test bit unless the block ends there
            const int last = nsig + top == N - 1;
            const int lt = top + 1 + ones - last;
            const int len = lt + (nsig + top + 1 < N ? 1 : 0);
            const int emit = min(len, bits);
            code &= low_bits(min(lt, emit));
            bw.put(code, emit);
            bits -= emit;
            nsig += top + 1;
        }
    };
    if constexpr (N == 16) {
        // planes 31..16 by one bit transpose of the coefficients' upper halves
        uint32_t w[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) w[j] = (u[2 * j] >> 16) | (u[2 * j + 1] & 0xffff0000u);
        transpose16(w);
#pragma unroll
        for (int k = 15; k >= 0; --k)
            if (bits > 0) code_plane((k & 1) ? w[k >> 1] >> 16 : w[k >> 1] & 0xffffu);
        for (int k = 15; k >= 0 && bits > 0; --k) {
            uint32_t x = 0;
#pragma unroll
            for (int i = 0; i < N; ++i) x |= ((u[i] >> k) & 1u) << i;
            code_plane(x);
        }
    } else {
        for (int k = 31; k >= 0 && bits > 0; --k) {
            uint32_t x = 0;
#pragma unroll
            for (int i = 0; i < N; ++i) x |= ((u[i] >> k) & 1u) << i;
            code_plane(x);
        }
    }
    bw.finish();
}

// ---- group tests of a 2-D block's bit plane, eight stream bits at a time
// The group-test bits of a plane are a walk with two states: a test bit is due (T), or the zeros of
// a run up to the next one bit are being read (R).  What eight stream bits do to that walk depends
// on the state and on how far away the block's last value is (its one is implied, and after it the
// plane ends without another test bit).  gt16_step works that out once per (state, distance, byte):
// bits 0..7 the one bits found (relative to the first value that was not significant), bits 8..11
// the values passed, bits 12..15 a code c: c <= 8 = the plane ended after c bits; 9 / 10 = all eight
// bits used and the walk goes on in state T / R.  The walk is zfp's own (decode_ints), minus the
// budget: a step that would use up the budget is not taken, see fast_plane16.
__host__ __device__ constexpr uint16_t gt16_step(int state, int r, uint32_t byte)
{
    const int last = r < 8 ? r : 99;            // the block's last value, if this step can reach it
    int n = 0, used = 0, st = state;
    uint32_t mask = 0;
    bool done = false;
    while (true) {
        if (st == 0) {
            if (n > last) { done = true; break; }
            if (used == 8) break;
            const uint32_t b = (byte >> used) & 1u; ++used;
            if (!b) { done = true; break; }
            st = 1;
        }
        bool out_of_bits = false;
        while (n != last) {
            if (used == 8) { out_of_bits = true; break; }
            const uint32_t b = (byte >> used) & 1u; ++used;
            if (b) break;
            ++n;
        }
        if (out_of_bits) break;
        mask |= 1u << n; ++n; st = 0;
        if (n > last) { done = true; break; }
    }
    const int c = done ? used : (st ? 10 : 9);
    return (uint16_t)(mask | ((uint32_t)n << 8) | ((uint32_t)c << 12));
}
constexpr int GT16_ENTRIES = 9 * 2 * 256;      // [min(15 - nsig, 8)][state][byte]
struct Gt16Table {
    uint16_t step[GT16_ENTRIES];
    constexpr Gt16Table() : step()
    {
        for (int i = 0; i < GT16_ENTRIES; ++i) step[i] = gt16_step((i >> 8) & 1, i >> 9, (uint32_t)i & 255u);
    }
};
__constant__ const Gt16Table gt16_table = Gt16Table();

// all 256 threads of the work-group copy the table into LDS (9 KB); a barrier follows
__device__ __forceinline__ void gt16_load(uint16_t *tab)
{
    const uint32_t *src = reinterpret_cast<const uint32_t *>(gt16_table.step);
    uint32_t *dst = reinterpret_cast<uint32_t *>(tab);
#pragma unroll
    for (int i = 0; i < GT16_ENTRIES / 2 / 256; ++i) dst[threadIdx.x + 256 * i] = src[threadIdx.x + 256 * i];
    __syncthreads();
}

// One bit plane of a 2-D block, bit by bit as zfp walks it: look = the next 64 stream bits (a plane
// never uses more than 48), bits = what is left of the block's budget, nsig = values significant so
// far.  nsig verbatim bits, then segment by segment the test bit and the zeros up to the next one
// bit (cut short by the budget or by the block's last value, whose one is implied).
__device__ __forceinline__ uint32_t slow_plane16(uint64_t look, int &bits, int &nsig)
{
    constexpr int N = 16;
    const int mm = min(nsig, bits);
    bits -= mm;
    uint32_t x = (uint32_t)look & ((1u << mm) - 1u);
    look >>= mm;
    while (nsig < N && bits > 0) {
        const uint32_t lo = (uint32_t)look;
        if (!(lo & 1u)) { --bits; break; }
        const int lim = min(N - 1 - nsig, bits - 1);
        const uint32_t win = (lo >> 1) & ((1u << lim) - 1u);
        const int z = win != 0u ? __builtin_ctz(win) : lim;       // zeros read
        const int used = 1 + (win != 0u ? z + 1 : lim);
        look >>= used; bits -= used; nsig += z;
        x |= 1u << nsig;
        ++nsig;
    }
    return x;
}

// The same plane by table, as long as the budget does not end inside it: false = it would (bits and
// nsig are then whatever the walk left them at: the caller keeps its own copies and has
// slow_plane16 do that plane, the block's last).  One exit and selects instead of branches: the
// lanes of a wave are at different points of their walks.
__device__ __forceinline__ bool fast_plane16(uint64_t look, int &bits, int &nsig, uint32_t &x, const uint16_t *tab)
{
    const int mm = min(nsig, bits);
    bits -= mm;
    x = (uint32_t)look & ((1u << mm) - 1u);
    look >>= mm;
    bool over = false, go = nsig < 16 && bits > 0;
    uint32_t st = 0u;                          // state * 256
    while (go) {
        const uint32_t r = (uint32_t)min(15 - nsig, 8);
        const uint32_t e = tab[(r << 9) | st | ((uint32_t)look & 255u)];
        const uint32_t c = e >> 12;
        const int used = (int)min(c, 8u);
        over = used >= bits;
        const int u = over ? 0 : used;
        x |= (over ? 0u : (e & 255u)) << nsig;
        nsig += over ? 0 : (int)((e >> 8) & 15u);
        look >>= u; bits -= u;
        st = (c & 1u) ? 0u : 256u;             // c = 9: state T, c = 10: state R (other values end the walk)
        go = !over && c >= 9u;
    }
    return !over;
}

// tab: the group-test table in LDS (gt16_load), used by 2-D blocks only
template <int N, int NW>
__device__ __forceinline__ void decode_block(BitReader<NW> &br, float *f, const uint16_t *tab = nullptr)
{
    if (!br.get(1)) {
#pragma unroll
        for (int i = 0; i < N; ++i) f[i] = 0.f;
        return;
    }
    const int emax = (int)br.get(8) - 127;
    uint32_t u[N];
#pragma unroll
    for (int i = 0; i < N; ++i) u[i] = 0u;
    int bits = 32 * NW - 9;
    int nsig = 0;
    auto read_plane = [&]() __attribute__((always_inline)) {
        if constexpr (N == 4) {
            const int mm = min(nsig, bits);
            bits -= mm;
            uint32_t x = br.get(mm);
            while (nsig < N && bits > 0) {
                // tiny blocks: test bit and run are read separately (measured faster here)
                --bits;
                if (!br.get(1)) break;
                const int lim = min(N - 1 - nsig, bits);
                const uint32_t win = br.peek() & ((1u << lim) - 1u);
                const int z = win != 0u ? __builtin_ctz(win) : lim;
                const int used = win != 0u ? z + 1 : lim;
                br.skip(used); bits -= used; nsig += z;
                x |= 1u << nsig;
                ++nsig;
            }
            return x;
        } else {
            // one look at the stream per plane
            const int before = bits;
            const uint32_t x = slow_plane16(br.peek64(), bits, nsig);
            br.skip(before - bits);
            return x;
        }
    };
    if constexpr (N == 16) {
        // planes 31..16 are collected as rows and transposed into the coefficients' upper halves
        uint32_t w[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) w[j] = 0u;
        // by table, up to the plane the budget ends in: that one is set aside (every lane has one, each
        // at a plane of its own) and walked bit by bit afterwards, by all lanes at once
        int last_k = -1, last_bits = 0, last_nsig = 0;
        uint64_t last_look = 0;
#pragma unroll
        for (int k = 15; k >= 0; --k) {
            // (a branch of the whole wave; a lane whose budget is spent walks a plane of no bits)
            if (__builtin_amdgcn_ballot_w64(bits > 0) != 0) {
                const uint64_t look = br.peek64();
                const int before = bits, nsig0 = nsig;
                uint32_t x;
                const bool ok = fast_plane16(look, bits, nsig, x, tab);
                br.skip(ok ? before - bits : 0);
                w[k >> 1] |= ok ? x << (16 * (k & 1)) : 0u;
                last_k = ok ? last_k : k;
                last_look = ok ? last_look : look;
                last_bits = ok ? last_bits : before;
                last_nsig = ok ? last_nsig : nsig0;
                bits = ok ? bits : 0;
            }
        }
        if (last_k >= 0) {
            const uint32_t x = slow_plane16(last_look, last_bits, last_nsig) << (16 * (last_k & 1));
#pragma unroll
            for (int j = 0; j < 8; ++j) w[j] |= (last_k >> 1) == j ? x : 0u;
        }
        transpose16(w);
#pragma unroll
        for (int j = 0; j < 8; ++j) { u[2 * j] = w[j] << 16; u[2 * j + 1] = w[j] & 0xffff0000u; }
        for (int k = 15; k >= 0 && bits > 0; --k) {
            const uint32_t x = read_plane();
#pragma unroll
            for (int i = 0; i < N; ++i) u[i] |= ((x >> i) & 1u) << k;
        }
    } else {
        for (int k = 31; k >= 0 && bits > 0; --k) {
            const uint32_t x = read_plane();
#pragma unroll
            for (int i = 0; i < N; ++i) u[i] |= ((x >> i) & 1u) << k;
        }
    }
    int32_t q[N];
    if constexpr (N == 4) {
#pragma unroll
        for (int i = 0; i < 4; ++i) q[i] = from_negabinary(u[i]);
        inv_lift(q[0], q[1], q[2], q[3]);
    } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) q[perm2(i)] = from_negabinary(u[i]);
#pragma unroll
        for (int x = 0; x < 4; ++x) inv_lift(q[x], q[x + 4], q[x + 8], q[x + 12]);
#pragma unroll
        for (int y = 0; y < 4; ++y) inv_lift(q[4 * y], q[4 * y + 1], q[4 * y + 2], q[4 * y + 3]);
    }
    const float s = ldexpf(1.0f, emax - 30);
#pragma unroll
    for (int i = 0; i < N; ++i) f[i] = (float)q[i] * s;
}

template <int NW>
__device__ __forceinline__ void store_words(uint32_t *dst, const uint32_t *w)
{
    if constexpr (NW == 1) dst[0] = w[0];
    else if constexpr (NW == 2) *reinterpret_cast<uint2 *>(dst) = make_uint2(w[0], w[1]);
    else {
#pragma unroll
        for (int i = 0; i < NW / 4; ++i)
            reinterpret_cast<uint4 *>(dst)[i] = make_uint4(w[4 * i], w[4 * i + 1], w[4 * i + 2], w[4 * i + 3]);
    }
}

template <int NW>
__device__ __forceinline__ void load_words(const uint32_t *src, uint32_t *w)
{
    if constexpr (NW == 1) w[0] = src[0];
    else if constexpr (NW == 2) { const uint2 v = *reinterpret_cast<const uint2 *>(src); w[0] = v.x; w[1] = v.y; }
    else {
#pragma unroll
        for (int i = 0; i < NW / 4; ++i) {
            const uint4 v = reinterpret_cast<const uint4 *>(src)[i];
            w[4 * i] = v.x; w[4 * i + 1] = v.y; w[4 * i + 2] = v.z; w[4 * i + 3] = v.w;
        }
    }
}

template <int NW>
__global__ __launch_bounds__(256) void zfp_encode1_kernel(const float *__restrict__ field, int64_t blocks,
                                                          uint32_t *__restrict__ out)
{
    __shared__ uint32_t lds[NW * 256];
    __shared__ uint32_t tab[512];
    group_code_table(tab);
    const int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (b >= blocks) return;
    const float4 v = reinterpret_cast<const float4 *>(field)[b];
    const float f[4] = {v.x, v.y, v.z, v.w};
    BitWriter<NW> bw;
    encode_block<4, NW>(f, bw, lds, tab);
    uint32_t w[NW];
    bw.words(lds, w);
    store_words<NW>(out + b * NW, w);
    // an odd count of 32-bit words leaves half of the last 64-bit stream word as padding
    if (b == blocks - 1 && ((blocks * NW) & 1)) out[blocks * NW] = 0u;
}

template <int NW>
__global__ __launch_bounds__(256) void zfp_decode1_kernel(const uint32_t *__restrict__ in, int64_t blocks,
                                                          float *__restrict__ field)
{
    const int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (b >= blocks) return;
    __shared__ uint32_t lds[NW <= 2 ? 1 : BitReader<NW>::STRIDE * 256];
    uint32_t w[NW];
    load_words<NW>(in + b * NW, w);
    BitReader<NW> br;
    br.init(lds, w);
    float f[4];
    decode_block<4, NW>(br, f);
    reinterpret_cast<float4 *>(field)[b] = make_float4(f[0], f[1], f[2], f[3]);
}

// ---------------------------------------------------------------- 1-D blocks of 32 bits (rate 8)
// A block is 4 values and one 32-bit word: 9 header bits and a budget of 23.  Everything a bit
// plane contributes follows from two small numbers, the count of values that are significant
// already and the plane's 4 bits, so both directions look their group tests up instead of
// walking them: the coder in a table of 4 x 16 entries (code, length, newly significant values),
// the decoder in one of 4 x 128 entries indexed by the next 7 stream bits (the longest group-test
// code of a plane has 7 bits), and the block's word never leaves its register.

// group-test code of the 4 - nsig values that are not significant yet, whose plane bits are r:
// code in bits 0..7, its length in bits 8..11, the values that become significant in bits 12..14
__host__ __device__ constexpr uint32_t gt4_code(int nsig, uint32_t r)
{
    uint32_t code = 0, x = r;
    int len = 0, n = nsig;
    while (n < 4) {
        const uint32_t any = x != 0u;
        code |= any << len; ++len;
        if (!any) break;
        while (n < 3) {
            const uint32_t one = x & 1u;
            code |= one << len; ++len;
            if (one) break;
            x >>= 1; ++n;
        }
        x >>= 1; ++n;
    }
    return code | ((uint32_t)len << 8) | ((uint32_t)(n - nsig) << 12);
}

// the inverse, for a stream whose next 7 bits are s and of which `budget` >= 1 bits are left (7
// stands for "7 or more": the longest code has 7 bits); the walk is zfp's own, budget checks
// included.  Plane bits (at their absolute positions) in bits 0..3, bits used in 4..7, newly
// significant values in 8..10
__host__ __device__ constexpr uint32_t gt4_parse(int nsig, uint32_t s, int budget)
{
    uint32_t x = 0;
    int used = 0, n = nsig, bits = budget;
    while (n < 4 && bits > 0) {
        --bits;
        const uint32_t any = (s >> used) & 1u; ++used;
        if (!any) break;
        while (n < 3 && bits > 0) {
            --bits;
            const uint32_t one = (s >> used) & 1u; ++used;
            if (one) break;
            ++n;
        }
        x |= 1u << n; ++n;
    }
    return x | ((uint32_t)used << 4) | ((uint32_t)(n - nsig) << 8);
}

// The 32 bit planes of a 1-D block as nibbles: word c holds the planes k = c (mod 4), plane k in
// bits k - c .. k - c + 3 (bit i of the nibble = bit k of value i).  32 operations for all planes
// instead of 8 per plane.
__device__ __forceinline__ void planes_of(const uint32_t (&u)[4], uint32_t (&pl)[4])
{
#pragma unroll
    for (int c = 0; c < 4; ++c)
        pl[c] = ((u[0] >> c) & 0x11111111u) | (((u[1] >> c) & 0x11111111u) << 1) |
                (((u[2] >> c) & 0x11111111u) << 2) | (((u[3] >> c) & 0x11111111u) << 3);
}
__device__ __forceinline__ void values_of(const uint32_t (&pl)[4], uint32_t (&u)[4])
{
#pragma unroll
    for (int i = 0; i < 4; ++i)
        u[i] = ((pl[0] >> i) & 0x11111111u) | (((pl[1] >> i) & 0x11111111u) << 1) |
               (((pl[2] >> i) & 0x11111111u) << 2) | (((pl[3] >> i) & 0x11111111u) << 3);
}

// both tables worked out by the compiler; a work-group copies them into LDS
struct Gt4Tables {
    uint32_t code[64];      // [nsig][plane bits]: code, length, newly significant values, a byte each
    uint16_t parse[7 * 512];    // [min(budget, 7) - 1][nsig][next 7 stream bits]
    constexpr Gt4Tables() : code(), parse()
    {
        for (int i = 0; i < 64; ++i) {
            const uint32_t e = gt4_code(i >> 4, (uint32_t)i & 15u);
            code[i] = (e & 0xffu) | (((e >> 8) & 15u) << 8) | ((e >> 12) << 16);
        }
        for (int i = 0; i < 7 * 512; ++i) parse[i] = (uint16_t)gt4_parse((i >> 7) & 3, (uint32_t)i & 127u, (i >> 9) + 1);
    }
};
__constant__ const Gt4Tables gt4_tables = Gt4Tables();

__global__ __launch_bounds__(256) void zfp_encode1_word_kernel(const float *__restrict__ field, int64_t blocks,
                                                               uint32_t *__restrict__ out)
{
    __shared__ uint32_t tab[64];
    if (threadIdx.x < 64) tab[threadIdx.x] = gt4_tables.code[threadIdx.x];
    __syncthreads();
    const int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (b >= blocks) return;
    if (b == blocks - 1 && (blocks & 1)) out[blocks] = 0u;      // the other half of the last 64-bit stream word
    const float4 v = reinterpret_cast<const float4 *>(field)[b];
    const float f[4] = {v.x, v.y, v.z, v.w};
    const float m = fmaxf(fmaxf(fabsf(f[0]), fabsf(f[1])), fmaxf(fabsf(f[2]), fabsf(f[3])));
    if (!(m > 0.f)) { out[b] = 0u; return; }                     // all-zero block: '0' flag and zero padding
    const int emax = (int)((__float_as_uint(m) >> 23) & 0xffu) - 126;
    const int se = 30 - emax;
    const float s = se > 127 ? INFINITY : __uint_as_float((uint32_t)(se + 127) << 23);
    int32_t q[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const float t = f[i] * s;
        q[i] = fabsf(t) < 2147483648.0f ? (int32_t)t : (int32_t)0x80000000;
    }
    fwd_lift(q[0], q[1], q[2], q[3]);
    const uint32_t u[4] = {to_negabinary(q[0]), to_negabinary(q[1]), to_negabinary(q[2]), to_negabinary(q[3])};
    uint32_t pl[4];
    planes_of(u, pl);

    // The word fills from bit 9 up.  What does not fit falls off the top of the 32-bit register, which
    // is exactly where the budget cuts the stream, so nothing is masked to the remaining budget.
    uint32_t acc = 2u * (uint32_t)(emax + 127) + 1u;
    int fill = 9, nsig = 0;
    uint32_t sigmask = 0u;                                       // (1 << nsig) - 1
    auto plane = [&](uint32_t x) __attribute__((always_inline)) {
        acc |= (x & sigmask) << fill;
        fill += nsig;
        if (nsig < 4 && fill < 32) {
            const uint32_t e = tab[nsig * 16 + (int)(x >> nsig)];
            acc |= (e & 0xffu) << fill;
            fill += (int)((e >> 8) & 0xffu);
            nsig += (int)(e >> 16);
            sigmask = (1u << nsig) - 1u;
        }
    };
    for (int kb = 28; kb >= 0 && fill < 32; kb -= 4) {
        plane((pl[3] >> kb) & 15u);
        if (fill < 32) plane((pl[2] >> kb) & 15u);
        if (fill < 32) plane((pl[1] >> kb) & 15u);
        if (fill < 32) plane((pl[0] >> kb) & 15u);
    }
    out[b] = acc;
}

// blocks per thread: the parse table (7 KB) is copied into LDS once per work-group
constexpr int ZD1_PER_THREAD = 4;

__global__ __launch_bounds__(256) void zfp_decode1_word_kernel(const uint32_t *__restrict__ in, int64_t blocks,
                                                               float *__restrict__ field)
{
    __shared__ uint16_t tab[7 * 512];
    {
        const uint32_t *src = reinterpret_cast<const uint32_t *>(gt4_tables.parse);
        uint32_t *dst = reinterpret_cast<uint32_t *>(tab);
#pragma unroll
        for (int i = 0; i < 7; ++i) dst[threadIdx.x + 256 * i] = src[threadIdx.x + 256 * i];
    }
    __syncthreads();
    const int64_t b0 = (int64_t)blockIdx.x * (256 * ZD1_PER_THREAD) + threadIdx.x;
    uint32_t win[ZD1_PER_THREAD];
#pragma unroll
    for (int it = 0; it < ZD1_PER_THREAD; ++it) win[it] = in[min(b0 + 256 * it, blocks - 1)];
#pragma unroll
    for (int it = 0; it < ZD1_PER_THREAD; ++it) {
        const int64_t b = b0 + 256 * it;
        if (b >= blocks) break;
        const uint32_t w = win[it];
        float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
        if (w & 1u) {
            const int emax = (int)((w >> 1) & 0xffu) - 127;
            uint32_t s = w >> 9;                                     // the 23 coded bits, zeros above them
            uint32_t pl[4] = {0u, 0u, 0u, 0u};
            int bits = 23, nsig = 0;
            uint32_t sigmask = 0u;
            // the bits of one plane: the verbatim ones (past the budget the register holds zeros, as the
            // budget's end demands), then the group tests by table, whatever is left of the budget
            auto plane = [&]() __attribute__((always_inline)) {
                uint32_t x = s & sigmask;
                s >>= nsig; bits -= nsig;
                if (nsig < 4 && bits > 0) {
                    const uint32_t e = tab[(min(bits, 7) - 1) * 512 + nsig * 128 + (int)(s & 127u)];
                    const int used = (int)((e >> 4) & 15u);
                    x |= e & 15u;
                    s >>= used; bits -= used;
                    nsig += (int)(e >> 8);
                    sigmask = (1u << nsig) - 1u;
                }
                return x;
            };
            for (int kb = 28; kb >= 0 && bits > 0; kb -= 4) {
                pl[3] |= plane() << kb;
                if (bits > 0) pl[2] |= plane() << kb;
                if (bits > 0) pl[1] |= plane() << kb;
                if (bits > 0) pl[0] |= plane() << kb;
            }
            uint32_t u[4];
            values_of(pl, u);
            int32_t q0 = from_negabinary(u[0]), q1 = from_negabinary(u[1]), q2 = from_negabinary(u[2]), q3 = from_negabinary(u[3]);
            inv_lift(q0, q1, q2, q3);
            // 2^(emax - 30): a normal number unless the block's values are next to the denormals
            const int se = emax - 30 + 127;
            const float sc = se >= 1 ? __uint_as_float((uint32_t)se << 23) : ldexpf(1.0f, emax - 30);
            o = make_float4((float)q0 * sc, (float)q1 * sc, (float)q2 * sc, (float)q3 * sc);
        }
        reinterpret_cast<float4 *>(field)[b] = o;
    }
}

template <int NW>
__global__ __launch_bounds__(256) void zfp_encode2_kernel(const float *__restrict__ field, int64_t nx,
                                                          int64_t nbx, int64_t blocks,
                                                          uint32_t *__restrict__ out)
{
    __shared__ uint32_t lds[NW * 256];
    __shared__ uint32_t tab[512];
    group_code_table(tab);
    const int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (b >= blocks) return;
    const int64_t by = b / nbx, bx = b - by * nbx;
    const float *p = field + 4 * by * nx + 4 * bx;
    float f[16];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float4 v = *reinterpret_cast<const float4 *>(p + j * nx);
        f[4 * j] = v.x; f[4 * j + 1] = v.y; f[4 * j + 2] = v.z; f[4 * j + 3] = v.w;
    }
    BitWriter<NW> bw;
    encode_block<16, NW>(f, bw, lds, tab);
    uint32_t w[NW];
    bw.words(lds, w);
    store_words<NW>(out + b * NW, w);
}

// blocks per thread: the group-test table (9 KB) is copied into LDS once per work-group
constexpr int ZD2_PER_THREAD = 4;

template <int NW>
__global__ __launch_bounds__(256) void zfp_decode2_kernel(const uint32_t *__restrict__ in, int64_t nx,
                                                          int64_t nbx, int64_t blocks,
                                                          float *__restrict__ field)
{
    __shared__ uint32_t lds[NW <= 2 ? 1 : BitReader<NW>::STRIDE * 256];
    __shared__ uint16_t tab[GT16_ENTRIES];
    gt16_load(tab);
    const int64_t b0 = (int64_t)blockIdx.x * (256 * ZD2_PER_THREAD) + threadIdx.x;
    for (int it = 0; it < ZD2_PER_THREAD; ++it) {
        const int64_t b = b0 + 256 * it;
        if (b >= blocks) break;
        uint32_t w[NW];
        load_words<NW>(in + b * NW, w);
        BitReader<NW> br;
        br.init(lds, w);
        float f[16];
        decode_block<16, NW>(br, f, tab);
        const int64_t by = b / nbx, bx = b - by * nbx;
        float *p = field + 4 * by * nx + 4 * bx;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            *reinterpret_cast<float4 *>(p + j * nx) = make_float4(f[4 * j], f[4 * j + 1], f[4 * j + 2], f[4 * j + 3]);
    }
}

// ---------------------------------------------------------------- dispatch fused with the 2-D encoder
// fast_encode followed by ZfpCompressor::compress (fast_dispatch.py:26-29 + zfpc.cpp:23-51) without
// the [experts * capacity, model_dim] buffer in between: a block of the field is 4 consecutive
// slot rows x 4 columns, so the encoder fetches its 4 rows from the tokens that fill those slots.

// slot -> token that fills it (-1 = empty: pre-filled) and, for the gated variant, its gate
__global__ __launch_bounds__(256) void slot_source_mark(int32_t *__restrict__ src, float *__restrict__ sgate,
                                                       int32_t *__restrict__ splane,
                                                       const float *__restrict__ gates,
                                                       const int32_t *__restrict__ indices,
                                                       const int32_t *__restrict__ locations, int64_t stride,
                                                       int top_k, int samples, int experts, int capacity)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= samples * top_k) return;
    const int j = i / samples, t = i - j * samples;
    const int64_t o = (int64_t)j * stride + t;
    const int e = indices[o], l = locations[o];
    if (e < 0 || e >= experts || l < 0 || l >= capacity) return;
    const int slot = e * capacity + l;
    src[slot] = t;
    if (gates) sgate[slot] = gates[o];
    if (splane) splane[slot] = j;
}

template <int NW, bool GATED>
__global__ __launch_bounds__(256) void dispatch_zfp2_kernel(const float *__restrict__ x,
                                                           const int32_t *__restrict__ src,
                                                           const float *__restrict__ sgate, int64_t model_dim,
                                                           int64_t nbx, int64_t blocks,
                                                           uint32_t *__restrict__ out)
{
    __shared__ uint32_t lds[NW * 256];
    __shared__ uint32_t tab[512];
    group_code_table(tab);
    const int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (b >= blocks) return;
    const int64_t by = b / nbx, bx = b - by * nbx;
    const int4 tok = *reinterpret_cast<const int4 *>(src + 4 * by);
    const int t[4] = {tok.x, tok.y, tok.z, tok.w};
    float g[4] = {1.f, 1.f, 1.f, 1.f};
    if constexpr (GATED) {
        const float4 gv = *reinterpret_cast<const float4 *>(sgate + 4 * by);
        g[0] = gv.x; g[1] = gv.y; g[2] = gv.z; g[3] = gv.w;
    }
    float f[16];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        // straight-line load at a clamped row; an empty slot is a row of zeros
        const float4 v = *reinterpret_cast<const float4 *>(x + (int64_t)max(t[j], 0) * model_dim + 4 * bx);
        const bool live = t[j] >= 0;
        // the dispatch kernel stores 0 + g * x (x itself without gates); the sign of a zero does not
        // reach the stream
        f[4 * j] = live ? (GATED ? g[j] * v.x : v.x) : 0.f;
        f[4 * j + 1] = live ? (GATED ? g[j] * v.y : v.y) : 0.f;
        f[4 * j + 2] = live ? (GATED ? g[j] * v.z : v.z) : 0.f;
        f[4 * j + 3] = live ? (GATED ? g[j] * v.w : v.w) : 0.f;
    }
    BitWriter<NW> bw;
    encode_block<16, NW>(f, bw, lds, tab);
    uint32_t w[NW];
    bw.words(lds, w);
    store_words<NW>(out + b * NW, w);
}

// ---------------------------------------------------------------- 2-D decoder fused with combine
// ZfpCompressor::decompress followed by fast_decode (zfpc.cpp:66-86 + fast_dispatch.py:59-64)
// without the decoded [experts * capacity, model_dim] buffer: a decoded block holds 4 slot rows,
// and every row goes to the token that owns the slot.  The reference adds the choices of a token
// left to right, so one launch per choice plane: plane 0 stores gate * row, plane j adds to what
// is there; blocks without a row of the plane leave before decoding (the slots of an expert are
// filled plane after plane, so almost every block belongs to one plane), and empty slots are
// never decoded.  A small launch per plane gives the tokens whose choice was dropped the
// reference's "+ 0" (a zero row for plane 0).
template <int NW>
__global__ __launch_bounds__(256) void combine_zfp2_kernel(const uint32_t *__restrict__ in,
                                                          const int32_t *__restrict__ src,
                                                          const float *__restrict__ sgate,
                                                          const int32_t *__restrict__ splane, int plane,
                                                          int64_t model_dim, int64_t nbx, int64_t blocks,
                                                          float *__restrict__ out)
{
    // (one block per thread: with four, so that the table is copied once per 1024 blocks, the launch
    // takes 10 % longer: half the work-groups leave early and the rest run four times as long)
    __shared__ uint32_t lds[NW <= 2 ? 1 : BitReader<NW>::STRIDE * 256];
    __shared__ uint16_t tab[GT16_ENTRIES];
    const int64_t b = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const bool in_field = b < blocks;
    const int64_t by = (in_field ? b : blocks - 1) / nbx, bx = b - by * nbx;
    const int4 tok = *reinterpret_cast<const int4 *>(src + 4 * by);
    const int4 pl = *reinterpret_cast<const int4 *>(splane + 4 * by);
    const int t[4] = {tok.x, tok.y, tok.z, tok.w};
    const bool mine[4] = {in_field && tok.x >= 0 && pl.x == plane, in_field && tok.y >= 0 && pl.y == plane,
                          in_field && tok.z >= 0 && pl.z == plane, in_field && tok.w >= 0 && pl.w == plane};
    const bool any_mine = mine[0] || mine[1] || mine[2] || mine[3];
    if (!__syncthreads_or(any_mine)) return;          // a work-group without a row of this plane leaves before the table
    gt16_load(tab);
    if (!any_mine) return;
    float g[4] = {1.f, 1.f, 1.f, 1.f};
    if (sgate) {
        const float4 gv = *reinterpret_cast<const float4 *>(sgate + 4 * by);
        g[0] = gv.x; g[1] = gv.y; g[2] = gv.z; g[3] = gv.w;
    }
    // what is there so far, requested before the decode (straight-line loads at clamped rows)
    float4 acc[4];
    if (plane > 0) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            acc[j] = *reinterpret_cast<const float4 *>(out + (int64_t)max(t[j], 0) * model_dim + 4 * bx);
    }
    uint32_t w[NW];
    load_words<NW>(in + b * NW, w);
    BitReader<NW> br;
    br.init(lds, w);
    float f[16];
    decode_block<16, NW>(br, f, tab);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if (!mine[j]) continue;
        float4 v = make_float4(g[j] * f[4 * j], g[j] * f[4 * j + 1], g[j] * f[4 * j + 2], g[j] * f[4 * j + 3]);
        if (plane > 0) v = make_float4(acc[j].x + v.x, acc[j].y + v.y, acc[j].z + v.z, acc[j].w + v.w);
        *reinterpret_cast<float4 *>(out + (int64_t)t[j] * model_dim + 4 * bx) = v;
    }
}

// GatingDecoder.backward's gate gradients (create_backward_gate, fast_dispatch.py:73-78) straight
// from the stream of the expert output the decode consumed: grad_gate[plane][t] = <grad_out[t],
// decoded slot row>, so the backward pass never writes the decoded buffer.  One work-group owns
// the four slot rows of one row of blocks; a thread decodes its blocks along the row and keeps four
// partial sums, which the work-group adds in a fixed order.  grad_gates must be zero beforehand
// (choices that take no slot keep their zero).
template <int NW>
__global__ __launch_bounds__(256) void bwd_gate_zfp2_kernel(const uint32_t *__restrict__ in,
                                                           const int32_t *__restrict__ src,
                                                           const int32_t *__restrict__ splane,
                                                           const float *__restrict__ grad_out, int64_t stride,
                                                           int64_t model_dim, int64_t nbx,
                                                           float *__restrict__ grad_gates)
{
    __shared__ uint32_t lds[NW <= 2 ? 1 : BitReader<NW>::STRIDE * 256];
    __shared__ float s_part[4][4];
    __shared__ uint16_t tab[GT16_ENTRIES];
    const int64_t by = blockIdx.x;
    const int4 tok = *reinterpret_cast<const int4 *>(src + 4 * by);
    const int t[4] = {tok.x, tok.y, tok.z, tok.w};
    if (t[0] < 0 && t[1] < 0 && t[2] < 0 && t[3] < 0) return;        // four empty slots (the whole work-group leaves)
    gt16_load(tab);
    float acc[4] = {0.f, 0.f, 0.f, 0.f};
    for (int64_t bx0 = 0; bx0 < nbx; bx0 += 256) {
        const int64_t bx = bx0 + threadIdx.x;
        const bool in_row = bx < nbx;
        const int64_t bxc = in_row ? bx : nbx - 1;                   // clamped: straight-line loads
        float4 g[4];
#pragma unroll
        for (int j = 0; j < 4; ++j)
            g[j] = *reinterpret_cast<const float4 *>(grad_out + (int64_t)max(t[j], 0) * model_dim + 4 * bxc);
        uint32_t w[NW];
        load_words<NW>(in + (by * nbx + bxc) * NW, w);
        BitReader<NW> br;
        br.init(lds, w);
        float f[16];
        decode_block<16, NW>(br, f, tab);
        if (in_row) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[j] += ((f[4 * j] * g[j].x + f[4 * j + 1] * g[j].y) + f[4 * j + 2] * g[j].z) + f[4 * j + 3] * g[j].w;
        }
    }
    const int wave = threadIdx.x >> 6;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float r = wave_sum(acc[j]);
        if (lane_id() == 0) s_part[wave][j] = r;
    }
    __syncthreads();
    if (threadIdx.x < 4) {
        const int j = threadIdx.x;
        if (t[j] >= 0)
            grad_gates[(int64_t)splane[4 * by + j] * stride + t[j]] =
                ((s_part[0][j] + s_part[1][j]) + s_part[2][j]) + s_part[3][j];
    }
}

// tokens whose choice `plane` takes no slot: a zero row (plane 0) or row + 0 (later planes)
__global__ __launch_bounds__(256) void combine_dropped_kernel(const int32_t *__restrict__ indices,
                                                             const int32_t *__restrict__ locations,
                                                             int64_t stride, int plane, int samples,
                                                             int model_dim, int experts, int capacity,
                                                             float *__restrict__ out)
{
    const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= samples) return;
    const int64_t o = (int64_t)plane * stride + t;
    const int e = indices[o], l = locations[o];
    if (e >= 0 && e < experts && l >= 0 && l < capacity) return;
    float4 *row = reinterpret_cast<float4 *>(out + (int64_t)t * model_dim);
    for (int u = lane_id(); u < model_dim / 4; u += WAVE) {
        float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
        if (plane > 0) {
            v = row[u];
            v = make_float4(v.x + 0.f, v.y + 0.f, v.z + 0.f, v.w + 0.f);
        }
        row[u] = v;
    }
}

static int zfp_maxbits(int dims, double rate)
{
    const int n = dims == 1 ? 4 : 16;
    int bits = (int)std::floor(n * rate + 0.5);
    if (bits < 9) bits = 9;
    return bits;
}

static int zfp_check(const char *who, int dims, int64_t nx, int64_t ny, double rate, int &nw,
                     int64_t &blocks)
{
    PM_REQUIRE(dims == 1 || dims == 2, "%s: dims must be 1 or 2 (got %d)", who, dims);
    PM_REQUIRE(nx >= 0 && ny >= 0, "%s: negative extent", who);
    PM_REQUIRE(nx % 4 == 0 && ny % 4 == 0, "%s: zfp fails. (every extent must be a multiple of 4, got nx=%lld ny=%lld)",
               who, (long long)nx, (long long)ny);
    PM_REQUIRE(rate > 0, "%s: rate must be > 0", who);
    const int maxbits = zfp_maxbits(dims, rate);
    PM_REQUIRE(maxbits % 32 == 0 && (maxbits / 32 == 1 || maxbits / 32 == 2 || maxbits / 32 == 4 || maxbits / 32 == 8),
               "%s: rate %.3f gives %d bits per block; supported block sizes are 32, 64, 128 and 256 bits",
               who, rate, maxbits);
    nw = maxbits / 32;
    blocks = dims == 1 ? (nx * ny) / 4 : (nx / 4) * (ny / 4);
    PM_REQUIRE((blocks + 255) / 256 < (1ll << 31), "%s: field too large", who);
    return 0;
}

} // namespace pm

using namespace pm;

extern "C" size_t planmoe_zfp_max_bytes(int dims, int64_t nx, int64_t ny, double rate)
{
    if ((dims != 1 && dims != 2) || nx < 0 || ny < 0 || !(rate > 0)) return 0;
    const uint64_t blocks = dims == 1 ? (uint64_t)(nx * ny + 3) / 4 : (uint64_t)((nx + 3) / 4) * (uint64_t)((ny + 3) / 4);
    const uint64_t bits = 148u + blocks * (uint64_t)zfp_maxbits(dims, rate);   // header allowance
    return (size_t)(((bits + 63u) / 64u) * 8u);
}

extern "C" size_t planmoe_zfp_stream_bytes(int dims, int64_t nx, int64_t ny, double rate)
{
    if ((dims != 1 && dims != 2) || nx < 0 || ny < 0 || !(rate > 0)) return 0;
    const uint64_t blocks = dims == 1 ? (uint64_t)(nx * ny) / 4 : (uint64_t)(nx / 4) * (uint64_t)(ny / 4);
    const uint64_t bits = blocks * (uint64_t)zfp_maxbits(dims, rate);
    return (size_t)(((bits + 63u) / 64u) * 8u);
}

#define PM_NW_SWITCH(nw, NW, ...)                              \
    switch (nw) {                                              \
    case 1: { constexpr int NW = 1; __VA_ARGS__; break; }      \
    case 2: { constexpr int NW = 2; __VA_ARGS__; break; }      \
    case 4: { constexpr int NW = 4; __VA_ARGS__; break; }      \
    default: { constexpr int NW = 8; __VA_ARGS__; break; }     \
    }

extern "C" int planmoe_zfp_compress(const float *field, int dims, int64_t nx, int64_t ny, double rate,
                                    void *stream_out, size_t stream_capacity, void *stream)
{
    int nw; int64_t blocks;
    if (zfp_check("planmoe_zfp_compress", dims, nx, ny, rate, nw, blocks)) return 1;
    if (blocks == 0) return 0;
    PM_REQUIRE(field && stream_out, "planmoe_zfp_compress: NULL argument");
    PM_REQUIRE(aligned16(field) && aligned16(stream_out), "planmoe_zfp_compress: buffers must be 16-byte aligned");
    const size_t need = planmoe_zfp_stream_bytes(dims, nx, ny, rate);
    PM_REQUIRE(stream_capacity >= need, "planmoe_zfp_compress: stream buffer too small (%zu < %zu)",
               stream_capacity, need);
    hipStream_t st = (hipStream_t)stream;
    const unsigned grid = (unsigned)((blocks + 255) / 256);
    if (dims == 1 && nw == 1) {
        zfp_encode1_word_kernel<<<grid, 256, 0, st>>>(field, blocks, (uint32_t *)stream_out);
        PM_LAUNCH_CHECK("planmoe_zfp_compress");
        return 0;
    }
    PM_NW_SWITCH(nw, NW, {
        if (dims == 1) zfp_encode1_kernel<NW><<<grid, 256, 0, st>>>(field, blocks, (uint32_t *)stream_out);
        else zfp_encode2_kernel<NW><<<grid, 256, 0, st>>>(field, nx, nx / 4, blocks, (uint32_t *)stream_out);
    });
    PM_LAUNCH_CHECK("planmoe_zfp_compress");
    return 0;
}

extern "C" int planmoe_zfp_decompress(const void *stream_in, int dims, int64_t nx, int64_t ny, double rate,
                                      float *field, void *stream)
{
    int nw; int64_t blocks;
    if (zfp_check("planmoe_zfp_decompress", dims, nx, ny, rate, nw, blocks)) return 1;
    if (blocks == 0) return 0;
    PM_REQUIRE(field && stream_in, "planmoe_zfp_decompress: NULL argument");
    PM_REQUIRE(aligned16(field) && aligned16(stream_in), "planmoe_zfp_decompress: buffers must be 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    const unsigned grid = (unsigned)((blocks + 255) / 256);
    if (dims == 1 && nw == 1) {
        const unsigned grid1 = (unsigned)((blocks + 256 * ZD1_PER_THREAD - 1) / (256 * ZD1_PER_THREAD));
        zfp_decode1_word_kernel<<<grid1, 256, 0, st>>>((const uint32_t *)stream_in, blocks, field);
        PM_LAUNCH_CHECK("planmoe_zfp_decompress");
        return 0;
    }
    PM_NW_SWITCH(nw, NW, {
        if (dims == 1) zfp_decode1_kernel<NW><<<grid, 256, 0, st>>>((const uint32_t *)stream_in, blocks, field);
        else zfp_decode2_kernel<NW><<<(unsigned)((blocks + 256 * ZD2_PER_THREAD - 1) / (256 * ZD2_PER_THREAD)), 256, 0, st>>>(
                 (const uint32_t *)stream_in, nx, nx / 4, blocks, field);
    });
    PM_LAUNCH_CHECK("planmoe_zfp_decompress");
    return 0;
}

extern "C" size_t planmoe_dispatch_zfp_workspace_bytes(int experts, int capacity)
{
    if (experts <= 0 || capacity <= 0) return 16;
    return round_up((size_t)experts * (size_t)capacity * 8u, 256);        // slot -> token, slot -> gate
}

extern "C" int planmoe_dispatch_zfp(const float *x, const float *gates, const int32_t *indices,
                                    const int32_t *locations, int64_t plane_stride, int top_k, int samples,
                                    int model_dim, int experts, int capacity, double rate, void *stream_out,
                                    size_t stream_capacity, void *workspace, size_t workspace_bytes, void *stream)
{
    const char *who = "planmoe_dispatch_zfp";
    PM_REQUIRE((indices && locations) || samples == 0, "%s: indices/locations must not be NULL", who);
    PM_REQUIRE(top_k >= 1 && samples >= 0 && plane_stride >= samples, "%s: bad routing planes", who);
    PM_REQUIRE(model_dim >= 1 && experts >= 1 && capacity >= 0, "%s: bad shape", who);
    PM_REQUIRE((int64_t)experts * capacity < (1ll << 31) && (int64_t)samples * top_k < (1ll << 31),
               "%s: experts*capacity or samples*top_k overflows int32", who);
    const int64_t rows = (int64_t)experts * capacity;
    int nw; int64_t blocks;
    if (zfp_check(who, 2, model_dim, rows, rate, nw, blocks)) return 1;
    if (blocks == 0) return 0;
    PM_REQUIRE((x || samples == 0) && stream_out, "%s: NULL argument", who);
    PM_REQUIRE(aligned16(x) && aligned16(stream_out), "%s: buffers must be 16-byte aligned", who);
    const size_t need = planmoe_zfp_stream_bytes(2, model_dim, rows, rate);
    PM_REQUIRE(stream_capacity >= need, "%s: stream buffer too small (%zu < %zu)", who, stream_capacity, need);
    hipStream_t st = (hipStream_t)stream;
    if (samples == 0) {
        // every slot is empty, and a field of zeros codes as a stream of zeros
        fill_u32((uint32_t *)stream_out, need / 4, 0u, st);
        PM_LAUNCH_CHECK(who);
        return 0;
    }
    PM_REQUIRE(workspace && aligned16(workspace) &&
               workspace_bytes >= planmoe_dispatch_zfp_workspace_bytes(experts, capacity),
               "%s: workspace too small or not 16-byte aligned", who);
    int32_t *src = (int32_t *)workspace;
    float *sgate = (float *)(src + rows);
    fill_u32((uint32_t *)src, (size_t)rows, 0xffffffffu, st);
    slot_source_mark<<<(unsigned)(((int64_t)samples * top_k + 255) / 256), 256, 0, st>>>(
        src, sgate, nullptr, gates, indices, locations, plane_stride, top_k, samples, experts, capacity);
    const unsigned grid = (unsigned)((blocks + 255) / 256);
    PM_NW_SWITCH(nw, NW, {
        if (gates) dispatch_zfp2_kernel<NW, true><<<grid, 256, 0, st>>>(x, src, sgate, model_dim, model_dim / 4, blocks,
                                                                       (uint32_t *)stream_out);
        else dispatch_zfp2_kernel<NW, false><<<grid, 256, 0, st>>>(x, src, sgate, model_dim, model_dim / 4, blocks,
                                                                  (uint32_t *)stream_out);
    });
    PM_LAUNCH_CHECK(who);
    return 0;
}

extern "C" size_t planmoe_combine_zfp_workspace_bytes(int experts, int capacity)
{
    if (experts <= 0 || capacity <= 0) return 16;
    return round_up((size_t)experts * (size_t)capacity * 12u, 256);       // slot -> token, gate, plane
}

extern "C" int planmoe_combine_zfp(const void *stream_in, double rate, const float *gates,
                                   const int32_t *indices, const int32_t *locations, int64_t plane_stride,
                                   int top_k, int samples, int model_dim, int experts, int capacity,
                                   float *out, void *workspace, size_t workspace_bytes, void *stream)
{
    const char *who = "planmoe_combine_zfp";
    PM_REQUIRE((indices && locations) || samples == 0, "%s: indices/locations must not be NULL", who);
    PM_REQUIRE(top_k >= 1 && samples >= 0 && plane_stride >= samples, "%s: bad routing planes", who);
    PM_REQUIRE(model_dim >= 1 && experts >= 1 && capacity >= 0, "%s: bad shape", who);
    PM_REQUIRE((int64_t)experts * capacity < (1ll << 31) && (int64_t)samples * top_k < (1ll << 31),
               "%s: experts*capacity or samples*top_k overflows int32", who);
    const int64_t rows = (int64_t)experts * capacity;
    int nw; int64_t blocks;
    if (zfp_check(who, 2, model_dim, rows, rate, nw, blocks)) return 1;
    if (samples == 0) return 0;
    PM_REQUIRE(out && aligned16(out), "%s: out must be a 16-byte aligned buffer", who);
    hipStream_t st = (hipStream_t)stream;
    if (blocks == 0) {                                  // no slot at all: every token row is zero
        fill_u32((uint32_t *)out, (size_t)samples * model_dim, 0u, st);
        PM_LAUNCH_CHECK(who);
        return 0;
    }
    PM_REQUIRE(stream_in && aligned16(stream_in), "%s: the stream must be a 16-byte aligned buffer", who);
    PM_REQUIRE(workspace && aligned16(workspace) &&
               workspace_bytes >= planmoe_combine_zfp_workspace_bytes(experts, capacity),
               "%s: workspace too small or not 16-byte aligned", who);
    int32_t *src = (int32_t *)workspace;
    float *sgate = (float *)(src + rows);
    int32_t *splane = (int32_t *)(sgate + rows);
    fill_u32((uint32_t *)src, (size_t)rows, 0xffffffffu, st);
    slot_source_mark<<<(unsigned)(((int64_t)samples * top_k + 255) / 256), 256, 0, st>>>(
        src, sgate, splane, gates, indices, locations, plane_stride, top_k, samples, experts, capacity);
    const unsigned grid = (unsigned)((blocks + 255) / 256);
    for (int j = 0; j < top_k; ++j) {
        PM_NW_SWITCH(nw, NW, {
            combine_zfp2_kernel<NW><<<grid, 256, 0, st>>>((const uint32_t *)stream_in, src, gates ? sgate : nullptr,
                                                         splane, j, model_dim, model_dim / 4, blocks, out);
        });
        combine_dropped_kernel<<<(unsigned)((samples + 3) / 4), 256, 0, st>>>(indices, locations, plane_stride, j,
                                                                            samples, model_dim, experts, capacity, out);
    }
    PM_LAUNCH_CHECK(who);
    return 0;
}

extern "C" int planmoe_bwd_gate_zfp(const void *stream_in, double rate, const float *grad_out,
                                    const int32_t *indices, const int32_t *locations, int64_t plane_stride,
                                    int top_k, int samples, int model_dim, int experts, int capacity,
                                    float *grad_gates, void *workspace, size_t workspace_bytes, void *stream)
{
    const char *who = "planmoe_bwd_gate_zfp";
    PM_REQUIRE((indices && locations) || samples == 0, "%s: indices/locations must not be NULL", who);
    PM_REQUIRE(top_k >= 1 && samples >= 0 && plane_stride >= samples, "%s: bad routing planes", who);
    PM_REQUIRE(model_dim >= 1 && experts >= 1 && capacity >= 0, "%s: bad shape", who);
    PM_REQUIRE((int64_t)experts * capacity < (1ll << 31) && (int64_t)samples * top_k < (1ll << 31),
               "%s: experts*capacity or samples*top_k overflows int32", who);
    const int64_t rows = (int64_t)experts * capacity;
    int nw; int64_t blocks;
    if (zfp_check(who, 2, model_dim, rows, rate, nw, blocks)) return 1;
    if (samples == 0) return 0;
    PM_REQUIRE(grad_gates, "%s: grad_gates is NULL", who);
    hipStream_t st = (hipStream_t)stream;
    // every plane row in full: plane_stride may exceed samples, the padding is the caller's
    for (int j = 0; j < top_k; ++j)
        fill_u32((uint32_t *)(grad_gates + (int64_t)j * plane_stride), (size_t)samples, 0u, st);
    if (blocks == 0) {                                  // no slot at all: every gradient is zero
        PM_LAUNCH_CHECK(who);
        return 0;
    }
    PM_REQUIRE(stream_in && aligned16(stream_in), "%s: the stream must be a 16-byte aligned buffer", who);
    PM_REQUIRE(grad_out && aligned16(grad_out), "%s: grad_out must be a 16-byte aligned buffer", who);
    PM_REQUIRE(workspace && aligned16(workspace) &&
               workspace_bytes >= planmoe_combine_zfp_workspace_bytes(experts, capacity),
               "%s: workspace too small or not 16-byte aligned", who);
    int32_t *src = (int32_t *)workspace;
    float *sgate = (float *)(src + rows);
    int32_t *splane = (int32_t *)(sgate + rows);
    fill_u32((uint32_t *)src, (size_t)rows, 0xffffffffu, st);
    slot_source_mark<<<(unsigned)(((int64_t)samples * top_k + 255) / 256), 256, 0, st>>>(
        src, sgate, splane, nullptr, indices, locations, plane_stride, top_k, samples, experts, capacity);
    PM_NW_SWITCH(nw, NW, {
        bwd_gate_zfp2_kernel<NW><<<(unsigned)(rows / 4), 256, 0, st>>>((const uint32_t *)stream_in, src, splane, grad_out,
                                                                     plane_stride, model_dim, model_dim / 4, grad_gates);
    });
    PM_LAUNCH_CHECK(who);
    return 0;
}
