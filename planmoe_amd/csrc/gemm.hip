// Batched bf16 GEMM of the expert FFN, written for gfx950's matrix cores, and the transpose that
// brings an operand into k-major form where the direct forms do not apply.
//
//   C[e][m][n] = act( bf16( bf16( sum_k A[e][m][k] * B[e][n][k] ) + bias[e][n] ) )
//
// A matrix-core operand is eight consecutive k per lane.  An operand stored with k running fastest
// ("N" for A, "T" for B) gives that as one 16-byte read of LDS; an operand stored the other way round
// is read through LDS reads that transpose (ds_read_b64_tr_b16), so the direct-to-LDS kernel below
// takes either operand either way.  The reference's experts (experts/ffn.py:63-82) compute
// x @ fc1_w -> activation -> @ fc2_w with weights stored [experts, in, out]; the GEMM shapes of its
// forward and backward pass are
//   forward   y  = x  @ W          A = x  [rows, in],   B = W  [in, out]      planmoe_gemm_nn_bf16
//   backward  dx = dy @ W^T        A = dy [rows, out],  B = W  [in, out]      planmoe_gemm_nt_bf16
//             dW = x^T @ dy        A = x  [rows, in],   B = dy [rows, out]    planmoe_gemm_tn_bf16
// all with the operands as they lie in memory when the reduction length is a multiple of 64; for other
// lengths planmoe_gemm_nt_bf16 serves on transposed copies (the register-staged kernel, any k % 8 == 0).
//
// Tile 256 x 256 x 64 per work-group of four waves; a wave owns 128 x 128 as 4 x 4 tiles of
// v_mfma_f32_32x32x16_bf16 (256 accumulator registers, so one wave per SIMD: latency is covered by
// what the wave itself has in flight).  Per k-step of 16 a wave reads 8 fragments of 1 KB from LDS
// for 16 MFMAs of 32 cycles: LDS carries 64 bytes per clock for the four waves where 128 x 128
// tiles of 16 x 16 x 32 MFMAs (64 x 64 per wave) need 256.  LDS rows are 144 bytes apart (128 of
// data + 16): consecutive rows shift by one 16-byte unit, so the 8 / 16 rows that one pass of a
// fragment read or of a tile write touches fall into different banks whether the LDS serves 32 or
// 64 banks per clock.  LDS holds two k-tiles of both operands (144 KB); global loads run two
// k-tiles ahead in two register sets; one LDS-only barrier per k-tile, so the loads in flight
// stay in flight across it.  Epilogue: every wave passes its 128 x 128 quadrant through its own
// LDS region and stores whole 16-byte pieces of rows.
#include "common.hpp"

namespace pm {

typedef float  f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 gemm_bf16x8 __attribute__((ext_vector_type(8)));

constexpr int GEMM_BM = 256, GEMM_BN = 256, GEMM_BK = 64;
constexpr int GEMM_PITCH = 144;                             // bytes between LDS rows of a k-tile
constexpr int GEMM_TILE = 256 * GEMM_PITCH;                 // one operand's k-tile in LDS
constexpr int GEMM_CPITCH = 272;                            // bytes between rows of a wave's output quadrant in LDS
constexpr int GEMM_LDS = 4 * GEMM_TILE;                     // A0 B0 A1 B1 (the epilogue's 4 x 128 x 272 fits inside)
static_assert(4 * 128 * GEMM_CPITCH <= GEMM_LDS, "the output quadrants reuse the operand space");

__device__ __forceinline__ void gemm_lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

struct GemmArgs {
    const uint16_t *A, *B, *bias;
    uint16_t *C;
    int M, N, K;                  // rows of A, rows of B, reduction length
    int lda, ldb, ldc;            // elements between rows
    int64_t sA, sB, sC, sBias;    // elements between batches
    int batches;
};

template <int ACT>
__global__ __launch_bounds__(256, 1) void gemm_nt_bf16_kernel(const GemmArgs p)
{
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int wm = wave >> 1, wn = wave & 1;
    const int e = blockIdx.z, m0 = blockIdx.y * GEMM_BM, n0 = blockIdx.x * GEMM_BN;
    const uint8_t *A = reinterpret_cast<const uint8_t *>(p.A + (int64_t)e * p.sA);
    const uint8_t *B = reinterpret_cast<const uint8_t *>(p.B + (int64_t)e * p.sB);

    // what a thread fetches of one k-tile: chunk lc (8 values) of rows lr + 32 i of both operands.
    // Byte offsets from the batch's base (the host checks that they fit 32 bits); rows past the end
    // read the last row again (their products land in rows / columns nobody stores).
    const int lr = tid >> 3, lc = tid & 7;
    uint32_t ao[8], bo[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        ao[i] = (uint32_t)min(m0 + lr + 32 * i, p.M - 1) * (uint32_t)p.lda * 2u;
        bo[i] = (uint32_t)min(n0 + lr + 32 * i, p.N - 1) * (uint32_t)p.ldb * 2u;
    }
    // Every load is unconditional and straight-line (a chunk past
    // the end of K reads the row's last chunk instead and is zeroed by `keep` on its way into LDS).
    struct Fetched { uint4 a0, a1, a2, a3, a4, a5, a6, a7, b0, b1, b2, b3, b4, b5, b6, b7; uint32_t keep; } f0;
    const int KT = (p.K + GEMM_BK - 1) / GEMM_BK;
    const uint32_t last_chunk = (uint32_t)(p.K - 8) * 2u;
    auto load_tile = [&](Fetched &f, int kt) {
        const uint32_t kb = min((uint32_t)(kt * GEMM_BK + lc * 8) * 2u, last_chunk);
        f.keep = (kt < KT && kt * GEMM_BK + lc * 8 < p.K) ? 0xffffffffu : 0u;
#define PM_LD(dst, base, o) f.dst = *reinterpret_cast<const uint4 *>(base + (o + kb))
        PM_LD(a0, A, ao[0]); PM_LD(a1, A, ao[1]); PM_LD(a2, A, ao[2]); PM_LD(a3, A, ao[3]);
        PM_LD(a4, A, ao[4]); PM_LD(a5, A, ao[5]); PM_LD(a6, A, ao[6]); PM_LD(a7, A, ao[7]);
        PM_LD(b0, B, bo[0]); PM_LD(b1, B, bo[1]); PM_LD(b2, B, bo[2]); PM_LD(b3, B, bo[3]);
        PM_LD(b4, B, bo[4]); PM_LD(b5, B, bo[5]); PM_LD(b6, B, bo[6]); PM_LD(b7, B, bo[7]);
#undef PM_LD
    };
    auto store_tile = [&](const Fetched &f, int buf) {
        uint8_t *sa = lds + buf * 2 * GEMM_TILE + lr * GEMM_PITCH + lc * 16, *sb = sa + GEMM_TILE;
        const uint32_t k = f.keep;
#define PM_ST(base, i, v) *reinterpret_cast<uint4 *>(base + (i) * 32 * GEMM_PITCH) = make_uint4(f.v.x & k, f.v.y & k, f.v.z & k, f.v.w & k)
        PM_ST(sa, 0, a0); PM_ST(sa, 1, a1); PM_ST(sa, 2, a2); PM_ST(sa, 3, a3);
        PM_ST(sa, 4, a4); PM_ST(sa, 5, a5); PM_ST(sa, 6, a6); PM_ST(sa, 7, a7);
        PM_ST(sb, 0, b0); PM_ST(sb, 1, b1); PM_ST(sb, 2, b2); PM_ST(sb, 3, b3);
        PM_ST(sb, 4, b4); PM_ST(sb, 5, b5); PM_ST(sb, 6, b6); PM_ST(sb, 7, b7);
#undef PM_ST
    };

    f32x16 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;

    // lane l of a fragment: row l % 32, k-chunk l / 32 of the step.  The fragments of step s + 1 are
    // requested before the MFMAs of step s are issued (two fragment sets, used in turn).
    const int fr = lane & 31, fc = lane >> 5;
    struct Frags { gemm_bf16x8 a0, a1, a2, a3, b0, b1, b2, b3; };
    auto read_frags = [&](Frags &f, const uint8_t *sa, const uint8_t *sb, int ks) {
        f.a0 = *reinterpret_cast<const gemm_bf16x8 *>(sa + 0 * 32 * GEMM_PITCH + ks * 32);
        f.a1 = *reinterpret_cast<const gemm_bf16x8 *>(sa + 1 * 32 * GEMM_PITCH + ks * 32);
        f.a2 = *reinterpret_cast<const gemm_bf16x8 *>(sa + 2 * 32 * GEMM_PITCH + ks * 32);
        f.a3 = *reinterpret_cast<const gemm_bf16x8 *>(sa + 3 * 32 * GEMM_PITCH + ks * 32);
        f.b0 = *reinterpret_cast<const gemm_bf16x8 *>(sb + 0 * 32 * GEMM_PITCH + ks * 32);
        f.b1 = *reinterpret_cast<const gemm_bf16x8 *>(sb + 1 * 32 * GEMM_PITCH + ks * 32);
        f.b2 = *reinterpret_cast<const gemm_bf16x8 *>(sb + 2 * 32 * GEMM_PITCH + ks * 32);
        f.b3 = *reinterpret_cast<const gemm_bf16x8 *>(sb + 3 * 32 * GEMM_PITCH + ks * 32);
    };
#define PM_MMA(i, j, x, y) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, acc[i][j], 0, 0, 0)
    auto mma_step = [&](const Frags &f) {
        PM_MMA(0, 0, f.a0, f.b0); PM_MMA(0, 1, f.a0, f.b1); PM_MMA(0, 2, f.a0, f.b2); PM_MMA(0, 3, f.a0, f.b3);
        PM_MMA(1, 0, f.a1, f.b0); PM_MMA(1, 1, f.a1, f.b1); PM_MMA(1, 2, f.a1, f.b2); PM_MMA(1, 3, f.a1, f.b3);
        PM_MMA(2, 0, f.a2, f.b0); PM_MMA(2, 1, f.a2, f.b1); PM_MMA(2, 2, f.a2, f.b2); PM_MMA(2, 3, f.a2, f.b3);
        PM_MMA(3, 0, f.a3, f.b0); PM_MMA(3, 1, f.a3, f.b1); PM_MMA(3, 2, f.a3, f.b2); PM_MMA(3, 3, f.a3, f.b3);
    };
#undef PM_MMA
    auto multiply = [&](int buf) {
        const uint8_t *sa = lds + buf * 2 * GEMM_TILE + (wm * 128 + fr) * GEMM_PITCH + fc * 16;
        const uint8_t *sb = lds + buf * 2 * GEMM_TILE + GEMM_TILE + (wn * 128 + fr) * GEMM_PITCH + fc * 16;
        Frags g0, g1;
        read_frags(g0, sa, sb, 0);
        read_frags(g1, sa, sb, 1);
        mma_step(g0);
        __builtin_amdgcn_sched_barrier(0);
        read_frags(g0, sa, sb, 2);
        mma_step(g1);
        __builtin_amdgcn_sched_barrier(0);
        read_frags(g1, sa, sb, 3);
        mma_step(g0);
        __builtin_amdgcn_sched_barrier(0);
        mma_step(g1);
    };

    // one k-tile in registers on its way to LDS while the tile before it is multiplied
    load_tile(f0, 0);
    store_tile(f0, 0);
    gemm_lds_barrier();
    for (int kt = 0; kt < KT; ++kt) {
        load_tile(f0, kt + 1);                   // (past the end: zeros, never multiplied)
        multiply(kt & 1);
        store_tile(f0, (kt + 1) & 1);
        gemm_lds_barrier();
    }
    // every wave is done with the operand tiles before a quadrant overwrites them
    __syncthreads();

    // epilogue: acc[i][j][q] is row 32 i + 8 (q / 4) + 4 (lane / 32) + q % 4, column 32 j + lane % 32 of the quadrant
    uint8_t *quad = lds + wave * 128 * GEMM_CPITCH;
    const uint16_t *bias = p.bias ? p.bias + (int64_t)e * p.sBias + n0 + wn * 128 : nullptr;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int col = 32 * j + fr;
        const float fb = bias && n0 + wn * 128 + col < p.N ? bf16_to_f32(bias[col]) : 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int q = 0; q < 16; ++q) {
                const int row = 32 * i + 8 * (q >> 2) + 4 * fc + (q & 3);
                float v = bf16_to_f32(f32_to_bf16(acc[i][j][q]));       // the matmul's own rounding
                if (bias) v = bf16_to_f32(f32_to_bf16(v + fb));         // torch.add in bf16
                if (ACT == 1) v = fmaxf(v, 0.f);
                *reinterpret_cast<uint16_t *>(quad + row * GEMM_CPITCH + col * 2) = (uint16_t)f32_to_bf16(v);
            }
    }
    __builtin_amdgcn_wave_barrier();
    uint16_t *C = p.C + (int64_t)e * p.sC;
#pragma unroll 4
    for (int t = 0; t < 32; ++t) {
        const int q = lane + 64 * t, row = q >> 4, c = q & 15;
        const int gr = m0 + wm * 128 + row, gc = n0 + wn * 128 + c * 8;
        if (gr < p.M && gc < p.N)
            *reinterpret_cast<uint4 *>(C + (int64_t)gr * p.ldc + gc) = *reinterpret_cast<const uint4 *>(quad + row * GEMM_CPITCH + c * 16);
    }
}

// ---- the same product with the operands loaded straight into LDS (global_load_lds_dwordx4: the
// memory pipeline writes LDS itself, 16 bytes per lane at consecutive addresses, no register and no
// LDS-store instruction in between).  k-tiles of 64; LDS holds two of them for both operands and
// the loads of a tile are in flight during the MFMAs of the tile before it.  A load instruction
// fills 1 KB = 8 rows of 128 bytes; which 16-byte chunk of its row a lane fetches is chosen so
// that chunk c of row r lies at unit c ^ (r >> 1) & 7 of the row.  The LDS of this GPU serves 64
// banks (256 bytes) per clock, a 16-byte read 16 lanes at a time: the 16 consecutive rows of such a
// pass are 8 pairs of rows, the rows of a pair in different halves of the 256 bytes, the pairs at
// 8 different units.  (Measured with SQ_LDS_BANK_CONFLICT: 1.3 M conflict cycles per launch at
// 8 x 5120 x 4096 x 4096 against 85 M with c ^ r & 7, which would suit an LDS of 32 banks.)
// Needs k % 64 == 0.
constexpr int DMA_BK = 64, DMA_STAGES = 2;
constexpr int DMA_ROW = DMA_BK * 2;                         // bytes of a row of a k-tile
constexpr int DMA_OPERAND = 256 * DMA_ROW;                  // bytes of one operand's k-tile
constexpr int DMA_STAGE = 2 * DMA_OPERAND;
constexpr int DMA_LOADS = DMA_OPERAND / 1024 / 4;           // load instructions per wave, operand and k-tile
static_assert(DMA_STAGES * DMA_STAGE <= GEMM_LDS, "the kernels share the launch's LDS size");

__device__ __forceinline__ void gemm_dma16(const void *gbase, uint32_t voff, uint32_t lds_addr)
{
    // 16 bytes per lane from gbase + voff to LDS at lds_addr + 16 * lane
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" :: "s"(lds_addr), "v"(voff), "s"(gbase) : "memory", "m0");
}
// where chunk c of row r lies in its row of 8 units
__device__ __forceinline__ int dma_unit(int row, int chunk) { return chunk ^ ((row >> 1) & 7); }

// TA / TB = true: the operand is stored the other way round, a[e][k][m] / b[e][k][n] (both: c = a^T b, the
// weight gradient x^T dy; only b: c = a b with a weight as experts/ffn.py stores it; no transposed copies
// either way): a k-tile of such an operand is 64 rows of 512 bytes,
// a load instruction fills two of them, chunk c of row k lies at unit c ^ (k & 3) << 2, and a fragment
// comes out of LDS through ds_read_b64_tr_b16, which hands lane i of every 16 lanes element i % 4 of
// the 8 bytes that lanes i / 4, i / 4 + 4, i / 4 + 8, i / 4 + 12 point at: with lane s pointing at row
// s / 4, columns 4 (s % 4) .. + 3 of a 4 x 16 patch, lane i receives 4 consecutive k of column i --
// the matrix cores' operand layout.  Two such reads make the 8 k of a step; the 4 rows of a patch lie
// in different quarters of the 256 bytes the LDS serves per clock.  Needs k % 64 == 0.
typedef short gemm_s16x4 __attribute__((ext_vector_type(4)));
typedef short gemm_s16x8 __attribute__((ext_vector_type(8)));
__device__ __forceinline__ gemm_bf16x8 gemm_read_tr(const uint8_t *lo, const uint8_t *hi)
{
    typedef gemm_s16x4 __attribute__((address_space(3))) *lds_s16x4;
    const gemm_s16x4 x = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4)lo);
    const gemm_s16x4 y = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4)hi);
    const gemm_s16x8 v = __builtin_shufflevector(x, y, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(gemm_bf16x8, v);
}

template <int ACT, bool TA = false, bool TB = false>
__global__ __launch_bounds__(256, 1) void gemm_nt_bf16_dma_kernel(const GemmArgs p)
{
    extern __shared__ __align__(16) uint8_t lds[];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int wm = wave >> 1, wn = wave & 1;
    // Work-groups go to the 8 XCDs in turn, each XCD with an L2 of its own: XCD j (work-groups j, j + 8,
    // ...) takes the j-th eighth of the tiles, in the order batch, panel of 8 tile columns, tile row,
    // column of the panel, so that the 32 tiles it works on at a time are a 4 x 8 block of one batch
    // (12 operand tiles for 32 products; measured at 8 x 5120 x 4096 x 4096: L2 hits 69 -> 80 %, HBM reads
    // 3.3 -> 2.0 GB per launch).  The grid is one-dimensional, a multiple of 8; the surplus returns.
    const int tiles_m = (p.M + GEMM_BM - 1) / GEMM_BM, tiles_n = (p.N + GEMM_BN - 1) / GEMM_BN;
    const int64_t tiles = (int64_t)tiles_m * tiles_n * p.batches, per_xcd = (tiles + 7) / 8;
    const int64_t tile = (int64_t)(blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    if (tile >= tiles) return;
    const int e = (int)(tile / (tiles_m * tiles_n));
    int in_batch = (int)(tile - (int64_t)e * tiles_m * tiles_n);
    const int panel = in_batch / (tiles_m * 8);
    in_batch -= panel * tiles_m * 8;
    const int panel_width = min(8, tiles_n - panel * 8);
    const int m0 = (in_batch / panel_width) * GEMM_BM, n0 = (panel * 8 + in_batch % panel_width) * GEMM_BN;
    const uint8_t *A = reinterpret_cast<const uint8_t *>(p.A + (int64_t)e * p.sA);
    const uint8_t *B = reinterpret_cast<const uint8_t *>(p.B + (int64_t)e * p.sB);
    const uint32_t lds0 = (uint32_t)(uintptr_t)lds;
    const int wave_u = __builtin_amdgcn_readfirstlane(wave);        // (in a scalar register: LDS addresses of the loads are)

    // wave w brings in rows 64 w .. 64 w + 63 of both operands: 8 loads of 8 rows each.  Lane l of a
    // load fills unit l % 8 of row l / 8 of the block, i.e. fetches the chunk that belongs there.
    uint32_t ao[DMA_LOADS], bo[DMA_LOADS];
#pragma unroll
    for (int i = 0; i < DMA_LOADS; ++i) {
        // an operand with the reduction index slow: wave w brings in rows (k) 16 w .. 16 w + 15 of its
        // tile, 8 loads of 2 rows of 512 bytes
        const int trow = 16 * wave + 2 * i + (lane >> 5), tchunk = (lane & 31) ^ ((trow & 3) << 2);
        const int row = 64 * wave + 8 * i + (lane >> 3), chunk = dma_unit(row, lane & 7);
        ao[i] = TA ? (uint32_t)trow * (uint32_t)p.lda * 2u + (uint32_t)min(m0 + tchunk * 8, p.M - 8) * 2u
                   : (uint32_t)min(m0 + row, p.M - 1) * (uint32_t)p.lda * 2u + chunk * 16;
        bo[i] = TB ? (uint32_t)trow * (uint32_t)p.ldb * 2u + (uint32_t)min(n0 + tchunk * 8, p.N - 8) * 2u
                   : (uint32_t)min(n0 + row, p.N - 1) * (uint32_t)p.ldb * 2u + chunk * 16;
    }
    const int KT = p.K / DMA_BK;
    // a quarter of the loads of tile kt (a tile's loads go out in four parts, one before each k-step
    // of the tile before: 16 loads in a row hold the wave up at the address unit, and arrive in one burst)
    auto load_part = [&](int kt, int part) {
        // past the end: the last tile once more, into a buffer nobody reads again (keeps the number
        // of loads in flight the same in every round, which the waits below count on)
        const int k = min(kt, KT - 1);
        const uint8_t *ga = A + (TA ? (int64_t)k * DMA_BK * p.lda * 2 : (int64_t)k * (DMA_BK * 2));
        const uint8_t *gb = B + (TB ? (int64_t)k * DMA_BK * p.ldb * 2 : (int64_t)k * (DMA_BK * 2));
        const uint32_t sa = lds0 + (kt % DMA_STAGES) * DMA_STAGE + wave_u * (64 * DMA_ROW), sb = sa + DMA_OPERAND;   // (a wave's share is 8 KB either way)
        constexpr int PER = DMA_LOADS / 4;
#pragma unroll
        for (int i = PER * part; i < PER * part + PER; ++i) gemm_dma16(ga, ao[i], sa + i * 1024);
#pragma unroll
        for (int i = PER * part; i < PER * part + PER; ++i) gemm_dma16(gb, bo[i], sb + i * 1024);
    };
    static_assert(DMA_LOADS % 4 == 0, "a tile's loads go out in four parts");

    f32x16 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int q = 0; q < 16; ++q) acc[i][j][q] = 0.f;

    // fragment of a step: lane l holds row l % 32, chunk 2 ks + l / 32 of its rows
    const int fr = lane & 31, fc = lane >> 5;
    struct Frags { gemm_bf16x8 a0, a1, a2, a3, b0, b1, b2, b3; };
    // an operand with the reduction index slow: lane = (group g of 16 lanes, s): row 8 (g / 2) + s / 4 of the step's 16, bytes 8 (s % 4) of the
    // 32 that columns 16 (g % 2) .. + 15 of the fragment take; unit of the row swizzled by s / 4 = row & 3
    const int tg = lane >> 4, ts = lane & 15;
    const int t_row = (8 * (tg >> 1) + (ts >> 2)) * 512;
    int t_col[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) t_col[i] = (4 * (i ^ (ts >> 2)) + 2 * (tg & 1) + ((ts & 3) >> 1)) * 16 + 8 * (ts & 1);
    auto read_frags = [&](Frags &f, const uint8_t *st, int ks) {
#define PM_FT(base, i) gemm_read_tr(base + t_col[i], base + t_col[i] + 4 * 512)
#define PM_FR(base, i) *reinterpret_cast<const gemm_bf16x8 *>(base + (i) * 32 * DMA_ROW + dma_unit(32 * (i) + fr, 2 * ks + fc) * 16)
        if constexpr (TA) {
            const uint8_t *sa = st + t_row + ks * (16 * 512) + wm * 256;
            f.a0 = PM_FT(sa, 0); f.a1 = PM_FT(sa, 1); f.a2 = PM_FT(sa, 2); f.a3 = PM_FT(sa, 3);
        } else {
            const uint8_t *sa = st + (wm * 128 + fr) * DMA_ROW;
            f.a0 = PM_FR(sa, 0); f.a1 = PM_FR(sa, 1); f.a2 = PM_FR(sa, 2); f.a3 = PM_FR(sa, 3);
        }
        if constexpr (TB) {
            const uint8_t *sb = st + DMA_OPERAND + t_row + ks * (16 * 512) + wn * 256;
            f.b0 = PM_FT(sb, 0); f.b1 = PM_FT(sb, 1); f.b2 = PM_FT(sb, 2); f.b3 = PM_FT(sb, 3);
        } else {
            const uint8_t *sb = st + DMA_OPERAND + (wn * 128 + fr) * DMA_ROW;
            f.b0 = PM_FR(sb, 0); f.b1 = PM_FR(sb, 1); f.b2 = PM_FR(sb, 2); f.b3 = PM_FR(sb, 3);
        }
#undef PM_FR
#undef PM_FT
    };
#define PM_MMA(i, j, x, y) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(x, y, acc[i][j], 0, 0, 0)
    auto mma_step = [&](const Frags &f) {
        PM_MMA(0, 0, f.a0, f.b0); PM_MMA(0, 1, f.a0, f.b1); PM_MMA(0, 2, f.a0, f.b2); PM_MMA(0, 3, f.a0, f.b3);
        PM_MMA(1, 0, f.a1, f.b0); PM_MMA(1, 1, f.a1, f.b1); PM_MMA(1, 2, f.a1, f.b2); PM_MMA(1, 3, f.a1, f.b3);
        PM_MMA(2, 0, f.a2, f.b0); PM_MMA(2, 1, f.a2, f.b1); PM_MMA(2, 2, f.a2, f.b2); PM_MMA(2, 3, f.a2, f.b3);
        PM_MMA(3, 0, f.a3, f.b0); PM_MMA(3, 1, f.a3, f.b1); PM_MMA(3, 2, f.a3, f.b2); PM_MMA(3, 3, f.a3, f.b3);
    };
#undef PM_MMA

#pragma unroll
    for (int part = 0; part < 4; ++part) load_part(0, part);
    for (int kt = 0; kt < KT; ++kt) {
        // this wave's loads of tile kt are in; behind the barrier everybody's are, and everybody is
        // done reading tile kt - 1, whose buffer the loads of tile kt + 1 then fill during this tile's MFMAs
        asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
        const uint8_t *st = lds + (kt % DMA_STAGES) * DMA_STAGE;
        Frags g0, g1;
        read_frags(g0, st, 0);
        read_frags(g1, st, 1);
        load_part(kt + 1, 0);
        mma_step(g0);
        __builtin_amdgcn_sched_barrier(0);
        read_frags(g0, st, 2);
        load_part(kt + 1, 1);
        mma_step(g1);
        __builtin_amdgcn_sched_barrier(0);
        read_frags(g1, st, 3);
        load_part(kt + 1, 2);
        mma_step(g0);
        __builtin_amdgcn_sched_barrier(0);
        load_part(kt + 1, 3);
        mma_step(g1);
    }
    // nothing may still be on its way into LDS when the quadrants overwrite it
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();

    uint8_t *quad = lds + wave * 128 * GEMM_CPITCH;
    const uint16_t *bias = p.bias ? p.bias + (int64_t)e * p.sBias + n0 + wn * 128 : nullptr;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int col = 32 * j + fr;
        const float fb = bias && n0 + wn * 128 + col < p.N ? bf16_to_f32(bias[col]) : 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int q = 0; q < 16; ++q) {
                const int row = 32 * i + 8 * (q >> 2) + 4 * fc + (q & 3);
                float v = bf16_to_f32(f32_to_bf16(acc[i][j][q]));
                if (bias) v = bf16_to_f32(f32_to_bf16(v + fb));
                if (ACT == 1) v = fmaxf(v, 0.f);
                *reinterpret_cast<uint16_t *>(quad + row * GEMM_CPITCH + col * 2) = (uint16_t)f32_to_bf16(v);
            }
    }
    __builtin_amdgcn_wave_barrier();
    uint16_t *C = p.C + (int64_t)e * p.sC;
#pragma unroll 4
    for (int t = 0; t < 32; ++t) {
        const int q = lane + 64 * t, row = q >> 4, c = q & 15;
        const int gr = m0 + wm * 128 + row, gc = n0 + wn * 128 + c * 8;
        if (gr < p.M && gc < p.N)
            *reinterpret_cast<uint4 *>(C + (int64_t)gr * p.ldc + gc) = *reinterpret_cast<const uint4 *>(quad + row * GEMM_CPITCH + c * 16);
    }
}

// out[e][c][r] = in[e][r][c] for r < rows, zero for rows <= r < rows_out (the padding of a k dimension):
// 64 x 64 tiles through LDS, 16-byte accesses on both sides
__global__ __launch_bounds__(256) void transpose_bf16_kernel(const uint16_t *__restrict__ in, uint16_t *__restrict__ out,
                                                             int rows, int cols, int rows_out, int64_t s_in, int64_t s_out)
{
    __shared__ uint16_t tile[64][64 + 2];
    const int e = blockIdx.z, r0 = blockIdx.y * 64, c0 = blockIdx.x * 64, tid = threadIdx.x;
    in += (int64_t)e * s_in;
    out += (int64_t)e * s_out;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int q = tid + 256 * i, r = q >> 3, c = (q & 7) * 8;
        uint4 v = make_uint4(0u, 0u, 0u, 0u);
        if (r0 + r < rows && c0 + c < cols) v = *reinterpret_cast<const uint4 *>(in + (int64_t)(r0 + r) * cols + c0 + c);
        uint32_t *dst = reinterpret_cast<uint32_t *>(&tile[r][c]);
        dst[0] = v.x; dst[1] = v.y; dst[2] = v.z; dst[3] = v.w;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int q = tid + 256 * i, c = q >> 3, r = (q & 7) * 8;
        if (c0 + c < cols && r0 + r < rows_out) {
            uint32_t w[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] = (uint32_t)tile[r + 2 * j][c] | ((uint32_t)tile[r + 2 * j + 1][c] << 16);
            *reinterpret_cast<uint4 *>(out + (int64_t)(c0 + c) * rows_out + r0 + r) = make_uint4(w[0], w[1], w[2], w[3]);
        }
    }
}

} // namespace pm

using namespace pm;

extern "C" int planmoe_gemm_nt_bf16(const void *a, const void *b, const void *bias, int activation, int batches,
                                    int m, int n, int k, int lda, int ldb, int ldc, int64_t batch_stride_a,
                                    int64_t batch_stride_b, int64_t batch_stride_c, void *c, void *stream)
{
    PM_REQUIRE(batches >= 0 && m >= 0 && n >= 0 && k >= 1, "planmoe_gemm_nt_bf16: bad shape");
    if (batches == 0 || m == 0 || n == 0) return 0;
    PM_REQUIRE(a && b && c, "planmoe_gemm_nt_bf16: NULL argument");
    PM_REQUIRE(activation == 0 || activation == 1, "planmoe_gemm_nt_bf16: activation is 0 (none) or 1 (relu)");
    PM_REQUIRE(k % 8 == 0 && n % 8 == 0 && lda % 8 == 0 && ldb % 8 == 0 && ldc % 8 == 0 && lda >= k && ldb >= k && ldc >= n,
               "planmoe_gemm_nt_bf16: k, n and the row pitches must be multiples of 8 (16-byte pieces); pitches cover their rows");
    PM_REQUIRE(batch_stride_a % 8 == 0 && batch_stride_b % 8 == 0 && batch_stride_c % 8 == 0 && aligned16(a) && aligned16(b) && aligned16(c),
               "planmoe_gemm_nt_bf16: operands must be 16-byte aligned");
    const int64_t tm = ((int64_t)m + GEMM_BM - 1) / GEMM_BM, tn = ((int64_t)n + GEMM_BN - 1) / GEMM_BN;
    PM_REQUIRE(tm <= 65535 && batches <= 65535, "planmoe_gemm_nt_bf16: too many row tiles or batches");
    PM_REQUIRE((int64_t)m * lda * 2 < ((int64_t)1 << 32) && (int64_t)n * ldb * 2 < ((int64_t)1 << 32),
               "planmoe_gemm_nt_bf16: an operand of one batch must stay under 4 GiB");
    GemmArgs p{(const uint16_t *)a, (const uint16_t *)b, (const uint16_t *)bias, (uint16_t *)c, m, n, k, lda, ldb, ldc,
               batch_stride_a, batch_stride_b, batch_stride_c, (int64_t)n, batches};
    const void *fn = activation == 0 ? (const void *)gemm_nt_bf16_kernel<0> : (const void *)gemm_nt_bf16_kernel<1>;
    PM_REQUIRE(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_LDS) == hipSuccess,
               "planmoe_gemm_nt_bf16: the kernel needs %d bytes of LDS", GEMM_LDS);
    const dim3 grid((unsigned)tn, (unsigned)tm, (unsigned)batches);
    if (k % DMA_BK == 0) {
        // operands straight into LDS, loads three k-tiles ahead
        const void *fd = activation == 0 ? (const void *)gemm_nt_bf16_dma_kernel<0> : (const void *)gemm_nt_bf16_dma_kernel<1>;
        PM_REQUIRE(hipFuncSetAttribute(fd, hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_LDS) == hipSuccess,
                   "planmoe_gemm_nt_bf16: the kernel needs %d bytes of LDS", GEMM_LDS);
        const int64_t per_xcd = (tm * tn * batches + 7) / 8;
        PM_REQUIRE(per_xcd * 8 < ((int64_t)1 << 31), "planmoe_gemm_nt_bf16: too many tiles");
        const dim3 tiles((unsigned)(per_xcd * 8));
        if (activation == 0) gemm_nt_bf16_dma_kernel<0><<<tiles, 256, GEMM_LDS, (hipStream_t)stream>>>(p);
        else gemm_nt_bf16_dma_kernel<1><<<tiles, 256, GEMM_LDS, (hipStream_t)stream>>>(p);
        PM_LAUNCH_CHECK("planmoe_gemm_nt_bf16");
        return 0;
    }
    if (activation == 0) gemm_nt_bf16_kernel<0><<<grid, 256, GEMM_LDS, (hipStream_t)stream>>>(p);
    else gemm_nt_bf16_kernel<1><<<grid, 256, GEMM_LDS, (hipStream_t)stream>>>(p);
    PM_LAUNCH_CHECK("planmoe_gemm_nt_bf16");
    return 0;
}

extern "C" int planmoe_gemm_nn_bf16(const void *a, const void *b, const void *bias, int activation, int batches,
                                    int m, int n, int k, int lda, int ldb, int ldc, int64_t batch_stride_a,
                                    int64_t batch_stride_b, int64_t batch_stride_c, void *c, void *stream)
{
    PM_REQUIRE(batches >= 0 && m >= 0 && n >= 0 && k >= 64, "planmoe_gemm_nn_bf16: bad shape");
    if (batches == 0 || m == 0 || n == 0) return 0;
    PM_REQUIRE(a && b && c, "planmoe_gemm_nn_bf16: NULL argument");
    PM_REQUIRE(activation == 0 || activation == 1, "planmoe_gemm_nn_bf16: activation is 0 (none) or 1 (relu)");
    PM_REQUIRE(k % DMA_BK == 0, "planmoe_gemm_nn_bf16: k must be a multiple of %d", DMA_BK);
    PM_REQUIRE(n % 8 == 0 && lda % 8 == 0 && ldb % 8 == 0 && ldc % 8 == 0 && lda >= k && ldb >= n && ldc >= n,
               "planmoe_gemm_nn_bf16: n and the row pitches must be multiples of 8 (16-byte pieces); pitches cover their rows");
    PM_REQUIRE(batch_stride_a % 8 == 0 && batch_stride_b % 8 == 0 && batch_stride_c % 8 == 0 && aligned16(a) && aligned16(b) && aligned16(c),
               "planmoe_gemm_nn_bf16: operands must be 16-byte aligned");
    PM_REQUIRE((int64_t)m * lda * 2 < ((int64_t)1 << 32) && (int64_t)DMA_BK * ldb * 2 < ((int64_t)1 << 31),
               "planmoe_gemm_nn_bf16: the first operand of one batch must stay under 4 GiB, 64 rows of the second under 2 GiB");
    const int64_t tm = ((int64_t)m + GEMM_BM - 1) / GEMM_BM, tn = ((int64_t)n + GEMM_BN - 1) / GEMM_BN;
    const int64_t per_xcd = (tm * tn * batches + 7) / 8;
    PM_REQUIRE(per_xcd * 8 < ((int64_t)1 << 31), "planmoe_gemm_nn_bf16: too many tiles");
    GemmArgs p{(const uint16_t *)a, (const uint16_t *)b, (const uint16_t *)bias, (uint16_t *)c, m, n, k, lda, ldb, ldc,
               batch_stride_a, batch_stride_b, batch_stride_c, (int64_t)n, batches};
    const void *fd = activation == 0 ? (const void *)gemm_nt_bf16_dma_kernel<0, false, true>
                                     : (const void *)gemm_nt_bf16_dma_kernel<1, false, true>;
    PM_REQUIRE(hipFuncSetAttribute(fd, hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_LDS) == hipSuccess,
               "planmoe_gemm_nn_bf16: the kernel needs %d bytes of LDS", GEMM_LDS);
    const dim3 tiles((unsigned)(per_xcd * 8));
    if (activation == 0) gemm_nt_bf16_dma_kernel<0, false, true><<<tiles, 256, GEMM_LDS, (hipStream_t)stream>>>(p);
    else gemm_nt_bf16_dma_kernel<1, false, true><<<tiles, 256, GEMM_LDS, (hipStream_t)stream>>>(p);
    PM_LAUNCH_CHECK("planmoe_gemm_nn_bf16");
    return 0;
}

extern "C" int planmoe_gemm_tn_bf16(const void *a, const void *b, int batches, int m, int n, int k, int lda, int ldb,
                                    int ldc, int64_t batch_stride_a, int64_t batch_stride_b, int64_t batch_stride_c,
                                    void *c, void *stream)
{
    PM_REQUIRE(batches >= 0 && m >= 0 && n >= 0 && k >= 64, "planmoe_gemm_tn_bf16: bad shape");
    if (batches == 0 || m == 0 || n == 0) return 0;
    PM_REQUIRE(a && b && c, "planmoe_gemm_tn_bf16: NULL argument");
    PM_REQUIRE(k % DMA_BK == 0, "planmoe_gemm_tn_bf16: k must be a multiple of %d", DMA_BK);
    PM_REQUIRE(m % 8 == 0 && n % 8 == 0 && lda % 8 == 0 && ldb % 8 == 0 && ldc % 8 == 0 && lda >= m && ldb >= n && ldc >= n,
               "planmoe_gemm_tn_bf16: m, n and the row pitches must be multiples of 8 (16-byte pieces); pitches cover their rows");
    PM_REQUIRE(batch_stride_a % 8 == 0 && batch_stride_b % 8 == 0 && batch_stride_c % 8 == 0 && aligned16(a) && aligned16(b) && aligned16(c),
               "planmoe_gemm_tn_bf16: operands must be 16-byte aligned");
    PM_REQUIRE((int64_t)DMA_BK * lda * 2 < ((int64_t)1 << 31) && (int64_t)DMA_BK * ldb * 2 < ((int64_t)1 << 31),
               "planmoe_gemm_tn_bf16: 64 rows of an operand must stay under 2 GiB");
    const int64_t tm = ((int64_t)m + GEMM_BM - 1) / GEMM_BM, tn = ((int64_t)n + GEMM_BN - 1) / GEMM_BN;
    const int64_t per_xcd = (tm * tn * batches + 7) / 8;
    PM_REQUIRE(per_xcd * 8 < ((int64_t)1 << 31), "planmoe_gemm_tn_bf16: too many tiles");
    GemmArgs p{(const uint16_t *)a, (const uint16_t *)b, nullptr, (uint16_t *)c, m, n, k, lda, ldb, ldc,
               batch_stride_a, batch_stride_b, batch_stride_c, 0, batches};
    const void *fd = (const void *)gemm_nt_bf16_dma_kernel<0, true, true>;
    PM_REQUIRE(hipFuncSetAttribute(fd, hipFuncAttributeMaxDynamicSharedMemorySize, GEMM_LDS) == hipSuccess,
               "planmoe_gemm_tn_bf16: the kernel needs %d bytes of LDS", GEMM_LDS);
    gemm_nt_bf16_dma_kernel<0, true, true><<<dim3((unsigned)(per_xcd * 8)), 256, GEMM_LDS, (hipStream_t)stream>>>(p);
    PM_LAUNCH_CHECK("planmoe_gemm_tn_bf16");
    return 0;
}

extern "C" int planmoe_transpose_bf16(const void *in, int batches, int rows, int cols, int rows_out, void *out, void *stream)
{
    PM_REQUIRE(batches >= 0 && rows >= 0 && cols >= 0 && rows_out >= rows, "planmoe_transpose_bf16: bad shape");
    if (batches == 0 || cols == 0 || rows_out == 0) return 0;
    PM_REQUIRE(in && out, "planmoe_transpose_bf16: NULL argument");
    PM_REQUIRE(cols % 8 == 0 && rows_out % 8 == 0 && aligned16(in) && aligned16(out),
               "planmoe_transpose_bf16: cols and rows_out must be multiples of 8, buffers 16-byte aligned");
    PM_REQUIRE((rows_out + 63) / 64 <= 65535 && batches <= 65535, "planmoe_transpose_bf16: too many tiles");
    const dim3 grid((unsigned)((cols + 63) / 64), (unsigned)((rows_out + 63) / 64), (unsigned)batches);
    transpose_bf16_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const uint16_t *)in, (uint16_t *)out, rows, cols, rows_out,
                                                                 (int64_t)rows * cols, (int64_t)cols * rows_out);
    PM_LAUNCH_CHECK("planmoe_transpose_bf16");
    return 0;
}
