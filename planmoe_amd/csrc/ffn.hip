// First GEMM of the expert FFN with the int8 decode as its prologue.
//
// On the receive side the reference decompresses the codes into a [experts, capacity, model_dim]
// tensor (Int8Compressor::decompress, int8.cpp:46-60, called from overlap.py:66) and the experts
// then read that tensor in their first batched GEMM (experts/ffn.py:77).  Here the GEMM reads the
// codes: a work-group decodes its 128 x 64 tile of codes to the very bf16 values the decompressor
// would have stored (the same three rounded steps per element) on the way into LDS, so the
// decoded tensor never exists in memory, and the matrix cores see ordinary bf16 operands.
//
//   out[e][r][n] = bf16( bf16( sum_k dec(e, r, k) * w[e][n][k] ) + fc_bias[e][n] )
//
// w is taken with k running fastest ([experts, hidden, model_dim]): both MFMA operands want eight
// consecutive k per lane.  Tile 128 x 128 x 64, four waves of 64 x 64 (4 x 4 tiles of
// v_mfma_f32_16x16x32_bf16), operands through LDS in 16-byte chunks placed at chunk ^ (row & 7) so
// that the 16 rows a fragment read touches fall into different banks; the next tile's global
// loads are in flight during the MFMAs of the current one.
#include "gate_core.hpp"
#include "int8_core.hpp"

namespace pm {

constexpr int FFN_BM = 128, FFN_BN = 128, FFN_BK = 64;

__device__ __forceinline__ uint32_t codes_to_bf16x2(uint32_t w, int first)
{
    // bf16 of two bytes of w: the upper halves of their fp32 conversions
    const float lo = (float)((w >> (first ? 16 : 0)) & 0xffu), hi = (float)((w >> (first ? 24 : 8)) & 0xffu);
    return __builtin_amdgcn_perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);
}

// AFFINE: the row's affine map is taken out of the sum,
//   sum_k dec(r, k) w[n][k]  ~  (scale_r / 255) * sum_k code[r][k] w[n][k]  +  bias_r * sum_k w[n][k]
// so the matrix cores multiply the codes themselves (0 .. 255 are exact in bf16; two instructions
// per four codes instead of the decompressor's fifteen per two) and the epilogue applies scale, bias
// and the column sums of the weights, which the caller computes once per weight.  What is lost are
// the three bf16 roundings the decompressor applies to every element: the result differs by about an
// ulp of the bf16 output (tolerance-level parity), where the other form multiplies exactly the
// decompressor's values.  (Larger tiles, which would cut the LDS traffic per MFMA, were tried and
// are slower as compiled: 256 x 256 with 128 x 128 per wave keeps half of its 256 accumulator
// registers in the other register file and copies them in every step, 340 TFLOP/s; 256 x 128 with
// 128 x 64 per wave takes 304 registers, one wave per SIMD, 476 TFLOP/s.)
template <bool AFFINE>
__global__ __launch_bounds__(256, 3) void ffn_fc1_int8_kernel(
    const uint8_t *__restrict__ codes, const uint16_t *__restrict__ qbias, const uint16_t *__restrict__ qscale,
    const uint16_t *__restrict__ w, const float *__restrict__ colsum, const uint16_t *__restrict__ fc_bias,
    int rows, int K, int N, uint16_t *__restrict__ out)
{
    using B16 = Elem<PLANMOE_BF16>;
    __shared__ uint4 smem[(FFN_BM + FFN_BN) * FFN_BK * 2 / 16];          // A tile, then B tile: 32 KB
    uint4 *sA = smem, *sB = smem + FFN_BM * FFN_BK * 2 / 16;
    const int tid = threadIdx.x, wave = tid >> 6, lane = lane_id(), m = lane & 15, g = lane >> 4;
    const int e = blockIdx.z, r0 = blockIdx.y * FFN_BM, n0 = blockIdx.x * FFN_BN;
    const int wm = wave >> 1, wn = wave & 1;

    // this thread's share of the A tile: 32 consecutive codes of one row; of the B tile: 4 chunks
    const int ar = tid >> 1, ah = tid & 1;
    const int arow = min(r0 + ar, rows - 1);                              // rows past the end re-read the last one
    const uint8_t *ap = codes + ((int64_t)e * rows + arow) * K + ah * 32;
    const RowDecoder<PLANMOE_BF16> dec(B16::load(qbias, (int64_t)e * rows + arow), B16::load(qscale, (int64_t)e * rows + arow));
    const uint16_t *wp = w + ((int64_t)e * N + n0) * K;

    // What a thread fetches of one k-tile.  Two sets: the loads of a tile are issued two tiles ahead,
    // since one tile's MFMAs (512 cycles per wave, three work-groups per CU) do not cover the latency
    // of a load.  (Named members: an array indexed inside these helpers ends up in private memory.)
    struct Fetched { uint4 ca0, ca1, cb0, cb1, cb2, cb3; } f0, f1;
    const int brow = tid >> 3, bc = tid & 7;                         // chunk tid + 256 i: row brow + 32 i, chunk bc
    const uint16_t *bsrc = wp + (int64_t)brow * K + bc * 8;
    const int64_t bstep = (int64_t)32 * K;
    auto load_tile = [&](Fetched &f, int kt) {
        const int k0 = kt * FFN_BK;
        f.ca0 = *reinterpret_cast<const uint4 *>(ap + k0);
        f.ca1 = *reinterpret_cast<const uint4 *>(ap + k0 + 16);
        f.cb0 = *reinterpret_cast<const uint4 *>(bsrc + k0);
        f.cb1 = *reinterpret_cast<const uint4 *>(bsrc + bstep + k0);
        f.cb2 = *reinterpret_cast<const uint4 *>(bsrc + 2 * bstep + k0);
        f.cb3 = *reinterpret_cast<const uint4 *>(bsrc + 3 * bstep + k0);
    };
    auto decode_chunk = [&](uint32_t lo, uint32_t hi, int j) {
        if constexpr (AFFINE) {
            sA[ar * 8 + ((ah * 4 + j) ^ (ar & 7))] = make_uint4(codes_to_bf16x2(lo, 0), codes_to_bf16x2(lo, 1),
                                                                 codes_to_bf16x2(hi, 0), codes_to_bf16x2(hi, 1));
        } else {
            float f[8];
            dec.word(lo, f);
            dec.word(hi, f + 4);
            sA[ar * 8 + ((ah * 4 + j) ^ (ar & 7))] = B16::pack(f);
        }
    };
    auto store_tile = [&](const Fetched &f) {
        // 32 codes -> 32 bf16 values = 4 chunks of this row
        decode_chunk(f.ca0.x, f.ca0.y, 0);
        decode_chunk(f.ca0.z, f.ca0.w, 1);
        decode_chunk(f.ca1.x, f.ca1.y, 2);
        decode_chunk(f.ca1.z, f.ca1.w, 3);
        // rows brow + 32 i share brow & 7, hence the chunk's place
        const int place = bc ^ (brow & 7);
        sB[brow * 8 + place] = f.cb0;
        sB[(brow + 32) * 8 + place] = f.cb1;
        sB[(brow + 64) * 8 + place] = f.cb2;
        sB[(brow + 96) * 8 + place] = f.cb3;
    };

    const int KT = K / FFN_BK;
    f32x4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

    auto multiply = [&]() {
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            uint4 af[4], bf[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int row = wm * 64 + i * 16 + m;
                af[i] = sA[row * 8 + ((ks * 4 + g) ^ (row & 7))];
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const int row = wn * 64 + j * 16 + m;
                bf[j] = sB[row * 8 + ((ks * 4 + g) ^ (row & 7))];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) Mma<PLANMOE_BF16>::run(af[i], bf[j], acc[i][j]);
        }
    };
    auto step = [&](Fetched &f, int kt) {
        store_tile(f);
        __syncthreads();
        load_tile(f, min(kt + 2, KT - 1));          // (past the end: the last tile once more, never used)
        multiply();
        __syncthreads();
    };

    load_tile(f0, 0);
    load_tile(f1, min(1, KT - 1));
    for (int kt = 0; kt < KT; kt += 2) {
        step(f0, kt);
        if (kt + 1 < KT) step(f1, kt + 1);
    }

    // epilogue: the tile goes through LDS (the operand space, 128 x 128 bf16) so that it leaves in
    // 16-byte pieces of whole rows; acc[i][j][q] is row 4 g + q of tile i, column m of tile j
    uint16_t *sC = reinterpret_cast<uint16_t *>(smem);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int col = wn * 64 + j * 16 + m;
        const float fb = fc_bias ? B16::load(fc_bias, (int64_t)e * N + n0 + col) : 0.f;
        const float cs = AFFINE ? colsum[(int64_t)e * N + n0 + col] : 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int row = wm * 64 + i * 16 + 4 * g + q;
                float v = acc[i][j][q];
                if constexpr (AFFINE) {
                    const int64_t gr = (int64_t)e * rows + min(r0 + row, rows - 1);
                    v = B16::load(qscale, gr) * (1.0f / 255.0f) * v + B16::load(qbias, gr) * cs;
                }
                v = B16::round(v);                                  // the matmul's own rounding
                if (fc_bias) v = v + fb;                            // torch.add in bf16
                sC[row * FFN_BN + col] = (uint16_t)f32_to_bf16(v);
            }
    }
    __syncthreads();
    const uint4 *sC4 = reinterpret_cast<const uint4 *>(smem);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int q = tid + 256 * i, row = q >> 4, c = q & 15;
        if (r0 + row < rows)
            *reinterpret_cast<uint4 *>(out + ((int64_t)e * rows + r0 + row) * N + n0 + c * 8) = sC4[q];
    }
}

} // namespace pm

using namespace pm;

extern "C" int planmoe_ffn_fc1_int8_affine(const uint8_t *codes, const void *bias, const void *scale, int dtype,
                                           const void *weight_k_major, const float *weight_colsum, const void *fc_bias,
                                           int experts, int rows, int model_dim, int hidden, void *out, void *stream)
{
    PM_REQUIRE(dtype == PLANMOE_BF16, "planmoe_ffn_fc1_int8_affine: bf16 only (got dtype tag %d)", dtype);
    PM_REQUIRE(experts >= 0 && rows >= 0 && model_dim >= 1 && hidden >= 1, "planmoe_ffn_fc1_int8_affine: bad shape");
    if (experts == 0 || rows == 0) return 0;
    PM_REQUIRE(model_dim % FFN_BK == 0 && hidden % FFN_BN == 0,
               "planmoe_ffn_fc1_int8_affine: model_dim must be a multiple of %d and hidden of %d (got %d, %d)", FFN_BK, FFN_BN,
               model_dim, hidden);
    PM_REQUIRE(codes && bias && scale && weight_k_major && weight_colsum && out, "planmoe_ffn_fc1_int8_affine: NULL argument");
    PM_REQUIRE(aligned16(codes) && aligned16(weight_k_major) && aligned16(out), "planmoe_ffn_fc1_int8_affine: buffers must be 16-byte aligned");
    PM_REQUIRE((rows + FFN_BM - 1) / FFN_BM <= 65535 && experts <= 65535, "planmoe_ffn_fc1_int8_affine: too many row tiles or experts");
    const dim3 grid((unsigned)(hidden / FFN_BN), (unsigned)((rows + FFN_BM - 1) / FFN_BM), (unsigned)experts);
    ffn_fc1_int8_kernel<true><<<grid, 256, 0, (hipStream_t)stream>>>(
        codes, (const uint16_t *)bias, (const uint16_t *)scale, (const uint16_t *)weight_k_major, weight_colsum,
        (const uint16_t *)fc_bias, rows, model_dim, hidden, (uint16_t *)out);
    PM_LAUNCH_CHECK("planmoe_ffn_fc1_int8_affine");
    return 0;
}

extern "C" int planmoe_ffn_fc1_int8(const uint8_t *codes, const void *bias, const void *scale, int dtype,
                                    const void *weight_k_major, const void *fc_bias, int experts, int rows,
                                    int model_dim, int hidden, void *out, void *stream)
{
    PM_REQUIRE(dtype == PLANMOE_BF16, "planmoe_ffn_fc1_int8: bf16 only (got dtype tag %d)", dtype);
    PM_REQUIRE(experts >= 0 && rows >= 0 && model_dim >= 1 && hidden >= 1, "planmoe_ffn_fc1_int8: bad shape");
    if (experts == 0 || rows == 0) return 0;
    PM_REQUIRE(model_dim % FFN_BK == 0 && hidden % FFN_BN == 0,
               "planmoe_ffn_fc1_int8: model_dim must be a multiple of %d and hidden of %d (got %d, %d)", FFN_BK, FFN_BN,
               model_dim, hidden);
    PM_REQUIRE(codes && bias && scale && weight_k_major && out, "planmoe_ffn_fc1_int8: NULL argument");
    PM_REQUIRE(aligned16(codes) && aligned16(weight_k_major) && aligned16(out), "planmoe_ffn_fc1_int8: buffers must be 16-byte aligned");
    PM_REQUIRE((rows + FFN_BM - 1) / FFN_BM <= 65535 && experts <= 65535, "planmoe_ffn_fc1_int8: too many row tiles or experts");
    const dim3 grid((unsigned)(hidden / FFN_BN), (unsigned)((rows + FFN_BM - 1) / FFN_BM), (unsigned)experts);
    ffn_fc1_int8_kernel<false><<<grid, 256, 0, (hipStream_t)stream>>>(
        codes, (const uint16_t *)bias, (const uint16_t *)scale, (const uint16_t *)weight_k_major, nullptr,
        (const uint16_t *)fc_bias, rows, model_dim, hidden, (uint16_t *)out);
    PM_LAUNCH_CHECK("planmoe_ffn_fc1_int8");
    return 0;
}
