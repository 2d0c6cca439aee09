// Kernel selection for Y = epilogue(X * dequant(W) + bias) with Bfp8_b weights: up to four tile rows ->
// weight streaming kernel, macro-tile aligned shapes -> the MFMA kernel of gemm_bfp8b_kernel.hpp in
// one of its tile shapes and forms, a row count that is not a multiple of 128 -> both (rows split), N an odd
// number of tiles -> both (columns split), everything else -> the bounds-checked general kernel.
#include <cstdlib>

#include "gemm_bfp8b_kernel.hpp"

namespace ttbfp {

#ifndef TTBFP_SLIM_BELOW_TILES
#define TTBFP_SLIM_BELOW_TILES 256  // fewer 128 x 128 tiles than this: 128 x 64 tiles, twice as many workgroups
#endif
#ifndef TTBFP_CUS
#define TTBFP_CUS 256  // compute units of the part this library is built for (MI355X)
#endif
#ifndef TTBFP_BIG_MIN_TILES
#define TTBFP_BIG_MIN_TILES 192  // fewer macro tiles than this leave too many of the 256 CUs idle
#endif

hipError_t launch_gemm_bfp8b_general(uint32_t M, uint32_t N, uint32_t K, const void *x, const void *w, const void *bias,
                                     int epilogue, void *y, uint8_t y_fmt, hipStream_t stream);
hipError_t launch_gemm_bfp8b_skinny(uint32_t M, uint32_t N, uint32_t K, uint32_t ldn, const void *x, const void *w, const void *bias,
                                    int epilogue, void *y, uint8_t y_fmt, hipStream_t stream);
hipError_t launch_gemm_bfp8b_column_rest(uint32_t M, uint32_t N, uint32_t K, uint32_t ldn, const void *x, const void *w, const void *bias,
                                         int epilogue, void *y, uint8_t y_fmt, hipStream_t stream);

static int force_tile()  // tuning aid: TTBFP_GEMM_TILE = 1 (128 x 64), 2 (128 x 128), 3 (256 x 256), 5 (384 x 128), all on two stages, 6 (192 x 64, two pipelines), each where it fits; 0 / unset: automatic
{
    static const int force = [] { const char *v = getenv("TTBFP_GEMM_TILE"); return v ? atoi(v) : 0; }();
    return force;
}

// N columns (from the one w, bias and y point at) of a problem with ldn columns
static hipError_t launch_tiled(uint32_t M, uint32_t N, uint32_t K, uint32_t ldn, const void *x, const void *w, const void *bias,
                               int epilogue, void *y, uint8_t y_fmt, hipStream_t stream)
{
    if (y_fmt != kFloat32 && y_fmt != kFloat16_b) return hipErrorInvalidValue;
    const bool f32 = y_fmt == kFloat32;
    // Large problems: 256 x 256 macro tiles (eight wavefronts); smaller ones 128 x 128 so that every CU gets work.
    const uint64_t big_tiles = (uint64_t)(M / 256) * (N / 256);
    const bool big_ok = gemm_fits<BigShape>(M, N, K) && big_tiles >= TTBFP_BIG_MIN_TILES;
    // 384 x 128 tiles where they fill the CUs better: a round of them costs 0.84 of a round of 256 x 256 tiles (three quarters
    // of the area at a higher cost per MFMA: 3072 x 4096 x 1024 36 us against 41 with 192 tiles of 256 x 256; 3072 x 4096 x 4096
    // 114 / 120; 6144 x 4096 x 1024 72 / 75.5)
    const uint64_t tall_tiles = (uint64_t)(M / 384) * (N / 128);
    const auto rounds = [](uint64_t tiles) { return (double)((tiles + TTBFP_CUS - 1) / TTBFP_CUS); };
    if (gemm_fits<TallShape>(M, N, K) && tall_tiles >= TTBFP_BIG_MIN_TILES && (force_tile() == 0 || force_tile() == 5) &&
        (force_tile() == 5 || !big_ok || 0.84 * rounds(tall_tiles) < rounds(big_tiles)))
        return f32 ? launch_gemm_bfp8b_tall_f32(M, N, K, ldn, x, w, bias, epilogue, y, stream)
                   : launch_gemm_bfp8b_tall_bf16(M, N, K, ldn, x, w, bias, epilogue, y, stream);
    if (big_ok && force_tile() != 1 && force_tile() != 2 && force_tile() != 5)
        return f32 ? launch_gemm_bfp8b_big_f32(M, N, K, ldn, x, w, bias, epilogue, y, stream)
                   : launch_gemm_bfp8b_big_bf16(M, N, K, ldn, x, w, bias, epilogue, y, stream);
    // Fewer tiles than that: which tile and form, by how many workgroups a CU gets.
    //   at most one 128 x 64 workgroup per CU: that tile with two pipelines per workgroup on rings (K a multiple of 128;
    //     else one pipeline on rings) - 512 x 4096 x 4096: 37 us, one pipeline on rings 41, on two stages 49, 128 x 128 54;
    //   else at most one 128 x 128 workgroup per CU: that tile on two stages with two pipelines (K a multiple of 128) -
    //     3072 x 1024 x 4096: 44.5 us against 53 for 384 workgroups of 128 x 64, 512 x 8192 x 2048: 29 against 33;
    //   else 128 x 64 on two stages below 256 tiles of 128 x 128 (three workgroups fit a CU), 128 x 128 above.
    // TTBFP_GEMM_TILE (1: 128 x 64 on two stages, 2: 128 x 128 on two stages, 3: 256 x 256 where it fits, 5: 384 x 128 where it fits, 6: 192 x 64 with two pipelines where it fits) and
    // TTBFP_GEMM_PIPELINES=1 (no workgroup with two pipelines) are tuning aids for measurements and override this.
    const int force = force_tile();
    static const bool duo = [] { const char *v = getenv("TTBFP_GEMM_PIPELINES"); return !v || atoi(v) != 1; }();
    const uint64_t small_tiles = (uint64_t)(M / 128) * (N / 128), slim_tiles = (uint64_t)(M / 128) * (N / 64);
    if (force == 0 && gemm_fits<SlimShape>(M, N, K) && slim_tiles <= TTBFP_CUS) {
        if (duo && (K / 64) % 2 == 0)
            return f32 ? launch_gemm_bfp8b_duo_slim_f32(M, N, K, ldn, x, w, bias, epilogue, y, stream)
                       : launch_gemm_bfp8b_duo_slim_bf16(M, N, K, ldn, x, w, bias, epilogue, y, stream);
        return f32 ? launch_gemm_bfp8b_ring_slim_f32(M, N, K, ldn, x, w, bias, epilogue, y, stream)
                   : launch_gemm_bfp8b_ring_slim_bf16(M, N, K, ldn, x, w, bias, epilogue, y, stream);
    }
    // 192 x 64 tiles with two pipelines where they give more workgroups than 128 x 128 tiles and still at most one per CU
    // (3072 x 1024 x 4096: 256 against 192)
    const uint64_t lean_tiles = (uint64_t)(M / 192) * (N / 64);
    if ((force == 0 || force == 6) && duo && gemm_fits<LeanShape>(M, N, K) && (K / 64) % 2 == 0 && lean_tiles <= TTBFP_CUS &&
        (force == 6 || (slim_tiles > TTBFP_CUS && lean_tiles > small_tiles)))
        return f32 ? launch_gemm_bfp8b_duo_lean_f32(M, N, K, ldn, x, w, bias, epilogue, y, stream)
                   : launch_gemm_bfp8b_duo_lean_bf16(M, N, K, ldn, x, w, bias, epilogue, y, stream);
    if (force == 0 && duo && gemm_fits<SmallShape>(M, N, K) && small_tiles <= TTBFP_CUS && (K / 64) % 2 == 0)
        return f32 ? launch_gemm_bfp8b_duo_small_f32(M, N, K, ldn, x, w, bias, epilogue, y, stream)
                   : launch_gemm_bfp8b_duo_small_bf16(M, N, K, ldn, x, w, bias, epilogue, y, stream);
    if (gemm_fits<SlimShape>(M, N, K) && (force == 1 || (force == 0 && small_tiles < TTBFP_SLIM_BELOW_TILES)))
        return f32 ? launch_gemm_bfp8b_slim_f32(M, N, K, ldn, x, w, bias, epilogue, y, stream)
                   : launch_gemm_bfp8b_slim_bf16(M, N, K, ldn, x, w, bias, epilogue, y, stream);
    if (gemm_fits<SmallShape>(M, N, K))
        return f32 ? launch_gemm_bfp8b_small_f32(M, N, K, ldn, x, w, bias, epilogue, y, stream)
                   : launch_gemm_bfp8b_small_bf16(M, N, K, ldn, x, w, bias, epilogue, y, stream);
    return hipErrorNotSupported;  // the caller falls back to the general kernel
}

// M rows of N columns out of ldn: the macro-tiled kernel where the shape suits a tile, with the last M mod 128 rows
// (the rows are independent) given to the weight-streaming kernel; hipErrorNotSupported if no tile suits.
static hipError_t launch_rows_tiled(uint32_t M, uint32_t N, uint32_t K, uint32_t ldn, const void *x, const void *w, const void *bias,
                                    int epilogue, void *y, uint8_t y_fmt, hipStream_t stream)
{
    const size_t y_item = y_fmt == kFloat32 ? 4 : 2;
    hipError_t e = launch_tiled(M, N, K, ldn, x, w, bias, epilogue, y, y_fmt, stream);
    if (e != hipErrorNotSupported) return e;
    // M = 128 q + r with 0 < r < 128: the first 128 q rows go to the macro-tiled kernel and the last r (a multiple of 32)
    // to the weight-streaming one, provided N and K suit the tiles
    const uint32_t rest = M % 128, body = M - rest;
    if (body != 0 && rest % 32 == 0 && gemm_fits<SlimShape>(body, N, K)) {
        e = launch_tiled(body, N, K, ldn, x, w, bias, epilogue, y, y_fmt, stream);
        if (e != hipSuccess) return e;
        return launch_gemm_bfp8b_skinny(rest, N, K, ldn, (const uint8_t *)x + (size_t)body * K * 2, w, bias, epilogue,
                                        (uint8_t *)y + (size_t)body * ldn * y_item, y_fmt, stream);
    }
    return hipErrorNotSupported;
}

hipError_t launch_gemm_bfp8b(uint32_t M, uint32_t N, uint32_t K, const void *x, const void *w, const void *bias,
                             int epilogue, void *y, uint8_t y_fmt, hipStream_t stream)
{
    if (M == 0 || N == 0) return hipSuccess;
    hipError_t e = launch_gemm_bfp8b_skinny(M, N, K, N, x, w, bias, epilogue, y, y_fmt, stream);  // M <= 128: weight streaming
    if (e != hipErrorNotSupported) return e;
    const size_t y_item = y_fmt == kFloat32 ? 4 : 2;
    if (M < 256 && M % 32 == 0) {  // five to seven tile rows: two passes of the weight-streaming kernel beat one 128-row macro tile
        e = launch_gemm_bfp8b_skinny(128, N, K, N, x, w, bias, epilogue, y, y_fmt, stream);
        if (e != hipSuccess) return e;
        return launch_gemm_bfp8b_skinny(M - 128, N, K, N, (const uint8_t *)x + (size_t)128 * K * 2, w, bias, epilogue,
                                        (uint8_t *)y + (size_t)128 * N * y_item, y_fmt, stream);
    }
    e = launch_rows_tiled(M, N, K, N, x, w, bias, epilogue, y, y_fmt, stream);
    if (e != hipErrorNotSupported) return e;
    // N is an odd number of tiles (tensors are padded to multiples of 32, not of 64: pybuda/pybuda/tensor.py:805-877): the
    // columns but the last 32 go to the macro-tiled kernel, the last tile column to one-row-tile workgroups of the
    // weight-streaming kernel.  The bias may be fp32 or bf16: the pointer moves by its element size.
    if (N % 64 == 32 && N > 32 && M % 32 == 0) {
        const uint32_t body = N - 32;
        e = launch_rows_tiled(M, body, K, N, x, w, bias, epilogue, y, y_fmt, stream);
        if (e == hipSuccess) {
            const size_t bias_item = (epilogue & kEpilogueBiasF32) ? 4 : 2;
            return launch_gemm_bfp8b_column_rest(M, 32, K, N, x, (const uint8_t *)w + (size_t)(body / kTile) * tile_bytes(kBfp8_b),
                                                 bias ? (const uint8_t *)bias + (size_t)body * bias_item : nullptr, epilogue,
                                                 (uint8_t *)y + (size_t)body * y_item, y_fmt, stream);
        }
        if (e != hipErrorNotSupported) return e;
    }
    return launch_gemm_bfp8b_general(M, N, K, x, w, bias, epilogue, y, y_fmt, stream);
}

}  // namespace ttbfp
