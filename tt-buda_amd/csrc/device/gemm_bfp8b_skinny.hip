// Bfp8_b-weight GEMM for one to four tile rows of activations (M = 32, 64, 96, 128): the decode-like case.  Its floor
// is streaming the packed weights from HBM once (1.0625 bytes per weight), but the work that fills
// the time is turning every weight byte into a bf16 MFMA operand, so the kernel is laid out to put
// that work on as many SIMDs as possible.
//
// One workgroup of 16 wavefronts owns HALF a tile column of W - 16 columns n, the left or the right
// pair of faces of every tile - and all of K: N/16 workgroups, 256 for N = 4096, one per CU.
// Wavefront v takes the K/16 slice [v K/16, (v+1) K/16) two tiles at a time:
//   * the two face halves of a tile (32 k rows x 16 bytes) are loaded coalesced, one 16-byte face row
//     per lane, lanes 0..31 for the first tile of a pair and 32..63 for the second, and go through a
//     small per-wave LDS image to be read back column-wise: the B operand of the 16x16x32 MFMA needs
//     the 8 consecutive k of one n in a lane;
//   * one transposing LDS read (ds_read_b64_tr_b8) then hands a lane its 8 k bytes as two dwords, which
//     are converted four at a time: byte-select conversions, one ldexp per datum, byte permutes for
//     packing and for the signs;
//   * every workgroup needs all of X (32 x K bf16), so X is the larger stream into a CU (per 1024 k:
//     64 KiB of X out of L2 against 17 KiB of W): a wavefront fetches the X rows of a tile pair as whole 128-byte
//     lines, one pair ahead, and passes them through LDS into the MFMA A operand layout (a lane holds
//     8 consecutive k of one row); all 16-row blocks of X share the dequantized B operand, so more rows cost MFMAs
//     and X traffic only;
//   * the W loads of up to four tile pairs are issued before the first is touched;
//   * the 16 partial 32x16 accumulators are summed through LDS in a fixed order, so the result does
//     not depend on timing; bias, optional exact GELU and the bf16/fp32 store follow.
#include <type_traits>

#include "bfp_codec.hpp"
#include "launch.hpp"

namespace ttbfp {

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

// RT = M / 32 row tiles of X (1..4).  One row tile runs on 16 wavefronts, more on 8: the X rows of a tile pair, 4 KiB
// per row tile and wavefront, must fit the LDS next to the W images, and their prefetch the register file.
template <int RT>
struct Skinny {
    static constexpr int kWaves = RT == 1 ? 16 : 8;
    static constexpr uint32_t kRegion = 2 * (4 * (8 * 16 + 16) + 32) + RT * 32 * 128;  // two W images, then the X rows of a tile pair
    static_assert(kRegion % 16 == 0 && kRegion >= RT * 32 * 17 * 4, "the region doubles as the wavefront's partial sum");
    static_assert(kWaves * kRegion <= 160 * 1024, "LDS of a CU");
};
constexpr int kBatch = 4;                  // tile pairs a wavefront keeps in flight
constexpr uint32_t kGroupPitch = 8 * 16 + 16;   // 8 k rows of 16 bytes, then a gap
constexpr uint32_t kHalfImage = 4 * kGroupPitch + 32;  // 32 k rows + their 32 exponent bytes
constexpr uint32_t kW8Tile = tile_bytes(kBfp8_b);

typedef int v2i __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) v2i *lds_v2i;


template <int RT, int EPILOGUE, typename OutT>
__global__ __launch_bounds__(64 * Skinny<RT>::kWaves) void gemm_bfp8b_skinny_kernel(uint32_t ldn, uint32_t K,
                                                                        const uint16_t *__restrict__ X,
                                                                        const uint8_t *__restrict__ Wp,
                                                                        const uint16_t *__restrict__ bias, int bias_f32,
                                                                        OutT *__restrict__ Y)
{
    constexpr int kWaves = Skinny<RT>::kWaves;
    constexpr uint32_t kRegion = Skinny<RT>::kRegion;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds[];  // kWaves regions of kRegion bytes

    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    // ldn: columns of the whole problem (the pitch of Y's rows and of W's tile rows).  The launch computes the columns from
    // the one W, Y and bias point at: gridDim.x / 2 tile columns, and gridDim.y groups of RT row tiles.
    const uint32_t tiles_n = ldn / kTile, tiles_k = K / kTile;
    X += (uint64_t)blockIdx.y * (RT * 32) * K;
    Y += (uint64_t)blockIdx.y * (RT * 32) * ldn;
    // Tile column, and its left (0) or right (1) faces.  Workgroups go to the XCDs in turn (id mod 8), and the two halves
    // of a tile column share the lines that straddle two faces, so they are ids b and b + 8: same XCD, same L2.
    uint32_t nt = blockIdx.x >> 1, half = blockIdx.x & 1;
    if (gridDim.x % 16 == 0) nt = (blockIdx.x >> 4) * 8 + (blockIdx.x & 7), half = (blockIdx.x >> 3) & 1;
    // tile rows of this wavefront: an even split of tiles_k over the wavefronts
    const uint32_t kt_begin = (uint64_t)tiles_k * wave / kWaves, kt_end = (uint64_t)tiles_k * (wave + 1) / kWaves;

    uint8_t *image = lds + wave * kRegion;  // two W half-tile images, then the X rows of a tile pair
    uint8_t *xrows = image + 2 * kHalfImage;
    // W load/store side: lanes 0..31 own the first tile of a pair, 32..63 the second; lane i of a tile owns k row
    // i & 31 = face row i & 15 of face (top or bottom) * 2 + half; lanes 0..7 of a tile also carry 4 exponent bytes
    const uint32_t which = lane >> 5, krow = lane & 31;
    const uint32_t src_data = kExpSection + ((krow >> 4) * 2 + half) * 256 + (krow & 15) * 16;
    const uint32_t src_exp = (((lane & 7) >> 2) * 2 + half) * 16 + (lane & 3) * 4;
    const uint32_t st_off = which * kHalfImage + (krow >> 3) * kGroupPitch + (krow & 7) * 16;
    const uint32_t st_exp = which * kHalfImage + 4 * kGroupPitch + (lane & 7) * 4;
    // W read side (B operand): lane (n = lane & 15, kq = lane >> 4) gets column n of k rows kq * 8 .. + 7 and their exponents
    const uint32_t n_l = lane & 15, kq = lane >> 4;
    const uint32_t ld_col = kq * kGroupPitch + n_l * 8;  // the transposing read: the 16 lanes of a k group cover its 128 bytes
    const uint32_t ld_exp = 4 * kGroupPitch + kq * 8;
    // X: the 64 k of a tile pair are 128 contiguous bytes of each of the 32 rows.  Load i (of 4) takes rows 8 i .. 8 i + 7,
    // a lane one 16-byte piece (8 k): whole lines, read from L2 once.  Piece q of row r is kept at q ^ (r & 7), so that
    // both this store and the operand reads below (16 rows, one piece) spread over the banks.
    const uint32_t x_row = lane >> 3, x_q = lane & 7;
    const uint8_t *x_src = (const uint8_t *)X + (uint64_t)x_row * K * 2 + x_q * 16;
    const uint32_t x_st = x_row * 128 + ((x_q ^ x_row) * 16);  // + 1024 i: (8 i + row) & 7 == row
    // A operand of tile p, rows n_l (+16): piece 4 p + kq
    const uint32_t x_ld = n_l * 128;

    constexpr int XL = 4 * RT;  // X loads per tile pair: 8 rows each
    constexpr int HB = 2 * RT;  // 16-row blocks of Y
    f32x4 acc[HB];              // acc[h]: rows 16 h .. 16 h + 15 of Y
#pragma unroll
    for (int h = 0; h < HB; ++h) acc[h] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    // FULL: the pair (kt, kt + 1) lies inside the slice for sure, so the loads carry no condition
    auto load_x = [&](uint32_t kt, uint4 (&v)[XL], auto fullc) {  // a second tile past the slice is not fetched
        const bool live = decltype(fullc)::value || (kt < kt_end && (x_q < 4 || kt + 1 < kt_end));
#pragma unroll
        for (int i = 0; i < XL; ++i)
            v[i] = live ? *(const uint4 *)(x_src + (uint64_t)i * 8 * K * 2 + (uint64_t)kt * (kTile * 2)) : make_uint4(0, 0, 0, 0);
    };

    // One batch of tile pairs from tile row kt0 on.  NP = 1 .. kBatch: exactly NP whole pairs, all inside the wavefront's
    // slice; that version is straight-line code without a single condition, so the compiler counts the outstanding
    // loads exactly and the X rows fetched for the following pair stay in flight while this pair is multiplied.  With
    // conditions in the way (NP = 0: up to kBatch pairs, the last possibly half) it waits for every load before each
    // pair (vmcnt(0)), which exposes a trip to L2 per pair.
    auto batch = [&](uint32_t kt0, auto npc) {
        constexpr int NP = decltype(npc)::value;
        constexpr bool FULL = NP > 0;
        constexpr int PAIRS = FULL ? NP : kBatch;
        const std::integral_constant<bool, FULL> fullc;
        uint4 data[kBatch];
        uint32_t exps[kBatch];
        uint4 xcur[XL], xnext[XL];
#pragma unroll
        for (int b = 0; b < PAIRS; ++b) {
            const uint32_t kt = kt0 + 2 * b + which;
            data[b] = make_uint4(0, 0, 0, 0);
            exps[b] = 0;
            if (FULL || kt < kt_end) {
                const uint8_t *t = Wp + ((uint64_t)kt * tiles_n + nt) * kW8Tile;
                data[b] = load_stream(t + src_data);
                // every lane fetches the exponent word of lane & 7 (a valid address for all), no divergence
                exps[b] = *(const uint32_t *)(t + src_exp);
            }
        }
        load_x(kt0, xcur, fullc);
        __builtin_amdgcn_sched_barrier(0);  // all W loads of the batch are issued here, not sunk to their uses
#pragma unroll
        for (int b = 0; b < PAIRS; ++b) {
            if (!FULL && kt0 + 2 * b >= kt_end) break;  // wave-uniform
            if (b + 1 < PAIRS) load_x(kt0 + 2 * (b + 1), xnext, fullc);
            __builtin_amdgcn_sched_barrier(0);  // the next pair's X loads go out before this pair's work
            *(uint4 *)(image + st_off) = data[b];
            *(uint32_t *)(image + st_exp) = exps[b];  // lanes with equal lane & 7 of a tile store the same word to the same place
#pragma unroll
            for (int i = 0; i < XL; ++i) *(uint4 *)(xrows + i * 1024 + x_st) = xcur[i];
            // this region is private to the wavefront: its own LDS writes are visible to its reads in order
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                if (!FULL && kt0 + 2 * b + p >= kt_end) break;  // wave-uniform
                const uint32_t piece = ((4 * p + kq) ^ (n_l & 7)) * 16;
                bf16x8 xa[HB];
#pragma unroll
                for (int h = 0; h < HB; ++h) xa[h] = *(const bf16x8 *)(xrows + h * 16 * 128 + x_ld + piece);
                // one transposing read hands every lane the 8 consecutive k of its column: bytes k0..k3, k4..k7
                const v2i d = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i)(image + p * kHalfImage + ld_col));
                const uint2 e8 = *(const uint2 *)(image + p * kHalfImage + ld_exp);
                const uint2 lo = datums4_to_bf16((uint32_t)d.x, e8.x), hi = datums4_to_bf16((uint32_t)d.y, e8.y);
                const uint4 packed = make_uint4(lo.x, lo.y, hi.x, hi.y);
                const bf16x8 wb = __builtin_bit_cast(bf16x8, packed);
#pragma unroll
                for (int h = 0; h < HB; ++h) acc[h] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(xa[h], wb, acc[h], 0, 0, 0);
            }
            if (b + 1 < PAIRS) {
#pragma unroll
                for (int i = 0; i < XL; ++i) xcur[i] = xnext[i];
            }
        }
    };
    static_assert(kBatch == 4, "the dispatch below names the pair counts");
    for (uint32_t kt0 = kt_begin; kt0 < kt_end; kt0 += 2 * kBatch) {
        const uint32_t left = kt_end - kt0;
        // the shorter straight-line versions only where registers allow (with three or four row tiles the extra code
        // paths made the allocator spill)
        if (left >= 2 * kBatch)
            batch(kt0, std::integral_constant<int, 4>{});
        else if (RT <= 2 && left == 6)
            batch(kt0, std::integral_constant<int, RT <= 2 ? 3 : 0>{});
        else if (RT <= 2 && left == 4)
            batch(kt0, std::integral_constant<int, RT <= 2 ? 2 : 0>{});
        else if (RT <= 2 && left == 2)
            batch(kt0, std::integral_constant<int, RT <= 2 ? 1 : 0>{});
        else
            batch(kt0, std::integral_constant<int, 0>{});
    }

    // D layout of the 16x16 MFMA: register r of lane l holds row 4 (l / 16) + r, column l % 16.
    // Every wavefront leaves its M x 16 partial in its own region (done with it by now); the threads then add
    // the partials of one output each in a fixed order.
    float *partial = (float *)(lds + wave * kRegion);
#pragma unroll
    for (int h = 0; h < HB; ++h)
#pragma unroll
        for (int r = 0; r < 4; ++r) partial[(h * 16 + kq * 4 + r) * 17 + n_l] = acc[h][r];
    __syncthreads();
    for (uint32_t o = threadIdx.x; o < RT * 32 * 16; o += 64 * kWaves) {
        const uint32_t row = o >> 4, c = o & 15, col = nt * kTile + half * 16 + c;
        float v = 0.0f;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) v += ((const float *)(lds + w * kRegion))[row * 17 + c];
        if (bias) v += load_bias(bias, col, bias_f32);
        v = apply_epilogue(EPILOGUE, v);
        if constexpr (sizeof(OutT) == 4)
            Y[(uint64_t)row * ldn + col] = v;
        else
            Y[(uint64_t)row * ldn + col] = f32_to_bf16_rne(__float_as_uint(v));
    }
}

template <int RT, int EPILOGUE, typename OutT>
hipError_t launch(uint32_t groups, uint32_t N, uint32_t K, uint32_t ldn, const void *x, const void *w, const void *bias, int bias_f32, void *y,
                  hipStream_t stream)
{
    constexpr uint32_t smem = Skinny<RT>::kWaves * Skinny<RT>::kRegion;
    auto kernel = gemm_bfp8b_skinny_kernel<RT, EPILOGUE, OutT>;
    if (groups == 0 || groups > 65535u) return hipErrorInvalidValue;
    if (hipError_t e = allow_dynamic_lds(kernel, smem); e != hipSuccess) return e;
    hipLaunchKernelGGL(kernel, dim3(N / kTile * 2, groups), dim3(64 * Skinny<RT>::kWaves), smem, stream, ldn, K, (const uint16_t *)x,
                       (const uint8_t *)w, (const uint16_t *)bias, bias_f32, (OutT *)y);
    return hipGetLastError();
}

// groups x RT row tiles of X, N columns from the one the pointers are at
template <int RT>
hipError_t launch_rows(uint32_t groups, uint32_t N, uint32_t K, uint32_t ldn, const void *x, const void *w, const void *bias, int epilogue, void *y,
                       uint8_t y_fmt, hipStream_t stream)
{
    const int bias_f32 = epilogue & kEpilogueBiasF32;
    epilogue &= kEpilogueMask;
    if (y_fmt == kFloat32)
        return epilogue == 2   ? launch<RT, 2, float>(groups, N, K, ldn, x, w, bias, bias_f32, y, stream)
               : epilogue == 1 ? launch<RT, 1, float>(groups, N, K, ldn, x, w, bias, bias_f32, y, stream)
                               : launch<RT, 0, float>(groups, N, K, ldn, x, w, bias, bias_f32, y, stream);
    if (y_fmt == kFloat16_b)
        return epilogue == 2   ? launch<RT, 2, uint16_t>(groups, N, K, ldn, x, w, bias, bias_f32, y, stream)
               : epilogue == 1 ? launch<RT, 1, uint16_t>(groups, N, K, ldn, x, w, bias, bias_f32, y, stream)
                               : launch<RT, 0, uint16_t>(groups, N, K, ldn, x, w, bias, bias_f32, y, stream);
    return hipErrorInvalidValue;
}

}  // namespace

// M = 32, 64, 96 or 128 rows and N columns of a problem with ldn columns (w, bias and y point at the first of the N);
// returns hipErrorNotSupported for another M so that the caller picks another kernel.
hipError_t launch_gemm_bfp8b_skinny(uint32_t M, uint32_t N, uint32_t K, uint32_t ldn, const void *x, const void *w, const void *bias,
                                    int epilogue, void *y, uint8_t y_fmt, hipStream_t stream)
{
    switch (M) {
        case 32: return launch_rows<1>(1, N, K, ldn, x, w, bias, epilogue, y, y_fmt, stream);
        case 64: return launch_rows<2>(1, N, K, ldn, x, w, bias, epilogue, y, y_fmt, stream);
        case 96: return launch_rows<3>(1, N, K, ldn, x, w, bias, epilogue, y, y_fmt, stream);
        case 128: return launch_rows<4>(1, N, K, ldn, x, w, bias, epilogue, y, y_fmt, stream);
        default: return hipErrorNotSupported;
    }
}

// Any number of rows (a multiple of 32) of a few columns: the column range a macro-tiled launch leaves over.  One row
// tile per workgroup, M / 32 groups of them: each streams its 16 columns of W over all of K, so the launch takes about
// as long as one decode-like call however many rows there are, as long as the workgroups fit the CUs at once.
hipError_t launch_gemm_bfp8b_column_rest(uint32_t M, uint32_t N, uint32_t K, uint32_t ldn, const void *x, const void *w, const void *bias,
                                         int epilogue, void *y, uint8_t y_fmt, hipStream_t stream)
{
    if (M == 0 || N == 0) return hipSuccess;
    if (M % kTile || N % kTile) return hipErrorInvalidValue;
    const uint32_t row_tiles = M / kTile;
    const size_t y_item = y_fmt == kFloat32 ? 4 : 2;
    for (uint32_t first = 0; first < row_tiles; first += 65535u) {  // the grid's y dimension holds 65535 groups
        const uint32_t groups = row_tiles - first < 65535u ? row_tiles - first : 65535u;
        if (hipError_t e = launch_rows<1>(groups, N, K, ldn, (const uint8_t *)x + (size_t)first * kTile * K * 2, w, bias, epilogue,
                                          (uint8_t *)y + (size_t)first * kTile * ldn * y_item, y_fmt, stream);
            e != hipSuccess)
            return e;
    }
    return hipSuccess;
}

}  // namespace ttbfp
