// Two-pass form of the Bfp8_b-weight GEMM for large M, for callers that can lend a workspace of
// 2 K N bytes.  In the fused kernel every workgroup dequantizes the W slabs it needs, so the same
// weight is converted M / 256 times and that conversion shares the instruction issue with the MFMAs.
// With many rows of X it is cheaper to convert W once: pass 1 below writes, for every (column of
// 256-wide macro tiles, 64-k slab), the 32 KiB image of the B stage exactly as the fused kernel's
// dequantization leaves it in LDS ([k/8][n'][8 k] bf16, n' = n ^ (((n >> 3) ^ (n >> 6)) & 7)); pass 2 is
// the same MFMA kernel with its B stage filled by direct loads from that panel.  Same bf16 operand
// values, same accumulation order: the results are bit-identical to the fused kernel's.
//
// Pass 1 is a streaming kernel: 1.0625 bytes read and 2 written per weight.  A wavefront takes two
// tiles at a time: the data sections come in with one coalesced 16-byte load per lane and tile, pass
// through a wave-private LDS image, and two transposing reads (ds_read_b64_tr_b8) per tile hand every
// lane the 8 consecutive k of one column, which it converts four at a time and stores as one 16-byte
// vector; the 32 lanes of a k chunk store 512 contiguous bytes of the panel.
#include "gemm_bfp8b_kernel.hpp"

#ifndef TTBFP_PANEL_BIG_MIN_TILES
#define TTBFP_PANEL_BIG_MIN_TILES 192  // as in the fused kernel's choice of the 256 x 256 tile
#endif
#ifndef TTBFP_PANEL_BIG_MIN_M
#define TTBFP_PANEL_BIG_MIN_M 4096    // measured: equal at 4096 rows, 6-8 % ahead at 8192
#endif
#ifndef TTBFP_PANEL_SMALL_MIN_M
#define TTBFP_PANEL_SMALL_MIN_M 6144  // measured against the fused forms: 6144 x 1024 x 4096 73 against 80 us, level at 3072 and 4096 rows (4096 x 2048 x 2048 behind)
#endif

namespace ttbfp {

namespace {


typedef int v2i __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) v2i *lds_v2i;
constexpr int kPanelWaves = 4;   // wavefronts per workgroup, independent of one another
constexpr int kPanelTiles = 2;   // tiles a wavefront converts per pass, neighbours along n

// panel_n: width BN of the macro tiles the panel is made for (256 or 128); one (tile column, slab) image is
// (BK / 8) * panel_n * 16 bytes.
__global__ __launch_bounds__(64 * kPanelWaves) void dequant_panel_kernel(uint32_t N, uint32_t K, const uint8_t *__restrict__ Wp,
                                                                         uint8_t *__restrict__ panel, uint32_t panel_n)
{
    __shared__ __attribute__((aligned(16))) uint8_t images[kPanelWaves][kPanelTiles][1024];
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t tiles_n = N / kTile, nslabs = K / BK;
    const uint64_t first = ((uint64_t)blockIdx.x * kPanelWaves + wave) * kPanelTiles;  // tile index kt * tiles_n + nt
    if (first >= (uint64_t)(K / kTile) * tiles_n) return;  // whole wavefronts only: tiles_n is a multiple of kPanelTiles
    const uint32_t kt = (uint32_t)(first / tiles_n), nt0 = (uint32_t)(first % tiles_n);
    const uint8_t *tile0 = Wp + first * kW8Tile;

    uint4 data[kPanelTiles];
#pragma unroll
    for (int p = 0; p < kPanelTiles; ++p) data[p] = load_stream(tile0 + p * kW8Tile + kExpSection + lane * 16);
    // Read r (0, 1) of a tile: lane l gets k chunk kc4 = 2 r + l / 32 (8 k), column nh * 16 + n16 with nh = (l / 16) & 1,
    // n16 = l & 15: the 16 lanes of one (kc4, nh) cover the 8 face rows of that chunk, 128 contiguous bytes of the image.
    const uint32_t nh = (lane >> 4) & 1, n16 = lane & 15;
    uint2 exps[kPanelTiles][2];
#pragma unroll
    for (int p = 0; p < kPanelTiles; ++p)
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const uint32_t kc4 = 2 * r + (lane >> 5), face = (kc4 >> 1) * 2 + nh;
            exps[p][r] = *(const uint2 *)(tile0 + p * kW8Tile + face * 16 + (kc4 & 1) * 8);
        }
#pragma unroll
    for (int p = 0; p < kPanelTiles; ++p) *(uint4 *)(images[wave][p] + lane * 16) = data[p];
    // the images are private to this wavefront: its own LDS writes are visible to its reads in order
#pragma unroll
    for (int p = 0; p < kPanelTiles; ++p) {
        const uint32_t n_tile = (nt0 + p) * kTile;  // first column of the tile
        uint8_t *block = panel + ((uint64_t)(n_tile / panel_n) * nslabs + kt / 2) * ((BK / 8) * 16) * panel_n;
        const uint32_t n_in = n_tile % panel_n + nh * 16 + n16;
#pragma unroll
        for (int r = 0; r < 2; ++r) {
            const uint32_t kc4 = 2 * r + (lane >> 5), face = (kc4 >> 1) * 2 + nh;
            const v2i d = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i)(images[wave][p] + face * 256 + (kc4 & 1) * 128 + n16 * 8));
            const uint2 lo = datums4_to_bf16((uint32_t)d.x, exps[p][r].x), hi = datums4_to_bf16((uint32_t)d.y, exps[p][r].y);
            const uint32_t kc = (kt & 1) * 4 + kc4;  // k chunk inside the slab
            store_stream(block + ((uint64_t)kc * panel_n + swizzle_n(n_in)) * 16, make_uint4(lo.x, lo.y, hi.x, hi.y));
        }
    }
}

}  // namespace

// Which macro tile the two-pass form would use: 256 (as the fused kernel chooses it), 128, or 0 for "stay fused".
// The conversion costs about 3 bytes of traffic per weight; it pays once enough rows share it.
static uint32_t panel_tile(uint32_t M, uint32_t N, uint32_t K)
{
    if (K % 64) return 0;  // the panel is cut into whole slabs
    const uint64_t big_tiles = (uint64_t)(M / 256) * (N / 256);
    if (gemm_fits<BigShape>(M, N, K) && big_tiles >= TTBFP_PANEL_BIG_MIN_TILES) return M >= TTBFP_PANEL_BIG_MIN_M ? 256 : 0;
    if (gemm_fits<SmallShape>(M, N, K)) return M >= TTBFP_PANEL_SMALL_MIN_M ? 128 : 0;
    return 0;
}

uint64_t gemm_bfp8b_panel_bytes(uint32_t M, uint32_t N, uint32_t K) { return panel_tile(M, N, K) ? (uint64_t)K * N * 2 : 0; }

hipError_t launch_gemm_bfp8b_panel(uint32_t M, uint32_t N, uint32_t K, const void *x, const void *w, const void *bias, int epilogue,
                                   void *y, uint8_t y_fmt, void *workspace, hipStream_t stream)
{
    if (y_fmt != kFloat32 && y_fmt != kFloat16_b) return hipErrorInvalidValue;
    const uint32_t tile = panel_tile(M, N, K);
    if (tile == 0) return hipErrorInvalidValue;
    const uint64_t tiles = (uint64_t)(N / kTile) * (K / kTile), per_group = kPanelWaves * kPanelTiles;
    hipLaunchKernelGGL(dequant_panel_kernel, dim3((uint32_t)((tiles + per_group - 1) / per_group)), dim3(64 * kPanelWaves), 0, stream, N, K,
                       (const uint8_t *)w, (uint8_t *)workspace, tile);
    if (hipError_t e = hipGetLastError(); e != hipSuccess) return e;
    if (tile == 256)
        return y_fmt == kFloat32 ? launch_gemm_bfp8b_panel_f32(M, N, K, N, x, workspace, bias, epilogue, y, stream)
                                 : launch_gemm_bfp8b_panel_bf16(M, N, K, N, x, workspace, bias, epilogue, y, stream);
    return y_fmt == kFloat32 ? launch_gemm_bfp8b_panel_small_f32(M, N, K, N, x, workspace, bias, epilogue, y, stream)
                             : launch_gemm_bfp8b_panel_small_bf16(M, N, K, N, x, workspace, bias, epilogue, y, stream);
}

}  // namespace ttbfp
