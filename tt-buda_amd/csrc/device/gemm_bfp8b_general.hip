// General form of the Bfp8_b-weight GEMM: any M, N, K that are multiples of 32.  Every access is
// bounds-tested, so it also serves the shapes the macro-tiled kernel (gemm_bfp8b.hip) does not take
// (ragged tile counts, K not a multiple of 64, very small M).  Same arithmetic, same results.
//
// W stays packed in HBM (1.0625 bytes per weight) in exactly the layout the pack kernel writes:
// tiles [K/32][N/32], 64 exponent bytes + four 16x16 faces, a face row being 16 consecutive n of
// one k.  The MFMA B operand wants 8 consecutive k per lane, so each thread fetches a 4(n) x 8(k)
// patch of one face as eight dwords, turns the bytes into bf16 (exact: a 7-bit magnitude fits the
// bf16 significand) and writes four k-contiguous 128-bit rows into an [n][k] LDS image.  X tiles go
// to an [m][k] LDS image unchanged.  Wavefronts then read both operands with ds_read_b128 and
// issue v_mfma_f32_32x32x16_bf16.
#include "bfp_codec.hpp"
#include "launch.hpp"

namespace ttbfp {

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int BM = 128, BN = 128, BK = 64;
constexpr int LDK = BK + 8;  // LDS row pitch in bf16: 144 bytes, keeps 128-bit reads of 16 rows on distinct banks
constexpr uint32_t kW8Tile = tile_bytes(kBfp8_b);

// bf16 bit pattern (upper half of the fp32 pattern) of one Bfp8_b byte under shared exponent e
__device__ __forceinline__ uint32_t bfp8_to_bf16(uint32_t byte, uint32_t e)
{
    return dequantize_datum<7>(byte, e) >> 16;
}

struct WPatch {
    uint32_t d[8];  // d[j]: 4 datums (n = 4g .. 4g+3) of face row 8*kh + j
    uint2 e;        // the 8 shared exponents of those rows
};

template <int EPILOGUE, typename OutT>
__global__ __launch_bounds__(256) void gemm_bfp8b_general_kernel(uint32_t M, uint32_t N, uint32_t K,
                                                         const uint16_t *__restrict__ X,
                                                         const uint8_t *__restrict__ Wp,
                                                         const uint16_t *__restrict__ bias, int bias_f32, OutT *__restrict__ Y)
{
    __shared__ __attribute__((aligned(16))) uint16_t As[BM * LDK];
    __shared__ __attribute__((aligned(16))) uint16_t Bs[BN * LDK];

    const uint32_t tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t wm = wave >> 1, wn = wave & 1;
    const uint32_t m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
    const uint32_t tiles_n = N / kTile, tiles_k = K / kTile;

    // W patch owned by this thread inside the BK x BN slab
    const uint32_t g = tid & 3, kh = (tid >> 2) & 1, face = (tid >> 3) & 3, wt = tid >> 5;
    const uint32_t kt_l = wt >> 2, nt_l = wt & 3;
    const uint32_t w_n = nt_l * 32 + (face & 1) * 16 + g * 4;   // first of 4 local n
    const uint32_t w_k = kt_l * 32 + (face >> 1) * 16 + kh * 8; // first of 8 local k
    const bool w_col_live = n0 / kTile + nt_l < tiles_n;

    uint4 xa[4];
    WPatch wp;

    auto fetch = [&](uint32_t k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t c = tid + 256 * i, row = c >> 3, kc = c & 7;
            const bool live = m0 + row < M && k0 + kc * 8 < K;
            xa[i] = live ? *(const uint4 *)(X + (uint64_t)(m0 + row) * K + k0 + kc * 8) : make_uint4(0, 0, 0, 0);
        }
        const uint32_t kt = k0 / kTile + kt_l;
        if (w_col_live && kt < tiles_k) {
            const uint8_t *t = Wp + ((uint64_t)kt * tiles_n + n0 / kTile + nt_l) * kW8Tile;
            wp.e = *(const uint2 *)(t + face * 16 + kh * 8);
            const uint8_t *dp = t + kExpSection + face * 256 + kh * 128 + g * 4;
#pragma unroll
            for (int j = 0; j < 8; ++j) wp.d[j] = *(const uint32_t *)(dp + j * 16);
        } else {
            wp.e = make_uint2(0, 0);
#pragma unroll
            for (int j = 0; j < 8; ++j) wp.d[j] = 0;
        }
    };

    auto stage = [&]() {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t c = tid + 256 * i, row = c >> 3, kc = c & 7;
            *(uint4 *)(As + row * LDK + kc * 8) = xa[i];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {  // local n = w_n + i
            uint32_t h[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const uint32_t e = ((j < 4 ? wp.e.x : wp.e.y) >> (8 * (j & 3))) & 0xffu;
                h[j] = bfp8_to_bf16((wp.d[j] >> (8 * i)) & 0xffu, e);
            }
            *(uint4 *)(Bs + (w_n + i) * LDK + w_k) =
                make_uint4(h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16));
        }
    };

    f32x16 acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.0f;

    fetch(0);
    stage();
    __syncthreads();

    for (uint32_t k0 = 0; k0 < K; k0 += BK) {
        const bool more = k0 + BK < K;
        if (more) fetch(k0 + BK);
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            const uint32_t kk = ks * 16 + (lane >> 5) * 8;
            bf16x8 a[2], b[2];
#pragma unroll
            for (int mb = 0; mb < 2; ++mb) a[mb] = *(const bf16x8 *)(As + (wm * 64 + mb * 32 + (lane & 31)) * LDK + kk);
#pragma unroll
            for (int nb = 0; nb < 2; ++nb) b[nb] = *(const bf16x8 *)(Bs + (wn * 64 + nb * 32 + (lane & 31)) * LDK + kk);
#pragma unroll
            for (int mb = 0; mb < 2; ++mb)
#pragma unroll
                for (int nb = 0; nb < 2; ++nb)
                    acc[mb][nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[mb], b[nb], acc[mb][nb], 0, 0, 0);
        }
        __syncthreads();
        if (more) {
            stage();
            __syncthreads();
        }
    }

    // D layout of the 32x32 MFMA: register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4, column l%32
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int nb = 0; nb < 2; ++nb) {
            const uint32_t col = n0 + wn * 64 + nb * 32 + (lane & 31);
            if (col >= N) continue;
            const float bv = bias ? load_bias(bias, col, bias_f32) : 0.0f;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const uint32_t row = m0 + wm * 64 + mb * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
                if (row >= M) continue;
                float v = acc[mb][nb][r] + bv;
                v = apply_epilogue(EPILOGUE, v);
                if constexpr (sizeof(OutT) == 4)
                    Y[(uint64_t)row * N + col] = v;
                else
                    Y[(uint64_t)row * N + col] = f32_to_bf16_rne(__float_as_uint(v));
            }
        }
}

template <int EPILOGUE, typename OutT>
hipError_t launch(uint32_t M, uint32_t N, uint32_t K, const void *x, const void *w, const void *bias, int bias_f32, void *y,
                  hipStream_t stream)
{
    dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
    if (grid.y > 65535u) return hipErrorInvalidValue;
    hipLaunchKernelGGL((gemm_bfp8b_general_kernel<EPILOGUE, OutT>), grid, dim3(256), 0, stream, M, N, K, (const uint16_t *)x,
                       (const uint8_t *)w, (const uint16_t *)bias, bias_f32, (OutT *)y);
    return hipGetLastError();
}

}  // namespace

hipError_t launch_gemm_bfp8b_general(uint32_t M, uint32_t N, uint32_t K, const void *x, const void *w, const void *bias,
                             int epilogue, void *y, uint8_t y_fmt, hipStream_t stream)
{
    if (M == 0 || N == 0) return hipSuccess;
    const int bias_f32 = epilogue & kEpilogueBiasF32;
    epilogue &= kEpilogueMask;
    if (y_fmt == kFloat32)
        return epilogue == 2   ? launch<2, float>(M, N, K, x, w, bias, bias_f32, y, stream)
               : epilogue == 1 ? launch<1, float>(M, N, K, x, w, bias, bias_f32, y, stream)
                               : launch<0, float>(M, N, K, x, w, bias, bias_f32, y, stream);
    if (y_fmt == kFloat16_b)
        return epilogue == 2   ? launch<2, uint16_t>(M, N, K, x, w, bias, bias_f32, y, stream)
               : epilogue == 1 ? launch<1, uint16_t>(M, N, K, x, w, bias, bias_f32, y, stream)
                               : launch<0, uint16_t>(M, N, K, x, w, bias, bias_f32, y, stream);
    return hipErrorInvalidValue;
}

}  // namespace ttbfp
