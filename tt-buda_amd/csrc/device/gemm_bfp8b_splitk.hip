// Split-K form of the Bfp8_b-weight GEMM for shapes whose 128 x 128 macro tiles leave CUs idle (M = 512 at N = 4096
// gives 128 tiles for 256 CUs), for callers that lend a workspace: the K loop is cut into `splits` runs, each
// (tile, run) pair is a workgroup of the MFMA kernel (SPLITK flag of gemm_bfp8b_kernel.hpp) that writes an fp32
// partial tile into the workspace, and a second, streaming kernel adds the planes in a fixed order, applies bias and
// epilogue and writes Y.  Deterministic; the sum is grouped differently from the fused kernel's, so the results agree
// with it to fp32 rounding, not bit for bit.
#include "gemm_bfp8b_kernel.hpp"

#ifndef TTBFP_SPLITK_MAX
#define TTBFP_SPLITK_MAX 8  // most runs K is cut into
#endif

namespace ttbfp {

namespace {

// four consecutive outputs per thread: planes added in order 0, 1, ...; N is a multiple of 4.  SPLITS is a template
// argument so that a thread issues the loads of all planes before it waits for the first.
template <typename OutT, int SPLITS>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(uint64_t quads, uint32_t N, const float *__restrict__ partials,
                                                            const uint16_t *__restrict__ bias, int epilogue, OutT *__restrict__ Y)
{
    const uint64_t q = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (q >= quads) return;
    const uint64_t plane = quads * 4;
    float4 v[SPLITS];
#pragma unroll
    for (int j = 0; j < SPLITS; ++j) v[j] = *(const float4 *)(partials + j * plane + q * 4);
    float4 acc = v[0];
#pragma unroll
    for (int j = 1; j < SPLITS; ++j) acc.x += v[j].x, acc.y += v[j].y, acc.z += v[j].z, acc.w += v[j].w;
    float r[4] = {acc.x, acc.y, acc.z, acc.w};
    const uint32_t col = (uint32_t)((q * 4) % N);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (bias) r[i] += load_bias(bias, col + i, epilogue & kEpilogueBiasF32);
        r[i] = apply_epilogue(epilogue & kEpilogueMask, r[i]);
    }
    if constexpr (sizeof(OutT) == 4) {
        *(float4 *)(Y + q * 4) = make_float4(r[0], r[1], r[2], r[3]);
    } else {
        const uint32_t lo = f32_to_bf16_rne(__float_as_uint(r[0])) | ((uint32_t)f32_to_bf16_rne(__float_as_uint(r[1])) << 16);
        const uint32_t hi = f32_to_bf16_rne(__float_as_uint(r[2])) | ((uint32_t)f32_to_bf16_rne(__float_as_uint(r[3])) << 16);
        *(uint2 *)(Y + q * 4) = make_uint2(lo, hi);
    }
}

template <typename OutT, int SPLITS>
void launch_reduce(uint64_t quads, uint32_t N, const float *partials, const void *bias, int epilogue, void *y, hipStream_t stream)
{
    hipLaunchKernelGGL((splitk_reduce_kernel<OutT, SPLITS>), dim3((uint32_t)((quads + 255) / 256)), dim3(256), 0, stream, quads, N, partials,
                       (const uint16_t *)bias, epilogue, (OutT *)y);
}

template <typename OutT>
hipError_t launch_reduce(uint32_t splits, uint64_t quads, uint32_t N, const float *partials, const void *bias, int epilogue, void *y,
                         hipStream_t stream)
{
    static_assert(TTBFP_SPLITK_MAX <= 8, "one case per number of runs");
    switch (splits) {
        case 2: launch_reduce<OutT, 2>(quads, N, partials, bias, epilogue, y, stream); break;
        case 3: launch_reduce<OutT, 3>(quads, N, partials, bias, epilogue, y, stream); break;
        case 4: launch_reduce<OutT, 4>(quads, N, partials, bias, epilogue, y, stream); break;
        case 5: launch_reduce<OutT, 5>(quads, N, partials, bias, epilogue, y, stream); break;
        case 6: launch_reduce<OutT, 6>(quads, N, partials, bias, epilogue, y, stream); break;
        case 7: launch_reduce<OutT, 7>(quads, N, partials, bias, epilogue, y, stream); break;
        case 8: launch_reduce<OutT, 8>(quads, N, partials, bias, epilogue, y, stream); break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace

// How many ways K is cut: 0 = this form does not apply.  A cost model of the measured pieces, in microseconds.  Launch,
// prologue and epilogue cost 5.5.  The fused kernel that the shape would get otherwise: the 128 x 64 tile with two pipelines
// takes 0.80 to 0.97 per pair of 64-k slabs (by how many of the CUs have a workgroup), with one pipeline 0.53 per slab; the
// 128 x 128 tile with two pipelines 1.25 per pair.  A workgroup of the 128 x 128 kernel of this form takes 0.735 per slab alone on
// its CU and two that share a CU 1.2 per pair of slabs (so up to 512 workgroups are worth having); the second launch costs 3
// plus the partial planes written and read once (s M N 8 bytes at 9 TB/s, most of it out of cache).  Predicted / measured:
// 256 x 4096 x 4096 fused 33.8 / 31.8, four runs 24.0 / 24.9; 1024 x 1024 x 4096 33.8 / 31.3 and 24.0 / 25.7; 256 x 1024 x 4096
// 31.7 / 29.6, eight runs 16.3 / 17.3; 512 x 4096 x 4096 36.5 / 36.4, four runs 35.2 / 37.3 (not taken); 512 x 2048 x 2048 19.7 / 18.1,
// four runs 18.1 / 21.2 (not taken).  The cut with the shortest prediction wins if it saves 3 us or more.
static uint32_t splitk_factor(uint32_t M, uint32_t N, uint32_t K)
{
    if (!gemm_fits<SmallShape>(M, N, K) || K % 64) return 0;  // fewer than 128 rows, and 160 to 224, go to the weight-streaming kernel
    const uint64_t tiles = (uint64_t)(M / 128) * (N / 128);
    if (tiles > 256) return 0;
    const uint32_t slabs = K / BK;
    double fused;
    if (M == 128)  // the weight-streaming kernel on four row tiles: every workgroup pulls all of X through its L2 (N = K = 4096: 20 us)
        fused = 4.3 + 16.0 * ((double)K / 4096.0) * (double)((N + 4095) / 4096);
    else if (2 * tiles <= 256)
        fused = K % 128 == 0 ? 5.5 + (slabs / 2) * (0.80 + 0.17 * (double)(2 * tiles) / 256.0) : 5.5 + slabs * 0.53;
    else
        fused = K % 128 == 0 ? 5.5 + (slabs / 2) * 1.25 : 5.5 + slabs * 0.735;
    auto mfma_time = [&](uint32_t s) {
        const uint64_t wgs = tiles * s;
        const double per_slab = wgs > 256 ? 1.2 : 0.735;  // a pair of workgroups per CU, or one
        return 5.5 + (double)(slabs / s) * per_slab;
    };
    uint32_t best = 0;
    double best_time = fused - 3.0;
    for (uint32_t s = 2; s <= TTBFP_SPLITK_MAX && tiles * s <= 512; ++s) {
        if (slabs % s || slabs / s < 4) continue;
        const double t = mfma_time(s) + 3.0 + (double)s * M * N * 8.0 / 9.0e6;
        if (t < best_time) best = s, best_time = t;
    }
    return best;
}

uint64_t gemm_bfp8b_splitk_bytes(uint32_t M, uint32_t N, uint32_t K) { return (uint64_t)splitk_factor(M, N, K) * M * N * 4; }

hipError_t launch_gemm_bfp8b_splitk(uint32_t M, uint32_t N, uint32_t K, const void *x, const void *w, const void *bias, int epilogue,
                                    void *y, uint8_t y_fmt, void *workspace, hipStream_t stream)
{
    if (y_fmt != kFloat32 && y_fmt != kFloat16_b) return hipErrorInvalidValue;
    const uint32_t splits = splitk_factor(M, N, K);
    if (splits == 0) return hipErrorInvalidValue;
    if (hipError_t e = launch_tile_splitk<SmallShape>(M, N, K, splits, x, w, (float *)workspace, stream); e != hipSuccess) return e;
    const uint64_t quads = (uint64_t)M * N / 4;
    if (y_fmt == kFloat32) return launch_reduce<float>(splits, quads, N, (const float *)workspace, bias, epilogue, y, stream);
    return launch_reduce<uint16_t>(splits, quads, N, (const float *)workspace, bias, epilogue, y, stream);
}

}  // namespace ttbfp
