// Y[M,N] = epilogue(X[M,K] * W[K,N] + bias), everything fp32, row-major: the matmul of the full-precision mode of the
// backend (BackendConfig's ignore_data_format_precision, pybuda/csrc/backend_api/backend_api.cpp:268-275: "run backend at
// full precision"), where queues keep their tensors unquantized and the golden evaluation
// (pybuda/pybuda/op/eval/buda/matmul.py:233-249) runs on them as they are.  A verification path, not a fast one: 64 x 64
// output tiles, K in steps of 16 through LDS, a 4 x 4 register tile per thread, plain fp32 FMAs so that the result is an
// ordinary fp32 dot product (no matrix-core rounding modes to account for).  Any M, N, K.
#include "bfp_codec.hpp"
#include "launch.hpp"

namespace ttbfp {

namespace {

constexpr int FT = 64, FK = 16;

__global__ __launch_bounds__(256) void gemm_f32_kernel(uint32_t M, uint32_t N, uint32_t K, const float *__restrict__ X,
                                                       const float *__restrict__ W, const float *__restrict__ bias, int epilogue,
                                                       float *__restrict__ Y)
{
    __shared__ float xs[FK][FT + 4];  // [k][m]: the thread's four m are contiguous
    __shared__ float ws[FK][FT + 4];  // [k][n]
    const uint32_t tid = threadIdx.x, tx = tid % 16, ty = tid / 16;
    const uint32_t m0 = blockIdx.y * FT, n0 = blockIdx.x * FT;
    float acc[4][4] = {};
    for (uint32_t k0 = 0; k0 < K; k0 += FK) {
        // X tile: 64 rows x 16 k, one row segment of four k per thread; W tile: 16 k x 64 n, four n per thread
        {
            const uint32_t r = tid / 4, kq = (tid % 4) * 4;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t m = m0 + r, k = k0 + kq + j;
                xs[kq + j][r] = (m < M && k < K) ? X[(uint64_t)m * K + k] : 0.0f;
            }
            const uint32_t kr = tid / 16, nq = (tid % 16) * 4;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t k = k0 + kr, n = n0 + nq + j;
                ws[kr][nq + j] = (k < K && n < N) ? W[(uint64_t)k * N + n] : 0.0f;
            }
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < FK; ++k) {
            float a[4], b[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) a[i] = xs[k][ty * 4 + i], b[i] = ws[k][tx * 4 + i];
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t m = m0 + ty * 4 + i, n = n0 + tx * 4 + j;
            if (m < M && n < N) Y[(uint64_t)m * N + n] = apply_epilogue(epilogue, acc[i][j] + (bias ? bias[n] : 0.0f));
        }
}

}  // namespace

hipError_t launch_gemm_f32(uint32_t M, uint32_t N, uint32_t K, const void *x, const void *w, const void *bias, int epilogue,
                           void *y, hipStream_t stream)
{
    if (M == 0 || N == 0) return hipSuccess;
    const dim3 grid((N + FT - 1) / FT, (M + FT - 1) / FT);
    if (grid.y > 65535u) return hipErrorInvalidValue;
    hipLaunchKernelGGL(gemm_f32_kernel, grid, dim3(256), 0, stream, M, N, K, (const float *)x, (const float *)w, (const float *)bias,
                       epilogue & kEpilogueMask, (float *)y);
    return hipGetLastError();
}

}  // namespace ttbfp
