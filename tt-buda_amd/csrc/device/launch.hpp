// Launchers of the HIP kernels, called by the C ABI (c_abi.hip) after it has validated arguments.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

namespace ttbfp {

// Row-major [W,Z,R,C] tensor view; strides in bytes, outermost first (tt_PytorchTensorDesc,
// pybuda/csrc/backend_api/backend_api.cpp:489-560).  R and C are multiples of 32: the extent of the tiles.
// The memory itself may hold fewer rows and columns, Rl x Cl (the tensor before pad_pytorch_tensor_to_buda,
// pybuda/pybuda/tensor.py:805-877): packing reads rows >= Rl / columns >= Cl as zeros, or as the last row / column where
// rep_r / rep_c is set (the reference's "replicate" mode, used for a dimension of one that is broadcast to a tile);
// unpacking writes the Rl x Cl corner only (narrow_buda_tensor_to_pytorch, tensor.py:879-954).  Rl == R and Cl == C:
// nothing to pad or narrow.
struct TensorGeom {
    uint32_t W, Z, R, C;
    uint64_t s0, s1, s2, s3;
    uint32_t Rl, Cl;
    uint32_t rep_r, rep_c;
    bool padded() const { return Rl != R || Cl != C; }
};

struct QueueLayout;  // queue_layout.hpp

// A kernel that wants more dynamic LDS than the default limit has to say so once per device.  Kernels of one
// signature share a function-pointer type, so the memory of who has been told is keyed by the kernel's address, not by
// its type: a small open-addressed table (the library has a few dozen such kernels), one 64-bit device mask per entry.
// Lock-free; a slot whose key is being claimed by another thread is simply told again, which is harmless.
struct DynamicLdsTold {
    static constexpr int kSlots = 256;
    std::atomic<const void *> key[kSlots];
    std::atomic<uint64_t> mask[kSlots];
};
inline DynamicLdsTold g_dynamic_lds_told{};

inline hipError_t allow_dynamic_lds_at(const void *kernel, uint32_t bytes)
{
    int device = 0;
    if (hipError_t e = hipGetDevice(&device); e != hipSuccess) return e;
    const uint64_t bit = device >= 0 && device < 64 ? 1ull << device : 0;
    DynamicLdsTold &t = g_dynamic_lds_told;
    int slot = -1;
    for (int i = 0, h = (int)(((uintptr_t)kernel >> 4) % DynamicLdsTold::kSlots); i < DynamicLdsTold::kSlots; ++i, h = (h + 1) % DynamicLdsTold::kSlots) {
        const void *k = t.key[h].load(std::memory_order_acquire);
        if (k == nullptr) {
            const void *expected = nullptr;
            if (t.key[h].compare_exchange_strong(expected, kernel, std::memory_order_acq_rel)) k = kernel;
            else k = expected;
        }
        if (k == kernel) { slot = h; break; }
    }
    if (slot >= 0 && bit && (t.mask[slot].load(std::memory_order_acquire) & bit)) return hipSuccess;
    if (hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes); e != hipSuccess) return e;
    if (slot >= 0) t.mask[slot].fetch_or(bit, std::memory_order_release);
    return hipSuccess;
}
template <typename Kernel>
hipError_t allow_dynamic_lds(Kernel kernel, uint32_t bytes)
{
    return allow_dynamic_lds_at((const void *)kernel, bytes);
}

// q == nullptr: header-less tiles in one run, order [w][z][r/32][c/32]; otherwise the tiles sit in
// the queue buffers q describes.
hipError_t launch_tilize_pack(const void *src, uint8_t src_fmt, const TensorGeom &g, uint8_t dst_fmt, int rounding,
                              void *dst, const QueueLayout *q, hipStream_t stream);

hipError_t launch_unpack_untilize(const void *src, uint8_t src_fmt, const TensorGeom &g, uint8_t dst_fmt, void *dst,
                                  const QueueLayout *q, hipStream_t stream);

// [W, C, H, W] (g.Z = channels, g.R x g.C the image) -> row-major [W, 1, rows, cols] of the same element size,
// prestrided by `stride` and zero-padded to rows x cols.
hipError_t launch_prestride(const void *src, uint32_t itemsize, const TensorGeom &g, uint32_t stride, void *dst, uint32_t rows,
                            uint32_t cols, hipStream_t stream);

hipError_t launch_gemm_bfp8b(uint32_t M, uint32_t N, uint32_t K, const void *x, const void *w, const void *bias,
                             int epilogue, void *y, uint8_t y_fmt, hipStream_t stream);

// Plain fp32 GEMM on row-major operands with an fp32 bias row: the matmul of the full-precision (unquantized) mode.
// the same conversions on host memory (cpu_twins.hip): no GPU involved, never called by a device entry point
bool cpu_tilize_pack(const void *src, uint8_t src_fmt, const TensorGeom &g, uint8_t dst_fmt, int rounding, void *dst);
bool cpu_unpack_untilize(const void *src, uint8_t src_fmt, const TensorGeom &g, uint8_t dst_fmt, void *dst);
bool cpu_gemm_bfp8b(uint32_t M, uint32_t N, uint32_t K, const void *x, const void *w, const void *bias, int epilogue, void *y, uint8_t y_fmt);

hipError_t launch_gemm_f32(uint32_t M, uint32_t N, uint32_t K, const void *x, const void *w, const void *bias, int epilogue, void *y,
                           hipStream_t stream);

// Two-pass form for large M with a caller's workspace: W is converted once into a bf16 panel, then the MFMA kernel
// runs on that.  gemm_bfp8b_panel_bytes is the workspace it needs, 0 when the fused kernel is the better choice.
uint64_t gemm_bfp8b_panel_bytes(uint32_t M, uint32_t N, uint32_t K);
hipError_t launch_gemm_bfp8b_panel(uint32_t M, uint32_t N, uint32_t K, const void *x, const void *w, const void *bias, int epilogue,
                                   void *y, uint8_t y_fmt, void *workspace, hipStream_t stream);

// Split-K form for shapes whose macro tiles leave CUs idle, with a caller's workspace of fp32 partial sums;
// gemm_bfp8b_splitk_bytes is the workspace it needs, 0 when it does not apply.
uint64_t gemm_bfp8b_splitk_bytes(uint32_t M, uint32_t N, uint32_t K);
hipError_t launch_gemm_bfp8b_splitk(uint32_t M, uint32_t N, uint32_t K, const void *x, const void *w, const void *bias, int epilogue,
                                    void *y, uint8_t y_fmt, void *workspace, hipStream_t stream);

}  // namespace ttbfp
