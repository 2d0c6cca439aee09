// The C ABI declared in include/ttbfp.h: argument checks, status codes, memory/stream plumbing,
// and dispatch to the kernel launchers.  Nothing here keeps state between calls except the
// thread-local text of the last failure.
#include "../../../include/ttbfp.h"

#include <atomic>
#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <thread>

#include "bfp_codec.hpp"
#include "launch.hpp"
#include "queue_layout.hpp"

// Scratch memory of ttbfp_gemm_bfp8b_bf16_static: the workspace that ttbfp_gemm_bfp8b_bf16_ws takes from its caller, held
// by the library instead, for callers that cannot allocate.  Every device the library's code is loaded on holds its
// own copy of the array at its own address until the process ends.  The name below is only a host-side handle of the
// symbol: host code uses the device address that hipGetSymbolAddress returns for the current device, never the name.
static __device__ __align__(256) unsigned char scratch[TTBFP_STATIC_SCRATCH_BYTES];

namespace {

thread_local char g_error[512] = "";

constexpr int kMaxDevices = 64;
std::atomic<void *> g_scratch_ptr[kMaxDevices];  // device address of `scratch` per device, nullptr until asked for

int32_t fail(const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_error, sizeof(g_error), fmt, ap);
    va_end(ap);
    return TTBFP_RUNTIME_ERROR;
}

int32_t hip_status(hipError_t err, const char *what)
{
    if (err == hipSuccess) return TTBFP_SUCCESS;
    return fail("%s: %s", what, hipGetErrorString(err));
}

// Device address of the static scratch array on `device`, which must be the calling thread's current device.  Asked
// for once per device (ttbfp_init, or the first ttbfp_gemm_bfp8b_bf16_static on a device that was never initialised);
// two threads that race here both get the same answer from the runtime.
int32_t static_scratch(int device, void **out)
{
    if (device < 0 || device >= kMaxDevices) return fail("static scratch: device %d is beyond the %d the library keeps track of", device, kMaxDevices);
    void *p = g_scratch_ptr[device].load(std::memory_order_acquire);
    if (!p) {
        const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) return fail("hipGetSymbolAddress(scratch) on device %d: %s", device, hipGetErrorString(e));
        g_scratch_ptr[device].store(p, std::memory_order_release);
    }
    *out = p;
    return TTBFP_SUCCESS;
}

// Integer formats (pybuda/csrc/lower_to_buda/common.hpp:92-111; sizes pybuda/csrc/lower_to_buda/common.cpp:180-186): index
// tensors travel as RawUInt32 (pybuda/pybuda/device_connector.py:270-277), int32 and int8 torch tensors as Int32 and Int8
// (pybuda/pybuda/tensor.py:667-670).  They are tiled without any conversion: the 32-bit ones by the Float32 -> Float32
// kernels, which move the bits they are given, the 16-bit ones by the Float16_b -> Float16_b kernels, the 8-bit ones by
// a byte permutation of their own.  An integer format pairs with itself only.
constexpr uint8_t kRawUInt8 = 0xF0, kRawUInt16 = 0xF1, kRawUInt32 = 0xF2, kInt32 = 8, kUInt16 = 12, kInt8 = 14;
bool is_integer(uint8_t fmt) { return fmt == kRawUInt8 || fmt == kRawUInt16 || fmt == kRawUInt32 || fmt == kInt32 || fmt == kUInt16 || fmt == kInt8; }
uint8_t canonical(uint8_t fmt)
{
    switch (fmt) {
        case kRawUInt32: case kInt32: return ttbfp::kFloat32;
        case kRawUInt16: case kUInt16: return ttbfp::kFloat16_b;
        case kRawUInt8: case kInt8: return ttbfp::kRaw8;
        default: return fmt;
    }
}
// true if the pair is legal as far as integers go (an integer format pairs with itself only); rewrites both to their kernel formats
bool raw_pair_ok(uint8_t &a, uint8_t &b)
{
    if ((is_integer(a) || is_integer(b)) && a != b) return false;
    a = canonical(a);
    b = canonical(b);
    return true;
}
// bytes per element of a row-major tensor in (kernel) format fmt
uint32_t plain_itemsize(uint8_t fmt) { return fmt == ttbfp::kFloat32 ? 4 : fmt == ttbfp::kRaw8 ? 1 : 2; }

bool is_plain(uint8_t fmt) { return fmt == ttbfp::kFloat32 || fmt == ttbfp::kFloat16_b || fmt == ttbfp::kFloat16 || fmt == ttbfp::kRaw8; }
bool is_bfp(uint8_t fmt) { return ttbfp::mantissa_bits(fmt) != 0; }

const char *fmt_name(uint8_t fmt)
{
    switch (fmt) {
        case ttbfp::kFloat32: return "Float32";
        case ttbfp::kFloat16_b: return "Float16_b";
        case ttbfp::kBfp8_b: return "Bfp8_b";
        case ttbfp::kBfp4_b: return "Bfp4_b";
        case ttbfp::kBfp2_b: return "Bfp2_b";
        case ttbfp::kFloat16: return "Float16";
        case ttbfp::kBfp8: return "Bfp8";
        case ttbfp::kBfp4: return "Bfp4";
        case ttbfp::kBfp2: return "Bfp2";
        case ttbfp::kRaw8: return "8-bit integer";
        default: return "unsupported";
    }
}

uint32_t align_up_tile(uint32_t d) { return (d + 31u) / 32u * 32u; }  // pybuda/csrc/tt_torch_device/tt_device.hpp:205-210

// Common checks of a [w,z,r,c] view; fills g.  itemsize is that of the row-major side.  With `ragged` the rows and
// columns of the memory need not be multiples of 32: the tiles then cover the shape rounded up (`tiled`), and what lies
// past the memory is padding (pack) or left out (unpack).
int32_t check_geom(const char *fn, const uint32_t shape[4], const uint64_t strides[4], uint32_t itemsize,
                   ttbfp::TensorGeom &g, bool ragged = false, uint32_t rep_r = 0, uint32_t rep_c = 0, uint32_t tiled[4] = nullptr)
{
    if (!shape || !strides) return fail("%s: shape and strides must not be NULL", fn);
    if (!ragged && (shape[2] % 32 || shape[3] % 32))
        return fail("%s: shape [%u,%u,%u,%u]: rows and columns must be multiples of the 32x32 tile", fn, shape[0],
                    shape[1], shape[2], shape[3]);
    if (ragged && (shape[2] == 0 || shape[3] == 0 || shape[2] > 0xffffffe0u || shape[3] > 0xffffffe0u))
        return fail("%s: shape [%u,%u,%u,%u]: rows and columns must lie between 1 and 2^32 - 32", fn, shape[0], shape[1], shape[2], shape[3]);
    if (rep_r > 1 || rep_c > 1) return fail("%s: the replicate flags are 0 or 1", fn);
    // the reference replicates only a dimension of one (pybuda/pybuda/tensor.py:852-856)
    if ((rep_r && shape[2] != 1) || (rep_c && shape[3] != 1))
        return fail("%s: shape [%u,%u,%u,%u]: only a dimension of size 1 can be replicated into its tile", fn, shape[0], shape[1], shape[2], shape[3]);
    for (int i = 0; i < 4; ++i)
        if (strides[i] % itemsize)
            return fail("%s: stride %d (%llu bytes) is not a multiple of the element size %u", fn, i,
                        (unsigned long long)strides[i], itemsize);
    const uint32_t R = align_up_tile(shape[2]), C = align_up_tile(shape[3]);
    const uint64_t elems = (uint64_t)shape[0] * shape[1] * R * C;
    if (elems / 1024 * 64 > 0x7fffffffull * 256ull) return fail("%s: tensor too large", fn);
    g = {shape[0], shape[1], R, C, strides[0], strides[1], strides[2], strides[3], shape[2], shape[3], rep_r, rep_c};
    if (tiled) tiled[0] = shape[0], tiled[1] = shape[1], tiled[2] = R, tiled[3] = C;
    return TTBFP_SUCCESS;
}

}  // namespace

extern "C" {

const char *ttbfp_last_error(void) { return g_error; }

int32_t ttbfp_device_count(void)
{
    int n = 0;
    if (hipGetDeviceCount(&n) != hipSuccess) return -1;
    return n > 0 ? n : -1;
}

int32_t ttbfp_init(int32_t device)
{
    int n = 0;
    hipError_t err = hipGetDeviceCount(&n);
    if (err != hipSuccess || n <= 0) return fail("ttbfp_init: no HIP device (%s)", hipGetErrorString(err));
    if (device < 0 || device >= n) return fail("ttbfp_init: device %d out of range (0..%d)", device, n - 1);
    if (int32_t s = hip_status(hipSetDevice(device), "hipSetDevice")) return s;
    hipDeviceProp_t prop;
    if (int32_t s = hip_status(hipGetDeviceProperties(&prop, device), "hipGetDeviceProperties")) return s;
    if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
        return fail("ttbfp_init: device %d is %s; this library holds gfx950 code only", device, prop.gcnArchName);
    void *p = nullptr;
    return static_scratch(device, &p);  // set-up work (it may load the code object) done here, not in the first GEMM call
}

uint32_t ttbfp_tile_bytes(uint8_t fmt) { return ttbfp::tile_bytes(canonical(fmt)); }

uint64_t ttbfp_packed_size(uint8_t fmt, const uint32_t shape[4])
{
    if (!shape || shape[2] % 32 || shape[3] % 32) return 0;
    return (uint64_t)shape[0] * shape[1] * (shape[2] / 32) * (shape[3] / 32) * ttbfp_tile_bytes(fmt);
}

int32_t ttbfp_alloc(uint64_t bytes, void **out_dev)
{
    if (!out_dev) return fail("ttbfp_alloc: out_dev is NULL");
    *out_dev = nullptr;
    if (bytes == 0) return TTBFP_SUCCESS;
    return hip_status(hipMalloc(out_dev, bytes), "hipMalloc");
}

int32_t ttbfp_free(void *dev) { return dev ? hip_status(hipFree(dev), "hipFree") : TTBFP_SUCCESS; }

int32_t ttbfp_host_alloc(uint64_t bytes, void **out_host)
{
    if (!out_host) return fail("ttbfp_host_alloc: out_host is NULL");
    *out_host = nullptr;
    if (bytes == 0) return TTBFP_SUCCESS;
    return hip_status(hipHostMalloc(out_host, bytes, hipHostMallocDefault), "hipHostMalloc");
}

int32_t ttbfp_host_free(void *host) { return host ? hip_status(hipHostFree(host), "hipHostFree") : TTBFP_SUCCESS; }

int32_t ttbfp_memcpy_h2d(void *dst_dev, const void *src_host, uint64_t bytes, void *stream)
{
    if (bytes == 0) return TTBFP_SUCCESS;
    return hip_status(hipMemcpyAsync(dst_dev, src_host, bytes, hipMemcpyHostToDevice, (hipStream_t)stream),
                      "hipMemcpyAsync(host to device)");
}

int32_t ttbfp_memcpy_d2h(void *dst_host, const void *src_dev, uint64_t bytes, void *stream)
{
    if (bytes == 0) return TTBFP_SUCCESS;
    return hip_status(hipMemcpyAsync(dst_host, src_dev, bytes, hipMemcpyDeviceToHost, (hipStream_t)stream),
                      "hipMemcpyAsync(device to host)");
}

int32_t ttbfp_memcpy_d2d(void *dst_dev, const void *src_dev, uint64_t bytes, void *stream)
{
    if (bytes == 0) return TTBFP_SUCCESS;
    return hip_status(hipMemcpyAsync(dst_dev, src_dev, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream),
                      "hipMemcpyAsync(device to device)");
}

int32_t ttbfp_pointer_is_device(const void *ptr)
{
    hipPointerAttribute_t attr;
    if (!ptr || hipPointerGetAttributes(&attr, ptr) != hipSuccess) {
        (void)hipGetLastError();  // an unregistered host pointer is reported as an error: not one here
        return 0;
    }
    return attr.type == hipMemoryTypeDevice ? 1 : 0;
}

int32_t ttbfp_stream_create(void **out_stream)
{
    if (!out_stream) return fail("ttbfp_stream_create: out_stream is NULL");
    hipStream_t s = nullptr;
    const int32_t st = hip_status(hipStreamCreateWithFlags(&s, hipStreamNonBlocking), "hipStreamCreate");
    *out_stream = s;
    return st;
}

int32_t ttbfp_stream_destroy(void *stream)
{
    return stream ? hip_status(hipStreamDestroy((hipStream_t)stream), "hipStreamDestroy") : TTBFP_SUCCESS;
}

int32_t ttbfp_device_synchronize(void) { return hip_status(hipDeviceSynchronize(), "hipDeviceSynchronize"); }

int32_t ttbfp_stream_synchronize(void *stream, int32_t timeout_s)
{
    if (timeout_s <= 0) return hip_status(hipStreamSynchronize((hipStream_t)stream), "hipStreamSynchronize");
    const auto deadline = std::chrono::steady_clock::now() + std::chrono::seconds(timeout_s);
    for (;;) {
        const hipError_t q = hipStreamQuery((hipStream_t)stream);
        if (q == hipSuccess) return TTBFP_SUCCESS;
        if (q != hipErrorNotReady) return hip_status(q, "hipStreamQuery");
        if (std::chrono::steady_clock::now() >= deadline) {
            snprintf(g_error, sizeof(g_error), "ttbfp_stream_synchronize: work not finished after %d s", timeout_s);
            return TTBFP_TIMEOUT_ERROR;
        }
        std::this_thread::sleep_for(std::chrono::microseconds(50));
    }
}

}  // extern "C"

namespace {

int32_t check_pack_formats(const char *fn, uint8_t src_fmt, uint8_t dst_fmt, int32_t rounding)
{
    if (!is_plain(src_fmt))
        return fail("%s: source format %u (%s): the source must be Float32, Float16_b or Float16", fn, src_fmt, fmt_name(src_fmt));
    if (!(is_bfp(dst_fmt) || is_plain(dst_fmt)))
        return fail("%s: destination format %u is not one of Bfp8[_b], Bfp4[_b], Bfp2[_b], Float16[_b], Float32", fn, dst_fmt);
    if ((src_fmt == ttbfp::kRaw8) != (dst_fmt == ttbfp::kRaw8)) return fail("%s: one-byte elements go into one-byte tiles and nothing else does", fn);
    // queues with a 5-bit exponent take IEEE half sources and nothing else does (pybuda/pybuda/device_connector.py:177-201)
    if (ttbfp::is_a_format(dst_fmt) != (src_fmt == ttbfp::kFloat16))
        return fail("%s: %s source with %s destination: Float16 sources go with Float16/Bfp8/Bfp4/Bfp2 only", fn, fmt_name(src_fmt),
                    fmt_name(dst_fmt));
    // a Float16_b source widens exactly into Float32 tiles (the full-precision mode of the host layer keeps queues that way)
    if (rounding != TTBFP_ROUND_TRUNCATE && rounding != TTBFP_ROUND_NEAREST)
        return fail("%s: rounding %d is neither truncate (0) nor nearest (1)", fn, rounding);
    return TTBFP_SUCCESS;
}

int32_t check_unpack_formats(const char *fn, uint8_t src_fmt, uint8_t dst_fmt)
{
    if (!(is_bfp(src_fmt) || is_plain(src_fmt)))
        return fail("%s: source format %u is not one of Bfp8[_b], Bfp4[_b], Bfp2[_b], Float16[_b], Float32", fn, src_fmt);
    if (!is_plain(dst_fmt))
        return fail("%s: destination format %u (%s): the output must be Float32, Float16_b or Float16", fn, dst_fmt,
                    fmt_name(dst_fmt));
    if ((src_fmt == ttbfp::kRaw8) != (dst_fmt == ttbfp::kRaw8)) return fail("%s: one-byte tiles read back as one-byte elements and nothing else does", fn);
    if (ttbfp::is_a_format(src_fmt) != (dst_fmt == ttbfp::kFloat16))
        return fail("%s: %s tiles read back as %s: Float16/Bfp8/Bfp4/Bfp2 read back as Float16 and nothing else does", fn,
                    fmt_name(src_fmt), fmt_name(dst_fmt));
    if (src_fmt == ttbfp::kFloat32 && dst_fmt != ttbfp::kFloat32)
        return fail("%s: Float32 tiles can only be read back as Float32", fn);
    return TTBFP_SUCCESS;
}

// Checks a queue geometry against a [w,t,R,C] shape and fills the kernels' view of it.
int32_t check_layout(const char *fn, uint8_t fmt, const uint32_t shape[4], const ttbfp_queue_layout *l, uint64_t pitch,
                     ttbfp::QueueLayout &q)
{
    if (!l) return fail("%s: layout is NULL", fn);
    if (!l->grid_r || !l->grid_c || !l->mblock_m || !l->mblock_n || !l->ublock_rt || !l->ublock_ct)
        return fail("%s: zero in the queue geometry", fn);
    if (l->ublock_order > 1 || l->tile_header > 1) return fail("%s: ublock_order and tile_header must be 0 or 1", fn);
    const uint64_t rt = (uint64_t)l->grid_r * l->mblock_m * l->ublock_rt, ct = (uint64_t)l->grid_c * l->mblock_n * l->ublock_ct;
    if (rt * 32 != shape[2] || ct * 32 != shape[3])
        return fail("%s: grid [%u,%u] x mblock [%u,%u] x ublock [%u,%u] covers %llu x %llu tiles, the tensor has %u x %u", fn, l->grid_r,
                    l->grid_c, l->mblock_m, l->mblock_n, l->ublock_rt, l->ublock_ct, (unsigned long long)rt, (unsigned long long)ct,
                    shape[2] / 32, shape[3] / 32);
    const uint64_t need = ttbfp_queue_buffer_bytes(fmt, shape, l);
    if (pitch % 16) return fail("%s: buffer pitch %llu is not a multiple of 16", fn, (unsigned long long)pitch);
    if (pitch < need && (uint64_t)l->grid_r * l->grid_c > 1)
        return fail("%s: buffer pitch %llu is below the %llu bytes one buffer holds", fn, (unsigned long long)pitch, (unsigned long long)need);
    q = {l->grid_r, l->grid_c, l->mblock_m, l->mblock_n, l->ublock_rt, l->ublock_ct, l->ublock_order, shape[1],
         l->tile_header ? 16u : 0u, ttbfp_tile_bytes(fmt) + (l->tile_header ? 32u : 0u), pitch};
    return TTBFP_SUCCESS;
}

}  // namespace

extern "C" {

uint64_t ttbfp_queue_buffer_bytes(uint8_t fmt, const uint32_t shape[4], const ttbfp_queue_layout *l)
{
    const uint32_t tb = ttbfp_tile_bytes(fmt);
    if (!shape || !l || !tb || !l->grid_r || !l->grid_c) return 0;
    if ((uint64_t)l->grid_r * l->mblock_m * l->ublock_rt * 32 != shape[2] || (uint64_t)l->grid_c * l->mblock_n * l->ublock_ct * 32 != shape[3])
        return 0;
    return (uint64_t)shape[0] * shape[1] * l->mblock_m * l->mblock_n * l->ublock_rt * l->ublock_ct * (tb + (l->tile_header ? 32u : 0u));
}

int32_t ttbfp_tilize_pack(const void *src_dev, uint8_t src_fmt, const uint32_t shape[4],
                          const uint64_t strides_bytes[4], uint8_t dst_fmt, int32_t rounding, void *dst_dev,
                          uint64_t dst_bytes, void *stream)
{
    const char *fn = "ttbfp_tilize_pack";
    if (!raw_pair_ok(src_fmt, dst_fmt)) return fail("%s: an integer format (Int8, UInt16, Int32, RawUInt8, RawUInt16, RawUInt32) pairs with itself only", fn);
    if (int32_t s = check_pack_formats(fn, src_fmt, dst_fmt, rounding)) return s;
    ttbfp::TensorGeom g;
    if (int32_t s = check_geom(fn, shape, strides_bytes, plain_itemsize(src_fmt), g)) return s;
    const uint64_t need = ttbfp_packed_size(dst_fmt, shape);
    if (dst_bytes < need)
        return fail("%s: destination holds %llu bytes, %llu needed", fn, (unsigned long long)dst_bytes,
                    (unsigned long long)need);
    if (need == 0) return TTBFP_SUCCESS;
    if (!src_dev || !dst_dev) return fail("%s: NULL device pointer", fn);
    return hip_status(ttbfp::launch_tilize_pack(src_dev, src_fmt, g, dst_fmt, rounding, dst_dev, nullptr, (hipStream_t)stream), fn);
}

int32_t ttbfp_tilize_pack_queue(const void *src_dev, uint8_t src_fmt, const uint32_t shape[4], const uint64_t strides_bytes[4],
                                uint8_t dst_fmt, int32_t rounding, const ttbfp_queue_layout *layout, uint64_t buffer_pitch_bytes,
                                void *dst_dev, uint64_t dst_bytes, void *stream)
{
    const char *fn = "ttbfp_tilize_pack_queue";
    if (!raw_pair_ok(src_fmt, dst_fmt)) return fail("%s: an integer format (Int8, UInt16, Int32, RawUInt8, RawUInt16, RawUInt32) pairs with itself only", fn);
    if (int32_t s = check_pack_formats(fn, src_fmt, dst_fmt, rounding)) return s;
    ttbfp::TensorGeom g;
    if (int32_t s = check_geom(fn, shape, strides_bytes, plain_itemsize(src_fmt), g)) return s;
    ttbfp::QueueLayout q;
    if (int32_t s = check_layout(fn, dst_fmt, shape, layout, buffer_pitch_bytes, q)) return s;
    const uint64_t per_buffer = ttbfp_queue_buffer_bytes(dst_fmt, shape, layout);
    const uint64_t need = per_buffer ? ((uint64_t)q.grid_r * q.grid_c - 1) * buffer_pitch_bytes + per_buffer : 0;
    if (dst_bytes < need)
        return fail("%s: destination holds %llu bytes, %llu needed", fn, (unsigned long long)dst_bytes, (unsigned long long)need);
    if (need == 0) return TTBFP_SUCCESS;
    if (!src_dev || !dst_dev) return fail("%s: NULL device pointer", fn);
    return hip_status(ttbfp::launch_tilize_pack(src_dev, src_fmt, g, dst_fmt, rounding, dst_dev, &q, (hipStream_t)stream), fn);
}

int32_t ttbfp_unpack_untilize(const void *src_dev, uint8_t src_fmt, const uint32_t shape[4], uint8_t dst_fmt,
                              const uint64_t dst_strides_bytes[4], void *dst_dev, void *stream)
{
    const char *fn = "ttbfp_unpack_untilize";
    if (!raw_pair_ok(src_fmt, dst_fmt)) return fail("%s: an integer format (Int8, UInt16, Int32, RawUInt8, RawUInt16, RawUInt32) pairs with itself only", fn);
    if (int32_t s = check_unpack_formats(fn, src_fmt, dst_fmt)) return s;
    ttbfp::TensorGeom g;
    if (int32_t s = check_geom(fn, shape, dst_strides_bytes, plain_itemsize(dst_fmt), g)) return s;
    if (ttbfp_packed_size(src_fmt, shape) == 0) return TTBFP_SUCCESS;
    if (!src_dev || !dst_dev) return fail("%s: NULL device pointer", fn);
    return hip_status(ttbfp::launch_unpack_untilize(src_dev, src_fmt, g, dst_fmt, dst_dev, nullptr, (hipStream_t)stream), fn);
}

int32_t ttbfp_unpack_untilize_queue(const void *src_dev, uint8_t src_fmt, const uint32_t shape[4], const ttbfp_queue_layout *layout,
                                    uint64_t buffer_pitch_bytes, uint8_t dst_fmt, const uint64_t dst_strides_bytes[4], void *dst_dev,
                                    void *stream)
{
    const char *fn = "ttbfp_unpack_untilize_queue";
    if (!raw_pair_ok(src_fmt, dst_fmt)) return fail("%s: an integer format (Int8, UInt16, Int32, RawUInt8, RawUInt16, RawUInt32) pairs with itself only", fn);
    if (int32_t s = check_unpack_formats(fn, src_fmt, dst_fmt)) return s;
    ttbfp::TensorGeom g;
    if (int32_t s = check_geom(fn, shape, dst_strides_bytes, plain_itemsize(dst_fmt), g)) return s;
    ttbfp::QueueLayout q;
    if (int32_t s = check_layout(fn, src_fmt, shape, layout, buffer_pitch_bytes, q)) return s;
    if (ttbfp_queue_buffer_bytes(src_fmt, shape, layout) == 0) return TTBFP_SUCCESS;
    if (!src_dev || !dst_dev) return fail("%s: NULL device pointer", fn);
    return hip_status(ttbfp::launch_unpack_untilize(src_dev, src_fmt, g, dst_fmt, dst_dev, &q, (hipStream_t)stream), fn);
}

int32_t ttbfp_tilize_pack_padded(const void *src_dev, uint8_t src_fmt, const uint32_t shape[4], const uint64_t strides_bytes[4],
                                 uint32_t replicate_rows, uint32_t replicate_cols, uint8_t dst_fmt, int32_t rounding,
                                 const ttbfp_queue_layout *layout, uint64_t buffer_pitch_bytes, void *dst_dev, uint64_t dst_bytes, void *stream)
{
    const char *fn = "ttbfp_tilize_pack_padded";
    if (!raw_pair_ok(src_fmt, dst_fmt)) return fail("%s: an integer format (Int8, UInt16, Int32, RawUInt8, RawUInt16, RawUInt32) pairs with itself only", fn);
    if (int32_t s = check_pack_formats(fn, src_fmt, dst_fmt, rounding)) return s;
    ttbfp::TensorGeom g;
    uint32_t tiled[4];
    if (int32_t s = check_geom(fn, shape, strides_bytes, plain_itemsize(src_fmt), g, true, replicate_rows, replicate_cols, tiled)) return s;
    ttbfp::QueueLayout q;
    uint64_t need;
    if (layout) {
        if (int32_t s = check_layout(fn, dst_fmt, tiled, layout, buffer_pitch_bytes, q)) return s;
        const uint64_t per_buffer = ttbfp_queue_buffer_bytes(dst_fmt, tiled, layout);
        need = per_buffer ? ((uint64_t)q.grid_r * q.grid_c - 1) * buffer_pitch_bytes + per_buffer : 0;
    } else {
        need = ttbfp_packed_size(dst_fmt, tiled);
    }
    if (dst_bytes < need)
        return fail("%s: destination holds %llu bytes, %llu needed", fn, (unsigned long long)dst_bytes, (unsigned long long)need);
    if (need == 0) return TTBFP_SUCCESS;
    if (!src_dev || !dst_dev) return fail("%s: NULL device pointer", fn);
    return hip_status(ttbfp::launch_tilize_pack(src_dev, src_fmt, g, dst_fmt, rounding, dst_dev, layout ? &q : nullptr, (hipStream_t)stream), fn);
}

int32_t ttbfp_unpack_untilize_narrow(const void *src_dev, uint8_t src_fmt, const uint32_t shape[4], const ttbfp_queue_layout *layout,
                                     uint64_t buffer_pitch_bytes, uint8_t dst_fmt, const uint64_t dst_strides_bytes[4], void *dst_dev,
                                     void *stream)
{
    const char *fn = "ttbfp_unpack_untilize_narrow";
    if (!raw_pair_ok(src_fmt, dst_fmt)) return fail("%s: an integer format (Int8, UInt16, Int32, RawUInt8, RawUInt16, RawUInt32) pairs with itself only", fn);
    if (int32_t s = check_unpack_formats(fn, src_fmt, dst_fmt)) return s;
    ttbfp::TensorGeom g;
    uint32_t tiled[4];
    if (int32_t s = check_geom(fn, shape, dst_strides_bytes, plain_itemsize(dst_fmt), g, true, 0, 0, tiled)) return s;
    ttbfp::QueueLayout q;
    if (layout) {
        if (int32_t s = check_layout(fn, src_fmt, tiled, layout, buffer_pitch_bytes, q)) return s;
    }
    if (ttbfp_packed_size(src_fmt, tiled) == 0) return TTBFP_SUCCESS;
    if (!src_dev || !dst_dev) return fail("%s: NULL device pointer", fn);
    return hip_status(ttbfp::launch_unpack_untilize(src_dev, src_fmt, g, dst_fmt, dst_dev, layout ? &q : nullptr, (hipStream_t)stream), fn);
}

int32_t ttbfp_unpack_untilize_sized(const void *src_dev, uint64_t src_bytes, uint8_t src_fmt, const uint32_t shape[4],
                                    const ttbfp_queue_layout *layout, uint64_t buffer_pitch_bytes, uint8_t dst_fmt,
                                    const uint64_t dst_strides_bytes[4], void *dst_dev, uint64_t dst_bytes, void *stream)
{
    const char *fn = "ttbfp_unpack_untilize_sized";
    if (!shape || !dst_strides_bytes) return fail("%s: shape and strides must not be NULL", fn);
    if (shape[2] == 0 || shape[3] == 0) return fail("%s: shape [%u,%u,%u,%u]: rows and columns must be at least 1", fn, shape[0], shape[1], shape[2], shape[3]);
    const uint32_t tiled[4] = {shape[0], shape[1], align_up_tile(shape[2]), align_up_tile(shape[3])};
    // bytes the tiles take on the source side
    uint64_t need_src;
    if (layout) {
        const uint64_t per_buffer = ttbfp_queue_buffer_bytes(src_fmt, tiled, layout);
        need_src = per_buffer ? ((uint64_t)layout->grid_r * layout->grid_c - 1) * buffer_pitch_bytes + per_buffer : 0;
    } else {
        need_src = ttbfp_packed_size(src_fmt, tiled);
    }
    if (src_bytes < need_src)
        return fail("%s: source holds %llu bytes, the tiles of [%u,%u,%u,%u] take %llu", fn, (unsigned long long)src_bytes, shape[0], shape[1],
                    shape[2], shape[3], (unsigned long long)need_src);
    // bytes from the first to one past the last element written on the destination side
    const uint32_t item = plain_itemsize(dst_fmt);
    uint64_t last = 0;
    for (int i = 0; i < 4; ++i) {
        if (shape[i] == 0) return TTBFP_SUCCESS;  // nothing to write
        const uint64_t reach = (uint64_t)(shape[i] - 1) * dst_strides_bytes[i];
        if (shape[i] > 1 && reach / (shape[i] - 1) != dst_strides_bytes[i]) return fail("%s: stride %d overflows", fn, i);
        if (last + reach < last) return fail("%s: strides overflow", fn);
        last += reach;
    }
    if (item && dst_bytes < last + item)
        return fail("%s: destination holds %llu bytes, the strided result reaches %llu", fn, (unsigned long long)dst_bytes, (unsigned long long)(last + item));
    return ttbfp_unpack_untilize_narrow(src_dev, src_fmt, shape, layout, buffer_pitch_bytes, dst_fmt, dst_strides_bytes, dst_dev, stream);
}

uint64_t ttbfp_prestride_shape(uint32_t itemsize, const uint32_t shape[4], uint32_t stride, uint32_t rows_cols[2])
{
    if (!shape || !stride || (itemsize != 2 && itemsize != 4)) return 0;
    const uint64_t rows = ((uint64_t)stride * stride * shape[1] + 31) / 32 * 32;
    const uint64_t cols = ((uint64_t)((shape[2] + stride - 1) / stride) * ((shape[3] + stride - 1) / stride) + 31) / 32 * 32;
    if (rows > 0xffffffffull || cols > 0xffffffffull) return 0;
    if (rows_cols) rows_cols[0] = (uint32_t)rows, rows_cols[1] = (uint32_t)cols;
    return (uint64_t)shape[0] * rows * cols * itemsize;
}

int32_t ttbfp_prestride(const void *src_dev, uint32_t itemsize, const uint32_t shape[4], const uint64_t strides_bytes[4], uint32_t stride,
                        void *dst_dev, uint64_t dst_bytes, void *stream)
{
    const char *fn = "ttbfp_prestride";
    if (!shape || !strides_bytes) return fail("%s: shape and strides must not be NULL", fn);
    if (itemsize != 2 && itemsize != 4) return fail("%s: element size %u: 2 or 4 bytes", fn, itemsize);
    if (stride == 0) return fail("%s: stride 0", fn);
    for (int i = 0; i < 4; ++i)
        if (strides_bytes[i] % itemsize) return fail("%s: stride %d is not a multiple of the element size", fn, i);
    uint32_t rc[2] = {0, 0};
    const uint64_t need = ttbfp_prestride_shape(itemsize, shape, stride, rc);
    if (need == 0 && (uint64_t)shape[0] * shape[1] * shape[2] * shape[3] != 0) return fail("%s: result too large", fn);
    if (rc[0] > 65535 || shape[0] > 65535) return fail("%s: more than 65535 entries or %u result rows", fn, rc[0]);
    if (dst_bytes < need) return fail("%s: destination holds %llu bytes, %llu needed", fn, (unsigned long long)dst_bytes, (unsigned long long)need);
    if (need == 0) return TTBFP_SUCCESS;
    if (!src_dev || !dst_dev) return fail("%s: NULL device pointer", fn);
    if ((uintptr_t)src_dev % itemsize || (uintptr_t)dst_dev % itemsize) return fail("%s: pointers must be aligned to the element size", fn);
    const ttbfp::TensorGeom g = {shape[0], shape[1], shape[2], shape[3], strides_bytes[0], strides_bytes[1], strides_bytes[2], strides_bytes[3],
                                 shape[2], shape[3], 0, 0};
    return hip_status(ttbfp::launch_prestride(src_dev, itemsize, g, stride, dst_dev, rc[0], rc[1], (hipStream_t)stream), fn);
}

}  // extern "C"

namespace {

int32_t check_gemm(const char *fn, uint32_t M, uint32_t N, uint32_t K, const void *x_dev, const void *w_dev, const void *bias_dev,
                   int32_t epilogue, void *y_dev, uint8_t y_fmt, bool &nothing_to_do)
{
    nothing_to_do = false;
    if (M % 32 || N % 32 || K % 32 || K == 0)
        return fail("%s: M=%u N=%u K=%u must be multiples of 32 (K non-zero)", fn, M, N, K);
    const int32_t activation = epilogue & ~TTBFP_EPILOGUE_BIAS_F32;
    if (activation != TTBFP_EPILOGUE_NONE && activation != TTBFP_EPILOGUE_GELU && activation != TTBFP_EPILOGUE_GELU_TANH) return fail("%s: unknown epilogue %d", fn, epilogue);
    if (y_fmt != ttbfp::kFloat32 && y_fmt != ttbfp::kFloat16_b) return fail("%s: output format %u: must be Float16_b or Float32", fn, y_fmt);
    if (M == 0 || N == 0) {
        nothing_to_do = true;
        return TTBFP_SUCCESS;
    }
    if (!x_dev || !w_dev || !y_dev) return fail("%s: NULL device pointer", fn);
    if ((uintptr_t)x_dev % 16 || (uintptr_t)w_dev % 16 || (uintptr_t)y_dev % 16 ||
        (uintptr_t)bias_dev % ((epilogue & TTBFP_EPILOGUE_BIAS_F32) ? 4 : 2))
        return fail("%s: x, w and y must be 16-byte aligned, the bias to its element size", fn);
    return TTBFP_SUCCESS;
}

}  // namespace

extern "C" {

int32_t ttbfp_gemm_bfp8b_bf16(uint32_t M, uint32_t N, uint32_t K, const void *x_dev, const void *w_dev,
                              const void *bias_dev, int32_t epilogue, void *y_dev, uint8_t y_fmt, void *stream)
{
    const char *fn = "ttbfp_gemm_bfp8b_bf16";
    bool nothing = false;
    if (int32_t s = check_gemm(fn, M, N, K, x_dev, w_dev, bias_dev, epilogue, y_dev, y_fmt, nothing)) return s;
    if (nothing) return TTBFP_SUCCESS;
    return hip_status(ttbfp::launch_gemm_bfp8b(M, N, K, x_dev, w_dev, bias_dev, epilogue, y_dev, y_fmt, (hipStream_t)stream), fn);
}

uint64_t ttbfp_gemm_bfp8b_workspace_bytes(uint32_t M, uint32_t N, uint32_t K)
{
    if (M % 32 || N % 32 || K % 32) return 0;
    const uint64_t panel = ttbfp::gemm_bfp8b_panel_bytes(M, N, K);  // the two forms never apply to the same shape
    return panel ? panel : ttbfp::gemm_bfp8b_splitk_bytes(M, N, K);
}

int32_t ttbfp_gemm_bfp8b_bf16_ws(uint32_t M, uint32_t N, uint32_t K, const void *x_dev, const void *w_dev, const void *bias_dev,
                                 int32_t epilogue, void *y_dev, uint8_t y_fmt, void *workspace_dev, uint64_t workspace_bytes, void *stream)
{
    const char *fn = "ttbfp_gemm_bfp8b_bf16_ws";
    bool nothing = false;
    if (int32_t s = check_gemm(fn, M, N, K, x_dev, w_dev, bias_dev, epilogue, y_dev, y_fmt, nothing)) return s;
    if (nothing) return TTBFP_SUCCESS;
    const uint64_t panel = ttbfp::gemm_bfp8b_panel_bytes(M, N, K);
    const uint64_t need = panel ? panel : ttbfp::gemm_bfp8b_splitk_bytes(M, N, K);
    if (need == 0 || !workspace_dev || workspace_bytes < need)
        return hip_status(ttbfp::launch_gemm_bfp8b(M, N, K, x_dev, w_dev, bias_dev, epilogue, y_dev, y_fmt, (hipStream_t)stream), fn);
    if ((uintptr_t)workspace_dev % 16) return fail("%s: the workspace must be 16-byte aligned", fn);
    if (!panel)
        return hip_status(ttbfp::launch_gemm_bfp8b_splitk(M, N, K, x_dev, w_dev, bias_dev, epilogue, y_dev, y_fmt, workspace_dev, (hipStream_t)stream), fn);
    return hip_status(ttbfp::launch_gemm_bfp8b_panel(M, N, K, x_dev, w_dev, bias_dev, epilogue, y_dev, y_fmt, workspace_dev, (hipStream_t)stream), fn);
}

int32_t ttbfp_gemm_bfp8b_bf16_sized(uint32_t M, uint32_t N, uint32_t K, const void *x_dev, uint64_t x_bytes, const void *w_dev,
                                    uint64_t w_bytes, const void *bias_dev, uint64_t bias_bytes, int32_t epilogue, void *y_dev,
                                    uint64_t y_bytes, uint8_t y_fmt, void *workspace_dev, uint64_t workspace_bytes, void *stream)
{
    const char *fn = "ttbfp_gemm_bfp8b_bf16_sized";
    const uint64_t y_item = y_fmt == ttbfp::kFloat32 ? 4 : 2, bias_item = (epilogue & TTBFP_EPILOGUE_BIAS_F32) ? 4 : 2;
    const uint32_t w_shape[4] = {1, 1, K, N};
    if (x_bytes < (uint64_t)M * K * 2) return fail("%s: x holds %llu bytes, M x K bf16 values take %llu", fn, (unsigned long long)x_bytes, (unsigned long long)M * K * 2);
    if (M % 32 == 0 && N % 32 == 0 && K % 32 == 0 && w_bytes < ttbfp_packed_size(TTBFP_FMT_BFP8_B, w_shape))
        return fail("%s: w holds %llu bytes, the Bfp8_b tiles of [K, N] take %llu", fn, (unsigned long long)w_bytes,
                    (unsigned long long)ttbfp_packed_size(TTBFP_FMT_BFP8_B, w_shape));
    if (bias_dev && bias_bytes < (uint64_t)N * bias_item) return fail("%s: bias holds %llu bytes, N values take %llu", fn, (unsigned long long)bias_bytes, (unsigned long long)N * bias_item);
    if (y_bytes < (uint64_t)M * N * y_item) return fail("%s: y holds %llu bytes, M x N results take %llu", fn, (unsigned long long)y_bytes, (unsigned long long)M * N * y_item);
    return ttbfp_gemm_bfp8b_bf16_ws(M, N, K, x_dev, w_dev, bias_dev, epilogue, y_dev, y_fmt, workspace_dev, workspace_bytes, stream);
}

int32_t ttbfp_gemm_f32(uint32_t M, uint32_t N, uint32_t K, const void *x_dev, const void *w_dev, const void *bias_dev, int32_t epilogue,
                       void *y_dev, void *stream)
{
    const char *fn = "ttbfp_gemm_f32";
    if (K == 0) return fail("%s: K must not be zero", fn);
    if (epilogue != TTBFP_EPILOGUE_NONE && epilogue != TTBFP_EPILOGUE_GELU && epilogue != TTBFP_EPILOGUE_GELU_TANH) return fail("%s: unknown epilogue %d", fn, epilogue);
    if (M == 0 || N == 0) return TTBFP_SUCCESS;
    if (!x_dev || !w_dev || !y_dev) return fail("%s: NULL device pointer", fn);
    if ((uintptr_t)x_dev % 4 || (uintptr_t)w_dev % 4 || (uintptr_t)y_dev % 4 || (uintptr_t)bias_dev % 4) return fail("%s: pointers must be 4-byte aligned", fn);
    return hip_status(ttbfp::launch_gemm_f32(M, N, K, x_dev, w_dev, bias_dev, epilogue, y_dev, (hipStream_t)stream), fn);
}

// ---- host-memory twins (cpu_twins.hip): the same argument checks, no device, no stream ----------------------------

int32_t ttbfp_tilize_pack_cpu(const void *src_host, uint8_t src_fmt, const uint32_t shape[4], const uint64_t strides_bytes[4],
                              uint8_t dst_fmt, int32_t rounding, void *dst_host, uint64_t dst_bytes)
{
    const char *fn = "ttbfp_tilize_pack_cpu";
    if (!raw_pair_ok(src_fmt, dst_fmt)) return fail("%s: an integer format (Int8, UInt16, Int32, RawUInt8, RawUInt16, RawUInt32) pairs with itself only", fn);
    if (int32_t s = check_pack_formats(fn, src_fmt, dst_fmt, rounding)) return s;
    ttbfp::TensorGeom g;
    if (int32_t s = check_geom(fn, shape, strides_bytes, plain_itemsize(src_fmt), g)) return s;
    const uint64_t need = ttbfp_packed_size(dst_fmt, shape);
    if (dst_bytes < need) return fail("%s: destination holds %llu bytes, %llu needed", fn, (unsigned long long)dst_bytes, (unsigned long long)need);
    if (need == 0) return TTBFP_SUCCESS;
    if (!src_host || !dst_host) return fail("%s: NULL pointer", fn);
    return ttbfp::cpu_tilize_pack(src_host, src_fmt, g, dst_fmt, rounding, dst_host) ? TTBFP_SUCCESS : fail("%s: unsupported format pair", fn);
}

int32_t ttbfp_unpack_untilize_cpu(const void *src_host, uint8_t src_fmt, const uint32_t shape[4], uint8_t dst_fmt,
                                  const uint64_t dst_strides_bytes[4], void *dst_host)
{
    const char *fn = "ttbfp_unpack_untilize_cpu";
    if (!raw_pair_ok(src_fmt, dst_fmt)) return fail("%s: an integer format (Int8, UInt16, Int32, RawUInt8, RawUInt16, RawUInt32) pairs with itself only", fn);
    if (int32_t s = check_unpack_formats(fn, src_fmt, dst_fmt)) return s;
    ttbfp::TensorGeom g;
    if (int32_t s = check_geom(fn, shape, dst_strides_bytes, plain_itemsize(dst_fmt), g)) return s;
    if (ttbfp_packed_size(src_fmt, shape) == 0) return TTBFP_SUCCESS;
    if (!src_host || !dst_host) return fail("%s: NULL pointer", fn);
    return ttbfp::cpu_unpack_untilize(src_host, src_fmt, g, dst_fmt, dst_host) ? TTBFP_SUCCESS : fail("%s: unsupported format pair", fn);
}

int32_t ttbfp_gemm_bfp8b_bf16_cpu(uint32_t M, uint32_t N, uint32_t K, const void *x_host, const void *w_host, const void *bias_host,
                                  int32_t epilogue, void *y_host, uint8_t y_fmt)
{
    const char *fn = "ttbfp_gemm_bfp8b_bf16_cpu";
    bool nothing = false;
    if (int32_t s = check_gemm(fn, M, N, K, x_host, w_host, bias_host, epilogue, y_host, y_fmt, nothing)) return s;
    if (nothing) return TTBFP_SUCCESS;
    return ttbfp::cpu_gemm_bfp8b(M, N, K, x_host, w_host, bias_host, epilogue, y_host, y_fmt) ? TTBFP_SUCCESS : fail("%s: failed", fn);
}

uint64_t ttbfp_static_scratch_bytes(void) { return TTBFP_STATIC_SCRATCH_BYTES; }

int32_t ttbfp_gemm_bfp8b_bf16_static(uint32_t M, uint32_t N, uint32_t K, const void *x_dev, const void *w_dev, const void *bias_dev,
                                     int32_t epilogue, void *y_dev, uint8_t y_fmt, void *stream)
{
    const char *fn = "ttbfp_gemm_bfp8b_bf16_static";
    bool nothing = false;
    if (int32_t s = check_gemm(fn, M, N, K, x_dev, w_dev, bias_dev, epilogue, y_dev, y_fmt, nothing)) return s;
    if (nothing) return TTBFP_SUCCESS;
    const uint64_t need = ttbfp_gemm_bfp8b_workspace_bytes(M, N, K);
    if (need > TTBFP_STATIC_SCRATCH_BYTES)
        return fail("%s: M=%u N=%u K=%u needs %llu bytes of scratch, the library's static scratch holds %llu; "
                    "use ttbfp_gemm_bfp8b_bf16 (no scratch) or ttbfp_gemm_bfp8b_bf16_ws with a workspace of the caller's",
                    fn, M, N, K, (unsigned long long)need, (unsigned long long)TTBFP_STATIC_SCRATCH_BYTES);
    if (need == 0)  // the shape gains nothing from scratch memory: the fused kernels, which use none
        return hip_status(ttbfp::launch_gemm_bfp8b(M, N, K, x_dev, w_dev, bias_dev, epilogue, y_dev, y_fmt, (hipStream_t)stream), fn);
    int device = -1;
    if (int32_t s = hip_status(hipGetDevice(&device), "hipGetDevice")) return s;
    void *ws = nullptr;
    if (int32_t s = static_scratch(device, &ws)) return s;
    // Nothing in the scratch has to start at zero: the split-K planes and the panel are written in full by the first
    // kernel before the second one reads them, so what an earlier call left there is never seen.
    return ttbfp_gemm_bfp8b_bf16_ws(M, N, K, x_dev, w_dev, bias_dev, epilogue, y_dev, y_fmt, ws, TTBFP_STATIC_SCRATCH_BYTES, stream);
}

}  // extern "C"
