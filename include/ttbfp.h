/*
 * ttbfp.h - C ABI of the MI355X (gfx950) block-floating-point data-format library.
 *
 * This is the boundary a TT-Buda maintainer binds instead of the tensor-conversion half of
 * tt-budabackend: the functions behind pybuda._C.backend_api.{tilize_tensor, push_input,
 * get_output} (pybuda/csrc/backend_api/backend_api.cpp:688-704) reduce to the calls below plus
 * memory plumbing.  Plain pointers and sizes only; every pointer named *_dev is device memory of
 * the current HIP device, `stream` is a hipStream_t passed as void* (NULL = the default stream).
 *
 * Every function that can fail returns a status with the values of BackendStatusCode
 * (pybuda/csrc/backend_api/backend_api.cpp:622-625) and never throws; the text of the last failure
 * on the calling thread is returned by ttbfp_last_error().  The library keeps no mutable global
 * state apart from that thread-local text, so calls may run concurrently from several threads
 * (the reference calls this boundary without the GIL: backend_api.cpp:688-701).
 *
 * Format codes are the numeric values of tt::DataFormat
 * (pybuda/csrc/lower_to_buda/common.hpp:92-111): Float32 = 0, Float16_b = 5, Bfp8_b = 6,
 * Bfp4_b = 7, Bfp2_b = 15, and the family with the 5-bit exponent of IEEE half
 * (docs/public/dataformats.rst:32-41,68): Float16 = 1, Bfp8 = 2, Bfp4 = 3, Bfp2 = 11, whose
 * shared-exponent byte holds the half exponent in its low five bits.
 *
 * Packed layout (header-less tiles, tile order [w][z][r/32][c/32]):
 *   one 32x32 tile = 64 shared-exponent bytes (index face*16 + row) followed by the data of the
 *   four 16x16 faces in order (top-left, top-right, bottom-left, bottom-right), rows of 16 datums;
 *   datum = sign<<m | magnitude with m = 7/3/1; Bfp4: datum 2k in the low nibble of byte k;
 *   Bfp2: datum 4k+i at bits [2i+1:2i] of byte k.  Tile sizes 1088 / 576 / 320 bytes
 *   (pybuda/csrc/lower_to_buda/common.cpp:174-179).  Float32 / Float16_b destinations are plain
 *   tiles of faces, 4096 / 2048 bytes.
 */
#ifndef TTBFP_H
#define TTBFP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* BackendStatusCode: backend_api.cpp:622-625 */
#define TTBFP_SUCCESS 0
#define TTBFP_RUNTIME_ERROR 1
#define TTBFP_TIMEOUT_ERROR 2

/* tt::DataFormat values: common.hpp:92-111 */
#define TTBFP_FMT_FLOAT32 0
#define TTBFP_FMT_FLOAT16_B 5
#define TTBFP_FMT_BFP8_B 6
#define TTBFP_FMT_BFP4_B 7
#define TTBFP_FMT_BFP2_B 15
#define TTBFP_FMT_RAW_UINT32 0xF2 /* integer tensors (embedding indices): tiled as they are, pairs with itself only */

/* Step 7 of the Float->BFP conversion (docs/public/dataformats.rst:81): truncate, or add half a
 * unit of the kept field first and clamp to the largest magnitude. */
#define TTBFP_ROUND_TRUNCATE 0
#define TTBFP_ROUND_NEAREST 1

/* GEMM epilogues: none, or GELU in one of the two forms of pybuda/pybuda/op/eval/pybuda/eltwise_unary.py:42-49:
 * approximate == "none" (erf form) or "tanh" (0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3)))) */
#define TTBFP_EPILOGUE_NONE 0
#define TTBFP_EPILOGUE_GELU 1
#define TTBFP_EPILOGUE_GELU_TANH 2
/* ORed into the epilogue argument: bias_dev holds N fp32 values instead of N bf16 ones.  For the sum over a stack of z
 * weights (the matmul's accumulate attribute, pybuda/pybuda/op/eval/buda/matmul.py:236,306-307), whose bias term z * bias
 * is not a bf16 value in general. */
#define TTBFP_EPILOGUE_BIAS_F32 0x100

/* Text of the last failure on this thread ("" if none). The pointer stays valid until the next
 * failing call on the same thread. */
const char *ttbfp_last_error(void);

/* Makes `device` the calling thread's HIP device and checks that it is a gfx950 part.
 * Replaces the device-open half of tt_backend::initialize (backend_api.cpp:668-669). */
int32_t ttbfp_init(int32_t device);

/* Number of HIP devices visible, or -1 when the runtime reports none. */
int32_t ttbfp_device_count(void);

/* data_format_byte_size(fmt, 1024): bytes of one header-less tile, 0 for an unsupported format
 * (pybuda/csrc/lower_to_buda/common.cpp:167-190, pybuda/csrc/balancer/balancer_utils.hpp:24-51). */
uint32_t ttbfp_tile_bytes(uint8_t fmt);

/* Bytes of a whole [w,z,r,c] tensor stored in `fmt` tiles; 0 if r or c is not a multiple of 32 or
 * the format is unsupported.  The tiles-only part of tt::backend::get_io_size_in_bytes
 * (backend_api.cpp:710-722). */
uint64_t ttbfp_packed_size(uint8_t fmt, const uint32_t shape[4]);

/* ---- memory and streams: the plumbing around the conversions -------------------------------- */

/* Device memory (hipMalloc / hipFree). */
int32_t ttbfp_alloc(uint64_t bytes, void **out_dev);
int32_t ttbfp_free(void *dev);
/* Pinned host memory (hipHostMalloc / hipHostFree): what tilize_tensor / get_output results live in
 * until free_tensor (backend_api.cpp:702-704). */
int32_t ttbfp_host_alloc(uint64_t bytes, void **out_host);
int32_t ttbfp_host_free(void *host);
int32_t ttbfp_memcpy_h2d(void *dst_dev, const void *src_host, uint64_t bytes, void *stream);
int32_t ttbfp_memcpy_d2h(void *dst_host, const void *src_dev, uint64_t bytes, void *stream);
int32_t ttbfp_memcpy_d2d(void *dst_dev, const void *src_dev, uint64_t bytes, void *stream);
/* 1 if `ptr` is device memory of a HIP device, 0 if it is host memory (pinned or pageable).
 * Lets push_input accept a tt_PytorchTensorDesc whose tensor already lives in HBM. */
int32_t ttbfp_pointer_is_device(const void *ptr);
int32_t ttbfp_stream_create(void **out_stream);
int32_t ttbfp_stream_destroy(void *stream);
/* Waits for all work queued on the current device, on any stream.  The host layer calls it before it reads a tensor that
 * already lives in device memory: the stream that produced it is not known at this boundary. */
int32_t ttbfp_device_synchronize(void);
/* Waits at most timeout_s seconds (<= 0: forever); TTBFP_TIMEOUT_ERROR when the work has not
 * finished by then - the status get_output / push_input return on a timeout (backend.py:346-371). */
int32_t ttbfp_stream_synchronize(void *stream, int32_t timeout_s);

/* ---- the hot path --------------------------------------------------------------------------- */

/* Row-major [w,z,r,c] tensor (fp32 = Float32 or bf16 = Float16_b, strides in BYTES as in
 * tt_PytorchTensorDesc, backend_api.cpp:489-560) -> tiles of faces in dst_fmt.  This is the
 * conversion inside tt::backend::tilize_tensor and push_input (backend_api.cpp:688-693, 704).
 * dst_bytes must be at least ttbfp_packed_size(dst_fmt, shape).  Legal pairs: src in
 * {Float32, Float16_b}; dst in {Bfp8_b, Bfp4_b, Bfp2_b, Float32, Float16_b} (a Float16_b source widens exactly into
 * Float32 tiles through the general kernel: the host layer's full-precision mode, not a conversion of the hot path);
 * a Float16 source goes with dst in {Bfp8, Bfp4, Bfp2, Float16} and with nothing else
 * (pybuda/pybuda/device_connector.py:177-201); an integer format goes to tiles of the same format and nothing
 * else, a pure permutation of its elements: RawUInt32 (the queues of embedding indices: device_connector.py:203-225,
 * 270-277) and Int32 (int32 tensors, pybuda/pybuda/tensor.py:667-668) of 4-byte elements, RawUInt16 and UInt16 of 2-byte
 * elements, RawUInt8 and Int8 (int8 tensors, tensor.py:669-670) of single bytes; tile sizes
 * pybuda/csrc/lower_to_buda/common.cpp:180-186. */
int32_t ttbfp_tilize_pack(const void *src_dev, uint8_t src_fmt, const uint32_t shape[4],
                          const uint64_t strides_bytes[4], uint8_t dst_fmt, int32_t rounding,
                          void *dst_dev, uint64_t dst_bytes, void *stream);

/* Tiles in src_fmt -> row-major [w,z,r,c] in dst_fmt (Float32 or Float16_b) with the given byte
 * strides: the conversion inside tt::backend::get_output (backend_api.cpp:700-701).
 * Legal pairs: src in {Bfp8_b, Bfp4_b, Bfp2_b, Float16_b} to either destination;
 * Float32 tiles to Float32 only; src in {Bfp8, Bfp4, Bfp2, Float16} to Float16 only; tiles of an integer format
 * (see ttbfp_tilize_pack) to row-major elements of the same format only. */
int32_t ttbfp_unpack_untilize(const void *src_dev, uint8_t src_fmt, const uint32_t shape[4],
                              uint8_t dst_fmt, const uint64_t dst_strides_bytes[4], void *dst_dev,
                              void *stream);

/* ---- the same conversions into and out of the buffers of a queue ----------------------------- */

/* Geometry of a queue (tt_dram_io_desc: bufq_grid_dim_r/c, mblock_m/n, ublock_rt/ct, t,
 * backend_api.cpp:409-430; ublock_order comes with the netlist's queue line,
 * pybuda/csrc/lower_to_buda/queue.cpp:24-28).  An entry [t, R, C] with R/32 = grid_r*mblock_m*ublock_rt
 * and C/32 = grid_c*mblock_n*ublock_ct tiles is cut over grid_r x grid_c buffers.  Inside a buffer the
 * tiles of an entry follow the order of TileLayout::map (pybuda/csrc/balancer/types.cpp:629-648):
 * t slowest, then the micro blocks row-major (ublock_order 0, "r") or column-major (1, "c") in the
 * macro block, then the tiles of a micro block row-major.  The entries of a [w,t,R,C] tensor follow
 * one another inside each buffer; buffer (gr, gc) starts buffer_pitch_bytes * (gr*grid_c + gc) into
 * the memory.  With tile_header set every tile takes tile_bytes + 32 bytes (tile_size_bytes with
 * header and padding, pybuda/csrc/balancer/balancer_utils.hpp:24-27): a 16-byte header, the tile,
 * 16 bytes of padding; the header's content is the absent backend's and is written as zeros. */
typedef struct ttbfp_queue_layout {
    uint32_t grid_r, grid_c;
    uint32_t mblock_m, mblock_n;
    uint32_t ublock_rt, ublock_ct;
    uint32_t ublock_order; /* 0 = r, 1 = c */
    uint32_t tile_header;  /* 0 = header-less tiles, 1 = header + padding around every tile */
} ttbfp_queue_layout;

/* Bytes one buffer of the grid needs for the shape[0] entries of a [w,t,R,C] tensor; 0 when the
 * format is unsupported or the shape does not match the geometry.  With grid 1x1 this is
 * tt::backend::get_io_size_in_bytes without its queue header (backend_api.cpp:710-722). */
uint64_t ttbfp_queue_buffer_bytes(uint8_t fmt, const uint32_t shape[4], const ttbfp_queue_layout *layout);

/* ttbfp_tilize_pack with the tiles placed in the queue's buffers (what push_input does for a
 * queue with this geometry).  buffer_pitch_bytes must be a multiple of 16 and at least
 * ttbfp_queue_buffer_bytes(); dst_bytes at least grid_r*grid_c*buffer_pitch_bytes.  Legal format
 * pairs as for ttbfp_tilize_pack. */
int32_t ttbfp_tilize_pack_queue(const void *src_dev, uint8_t src_fmt, const uint32_t shape[4],
                                const uint64_t strides_bytes[4], uint8_t dst_fmt, int32_t rounding,
                                const ttbfp_queue_layout *layout, uint64_t buffer_pitch_bytes,
                                void *dst_dev, uint64_t dst_bytes, void *stream);

/* ttbfp_unpack_untilize reading the tiles from the queue's buffers (get_output). */
int32_t ttbfp_unpack_untilize_queue(const void *src_dev, uint8_t src_fmt, const uint32_t shape[4],
                                    const ttbfp_queue_layout *layout, uint64_t buffer_pitch_bytes,
                                    uint8_t dst_fmt, const uint64_t dst_strides_bytes[4], void *dst_dev,
                                    void *stream);

/* The two conversions for a tensor whose rows and columns are not multiples of 32, with the padding and the narrowing
 * that pybuda does on the host around the boundary (pad_pytorch_tensor_to_buda / narrow_buda_tensor_to_pytorch,
 * pybuda/pybuda/tensor.py:805-954; pad_to_buda_shape, pybuda/csrc/tt_torch_device/tt_device.cpp:153-189) done inside the
 * launch instead.  `shape` is the shape of the row-major memory, rows and columns >= 1; the tiles cover it rounded up to
 * multiples of 32 (align_up_tile, tt_device.hpp:205-210).
 *  - ttbfp_tilize_pack_padded: elements past the memory's rows / columns pack as zeros ("constant" mode), or, with
 *    replicate_rows / replicate_cols = 1, as copies of the single row / column ("replicate", legal only for a dimension
 *    of size 1: the tile-broadcast dims of tensor.py:848-856).  layout NULL: header-less tiles in one run as
 *    ttbfp_tilize_pack writes them (buffer_pitch_bytes ignored), else the buffers of a queue as ttbfp_tilize_pack_queue.
 *  - ttbfp_unpack_untilize_narrow: only the shape[2] x shape[3] corner of every slice is written to dst.
 * A shape that is tile aligned gives exactly the unpadded calls. */
int32_t ttbfp_tilize_pack_padded(const void *src_dev, uint8_t src_fmt, const uint32_t shape[4],
                                 const uint64_t strides_bytes[4], uint32_t replicate_rows, uint32_t replicate_cols,
                                 uint8_t dst_fmt, int32_t rounding, const ttbfp_queue_layout *layout,
                                 uint64_t buffer_pitch_bytes, void *dst_dev, uint64_t dst_bytes, void *stream);
int32_t ttbfp_unpack_untilize_narrow(const void *src_dev, uint8_t src_fmt, const uint32_t shape[4],
                                     const ttbfp_queue_layout *layout, uint64_t buffer_pitch_bytes, uint8_t dst_fmt,
                                     const uint64_t dst_strides_bytes[4], void *dst_dev, void *stream);

/* ttbfp_unpack_untilize / _queue / _narrow (layout NULL: header-less tiles in one run; shape need not be tile aligned) for
 * callers that want the library to check both buffers: src_bytes is what src_dev holds, dst_bytes what dst_dev holds.
 * The call fails, before anything is launched, when the tiles of `shape` take more than src_bytes or when the strided
 * result reaches past dst_bytes.  Same conversion as tt::backend::get_output (backend_api.cpp:700-701), whose result
 * tensor the backend sizes itself; here the caller owns the destination, so its size travels with it. */
int32_t ttbfp_unpack_untilize_sized(const void *src_dev, uint64_t src_bytes, uint8_t src_fmt, const uint32_t shape[4],
                                    const ttbfp_queue_layout *layout, uint64_t buffer_pitch_bytes, uint8_t dst_fmt,
                                    const uint64_t dst_strides_bytes[4], void *dst_dev, uint64_t dst_bytes, void *stream);

/* The prestriding transform that push_input applies when the queue descriptor carries a tt::Stride
 * (backend_api.cpp:392-407; set for the activation of a strided convolution by
 * pybuda/pybuda/ttdevice.py:1437-1444 with xy_offsets = [(x, y) for y in range(s) for x in range(s)]).
 * src: [w, C, H, W] of 2- or 4-byte elements, byte strides.  dst: row-major contiguous
 * [w, 1, rows, cols] with rows = s*s*C and cols = ceil(H/s)*ceil(W/s) each rounded up to a multiple
 * of 32: out[w, 0, k*C + ch, i*ceil(W/s) + j] = src[w, ch, i*s + k/s, j*s + k%s], zero past H or W and
 * in the padding - the golden op conv2d_prestride_act (pybuda/pybuda/op/eval/pybuda/tm.py:316-335)
 * followed by the zero padding to tiles.  ttbfp_prestride_shape fills rows_cols[2] and returns the
 * bytes dst needs. */
uint64_t ttbfp_prestride_shape(uint32_t itemsize, const uint32_t shape[4], uint32_t stride, uint32_t rows_cols[2]);
int32_t ttbfp_prestride(const void *src_dev, uint32_t itemsize, const uint32_t shape[4],
                        const uint64_t strides_bytes[4], uint32_t stride, void *dst_dev,
                        uint64_t dst_bytes, void *stream);

/* Y[M,N] = epilogue(X[M,K] * dequant(W)[K,N] + bias[N]) with fp32 accumulation: the device matmul
 * with a Bfp8_b weight operand and Float16_b activations that the golden model evaluates by
 * dequantize-then-matmul (pybuda/pybuda/op/eval/buda/matmul.py:233-249; operand formats chosen by
 * pybuda/csrc/passes/amp.cpp:474-484).
 *   x_dev     bf16 row-major, contiguous, M x K
 *   w_dev     W packed as by ttbfp_tilize_pack of the row-major [1,1,K,N] tensor to Bfp8_b
 *   bias_dev  bf16 [N] (fp32 [N] with TTBFP_EPILOGUE_BIAS_F32) or NULL (the row the reference broadcasts: matmul.py:247-249)
 *   y_dev     row-major, contiguous, M x N in y_fmt (Float16_b: round to nearest even; Float32)
 * M, N and K must be multiples of 32. */
int32_t ttbfp_gemm_bfp8b_bf16(uint32_t M, uint32_t N, uint32_t K, const void *x_dev,
                              const void *w_dev, const void *bias_dev, int32_t epilogue,
                              void *y_dev, uint8_t y_fmt, void *stream);

/* The same GEMM for callers that can lend scratch memory; ttbfp_gemm_bfp8b_workspace_bytes(M, N, K) says how
 * much a shape can use (0: none).  Two shapes of problem gain from it:
 *  - many rows of X (M >= 4096 or 6144 depending on the tile, macro-tile aligned, K a multiple of 64): W is converted to bf16 once
 *    into a panel of 2 K N bytes in the workspace instead of in every workgroup, and the MFMA kernel runs on the
 *    panel; the result is bit-identical to ttbfp_gemm_bfp8b_bf16;
 *  - few macro tiles (M = 128 or 256 <= M, at most 256 tiles of 128 x 128, K a multiple of 64): K is cut into s <= 8 runs, each (tile, run)
 *    workgroup writes an fp32 partial tile into the workspace (s M N 4 bytes) and a second kernel adds the
 *    partials in a fixed order, then applies bias and epilogue.  Deterministic; the sum is grouped differently
 *    from ttbfp_gemm_bfp8b_bf16's, so the two agree to fp32 rounding (about 1e-7 relative), not bit for bit.
 * Otherwise (workspace NULL or smaller than the function says, or a shape for which it returns 0) the call is
 * exactly ttbfp_gemm_bfp8b_bf16.  The workspace must be 16-byte aligned, holds nothing the caller needs
 * afterwards and may be reused as soon as the work queued on `stream` has finished.
 * No counterpart in the reference, whose device converts weights in its unpacker hardware. */
uint64_t ttbfp_gemm_bfp8b_workspace_bytes(uint32_t M, uint32_t N, uint32_t K);
int32_t ttbfp_gemm_bfp8b_bf16_ws(uint32_t M, uint32_t N, uint32_t K, const void *x_dev,
                                 const void *w_dev, const void *bias_dev, int32_t epilogue,
                                 void *y_dev, uint8_t y_fmt, void *workspace_dev,
                                 uint64_t workspace_bytes, void *stream);

/* ttbfp_gemm_bfp8b_bf16_ws with the size of every buffer stated (the golden matmul, pybuda/pybuda/op/eval/buda/matmul.py:233-249,
 * gets its sizes from the tensors themselves; a C caller has to say them): fails before anything is launched when x holds
 * fewer than 2 M K bytes, w fewer than the Bfp8_b tiles of [K, N], the bias (if any) fewer than N values, or y fewer
 * than M N results in y_fmt.  workspace_dev may be NULL. */
int32_t ttbfp_gemm_bfp8b_bf16_sized(uint32_t M, uint32_t N, uint32_t K, const void *x_dev, uint64_t x_bytes,
                                    const void *w_dev, uint64_t w_bytes, const void *bias_dev, uint64_t bias_bytes,
                                    int32_t epilogue, void *y_dev, uint64_t y_bytes, uint8_t y_fmt, void *workspace_dev,
                                    uint64_t workspace_bytes, void *stream);

/* Y[M,N] = epilogue(X[M,K] * W[K,N] + bias[N]), all fp32, row-major, contiguous, any M, N, K > 0; epilogue without
 * TTBFP_EPILOGUE_BIAS_F32 (the bias is always fp32).  The golden matmul (pybuda/pybuda/op/eval/buda/matmul.py:233-249) on
 * unquantized operands: what the backend evaluates when its configuration says ignore_data_format_precision
 * (pybuda/csrc/backend_api/backend_api.cpp:261-275).  Plain fp32 FMAs; a verification path, not a fast one. */
int32_t ttbfp_gemm_f32(uint32_t M, uint32_t N, uint32_t K, const void *x_dev, const void *w_dev,
                       const void *bias_dev, int32_t epilogue, void *y_dev, void *stream);

/* ttbfp_gemm_bfp8b_bf16_ws with the scratch memory held by the library: a file-scope device array of
 * TTBFP_STATIC_SCRATCH_BYTES that every GPU the library runs on keeps until the process ends.  For callers that
 * cannot allocate or lend device memory: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  The call allocates nothing (no hipMalloc / hipFree, no allocating library routine) and only launches
 * kernels on `stream`.  Same kernels, same kernel choice and therefore the same bits as ttbfp_gemm_bfp8b_bf16_ws
 * given a workspace of ttbfp_gemm_bfp8b_workspace_bytes(M, N, K).  A shape whose workspace would exceed
 * TTBFP_STATIC_SCRATCH_BYTES is refused with TTBFP_RUNTIME_ERROR (8192 x 8192 x 8192 wants 128 MiB: use one of the
 * other two entry points); a shape that uses no workspace runs exactly as ttbfp_gemm_bfp8b_bf16.
 * All calls on one GPU share that GPU's array: calls that overlap in time on the same GPU (two streams, two
 * threads) race on it - serialize them.  The array keeps what the last call left; nothing in it needs clearing,
 * each call writes every byte it later reads.  ttbfp_init resolves the array's device address (once per device);
 * without ttbfp_init the first call on a device does.
 * No counterpart in the reference. */
#define TTBFP_STATIC_SCRATCH_BYTES (64ull << 20)
uint64_t ttbfp_static_scratch_bytes(void);
int32_t ttbfp_gemm_bfp8b_bf16_static(uint32_t M, uint32_t N, uint32_t K, const void *x_dev,
                                     const void *w_dev, const void *bias_dev, int32_t epilogue,
                                     void *y_dev, uint8_t y_fmt, void *stream);

/* ---- host-memory twins ---------------------------------------------------------------------------
 * The boundary's contract lists a CPU twin of each conversion.  These run the same datum rules as the kernels (one
 * shared statement, compiled for the host) on tensors in HOST memory, single-threaded, without any device or stream:
 * for a host that has no GPU at hand (packing the weights of a device image on a build machine, checking a queue dump).
 * They are separate entry points and nothing else: no device entry point calls them, and a device entry point
 * without a GPU fails.  Same arguments, checks, legal format pairs and status codes as ttbfp_tilize_pack
 * (backend_api.cpp:688-693, 704), ttbfp_unpack_untilize (backend_api.cpp:700-701) and ttbfp_gemm_bfp8b_bf16
 * (pybuda/pybuda/op/eval/buda/matmul.py:233-249), with results equal bit for bit for the conversions and to fp32
 * rounding for the matmul (sums in k order, erf / tanh of the C library). */
int32_t ttbfp_tilize_pack_cpu(const void *src_host, uint8_t src_fmt, const uint32_t shape[4],
                              const uint64_t strides_bytes[4], uint8_t dst_fmt, int32_t rounding,
                              void *dst_host, uint64_t dst_bytes);
int32_t ttbfp_unpack_untilize_cpu(const void *src_host, uint8_t src_fmt, const uint32_t shape[4],
                                  uint8_t dst_fmt, const uint64_t dst_strides_bytes[4], void *dst_host);
int32_t ttbfp_gemm_bfp8b_bf16_cpu(uint32_t M, uint32_t N, uint32_t K, const void *x_host, const void *w_host,
                                  const void *bias_host, int32_t epilogue, void *y_host, uint8_t y_fmt);

#ifdef __cplusplus
}
#endif
#endif
