/*
 * CPU oracle for the block-floating-point data-format path.  TEST INFRASTRUCTURE ONLY.
 *
 * This is a scalar, plain-C restatement of the conversion that TT-Buda's backend performs on
 * push/tilize and get_output.  It exists to check the HIP kernels and to be timed as the CPU
 * baseline.  Nothing in the shipped library links, loads or calls it.
 *
 * What it follows in the reference (paths relative to the reference tree):
 *   - conversion steps 1..9:           docs/public/dataformats.rst:74-83
 *   - block/exponent section pictures: docs/public/images/bfp8_blocks.png, bfp4_blocks.png, bfp2_blocks.png
 *   - enum values and byte-size rule:  pybuda/csrc/lower_to_buda/common.hpp:92-111, common.cpp:167-190
 *   - tile byte sizes:                 pybuda/csrc/balancer/balancer_utils.hpp:24-51
 *   - tile order in queue buffers:     pybuda/csrc/balancer/types.cpp:629-666
 *   - prestriding at push:             pybuda/pybuda/op/eval/pybuda/tm.py:316-335
 *   - golden matmul / gelu:            pybuda/pybuda/op/eval/buda/matmul.py:233-249,
 *                                      pybuda/pybuda/op/eval/pybuda/eltwise_unary.py:42-49
 *
 * The arithmetic itself lives in tenstorrent/tt-budabackend (third_party/budabackend, an empty,
 * un-pinned submodule: .gitmodules:5-8), which is absent.  The reference's own tests hold no byte
 * level vector for this path, so the following choices are PARITY UNPINNED against that backend:
 *   face order inside a tile, default rounding (truncate), sign of zero magnitude (dropped),
 *   treatment of fp32/bf16 denormal inputs (flushed to zero), sub-byte datum order for Bfp4/Bfp2,
 *   fp32 -> Float16_b narrowing (follows the same rounding switch: truncate keeps the upper 16
 *   bits, nearest is round-to-nearest-even); for the family with the 5-bit exponent (Bfp8/Bfp4/Bfp2
 *   from Float16) additionally: the exponent byte holds the 5-bit exponent in its low bits, the
 *   upper bits are ignored on the way back, results beyond the half range become infinity;
 *   for queues with tile headers: the header's place in the tile slot (16 bytes before the data,
 *   16 bytes of padding after) and its content (zeros).
 * The order of tiles inside a queue's buffers IS in the reference (pybuda/csrc/balancer/types.cpp:629-666)
 * and is pinned by the reference's own property test and an independent statement in tests/.
 * Everything else (shared exponent = block maximum, explicit leading one, right shift by the
 * exponent delta, truncation to 7/3/1 bits, exponent section before data section, byte sizes) is
 * pinned by the cited documentation and checked in tests/ against the mathematical definition.
 */
#ifndef TTBFP_ORACLE_H
#define TTBFP_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* DataFormat codes: pybuda/csrc/lower_to_buda/common.hpp:92-111 */
enum {
    ORACLE_FMT_FLOAT32 = 0,
    ORACLE_FMT_FLOAT16 = 1, /* IEEE half: the "A" family, 5-bit exponent */
    ORACLE_FMT_BFP8 = 2,
    ORACLE_FMT_BFP4 = 3,
    ORACLE_FMT_BFP2 = 11,
    ORACLE_FMT_FLOAT16_B = 5,
    ORACLE_FMT_BFP8_B = 6,
    ORACLE_FMT_BFP4_B = 7,
    ORACLE_FMT_BFP2_B = 15,
    /* integer tensors: tiled as they are; an integer format pairs with itself only */
    ORACLE_FMT_INT32 = 8,
    ORACLE_FMT_UINT16 = 12,
    ORACLE_FMT_INT8 = 14,
    ORACLE_FMT_RAW_UINT8 = 0xF0,
    ORACLE_FMT_RAW_UINT16 = 0xF1,
    ORACLE_FMT_RAW_UINT32 = 0xF2,
};

enum { ORACLE_ROUND_TRUNCATE = 0, ORACLE_ROUND_NEAREST = 1 };

/* data_format_byte_size(df, 1024) for one header-less 32x32 tile; 0 for unsupported formats. */
uint32_t oracle_tile_bytes(int fmt);

/* Bytes of a packed [w,z,r,c] tensor (r, c multiples of 32); 0 on bad arguments. */
uint64_t oracle_packed_size(int fmt, const uint32_t shape[4]);

/* Row-major [w,z,r,c] with byte strides -> tile order [w][z][tile_r][tile_c], each tile as four
 * 16x16 faces, element width unchanged (itemsize 2 or 4).  Returns 0 on success. */
int oracle_tilize(const void *src, uint32_t itemsize, const uint32_t shape[4],
                  const uint64_t strides_bytes[4], void *dst);
int oracle_untilize(const void *src, uint32_t itemsize, const uint32_t shape[4],
                    const uint64_t strides_bytes[4], void *dst);

/* One 16-element block: returns the shared exponent and writes 16 datums (sign<<m | magnitude),
 * one per byte, unpacked.  src_bits are fp32 bit patterns. */
uint8_t oracle_quantize_block(const uint32_t src_bits[16], int mant_bits, int rounding,
                              uint8_t datums[16]);

/* fp32 bit pattern of one datum under a shared exponent. */
uint32_t oracle_dequantize_datum(uint8_t datum, uint8_t shared_exp, int mant_bits);

/* The "A" family (docs/public/dataformats.rst:32-41,68): the shared exponent is the 5-bit exponent
 * of Float16 stored in a byte ("5b padded to 8b"), sources and results are IEEE half.  Same steps
 * on the 11-bit significand.  Reading back uses the low five bits of the exponent byte; a result
 * beyond the half range becomes infinity.  PARITY UNPINNED like the rest of the byte layout. */
uint8_t oracle_quantize_block_a(const uint16_t src_half[16], int mant_bits, int rounding, uint8_t datums[16]);
uint16_t oracle_dequantize_datum_a(uint8_t datum, uint8_t shared_exp, int mant_bits);

/* Tiles already in tile-of-faces order (fp32 or bf16 elements; half for the A formats) -> packed tiles. */
int oracle_pack_tiles(const void *tiles, int src_fmt, uint64_t ntiles, int dst_fmt, int rounding,
                      uint8_t *dst);
int oracle_unpack_tiles(const uint8_t *packed, int src_fmt, uint64_t ntiles, int dst_fmt,
                        void *tiles);

/* The two composed conversions the boundary performs.  nthreads > 1 splits tiles over OpenMP
 * threads (used only when timing the all-cores CPU baseline). */
int oracle_tilize_pack(const void *src, int src_fmt, const uint32_t shape[4],
                       const uint64_t strides_bytes[4], int dst_fmt, int rounding, void *dst,
                       int nthreads);
int oracle_unpack_untilize(const void *src, int src_fmt, const uint32_t shape[4], int dst_fmt,
                           const uint64_t dst_strides_bytes[4], void *dst, int nthreads);

/* Queue geometry (tt_dram_io_desc grid / mblock / ublock, pybuda/csrc/backend_api/backend_api.cpp:409-430;
 * ublock_order from the netlist queue line, pybuda/csrc/lower_to_buda/queue.cpp:24-28). */
typedef struct oracle_queue_layout {
    uint32_t grid_r, grid_c, mblock_m, mblock_n, ublock_rt, ublock_ct;
    uint32_t ublock_order; /* 0 = r, 1 = c */
    uint32_t tile_header;  /* 1: 16-byte header + tile + 16 bytes padding per slot (balancer_utils.hpp:24-27) */
} oracle_queue_layout;

/* Canonical tile coordinate (t, r, c) -> (buffer row, buffer column, address in tiles within the
 * buffer's entry) and back: TileLayout::map both ways, pybuda/csrc/balancer/types.cpp:629-666.
 * t_dim is the entry's t.  Pinned in tests/ by the reference's own property (the two maps are
 * inverse for every layout, balancer/tests/test_tile_layout.cpp:248-281) and by an independent
 * reshape/transpose statement of the order. */
int oracle_queue_map(const oracle_queue_layout *l, uint32_t t, uint32_t r, uint32_t c, uint32_t *grid_r,
                     uint32_t *grid_c, uint64_t *address);
int oracle_queue_unmap(const oracle_queue_layout *l, uint32_t grid_r, uint32_t grid_c, uint64_t address,
                       uint32_t *t, uint32_t *r, uint32_t *c);

/* Header-less packed tiles in order [w][t][r/32][c/32] <-> the queue's buffers: buffer (gr, gc) at
 * pitch_bytes * (gr*grid_c + gc), entries one after another inside a buffer.  to_queue writes only
 * the tile slots (headers and padding as zeros); bytes between buffers are left alone.
 * The header position inside a slot (16 bytes before the data) is PARITY UNPINNED. */
int oracle_tiles_to_queue(const uint8_t *tiles, int fmt, const uint32_t shape[4], const oracle_queue_layout *l,
                          uint64_t pitch_bytes, uint8_t *queue);
int oracle_queue_to_tiles(const uint8_t *queue, int fmt, const uint32_t shape[4], const oracle_queue_layout *l,
                          uint64_t pitch_bytes, uint8_t *tiles);

/* Prestriding of a strided convolution's activation, as push_input applies it for a queue whose
 * descriptor carries a stride (pybuda/pybuda/ttdevice.py:1437-1444): the golden op conv2d_prestride_act,
 * pybuda/pybuda/op/eval/pybuda/tm.py:316-335, followed by zero padding of rows and columns to
 * multiples of 32.  src [w, C, H, W] with byte strides -> dst contiguous [w, 1, rows, cols];
 * rows_cols receives the padded sizes.  itemsize 2 or 4.  Returns 0 on success. */
int oracle_prestride(const void *src, uint32_t itemsize, const uint32_t shape[4], const uint64_t strides_bytes[4],
                     uint32_t stride, void *dst, uint32_t rows_cols[2]);

/* The EmbeddingIndex runtime transform (pybuda/pybuda/tensor.py:1382-1408): w index vectors of n elements, of which
 * the first `valid` are real, become the [w, 1, q_rt*32, cols] tensor the embedding queue takes.  The vector is zero-padded
 * to a multiple of 32 and every position from `valid` on is then set to all-ones (`valid` may exceed n: the positions in
 * between stay zero, as in the reference's pad-then-overwrite order), cut into q_rt equal groups (n padded must divide), each
 * group written as rows of 32; with L such rows per group (padded with zero rows to L' = a multiple of 32) element j of
 * row l = 32 a + b of group g lands at out[w, 0, 32 g + b, 32 a + j].  cols = L'.  Returns 0 on success. */
int oracle_embedding_index(const uint32_t *index, uint32_t w, uint32_t n, uint32_t valid, uint32_t q_rt, uint32_t *out,
                           uint32_t *cols);

/* Packed Bfp8_b weight W[K,N] (tiles [K/32][N/32]) -> fp32 row-major [K,N]. */
int oracle_dequant_weight(const uint8_t *w_packed, int w_fmt, uint32_t K, uint32_t N, float *w_out);

/* Y[M,N] = epilogue(X[M,K] (bf16) * dequant(W) + bias), fp32 accumulate in k order, fp32 out.
 * epilogue: 0 none, 1 exact (erf) GELU, 2 tanh-form GELU.  Naive triple loop: small shapes only. */
int oracle_gemm_bfp(uint32_t M, uint32_t N, uint32_t K, const uint16_t *x_bf16,
                    const uint8_t *w_packed, int w_fmt, const uint16_t *bias_bf16, int epilogue,
                    float *y_out);

/* Conversions shared by the tests. */
uint16_t oracle_f32_to_bf16_rne(uint32_t bits);
uint16_t oracle_f32_to_bf16_trunc(uint32_t bits);

#ifdef __cplusplus
}
#endif
#endif
