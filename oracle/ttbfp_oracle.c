/*
 * CPU oracle for the block-floating-point data-format path.  TEST INFRASTRUCTURE ONLY: it checks
 * the HIP kernels and is timed as the CPU baseline; the shipped library never calls it.
 * See ttbfp_oracle.h for the reference files each part follows and for what is parity unpinned.
 */
#include "ttbfp_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#define TILE 32
#define FACE 16
#define TILE_ELEMS 1024
#define EXP_SECTION 64 /* 4 faces x 16 rows, one exponent byte each (bfp8_blocks.png "Exponent 0-3 ...") */

/* ---- format tables: pybuda/csrc/lower_to_buda/common.cpp:167-190 ------------------------------ */

static int mantissa_bits(int fmt)
{
    switch (fmt) {
        case ORACLE_FMT_BFP8_B: case ORACLE_FMT_BFP8: return 7;
        case ORACLE_FMT_BFP4_B: case ORACLE_FMT_BFP4: return 3;
        case ORACLE_FMT_BFP2_B: case ORACLE_FMT_BFP2: return 1;
        default: return 0;
    }
}

/* 1 for the formats with a 5-bit (Float16) exponent */
static int is_a_format(int fmt)
{
    return fmt == ORACLE_FMT_FLOAT16 || fmt == ORACLE_FMT_BFP8 || fmt == ORACLE_FMT_BFP4 || fmt == ORACLE_FMT_BFP2;
}

uint32_t oracle_tile_bytes(int fmt)
{
    switch (fmt) {
        case ORACLE_FMT_FLOAT32: case ORACLE_FMT_RAW_UINT32: case ORACLE_FMT_INT32: return 4 * TILE_ELEMS;
        case ORACLE_FMT_FLOAT16_B: case ORACLE_FMT_FLOAT16: case ORACLE_FMT_RAW_UINT16: case ORACLE_FMT_UINT16: return 2 * TILE_ELEMS;
        case ORACLE_FMT_RAW_UINT8: case ORACLE_FMT_INT8: return TILE_ELEMS;
        case ORACLE_FMT_BFP8_B: case ORACLE_FMT_BFP8: return TILE_ELEMS + TILE_ELEMS / 16;
        case ORACLE_FMT_BFP4_B: case ORACLE_FMT_BFP4: return TILE_ELEMS / 2 + TILE_ELEMS / 16;
        case ORACLE_FMT_BFP2_B: case ORACLE_FMT_BFP2: return TILE_ELEMS / 4 + TILE_ELEMS / 16;
        default: return 0;
    }
}

/* The integer formats (pybuda/csrc/lower_to_buda/common.hpp:92-111, sizes common.cpp:180-186) are tiled without
 * conversion: the 32-bit ones as Float32 bits are, the 16-bit ones as Float16_b bits are, the 8-bit ones as bytes
 * (ORACLE_FMT_RAW_UINT8 stands for both of them below).  An integer format pairs with itself only. */
static int is_integer(int f)
{
    return f == ORACLE_FMT_RAW_UINT8 || f == ORACLE_FMT_RAW_UINT16 || f == ORACLE_FMT_RAW_UINT32 || f == ORACLE_FMT_INT8 ||
           f == ORACLE_FMT_UINT16 || f == ORACLE_FMT_INT32;
}
static int raw_pair(int *a, int *b)
{
    if ((is_integer(*a) || is_integer(*b)) && *a != *b) return 1;
    if (*a == ORACLE_FMT_RAW_UINT32 || *a == ORACLE_FMT_INT32) *a = *b = ORACLE_FMT_FLOAT32;
    if (*a == ORACLE_FMT_RAW_UINT16 || *a == ORACLE_FMT_UINT16) *a = *b = ORACLE_FMT_FLOAT16_B;
    if (*a == ORACLE_FMT_INT8) *a = *b = ORACLE_FMT_RAW_UINT8;
    return 0;
}

static uint32_t plain_itemsize(int fmt)
{
    if (fmt == ORACLE_FMT_FLOAT32 || fmt == ORACLE_FMT_RAW_UINT32 || fmt == ORACLE_FMT_INT32) return 4;
    if (fmt == ORACLE_FMT_FLOAT16_B || fmt == ORACLE_FMT_FLOAT16 || fmt == ORACLE_FMT_RAW_UINT16 || fmt == ORACLE_FMT_UINT16) return 2;
    if (fmt == ORACLE_FMT_RAW_UINT8 || fmt == ORACLE_FMT_INT8) return 1;
    return 0;
}

static int shape_ok(const uint32_t shape[4])
{
    return shape[2] % TILE == 0 && shape[3] % TILE == 0;
}

static uint64_t tile_count(const uint32_t shape[4])
{
    return (uint64_t)shape[0] * shape[1] * (shape[2] / TILE) * (shape[3] / TILE);
}

uint64_t oracle_packed_size(int fmt, const uint32_t shape[4])
{
    if (!shape_ok(shape)) return 0;
    return tile_count(shape) * oracle_tile_bytes(fmt);
}

/* ---- bf16 <-> fp32 bit helpers ---------------------------------------------------------------- */

uint16_t oracle_f32_to_bf16_trunc(uint32_t bits) { return (uint16_t)(bits >> 16); }

uint16_t oracle_f32_to_bf16_rne(uint32_t bits)
{
    if ((bits & 0x7f800000u) == 0x7f800000u && (bits & 0x007fffffu)) /* NaN stays NaN */
        return (uint16_t)((bits >> 16) | 0x0040u);
    uint32_t lsb = (bits >> 16) & 1u;
    return (uint16_t)((bits + 0x7fffu + lsb) >> 16);
}

static float bits_to_float(uint32_t b)
{
    float f;
    memcpy(&f, &b, 4);
    return f;
}

static uint32_t float_to_bits(float f)
{
    uint32_t b;
    memcpy(&b, &f, 4);
    return b;
}

/* ---- tilize / untilize: a pure permutation ----------------------------------------------------- */

/* offset (in elements) of (r, c) inside one tile stored as four 16x16 faces */
static uint32_t in_tile_offset(uint32_t r, uint32_t c)
{
    uint32_t face = (r / FACE) * 2 + (c / FACE);
    return face * FACE * FACE + (r % FACE) * FACE + (c % FACE);
}

static int permute(const uint8_t *rowmajor_in, uint8_t *rowmajor_out, const uint8_t *tiles_in,
                   uint8_t *tiles_out, uint32_t itemsize, const uint32_t shape[4],
                   const uint64_t st[4])
{
    if (!shape_ok(shape) || (itemsize != 2 && itemsize != 4)) return 1;
    uint32_t tr_n = shape[2] / TILE, tc_n = shape[3] / TILE;
    for (uint32_t w = 0; w < shape[0]; ++w)
        for (uint32_t z = 0; z < shape[1]; ++z)
            for (uint32_t r = 0; r < shape[2]; ++r)
                for (uint32_t c = 0; c < shape[3]; ++c) {
                    uint64_t tile = (((uint64_t)w * shape[1] + z) * tr_n + r / TILE) * tc_n + c / TILE;
                    uint64_t t_off = (tile * TILE_ELEMS + in_tile_offset(r % TILE, c % TILE)) * itemsize;
                    uint64_t r_off = w * st[0] + z * st[1] + r * st[2] + c * st[3];
                    if (tiles_out)
                        memcpy(tiles_out + t_off, rowmajor_in + r_off, itemsize);
                    else
                        memcpy(rowmajor_out + r_off, tiles_in + t_off, itemsize);
                }
    return 0;
}

int oracle_tilize(const void *src, uint32_t itemsize, const uint32_t shape[4],
                  const uint64_t strides_bytes[4], void *dst)
{
    return permute((const uint8_t *)src, NULL, NULL, (uint8_t *)dst, itemsize, shape, strides_bytes);
}

int oracle_untilize(const void *src, uint32_t itemsize, const uint32_t shape[4],
                    const uint64_t strides_bytes[4], void *dst)
{
    return permute(NULL, (uint8_t *)dst, (const uint8_t *)src, NULL, itemsize, shape, strides_bytes);
}

/* ---- one 16-element block: docs/public/dataformats.rst:74-83 ------------------------------------ */

uint8_t oracle_quantize_block(const uint32_t src_bits[16], int m, int rounding, uint8_t datums[16])
{
    /* step 3: maximum exponent of the block.  Inputs with a zero exponent field (zeros and
     * denormals) carry no leading one and are treated as zero. */
    uint32_t shared = 0;
    for (int i = 0; i < 16; ++i) {
        uint32_t e = (src_bits[i] >> 23) & 0xffu;
        if (e > shared) shared = e;
    }
    for (int i = 0; i < 16; ++i) {
        uint32_t bits = src_bits[i];
        uint32_t e = (bits >> 23) & 0xffu;
        uint32_t sign = bits >> 31;
        uint32_t mag = 0;
        if (e != 0) {
            uint32_t sig = (bits & 0x007fffffu) | 0x00800000u; /* step 4: explicit leading one, 24 bits */
            uint32_t delta = shared - e;                       /* step 5 */
            sig = delta >= 24 ? 0 : sig >> delta;              /* step 6 */
            if (rounding == ORACLE_ROUND_NEAREST) {            /* step 7, optional rounding */
                sig += 1u << (24 - m - 1);
                mag = sig >> (24 - m);
                if (mag > (1u << m) - 1) mag = (1u << m) - 1;  /* no exponent bump: clamp */
            } else {
                mag = sig >> (24 - m);                         /* step 7: keep the top m bits */
            }
        }
        if (mag == 0) sign = 0; /* a zero magnitude is stored as +0 */
        datums[i] = (uint8_t)((sign << m) | mag);
    }
    return (uint8_t)shared;
}

uint32_t oracle_dequantize_datum(uint8_t datum, uint8_t shared_exp, int m)
{
    uint32_t mag = datum & ((1u << m) - 1);
    uint32_t sign = (datum >> m) & 1u;
    if (mag == 0) return 0;
    int p = 0; /* position of the leading one of the magnitude */
    while ((mag >> (p + 1)) != 0) ++p;
    int e = (int)shared_exp - (m - 1 - p);
    uint32_t bits;
    if (e >= 1)
        bits = ((uint32_t)e << 23) | ((mag << (23 - p)) & 0x007fffffu);
    else
        bits = mag << (shared_exp + 23 - m); /* fp32 denormal: units of 2^-149 */
    return (sign << 31) | bits;
}

/* ---- the same block steps on IEEE half with a 5-bit shared exponent ------------------------------ */

uint8_t oracle_quantize_block_a(const uint16_t h[16], int m, int rounding, uint8_t datums[16])
{
    uint32_t shared = 0;
    for (int i = 0; i < 16; ++i) {
        uint32_t e = (h[i] >> 10) & 0x1fu;
        if (e > shared) shared = e;
    }
    for (int i = 0; i < 16; ++i) {
        uint32_t e = (h[i] >> 10) & 0x1fu;
        uint32_t sign = h[i] >> 15;
        uint32_t mag = 0;
        if (e != 0) { /* zeros and half denormals carry no leading one */
            uint32_t sig = (h[i] & 0x3ffu) | 0x400u; /* explicit leading one, 11 bits */
            uint32_t delta = shared - e;
            sig = delta >= 11 ? 0 : sig >> delta;
            if (rounding == ORACLE_ROUND_NEAREST) {
                sig += 1u << (11 - m - 1);
                mag = sig >> (11 - m);
                if (mag > (1u << m) - 1) mag = (1u << m) - 1;
            } else {
                mag = sig >> (11 - m);
            }
        }
        if (mag == 0) sign = 0;
        datums[i] = (uint8_t)((sign << m) | mag);
    }
    return (uint8_t)shared;
}

uint16_t oracle_dequantize_datum_a(uint8_t datum, uint8_t shared_exp, int m)
{
    uint32_t mag = datum & ((1u << m) - 1);
    uint32_t sign = (datum >> m) & 1u;
    uint32_t E = shared_exp & 0x1fu; /* five bits padded to eight */
    if (mag == 0) return 0;
    int p = 0;
    while ((mag >> (p + 1)) != 0) ++p;
    int e = (int)E - (m - 1 - p); /* value = mag * 2^(E - 15 - (m - 1)) = 1.xxx * 2^(e - 15) */
    uint32_t bits;
    if (e >= 31)
        bits = 0x7c00u; /* beyond the half range */
    else if (e >= 1)
        bits = ((uint32_t)e << 10) | ((mag << (10 - p)) & 0x3ffu);
    else
        bits = mag << (E + 10 - m); /* half denormal: units of 2^-24 */
    return (uint16_t)((sign << 15) | bits);
}

/* ---- packed tile layout -------------------------------------------------------------------------
 * [64 exponent bytes: index face*16 + row][data: face 0..3, each 16 rows of 16 datums]
 * Bfp8: datum j of a row at byte j.  Bfp4: datum 2k in the low nibble of byte k, 2k+1 in the high
 * nibble.  Bfp2: datum 4k+i at bits [2i+1:2i] of byte k. */

static void store_datums(uint8_t *row_out, const uint8_t datums[16], int m)
{
    int bits = m + 1;
    int per_byte = 8 / bits;
    memset(row_out, 0, 16 / per_byte);
    for (int j = 0; j < 16; ++j)
        row_out[j / per_byte] |= (uint8_t)(datums[j] << ((j % per_byte) * bits));
}

static void load_datums(const uint8_t *row_in, uint8_t datums[16], int m)
{
    int bits = m + 1;
    int per_byte = 8 / bits;
    for (int j = 0; j < 16; ++j)
        datums[j] = (row_in[j / per_byte] >> ((j % per_byte) * bits)) & ((1u << bits) - 1);
}

static uint32_t load_elem_bits(const void *tiles, int fmt, uint64_t idx)
{
    if (fmt == ORACLE_FMT_FLOAT32) return ((const uint32_t *)tiles)[idx];
    return (uint32_t)((const uint16_t *)tiles)[idx] << 16;
}

static void pack_one_tile(const void *tile_elems, int src_fmt, uint64_t elem_base, int dst_fmt,
                          int rounding, uint8_t *out)
{
    int m = mantissa_bits(dst_fmt);
    uint32_t row_bytes = 16 * (m + 1) / 8;
    for (int face = 0; face < 4; ++face)
        for (int row = 0; row < FACE; ++row) {
            uint32_t blk[16];
            uint8_t datums[16];
            if (is_a_format(dst_fmt)) {
                const uint16_t *hp = (const uint16_t *)tile_elems + elem_base + face * 256 + row * 16;
                out[face * 16 + row] = oracle_quantize_block_a(hp, m, rounding, datums);
            } else {
                for (int j = 0; j < 16; ++j)
                    blk[j] = load_elem_bits(tile_elems, src_fmt, elem_base + face * 256 + row * 16 + j);
                out[face * 16 + row] = oracle_quantize_block(blk, m, rounding, datums);
            }
            store_datums(out + EXP_SECTION + (face * 16 + row) * row_bytes, datums, m);
        }
}

static void unpack_one_tile(const uint8_t *in, int src_fmt, int dst_fmt, void *tile_elems,
                            uint64_t elem_base)
{
    int m = mantissa_bits(src_fmt);
    uint32_t row_bytes = 16 * (m + 1) / 8;
    for (int face = 0; face < 4; ++face)
        for (int row = 0; row < FACE; ++row) {
            uint8_t datums[16];
            uint8_t shared = in[face * 16 + row];
            load_datums(in + EXP_SECTION + (face * 16 + row) * row_bytes, datums, m);
            for (int j = 0; j < 16; ++j) {
                uint64_t idx = elem_base + face * 256 + row * 16 + j;
                if (is_a_format(src_fmt)) {
                    ((uint16_t *)tile_elems)[idx] = oracle_dequantize_datum_a(datums[j], shared, m);
                    continue;
                }
                uint32_t bits = oracle_dequantize_datum(datums[j], shared, m);
                if (dst_fmt == ORACLE_FMT_FLOAT32)
                    ((uint32_t *)tile_elems)[idx] = bits;
                else
                    ((uint16_t *)tile_elems)[idx] = (uint16_t)(bits >> 16); /* exact: <= 8 significant bits */
            }
        }
}

int oracle_pack_tiles(const void *tiles, int src_fmt, uint64_t ntiles, int dst_fmt, int rounding,
                      uint8_t *dst)
{
    if (!plain_itemsize(src_fmt) || !mantissa_bits(dst_fmt)) return 1;
    if (is_a_format(dst_fmt) != (src_fmt == ORACLE_FMT_FLOAT16)) return 1; /* A formats take half sources only */
    uint32_t tb = oracle_tile_bytes(dst_fmt);
    for (uint64_t t = 0; t < ntiles; ++t)
        pack_one_tile(tiles, src_fmt, t * TILE_ELEMS, dst_fmt, rounding, dst + t * tb);
    return 0;
}

int oracle_unpack_tiles(const uint8_t *packed, int src_fmt, uint64_t ntiles, int dst_fmt, void *tiles)
{
    if (!plain_itemsize(dst_fmt) || !mantissa_bits(src_fmt)) return 1;
    if (is_a_format(src_fmt) != (dst_fmt == ORACLE_FMT_FLOAT16)) return 1; /* A formats read back as half only */
    uint32_t tb = oracle_tile_bytes(src_fmt);
    for (uint64_t t = 0; t < ntiles; ++t)
        unpack_one_tile(packed + t * tb, src_fmt, dst_fmt, tiles, t * TILE_ELEMS);
    return 0;
}

/* ---- composed conversions (what push/tilize and get_output do) ---------------------------------- */

/* plain (non-Bfp) destination element from a source element */
static void convert_plain(uint32_t src_bits_f32, int dst_fmt, int rounding, void *dst, uint64_t idx)
{
    if (dst_fmt == ORACLE_FMT_FLOAT16) /* half to half: load_elem_bits left the 16 bits in the upper half */
        ((uint16_t *)dst)[idx] = (uint16_t)(src_bits_f32 >> 16);
    else if (dst_fmt == ORACLE_FMT_FLOAT32)
        ((uint32_t *)dst)[idx] = src_bits_f32;
    else
        ((uint16_t *)dst)[idx] = rounding == ORACLE_ROUND_NEAREST ? oracle_f32_to_bf16_rne(src_bits_f32)
                                                                  : oracle_f32_to_bf16_trunc(src_bits_f32);
}

int oracle_tilize_pack(const void *src, int src_fmt, const uint32_t shape[4],
                       const uint64_t st[4], int dst_fmt, int rounding, void *dst, int nthreads)
{
    if (raw_pair(&src_fmt, &dst_fmt)) return 1;
    uint32_t isz = plain_itemsize(src_fmt);
    uint32_t tb = oracle_tile_bytes(dst_fmt);
    if (!isz || !tb || !shape_ok(shape)) return 1;
    if (is_a_format(dst_fmt) != (src_fmt == ORACLE_FMT_FLOAT16)) return 1; /* half sources feed the A formats, nothing else */
    uint32_t tr_n = shape[2] / TILE, tc_n = shape[3] / TILE;
    int64_t bands = (int64_t)shape[0] * shape[1] * tr_n;
    int is_bfp = mantissa_bits(dst_fmt) != 0;
    (void)nthreads;
#pragma omp parallel for num_threads(nthreads > 1 ? nthreads : 1) schedule(static)
    for (int64_t band = 0; band < bands; ++band) {
        uint32_t tr = (uint32_t)(band % tr_n);
        uint32_t z = (uint32_t)((band / tr_n) % shape[1]);
        uint32_t w = (uint32_t)(band / tr_n / shape[1]);
        uint8_t gathered[TILE_ELEMS * 4];
        for (uint32_t tc = 0; tc < tc_n; ++tc) {
            /* gather one tile into face order, element width kept */
            for (uint32_t r = 0; r < TILE; ++r)
                for (uint32_t c = 0; c < TILE; ++c) {
                    const uint8_t *p = (const uint8_t *)src + w * st[0] + z * st[1] +
                                       (uint64_t)(tr * TILE + r) * st[2] + (uint64_t)(tc * TILE + c) * st[3];
                    memcpy(gathered + (size_t)in_tile_offset(r, c) * isz, p, isz);
                }
            uint64_t tile = (uint64_t)band * tc_n + tc;
            if (is_bfp) {
                pack_one_tile(gathered, src_fmt, 0, dst_fmt, rounding, (uint8_t *)dst + tile * tb);
            } else if (isz == 1) { /* bytes: the permutation is all there is */
                memcpy((uint8_t *)dst + tile * tb, gathered, TILE_ELEMS);
            } else {
                for (uint32_t i = 0; i < TILE_ELEMS; ++i)
                    convert_plain(load_elem_bits(gathered, src_fmt, i), dst_fmt, rounding, dst,
                                  tile * TILE_ELEMS + i);
            }
        }
    }
    return 0;
}

int oracle_unpack_untilize(const void *src, int src_fmt, const uint32_t shape[4], int dst_fmt,
                           const uint64_t st[4], void *dst, int nthreads)
{
    if (raw_pair(&src_fmt, &dst_fmt)) return 1;
    uint32_t isz = plain_itemsize(dst_fmt);
    uint32_t tb = oracle_tile_bytes(src_fmt);
    if (!isz || !tb || !shape_ok(shape)) return 1;
    /* a Float32 queue read back as Float16_b would need a narrowing rule: not part of this path */
    if (src_fmt == ORACLE_FMT_FLOAT32 && dst_fmt != ORACLE_FMT_FLOAT32) return 1;
    if (is_a_format(src_fmt) != (dst_fmt == ORACLE_FMT_FLOAT16)) return 1;
    uint32_t tr_n = shape[2] / TILE, tc_n = shape[3] / TILE;
    int64_t bands = (int64_t)shape[0] * shape[1] * tr_n;
    int is_bfp = mantissa_bits(src_fmt) != 0;
    (void)nthreads;
#pragma omp parallel for num_threads(nthreads > 1 ? nthreads : 1) schedule(static)
    for (int64_t band = 0; band < bands; ++band) {
        uint32_t tr = (uint32_t)(band % tr_n);
        uint32_t z = (uint32_t)((band / tr_n) % shape[1]);
        uint32_t w = (uint32_t)(band / tr_n / shape[1]);
        uint8_t elems[TILE_ELEMS * 4];
        for (uint32_t tc = 0; tc < tc_n; ++tc) {
            uint64_t tile = (uint64_t)band * tc_n + tc;
            if (is_bfp) {
                unpack_one_tile((const uint8_t *)src + tile * tb, src_fmt, dst_fmt, elems, 0);
            } else if (isz == 1) {
                memcpy(elems, (const uint8_t *)src + tile * tb, TILE_ELEMS);
            } else {
                for (uint32_t i = 0; i < TILE_ELEMS; ++i)
                    convert_plain(load_elem_bits(src, src_fmt, tile * TILE_ELEMS + i), dst_fmt,
                                  ORACLE_ROUND_TRUNCATE, elems, i); /* widening or same width: exact */
            }
            for (uint32_t r = 0; r < TILE; ++r)
                for (uint32_t c = 0; c < TILE; ++c) {
                    uint8_t *p = (uint8_t *)dst + w * st[0] + z * st[1] +
                                 (uint64_t)(tr * TILE + r) * st[2] + (uint64_t)(tc * TILE + c) * st[3];
                    memcpy(p, elems + (size_t)in_tile_offset(r, c) * isz, isz);
                }
        }
    }
    return 0;
}

/* ---- dequantize-then-GEMM: pybuda/pybuda/op/eval/buda/matmul.py:233-249 ------------------------- */

/* ------------------------------------------------------------------------------------------------
 * queue geometry: pybuda/csrc/balancer/types.cpp:629-666
 * ---------------------------------------------------------------------------------------------- */

static int layout_ok(const oracle_queue_layout *l)
{
    return l && l->grid_r && l->grid_c && l->mblock_m && l->mblock_n && l->ublock_rt && l->ublock_ct && l->ublock_order <= 1;
}

int oracle_queue_map(const oracle_queue_layout *l, uint32_t t, uint32_t r, uint32_t c, uint32_t *grid_r, uint32_t *grid_c,
                     uint64_t *address)
{
    if (!layout_ok(l)) return -1;
    const uint32_t rows_per_buffer = l->mblock_m * l->ublock_rt, cols_per_buffer = l->mblock_n * l->ublock_ct;
    if (r >= l->grid_r * rows_per_buffer || c >= l->grid_c * cols_per_buffer) return -1;
    *grid_r = r / rows_per_buffer;
    *grid_c = c / cols_per_buffer;
    /* position of the micro block inside the macro block, and of the tile inside the micro block */
    const uint32_t m = (r / l->ublock_rt) % l->mblock_m, n = (c / l->ublock_ct) % l->mblock_n;
    const uint32_t in_r = r % l->ublock_rt, in_c = c % l->ublock_ct;
    const uint64_t per_ublock = (uint64_t)l->ublock_rt * l->ublock_ct;
    const uint64_t per_mblock = per_ublock * l->mblock_m * l->mblock_n;
    const uint64_t ublocks_before = l->ublock_order == 0 ? (uint64_t)m * l->mblock_n + n : (uint64_t)n * l->mblock_m + m;
    *address = (uint64_t)t * per_mblock + ublocks_before * per_ublock + (uint64_t)in_r * l->ublock_ct + in_c;
    return 0;
}

int oracle_queue_unmap(const oracle_queue_layout *l, uint32_t grid_r, uint32_t grid_c, uint64_t address, uint32_t *t,
                       uint32_t *r, uint32_t *c)
{
    if (!layout_ok(l) || grid_r >= l->grid_r || grid_c >= l->grid_c) return -1;
    const uint64_t per_ublock = (uint64_t)l->ublock_rt * l->ublock_ct;
    const uint64_t per_mblock = per_ublock * l->mblock_m * l->mblock_n;
    *t = (uint32_t)(address / per_mblock);
    const uint64_t in_mblock = address % per_mblock;
    const uint64_t ublock = in_mblock / per_ublock, in_ublock = in_mblock % per_ublock;
    const uint32_t m = l->ublock_order == 0 ? (uint32_t)(ublock / l->mblock_n) : (uint32_t)(ublock % l->mblock_m);
    const uint32_t n = l->ublock_order == 0 ? (uint32_t)(ublock % l->mblock_n) : (uint32_t)(ublock / l->mblock_m);
    *r = (grid_r * l->mblock_m + m) * l->ublock_rt + (uint32_t)(in_ublock / l->ublock_ct);
    *c = (grid_c * l->mblock_n + n) * l->ublock_ct + (uint32_t)(in_ublock % l->ublock_ct);
    return 0;
}

static int queue_copy(const uint8_t *tiles_in, uint8_t *tiles_out, const uint8_t *queue_in, uint8_t *queue_out, int fmt,
                      const uint32_t shape[4], const oracle_queue_layout *l, uint64_t pitch)
{
    const uint32_t tb = oracle_tile_bytes(fmt);
    if (!tb || !shape_ok(shape) || !layout_ok(l)) return -1;
    const uint32_t rt = shape[2] / 32, ct = shape[3] / 32;
    if (rt != l->grid_r * l->mblock_m * l->ublock_rt || ct != l->grid_c * l->mblock_n * l->ublock_ct) return -1;
    const uint64_t slot = tb + (l->tile_header ? 32u : 0u), before = l->tile_header ? 16u : 0u;
    const uint64_t entry_tiles = (uint64_t)shape[1] * l->mblock_m * l->mblock_n * l->ublock_rt * l->ublock_ct;
    uint64_t tile = 0;
    for (uint32_t w = 0; w < shape[0]; ++w)
        for (uint32_t t = 0; t < shape[1]; ++t)
            for (uint32_t r = 0; r < rt; ++r)
                for (uint32_t c = 0; c < ct; ++c, ++tile) {
                    uint32_t gr, gc;
                    uint64_t address;
                    if (oracle_queue_map(l, t, r, c, &gr, &gc, &address)) return -1;
                    const uint64_t at = (uint64_t)(gr * l->grid_c + gc) * pitch + (w * entry_tiles + address) * slot;
                    if (queue_out) {
                        memset(queue_out + at, 0, slot);
                        memcpy(queue_out + at + before, tiles_in + tile * tb, tb);
                    } else {
                        memcpy(tiles_out + tile * tb, queue_in + at + before, tb);
                    }
                }
    return 0;
}

int oracle_tiles_to_queue(const uint8_t *tiles, int fmt, const uint32_t shape[4], const oracle_queue_layout *l, uint64_t pitch,
                          uint8_t *queue)
{
    return queue_copy(tiles, NULL, NULL, queue, fmt, shape, l, pitch);
}

int oracle_queue_to_tiles(const uint8_t *queue, int fmt, const uint32_t shape[4], const oracle_queue_layout *l, uint64_t pitch,
                          uint8_t *tiles)
{
    return queue_copy(NULL, tiles, queue, NULL, fmt, shape, l, pitch);
}

/* ------------------------------------------------------------------------------------------------
 * prestriding: pybuda/pybuda/op/eval/pybuda/tm.py:316-335
 * ---------------------------------------------------------------------------------------------- */

static uint32_t round_up_32(uint64_t n) { return (uint32_t)((n + 31) / 32 * 32); }

int oracle_prestride(const void *src, uint32_t itemsize, const uint32_t shape[4], const uint64_t st[4], uint32_t stride, void *dst,
                     uint32_t rows_cols[2])
{
    if (!stride || (itemsize != 2 && itemsize != 4)) return -1;
    const uint32_t W = shape[0], C = shape[1], H = shape[2], X = shape[3];
    const uint32_t out_h = (H + stride - 1) / stride, out_w = (X + stride - 1) / stride;  /* the image padded up to the stride */
    const uint32_t rows = round_up_32((uint64_t)stride * stride * C), cols = round_up_32((uint64_t)out_h * out_w);
    rows_cols[0] = rows;
    rows_cols[1] = cols;
    memset(dst, 0, (uint64_t)W * rows * cols * itemsize);
    uint32_t section = 0; /* the sub-images are concatenated along the channel dimension, y outer, x inner */
    for (uint32_t y0 = 0; y0 < stride; ++y0)
        for (uint32_t x0 = 0; x0 < stride; ++x0, ++section)
            for (uint32_t w = 0; w < W; ++w)
                for (uint32_t c = 0; c < C; ++c) {
                    uint32_t flat = 0; /* (out_h, out_w) flattened into the last dimension */
                    for (uint32_t y = y0; y < out_h * stride; y += stride)
                        for (uint32_t x = x0; x < out_w * stride; x += stride, ++flat) {
                            if (y >= H || x >= X) continue; /* the zero padding of the image */
                            const uint8_t *from = (const uint8_t *)src + w * st[0] + c * st[1] + (uint64_t)y * st[2] + (uint64_t)x * st[3];
                            uint8_t *to = (uint8_t *)dst + (((uint64_t)w * rows + section * C + c) * cols + flat) * itemsize;
                            memcpy(to, from, itemsize);
                        }
                }
    return 0;
}

/* ------------------------------------------------------------------------------------------------
 * embedding indices: pybuda/pybuda/tensor.py:1382-1408
 * ---------------------------------------------------------------------------------------------- */

int oracle_embedding_index(const uint32_t *index, uint32_t w, uint32_t n, uint32_t valid, uint32_t q_rt, uint32_t *out, uint32_t *cols)
{
    if (!q_rt) return -1;
    const uint32_t n_pad = (n + 31) / 32 * 32;
    if (n_pad % (q_rt * 32)) return -1;          /* the reference's view(w, q_rt, -1, 32) would fail */
    const uint32_t rows_per_group = n_pad / (q_rt * 32);
    const uint32_t width = (rows_per_group + 31) / 32 * 32; /* L' */
    *cols = width;
    memset(out, 0, (size_t)w * q_rt * 32 * width * 4);
    for (uint32_t iw = 0; iw < w; ++iw)
        for (uint32_t e = 0; e < n_pad; ++e) {
            /* zero padding first, then all-ones from position `valid` on: a vector shorter than `valid` keeps zeros in between */
            const uint32_t value = e >= valid ? 0xffffffffu : e < n ? index[(size_t)iw * n + e] : 0u;
            const uint32_t g = e / (rows_per_group * 32), in_group = e % (rows_per_group * 32);
            const uint32_t l = in_group / 32, j = in_group % 32, a = l / 32, b = l % 32;
            out[((size_t)iw * q_rt * 32 + g * 32 + b) * width + a * 32 + j] = value;
        }
    return 0;
}

int oracle_dequant_weight(const uint8_t *w_packed, int w_fmt, uint32_t K, uint32_t N, float *w_out)
{
    uint32_t shape[4] = {1, 1, K, N};
    uint64_t st[4] = {(uint64_t)K * N * 4, (uint64_t)K * N * 4, (uint64_t)N * 4, 4};
    return oracle_unpack_untilize(w_packed, w_fmt, shape, ORACLE_FMT_FLOAT32, st, w_out, 1);
}

/* exact GELU: pybuda/pybuda/op/eval/pybuda/eltwise_unary.py:42-44 (approximate == "none") */
static float gelu_erf(float x) { return 0.5f * x * (1.0f + erff(x * 0.70710678118654752440f)); }
/* tanh form: eltwise_unary.py:45-47 (approximate == "tanh"), evaluated in double and rounded once */
static float gelu_tanh(float x)
{
    const double v = x;
    return (float)(0.5 * v * (1.0 + tanh(0.79788456080286535588 * (v + 0.044715 * v * v * v))));
}

int oracle_gemm_bfp(uint32_t M, uint32_t N, uint32_t K, const uint16_t *x_bf16,
                    const uint8_t *w_packed, int w_fmt, const uint16_t *bias_bf16, int epilogue,
                    float *y_out)
{
    float *w = (float *)malloc((size_t)K * N * sizeof(float));
    if (!w) return 1;
    if (oracle_dequant_weight(w_packed, w_fmt, K, N, w)) {
        free(w);
        return 1;
    }
    for (uint32_t m = 0; m < M; ++m)
        for (uint32_t n = 0; n < N; ++n) {
            float acc = 0.0f;
            for (uint32_t k = 0; k < K; ++k)
                acc += bits_to_float((uint32_t)x_bf16[(size_t)m * K + k] << 16) * w[(size_t)k * N + n];
            if (bias_bf16) acc += bits_to_float((uint32_t)bias_bf16[n] << 16);
            if (epilogue == 1) acc = gelu_erf(acc);
            if (epilogue == 2) acc = gelu_tanh(acc);
            y_out[(size_t)m * N + n] = acc;
        }
    free(w);
    (void)float_to_bits;
    return 0;
}
