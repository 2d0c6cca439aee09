// Host-memory twins of the three conversions: the same arithmetic as the device kernels (the datum rules of bfp_codec.hpp are
// shared, compiled for the host here), on tensors in host memory, with no GPU involved.  For a host without a device at
// hand - packing the weights of a device image on a build machine, checking a queue dump - and for nothing else: no device
// entry point ever calls them, and a device entry point without a GPU fails.  Scalar loops, one thread: they are not
// tuned and not timed.
#include <cmath>
#include <cstring>
#include <vector>

#include "bfp_codec.hpp"
#include "launch.hpp"

namespace ttbfp {

namespace {

// element (w, z, r, c) of a row-major tensor as an fp32 bit pattern (bf16: upper half; half: the pattern the A family computes on)
inline uint32_t load_bits(const uint8_t *p, uint8_t fmt, uint16_t *raw_half)
{
    if (fmt == kFloat32) {
        uint32_t v;
        std::memcpy(&v, p, 4);
        return v;
    }
    uint16_t h;
    std::memcpy(&h, p, 2);
    if (fmt == kFloat16) {
        *raw_half = h;
        return half_to_f32_pattern(h);
    }
    return (uint32_t)h << 16;
}

template <int M, int ROUNDING>
void pack_face_row(const uint32_t bits[16], bool a_family, uint8_t *tile, uint32_t face_row)
{
    uint32_t e = 0;
    for (int j = 0; j < 16; ++j) e = std::max(e, biased_exponent(bits[j]));
    constexpr int ROW_BYTES = 16 * (M + 1) / 8, PER_BYTE = 8 / (M + 1);
    tile[face_row] = (uint8_t)(a_family && e ? e - kHalfExponentRebase : e);
    for (int k = 0; k < ROW_BYTES; ++k) {
        uint32_t byte = 0;
        for (int i = 0; i < PER_BYTE; ++i) byte |= quantize_datum<M, ROUNDING>(bits[k * PER_BYTE + i], e) << (i * (M + 1));
        tile[kExpSection + face_row * ROW_BYTES + k] = (uint8_t)byte;
    }
}

template <int M>
void unpack_face_row(const uint8_t *tile, bool a_family, uint32_t face_row, uint32_t bits[16])
{
    constexpr int ROW_BYTES = 16 * (M + 1) / 8, PER_BYTE = 8 / (M + 1);
    const uint32_t e = a_family ? (tile[face_row] & 0x1fu) + kHalfExponentRebase : tile[face_row];
    for (int j = 0; j < 16; ++j) {
        const uint32_t byte = tile[kExpSection + face_row * ROW_BYTES + j / PER_BYTE];
        bits[j] = dequantize_datum<M>((byte >> ((j % PER_BYTE) * (M + 1))) & ((2u << M) - 1u), e);
    }
}

// position of (face row, j) of tile (tr, tc) in the row-major tensor
inline uint64_t element_offset(const TensorGeom &g, uint32_t w, uint32_t z, uint32_t tr, uint32_t tc, uint32_t face_row, uint32_t j)
{
    const uint32_t face = face_row / kFace, row = face_row % kFace;
    const uint32_t r = tr * kTile + (face / 2) * kFace + row, c = tc * kTile + (face % 2) * kFace + j;
    return w * g.s0 + z * g.s1 + (uint64_t)r * g.s2 + (uint64_t)c * g.s3;
}

}  // namespace

bool cpu_tilize_pack(const void *src, uint8_t src_fmt, const TensorGeom &g, uint8_t dst_fmt, int rounding, void *dst)
{
    const uint32_t tiles_r = g.R / kTile, tiles_c = g.C / kTile, TB = tile_bytes(dst_fmt);
    const int m = mantissa_bits(dst_fmt);
    const bool a_family = is_a_format(dst_fmt);
    uint64_t tile = 0;
    for (uint32_t w = 0; w < g.W; ++w)
        for (uint32_t z = 0; z < g.Z; ++z)
            for (uint32_t tr = 0; tr < tiles_r; ++tr)
                for (uint32_t tc = 0; tc < tiles_c; ++tc, ++tile) {
                    uint8_t *out = (uint8_t *)dst + tile * TB;
                    for (uint32_t face_row = 0; face_row < 64; ++face_row) {
                        if (src_fmt == kRaw8) {  // bytes as they are
                            for (uint32_t j = 0; j < 16; ++j) out[face_row * 16 + j] = ((const uint8_t *)src)[element_offset(g, w, z, tr, tc, face_row, j)];
                            continue;
                        }
                        uint32_t bits[16];
                        uint16_t raw[16] = {};
                        for (uint32_t j = 0; j < 16; ++j)
                            bits[j] = load_bits((const uint8_t *)src + element_offset(g, w, z, tr, tc, face_row, j), src_fmt, &raw[j]);
                        if (m == 7)
                            rounding ? pack_face_row<7, 1>(bits, a_family, out, face_row) : pack_face_row<7, 0>(bits, a_family, out, face_row);
                        else if (m == 3)
                            rounding ? pack_face_row<3, 1>(bits, a_family, out, face_row) : pack_face_row<3, 0>(bits, a_family, out, face_row);
                        else if (m == 1)
                            rounding ? pack_face_row<1, 1>(bits, a_family, out, face_row) : pack_face_row<1, 0>(bits, a_family, out, face_row);
                        else if (dst_fmt == kFloat32)
                            std::memcpy(out + face_row * 64, bits, 64);
                        else
                            for (uint32_t j = 0; j < 16; ++j) {
                                const uint16_t v = dst_fmt == kFloat16                  ? raw[j]
                                                   : rounding && src_fmt == kFloat32 ? f32_to_bf16_rne(bits[j])
                                                                                     : (uint16_t)(bits[j] >> 16);
                                std::memcpy(out + (face_row * 16 + j) * 2, &v, 2);
                            }
                    }
                }
    return true;
}

bool cpu_unpack_untilize(const void *src, uint8_t src_fmt, const TensorGeom &g, uint8_t dst_fmt, void *dst)
{
    const uint32_t tiles_r = g.R / kTile, tiles_c = g.C / kTile, TB = tile_bytes(src_fmt);
    const int m = mantissa_bits(src_fmt);
    const bool a_family = is_a_format(src_fmt);
    uint64_t tile = 0;
    for (uint32_t w = 0; w < g.W; ++w)
        for (uint32_t z = 0; z < g.Z; ++z)
            for (uint32_t tr = 0; tr < tiles_r; ++tr)
                for (uint32_t tc = 0; tc < tiles_c; ++tc, ++tile) {
                    const uint8_t *in = (const uint8_t *)src + tile * TB;
                    for (uint32_t face_row = 0; face_row < 64; ++face_row) {
                        uint32_t bits[16];
                        if (m == 7)
                            unpack_face_row<7>(in, a_family, face_row, bits);
                        else if (m == 3)
                            unpack_face_row<3>(in, a_family, face_row, bits);
                        else if (m == 1)
                            unpack_face_row<1>(in, a_family, face_row, bits);
                        for (uint32_t j = 0; j < 16; ++j) {
                            uint8_t *p = (uint8_t *)dst + element_offset(g, w, z, tr, tc, face_row, j);
                            if (src_fmt == kRaw8) {
                                *p = in[face_row * 16 + j];
                            } else if (m == 0 && src_fmt == kFloat32) {
                                std::memcpy(p, in + (face_row * 16 + j) * 4, 4);
                            } else if (m == 0) {  // Float16_b or Float16 tiles
                                uint16_t v;
                                std::memcpy(&v, in + (face_row * 16 + j) * 2, 2);
                                if (dst_fmt == kFloat32) {
                                    const uint32_t wide = (uint32_t)v << 16;
                                    std::memcpy(p, &wide, 4);
                                } else {
                                    std::memcpy(p, &v, 2);
                                }
                            } else if (dst_fmt == kFloat32) {
                                std::memcpy(p, &bits[j], 4);
                            } else {
                                const uint16_t v = dst_fmt == kFloat16 ? (uint16_t)f32_pattern_to_half(bits[j]) : (uint16_t)(bits[j] >> 16);
                                std::memcpy(p, &v, 2);
                            }
                        }
                    }
                }
    return true;
}

// Y = activation(X W + bias): W dequantized into fp32 once, then row by row with fp32 sums in k order
bool cpu_gemm_bfp8b(uint32_t M, uint32_t N, uint32_t K, const void *x, const void *w, const void *bias, int epilogue, void *y, uint8_t y_fmt)
{
    std::vector<float> wd((size_t)K * N);
    const TensorGeom gw{1, 1, K, N, (uint64_t)K * N * 4, (uint64_t)K * N * 4, (uint64_t)N * 4, 4, K, N, 0, 0};
    cpu_unpack_untilize(w, kBfp8_b, gw, kFloat32, wd.data());
    std::vector<float> row(N);
    const uint16_t *xb = (const uint16_t *)x;
    for (uint32_t m = 0; m < M; ++m) {
        std::fill(row.begin(), row.end(), 0.0f);
        for (uint32_t k = 0; k < K; ++k) {
            const float xv = __builtin_bit_cast(float, (uint32_t)xb[(size_t)m * K + k] << 16);
            const float *wr = wd.data() + (size_t)k * N;
            for (uint32_t n = 0; n < N; ++n) row[n] += xv * wr[n];
        }
        for (uint32_t n = 0; n < N; ++n) {
            float v = row[n];
            if (bias)
                v += (epilogue & kEpilogueBiasF32) ? ((const float *)bias)[n] : __builtin_bit_cast(float, (uint32_t)((const uint16_t *)bias)[n] << 16);
            const int act = epilogue & kEpilogueMask;
            if (act == 1) v = 0.5f * v * (1.0f + std::erf(v * 0.70710678118654752440f));
            if (act == 2) v = 0.5f * v * (1.0f + std::tanh(0.7978845608028654f * (v + 0.044715f * v * v * v)));
            if (y_fmt == kFloat32)
                ((float *)y)[(size_t)m * N + n] = v;
            else
                ((uint16_t *)y)[(size_t)m * N + n] = f32_to_bf16_rne(__builtin_bit_cast(uint32_t, v));
        }
    }
    return true;
}

}  // namespace ttbfp
