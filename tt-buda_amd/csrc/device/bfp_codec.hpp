// Device-side building blocks of the Bfp*_b codec, shared by the pack, unpack and GEMM kernels.
// The conversion is steps 3-7 of docs/public/dataformats.rst:74-83 on fp32 bit patterns; a bf16
// source is widened by a 16-bit shift, which changes nothing since bf16 is the upper half of fp32.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ttbfp {

constexpr int kTile = 32;
constexpr int kFace = 16;
constexpr int kTileElems = 1024;
constexpr int kExpSection = 64;  // 4 faces x 16 rows, one shared exponent byte each

// DataFormat codes (pybuda/csrc/lower_to_buda/common.hpp:92-111)
constexpr uint8_t kFloat32 = 0, kFloat16_b = 5, kBfp8_b = 6, kBfp4_b = 7, kBfp2_b = 15;
// the "A" family: 5-bit exponent of IEEE half, shared exponent byte = that exponent padded to 8 bits
// (docs/public/dataformats.rst:32-41,68)
constexpr uint8_t kFloat16 = 1, kBfp8 = 2, kBfp4 = 3, kBfp2 = 11;
// One-byte elements tiled as they are (Int8 and RawUInt8 queues): a tile is 1024 bytes, a face row 16 of them.  The 16-bit
// and 32-bit integer formats need no code of their own: the Float16_b -> Float16_b and Float32 -> Float32 kernels move
// bits without looking at them.
constexpr uint8_t kRaw8 = 0xF0;

__host__ __device__ constexpr int mantissa_bits(uint8_t fmt)
{
    return (fmt == kBfp8_b || fmt == kBfp8) ? 7 : (fmt == kBfp4_b || fmt == kBfp4) ? 3 : (fmt == kBfp2_b || fmt == kBfp2) ? 1 : 0;
}

__host__ __device__ constexpr bool is_a_format(uint8_t fmt)
{
    return fmt == kFloat16 || fmt == kBfp8 || fmt == kBfp4 || fmt == kBfp2;
}

// An IEEE half travelling through the kernels (a distinct type so that it is not taken for bf16).
struct half_t {
    uint16_t bits;
};

// The A family is computed on the fp32 pattern of the half: an exponent field e becomes e + 112 (31,
// Inf/NaN, becomes 143 on purpose: the shared exponent is the plain maximum of the 5-bit fields) and
// a zero field (zeros, half denormals) gives a signed zero, so the shared-exponent byte is the fp32
// block exponent minus 112 and the magnitudes are those of the 11-bit significand.
constexpr uint32_t kHalfExponentRebase = 112;
__host__ __device__ __forceinline__ uint32_t half_to_f32_pattern(uint32_t h)
{
    const uint32_t e = (h >> 10) & 0x1fu;
    return ((h & 0x8000u) << 16) | (e ? ((e + kHalfExponentRebase) << 23) | ((h & 0x3ffu) << 13) : 0u);
}
// exact for every value the A family produces; beyond the half range the result is infinity
__host__ __device__ __forceinline__ uint32_t f32_pattern_to_half(uint32_t f32_bits)
{
    return __builtin_bit_cast(uint16_t, (_Float16)__builtin_bit_cast(float, f32_bits));
}

// data_format_byte_size(fmt, 1024): pybuda/csrc/lower_to_buda/common.cpp:167-190
__host__ __device__ constexpr uint32_t tile_bytes(uint8_t fmt)
{
    return fmt == kFloat32     ? 4096u
           : fmt == kRaw8      ? 1024u
           : fmt == kFloat16_b ? 2048u
           : fmt == kFloat16   ? 2048u
           : mantissa_bits(fmt) == 7 ? 1024u + 64u
           : mantissa_bits(fmt) == 3 ? 512u + 64u
           : mantissa_bits(fmt) == 1 ? 256u + 64u
                                     : 0u;
}

// 128-bit global accesses with the non-temporal hint: every byte of these tensors is touched once,
// so it should stream past the caches instead of displacing lines.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

// Dynamic LDS bytes that, added to a kernel's `static_bytes`, leave room for `resident` workgroups per CU (160 KiB of LDS)
// and no more: the streaming kernels run faster with fewer workgroups in flight than their own LDS and registers allow
// (fewer concurrent streams into HBM), and unused LDS is the handle on that number.
inline uint32_t resident_cap_bytes(uint32_t static_bytes, uint32_t resident)
{
    const uint32_t share = 160u * 1024u / resident;
    const uint32_t dynamic = share > static_bytes + 1024u ? (share - static_bytes - 1024u) & ~255u : 0u;
    return static_bytes + dynamic > 64u * 1024u ? 64u * 1024u - ((static_bytes + 255u) & ~255u) : dynamic;  // stay within the default limit
}

__device__ __forceinline__ uint4 load_stream(const void *p)
{
    const u32x4_t v = __builtin_nontemporal_load((const u32x4_t *)p);
    return make_uint4(v.x, v.y, v.z, v.w);
}

__device__ __forceinline__ void store_stream(void *p, const uint4 &v)
{
    const u32x4_t t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, (u32x4_t *)p);
}

// The same 16-byte accesses at an address that is only known to be a multiple of ALIGN (the element size of a row-major
// tensor: a sliced view starts anywhere).  The device's memory path takes such accesses as they are (the hardware runs
// in its unaligned mode under this runtime), so the instruction is the same global_load/store_dwordx4; the type only
// keeps the compiler from assuming more alignment than there is.  A wavefront's 1 KiB then touches nine lines instead
// of eight.
template <int ALIGN>
struct UnderAligned;
template <>
struct UnderAligned<2> {
    typedef u32x4_t type __attribute__((aligned(2)));
};
template <>
struct UnderAligned<4> {
    typedef u32x4_t type __attribute__((aligned(4)));
};
template <int ALIGN>
__device__ __forceinline__ uint4 load_stream_at(const void *p)
{
    const u32x4_t v = __builtin_nontemporal_load((const typename UnderAligned<ALIGN>::type *)p);
    return make_uint4(v.x, v.y, v.z, v.w);
}
template <int ALIGN>
__device__ __forceinline__ void store_stream_at(void *p, const uint4 &v)
{
    const u32x4_t t = {v.x, v.y, v.z, v.w};
    __builtin_nontemporal_store(t, (typename UnderAligned<ALIGN>::type *)p);
}

__host__ __device__ __forceinline__ uint32_t biased_exponent(uint32_t f32_bits) { return (f32_bits >> 23) & 0xffu; }

// One datum (sign << M | magnitude) of an fp32 bit pattern under the block's shared exponent.
// Inputs with a zero exponent field have no leading one and quantize to zero; a zero magnitude is
// stored without its sign.
template <int M, int ROUNDING>
__host__ __device__ __forceinline__ uint32_t quantize_datum(uint32_t bits, uint32_t shared_exp)
{
    const uint32_t e = biased_exponent(bits);
    uint32_t sig = (bits & 0x007fffffu) | 0x00800000u;  // explicit leading one: 24 bits
    uint32_t delta = shared_exp - e;
    delta = delta > 31u ? 31u : delta;  // 24-bit value: any shift >= 24 clears it
    sig = e == 0u ? 0u : sig >> delta;
    uint32_t mag;
    if (ROUNDING) {
        sig += 1u << (23 - M);
        mag = sig >> (24 - M);
        mag = mag > (1u << M) - 1u ? (1u << M) - 1u : mag;
    } else {
        mag = sig >> (24 - M);
    }
    const uint32_t sign = (bits >> 31) << M;
    return mag ? (sign | mag) : 0u;
}

// fp32 bit pattern of a datum: (-1)^s * mag * 2^(E - 127 - (M - 1)), exact (denormals included).
template <int M>
__host__ __device__ __forceinline__ uint32_t dequantize_datum(uint32_t datum, uint32_t shared_exp)
{
    const uint32_t mag = datum & ((1u << M) - 1u);
    const int p = 31 - __builtin_clz(mag ? mag : 1u);  // leading one of the magnitude (unused when mag == 0)
    const int e = (int)shared_exp - (M - 1 - p);
    const uint32_t normal = ((uint32_t)e << 23) | ((mag << (23 - p)) & 0x007fffffu);
    const uint32_t denorm = mag << (shared_exp + 23 - M);
    uint32_t bits = e >= 1 ? normal : denorm;
    bits |= (datum >> M) << 31;
    return mag ? bits : 0u;
}

// max over the `LANES` (2 or 4) neighbouring lanes that share one 16-datum block, by DPP quad
// permutes (no LDS traffic).
template <int LANES>
__device__ __forceinline__ uint32_t block_max(uint32_t v)
{
    static_assert(LANES == 2 || LANES == 4, "a block spans 2 or 4 lanes");
    uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
    v = v > o ? v : o;
    if (LANES == 4) {
        o = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
        v = v > o ? v : o;
    }
    return v;
}

// ---- lean bf16 <-> Bfp8_b paths -------------------------------------------------------------------
// Two bf16 travel in one 32-bit word, so exponent extraction, the hidden one, the delta, the shift
// and the sign handling are done on both halves at once with packed 16-bit VALU operations.

typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b)
{
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2, a), __builtin_bit_cast(u16x2, b)));
}
__device__ __forceinline__ uint32_t pk_min_u16(uint32_t a, uint32_t b)
{
    return __builtin_bit_cast(uint32_t, __builtin_elementwise_min(__builtin_bit_cast(u16x2, a), __builtin_bit_cast(u16x2, b)));
}
__device__ __forceinline__ uint32_t pk_shr_u16(uint32_t v, uint32_t sh)
{
    return __builtin_bit_cast(uint32_t, __builtin_bit_cast(u16x2, v) >> __builtin_bit_cast(u16x2, sh));
}

// biased exponents of the two bf16 in a word, one per 16-bit half
__device__ __forceinline__ uint32_t bf16_pair_exponents(uint32_t w) { return (w >> 7) & 0x00ff00ffu; }

// max biased exponent of the 8 bf16 in a 16-byte chunk
__device__ __forceinline__ uint32_t bf16_chunk_max_exponent(const uint4 &v)
{
    const uint32_t m = pk_max_u16(pk_max_u16(bf16_pair_exponents(v.x), bf16_pair_exponents(v.y)),
                                  pk_max_u16(bf16_pair_exponents(v.z), bf16_pair_exponents(v.w)));
    return max(m & 0xffffu, m >> 16);
}

// Two Bfp8_b datums (truncation) of the two bf16 in `w`, one per 16-bit half, under shared exponent
// E >= 8.  The 8-bit significand 1.m7 shifted right by (E - e) + 1 is the 7-bit magnitude; a shift
// of 8 or more clears it, which also covers inputs with a zero exponent field.
__device__ __forceinline__ uint32_t bf16_pair_to_bfp8(uint32_t w, uint32_t e1_pair)
{
    const uint32_t sig = (w & 0x007f007fu) | 0x00800080u;
    const uint32_t sh = pk_min_u16(e1_pair - bf16_pair_exponents(w), 0x000f000fu);  // no borrow: E + 1 > e in both halves
    const uint32_t mag = pk_shr_u16(sig, sh);
    const uint32_t keep_sign = (mag + 0x007f007fu) & (w >> 8);  // bit 7 of a half: sign, if the magnitude is non-zero
    return (keep_sign & 0x00800080u) | mag;
}

// 8 bf16 (one 16-byte chunk) -> 8 Bfp8_b datum bytes.  Requires E == 0 or E >= 8.
__device__ __forceinline__ uint2 bf16_chunk_to_bfp8(const uint4 &v, uint32_t E)
{
    const uint32_t e1 = (E + 1u) | ((E + 1u) << 16);
    const uint32_t live = E ? 0xffffffffu : 0u;  // an all-zero block stores zeros
    const uint32_t d0 = bf16_pair_to_bfp8(v.x, e1), d1 = bf16_pair_to_bfp8(v.y, e1);
    const uint32_t d2 = bf16_pair_to_bfp8(v.z, e1), d3 = bf16_pair_to_bfp8(v.w, e1);
    return make_uint2(__builtin_amdgcn_perm(d1, d0, 0x06040200u) & live, __builtin_amdgcn_perm(d3, d2, 0x06040200u) & live);
}

// Four Bfp8_b datum bytes -> four bf16 (two words), shared exponent E >= 7 so every result is a
// normal number: float(mag) * 2^(E-133) is exact and its upper half is the bf16 pattern.
__device__ __forceinline__ uint2 bfp8_word_to_bf16(uint32_t w, float scale)
{
    const uint32_t m = w & 0x7f7f7f7fu;
    const uint32_t sgn = (m + 0x7f7f7f7fu) & w;  // bit 7 of each byte: sign, if the magnitude is non-zero
    const float f0 = (float)(m & 0xffu) * scale, f1 = (float)((m >> 8) & 0xffu) * scale;
    const float f2 = (float)((m >> 16) & 0xffu) * scale, f3 = (float)(m >> 24) * scale;
    const uint32_t p01 = __builtin_amdgcn_perm(__float_as_uint(f1), __float_as_uint(f0), 0x07060302u);
    const uint32_t p23 = __builtin_amdgcn_perm(__float_as_uint(f3), __float_as_uint(f2), 0x07060302u);
    const uint32_t s01 = __builtin_amdgcn_perm(sgn, sgn, 0x010c000cu);  // byte 0 -> byte 1, byte 1 -> byte 3
    const uint32_t s23 = __builtin_amdgcn_perm(sgn, sgn, 0x030c020cu);
    return make_uint2((s01 & 0x80008000u) | p01, (s23 & 0x80008000u) | p23);
}

// ---- lean paths through the float pipeline -----------------------------------------------------------
// Scaling by a power of two is exact, so for blocks whose shared exponent keeps every intermediate
// a normal number the shift-and-mask arithmetic can be replaced by one multiply and one conversion.

// Multiplier that turns |x| into its magnitude under shared exponent E: 2^(126 + M - E), doubled for
// round-to-nearest (the conversion then yields floor(2v) and the caller halves with rounding).
// Needs 8 <= E <= 250; E == 0 (an all-zero block) gets 0 so that every datum comes out 0.
template <int M, int ROUNDING>
__device__ __forceinline__ float quantize_multiplier(uint32_t E)
{
    return __uint_as_float(E ? (253u + M + ROUNDING - E) << 23 : 0u);
}

// One datum of an fp32 bit pattern: floor(|x| * mult) is the magnitude (inputs with a zero exponent
// field land below one and give 0), the sign is kept only beside a non-zero magnitude.
template <int M, int ROUNDING>
__device__ __forceinline__ uint32_t quantize_datum_scaled(uint32_t bits, float mult)
{
    uint32_t mag = (uint32_t)(fabsf(__uint_as_float(bits)) * mult);  // truncating conversion
    if (ROUNDING) mag = min((mag + 1u) >> 1, (1u << M) - 1u);
    const uint32_t keep_sign = (mag + ((1u << M) - 1u)) & (bits >> (31 - M));  // bit M: sign, if mag != 0
    return (keep_sign & (1u << M)) | mag;
}

// fp32 bit pattern of datum j of `piece` (datums of M + 1 bits, lowest first): mag * scale with the
// datum's sign moved into the scale; adding +0 turns the -0 of a signed zero magnitude into +0.
// `scale_bits` is the pattern of 2^(E - 127 - (M - 1)), which needs 8 <= E <= 254.
template <int M>
__device__ __forceinline__ uint32_t dequantize_datum_scaled(uint64_t piece, int j, uint32_t scale_bits)
{
    const uint32_t d = (uint32_t)(piece >> (j * (M + 1)));  // j is a constant after unrolling: one half of the piece, shifted
    const uint32_t signed_scale = ((d << (31 - M)) & 0x80000000u) | scale_bits;
    return __float_as_uint(fmaf((float)(d & ((1u << M) - 1u)), __uint_as_float(signed_scale), 0.0f));
}

__host__ __device__ __forceinline__ uint16_t f32_to_bf16_rne(uint32_t bits)
{
    if ((bits & 0x7f800000u) == 0x7f800000u && (bits & 0x007fffffu)) return (uint16_t)((bits >> 16) | 0x0040u);
    return (uint16_t)((bits + 0x7fffu + ((bits >> 16) & 1u)) >> 16);
}

// Four datum bytes of one column (four consecutive k) and the four shared exponents of their rows, byte j of
// each belonging to the same k -> the four bf16 values, two per dword.  float(mag) * 2^(E-133) is exact; the
// bytes are converted in place (byte-select conversions), the signs are moved to bits 15 and 31 by byte permutes.
__device__ __forceinline__ uint2 datums4_to_bf16(uint32_t d, uint32_t e4)
{
    // The masked word is hidden from the optimizer (no instruction is emitted): otherwise the 0x7f mask is folded into
    // each byte extraction, a bit-field extract per byte in front of a conversion that could have selected the byte.
    uint32_t m = d & 0x7f7f7f7fu;
    asm("" : "+v"(m));
    uint32_t f[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
        f[j] = __float_as_uint(__builtin_amdgcn_ldexpf((float)((m >> (8 * j)) & 0xffu), (int)((e4 >> (8 * j)) & 0xffu) - 133));
    // sign bytes to bits 15 and 31 (the other bytes of the permute carry magnitude bits, masked off in the merge)
    return make_uint2((__builtin_amdgcn_perm(0u, d, 0x010c000cu) & 0x80008000u) | __builtin_amdgcn_perm(f[1], f[0], 0x07060302u),
                      (__builtin_amdgcn_perm(0u, d, 0x030c020cu) & 0x80008000u) | __builtin_amdgcn_perm(f[3], f[2], 0x07060302u));
}

// GELU(x) = x Phi(x) in its erf form, the epilogue of the GEMM.  Phi comes from the complementary error function,
// erfc(z) = t (a1 + t (a2 + t (a3 + t (a4 + t a5)))) exp(-z^2), t = 1 / (1 + p z) for z >= 0 (Abramowitz & Stegun
// 7.1.26, absolute error below 1.5e-7 and shrinking with exp(-z^2)): Phi(x) = erfc(|x| / sqrt 2) / 2 for x < 0 and one
// minus that otherwise, so the negative tail keeps its relative accuracy instead of losing it in 1 + erf.  A dozen
// instructions without a branch, against the library erff's forty with one; the result is within 5e-7 of the exact
// value everywhere.
__device__ __forceinline__ float gelu_erf(float x)
{
    const float z = fabsf(x) * 0.70710678118654752440f;
    const float t = __builtin_amdgcn_rcpf(fmaf(0.3275911f, z, 1.0f));
    float p = fmaf(1.061405429f, t, -1.453152027f);
    p = fmaf(p, t, 1.421413741f);
    p = fmaf(p, t, -0.284496736f);
    p = fmaf(p, t, 0.254829592f);
    const float half_erfc = 0.5f * p * t * __builtin_amdgcn_exp2f(-1.4426950408889634f * z * z);
    return x * (x < 0.0f ? half_erfc : 1.0f - half_erfc);
}

// The tanh form of GELU, 0.5 x (1 + tanh(u)) with u = sqrt(2 / pi) (x + 0.044715 x^3)
// (pybuda/pybuda/op/eval/pybuda/eltwise_unary.py:45-47).  0.5 (1 + tanh u) is the logistic function of 2u, so the value
// is x / (1 + exp(-2u)): one exponential and one reciprocal, no branch, and the negative tail keeps its relative
// accuracy (exp overflows to infinity there and the quotient goes to -0 as the reference's product does).
__device__ __forceinline__ float gelu_tanh(float x)
{
    const float u = 0.7978845608028654f * fmaf(0.044715f * x, x * x, x);
    return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-2.8853900817779268f * u));
}

// The `epilogue` argument of the GEMM entry points: the low byte is the activation (0 none, 1 GELU in its erf form, 2 GELU
// in its tanh form), bit 8 says that the bias vector holds fp32 values instead of bf16 ones.
constexpr int kEpilogueMask = 0xff, kEpilogueBiasF32 = 0x100;

// element `col` of the bias row: bf16 (the Float16_b tensor the reference broadcasts) or fp32
__device__ __forceinline__ float load_bias(const uint16_t *bias, uint32_t col, bool f32)
{
    return f32 ? ((const float *)bias)[col] : __uint_as_float((uint32_t)bias[col] << 16);
}

__device__ __forceinline__ float apply_epilogue(int epilogue, float v)
{
    if (epilogue == 1) return gelu_erf(v);
    if (epilogue == 2) return gelu_tanh(v);
    return v;
}

}  // namespace ttbfp
