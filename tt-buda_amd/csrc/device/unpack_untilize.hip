// unpack + untilize: tiles of faces in Bfp8_b / Bfp4_b / Bfp2_b (or plain Float16_b / Float32
// tiles) -> row-major [w,z,r,c] fp32 or bf16.  This is the conversion behind
// tt::backend::get_output (pybuda/csrc/backend_api/backend_api.cpp:700-701); output formats are
// the ones pybuda accepts there (pybuda/pybuda/tensor.py:730-740).
//
// Mirror image of the pack kernel: a workgroup streams the packed tiles of one 32-row band segment
// (contiguous in memory) into LDS with 128-bit loads, then every lane rebuilds 16 bytes of one
// output row from its piece of the data section and the block's exponent byte, and a wave stores
// 1 KiB contiguous per row.
#include <type_traits>

#include "bfp_codec.hpp"
#include "launch.hpp"
#include "queue_layout.hpp"


#ifndef TTBFP_RESIDENT_MIN_GRID
#define TTBFP_RESIDENT_MIN_GRID 8192  // smallest grid (workgroups) whose residency is capped
#endif

namespace ttbfp {

namespace {

template <int BYTES>
__device__ __forceinline__ uint64_t lds_load(const uint8_t *p)
{
    if (BYTES == 1) return *p;
    if (BYTES == 2) return *(const uint16_t *)p;
    if (BYTES == 4) return *(const uint32_t *)p;
    const uint2 v = *(const uint2 *)p;
    return (uint64_t)v.x | ((uint64_t)v.y << 32);
}

// Fast path.  Requires: element stride == itemsize; dst base and outer strides multiples of the element size (a sliced
// view: its 16-byte stores then start anywhere); src 16-byte aligned.  1-D grid of bands x segments, segment index fastest (resident
// workgroups sweep contiguous memory on both sides).
// QUEUE: the tiles come from their slots of a queue's per-core buffers; only the read-in changes.
// NARROW: only the g.Rl x g.Cl corner of every [R, C] slice is written (g.Cl a multiple of the elements a lane stores).
// streaming: the result is stored with the non-temporal hint (it is larger than the last-level cache and would only push
// other data out of it); a smaller result is stored plainly and written back from the cache in whole lines.
template <uint8_t SRC, typename DstT, bool QUEUE, bool NARROW>
__global__ __launch_bounds__(256) void unpack_untilize_rows(const uint8_t *__restrict__ src, TensorGeom g,
                                                            uint8_t *__restrict__ dst, uint32_t segs, uint32_t streaming, QueueLayout q)
{
    constexpr int EPL = 16 / sizeof(DstT);
    constexpr int SEG_TILES = 64 * EPL / kTile;
    constexpr int M = mantissa_bits(SRC);
    constexpr uint32_t TB = tile_bytes(SRC);
    __shared__ __attribute__((aligned(16))) uint8_t image[SEG_TILES * TB];
    __shared__ uint64_t tile_src[QUEUE ? SEG_TILES : 1];

    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t tiles_c = g.C / kTile, tiles_r = g.R / kTile;
    const uint32_t band = blockIdx.x / segs;
    const uint32_t tr = band % tiles_r, wz = band / tiles_r;
    const uint32_t z = wz % g.Z, w = wz / g.Z;
    const uint32_t tile0 = (blockIdx.x % segs) * SEG_TILES;

    const uint32_t seg_tiles = min((uint32_t)SEG_TILES, tiles_c - tile0);
    const uint32_t bytes = seg_tiles * TB;
    if constexpr (QUEUE) {
        if (threadIdx.x < seg_tiles) tile_src[threadIdx.x] = tile_offset(q, w, z, tr, tile0 + threadIdx.x);
        __syncthreads();
    }
    // where byte o of the segment's packed tiles lies: one linear run, or tile by tile in the buffers of a queue
    const uint8_t *in = src + ((uint64_t)band * tiles_c + tile0) * TB;
    auto at = [&](uint32_t o) -> const uint8_t * {
        if constexpr (QUEUE) {
            const uint32_t tile = o / TB;
            return src + tile_src[tile] + (o - tile * TB);
        } else {
            return in + o;
        }
    };
    if (seg_tiles == SEG_TILES) {
        // A whole segment: every load of the thread is issued before the first is waited for (the loop below is a trip
        // to memory per turn).  The last, partial sweep is fetched by all threads - those past the end take the
        // segment's last 16 bytes again - so that no load sits under a condition; only the store is conditional.
        constexpr uint32_t BYTES = SEG_TILES * TB, NFULL = BYTES / 4096, REM = BYTES % 4096;
        uint4 t[NFULL + 1];
#pragma unroll
        for (uint32_t i = 0; i < NFULL; ++i) t[i] = load_stream(at(i * 4096 + threadIdx.x * 16));
        if constexpr (REM != 0) t[NFULL] = load_stream(at(min(NFULL * 4096 + threadIdx.x * 16, BYTES - 16)));
#pragma unroll
        for (uint32_t i = 0; i < NFULL; ++i) *(uint4 *)(image + i * 4096 + threadIdx.x * 16) = t[i];
        if constexpr (REM != 0) {
            if (threadIdx.x * 16 < REM) *(uint4 *)(image + NFULL * 4096 + threadIdx.x * 16) = t[NFULL];
        }
    } else {
        for (uint32_t o = threadIdx.x * 16; o < bytes; o += 256 * 16) *(uint4 *)(image + o) = load_stream(at(o));
    }
    __syncthreads();

    const uint32_t c0 = tile0 * kTile + lane * EPL;
    if (c0 >= (NARROW ? g.Cl : g.C)) return;
    uint8_t *row0 = dst + w * g.s0 + z * g.s1 + (uint64_t)(tr * kTile + wave * 8) * g.s2 + (uint64_t)c0 * sizeof(DstT);
    const uint32_t cc = lane * EPL % kTile;
    const uint32_t col_in_face = cc % kFace;
    const uint8_t *tile_img = image + (lane * EPL / kTile) * TB;
    // the eight rows of this wavefront, with one kind of store throughout (a branch per store would sit between the rows)
    auto rows = [&](auto ntc) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t rr = wave * 8 + i;
        const uint32_t face_row = ((rr / kFace) * 2 + cc / kFace) * kFace + rr % kFace;
        uint4 out;
        if constexpr (M != 0) {
            constexpr int ROW_BYTES = 16 * (M + 1) / 8;
            constexpr int PIECE_BYTES = EPL * (M + 1) / 8;
            // A family: five exponent bits padded to eight, rebased to the fp32 exponent of the same value
            const uint32_t e = is_a_format(SRC) ? (tile_img[face_row] & 0x1fu) + kHalfExponentRebase : tile_img[face_row];
            const uint64_t piece =
                lds_load<PIECE_BYTES>(tile_img + kExpSection + face_row * ROW_BYTES + col_in_face * (M + 1) / 8);
            constexpr bool LEAN8 = SRC == kBfp8_b && sizeof(DstT) == 2;
            // The multiply-based paths need a shared exponent that keeps every result a normal, finite
            // number (7 or 8 <= E <= 254); an all-zero piece is 0 under any exponent.  Other blocks
            // are rare and send the whole wavefront down the bit-assembly path for this row.
            if (LEAN8 && __builtin_amdgcn_ballot_w64(e - 7u >= 248u && piece != 0) == 0) {
                const float scale = __uint_as_float(e - 7u < 248u ? (e - 6u) << 23 : 0u);
                const uint2 lo = bfp8_word_to_bf16((uint32_t)piece, scale), hi = bfp8_word_to_bf16((uint32_t)(piece >> 32), scale);
                out = make_uint4(lo.x, lo.y, hi.x, hi.y);
            } else {
                uint32_t f[EPL];
                bool lean = false;
                if constexpr (!LEAN8) lean = __builtin_amdgcn_ballot_w64(e - 8u > 246u && piece != 0) == 0;
                if (lean) {
                    if constexpr (!LEAN8) {
                        const uint32_t scale = e - 8u <= 246u ? (e - (M - 1)) << 23 : 0u;
#pragma unroll
                        for (int j = 0; j < EPL; ++j) f[j] = dequantize_datum_scaled<M>(piece, j, scale);
                    }
                } else {
#pragma unroll
                    for (int j = 0; j < EPL; ++j)
                        f[j] = dequantize_datum<M>((uint32_t)(piece >> (j * (M + 1))) & ((2u << M) - 1u), e);
                }
                if constexpr (sizeof(DstT) == 4) {
                    out = make_uint4(f[0], f[1], f[2], f[3]);
                } else if constexpr (std::is_same<DstT, half_t>::value) {
                    uint32_t h[8];
#pragma unroll
                    for (int j = 0; j < 8; ++j) h[j] = f32_pattern_to_half(f[j % EPL]);
                    out = make_uint4(h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16));
                } else  // exact: at most 8 significant bits, so the low half of every pattern is zero
                    out = make_uint4(__builtin_amdgcn_perm(f[1], f[0], 0x07060302u), __builtin_amdgcn_perm(f[3], f[2], 0x07060302u),
                                     __builtin_amdgcn_perm(f[5 % EPL], f[4 % EPL], 0x07060302u),
                                     __builtin_amdgcn_perm(f[7 % EPL], f[6 % EPL], 0x07060302u));
            }
        } else if constexpr (SRC == kFloat32) {
            out = *(const uint4 *)(tile_img + (face_row * 16 + col_in_face) * 4);
        } else if constexpr (sizeof(DstT) == 2) {
            out = *(const uint4 *)(tile_img + (face_row * 16 + col_in_face) * 2);
        } else {
            const uint2 h = *(const uint2 *)(tile_img + (face_row * 16 + col_in_face) * 2);
            out = make_uint4(h.x << 16, h.x & 0xffff0000u, h.y << 16, h.y & 0xffff0000u);
        }
        if (!NARROW || tr * kTile + rr < g.Rl) {
            if constexpr (decltype(ntc)::value)
                store_stream_at<sizeof(DstT)>(row0 + i * g.s2, out);
            else
                *(typename UnderAligned<sizeof(DstT)>::type *)(row0 + i * g.s2) = u32x4_t{out.x, out.y, out.z, out.w};
        }
    }
    };
    if (streaming)  // uniform
        rows(std::true_type{});
    else
        rows(std::false_type{});
}

// General path: any strides and alignments.  One thread writes one element; the 16 lanes of a face row write neighbouring
// elements, so a wavefront's store covers four runs of 16 elements instead of 64 separate rows (a result with an element
// stride of 8 bytes, 256 MiB: 0.99 ms with one thread per face row).
template <uint8_t SRC, typename DstT, bool QUEUE>
__global__ __launch_bounds__(256) void unpack_untilize_blocks(const uint8_t *__restrict__ src, TensorGeom g,
                                                              uint8_t *__restrict__ dst, uint64_t nblocks, QueueLayout q)
{
    constexpr int M = mantissa_bits(SRC);
    constexpr uint32_t TB = tile_bytes(SRC);
    const uint64_t gid = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    const uint64_t blk = gid / 16;
    const uint32_t j = gid % 16;
    if (blk >= nblocks) return;
    const uint32_t tiles_c = g.C / kTile, tiles_r = g.R / kTile;
    const uint32_t face_row = blk % 64;
    const uint64_t tile = blk / 64;
    const uint32_t tc = tile % tiles_c;
    const uint64_t band = tile / tiles_c;
    const uint32_t tr = band % tiles_r;
    const uint64_t wz = band / tiles_r;
    const uint32_t z = wz % g.Z, w = wz / g.Z;
    const uint32_t face = face_row / kFace, row = face_row % kFace;
    const uint32_t r = tr * kTile + (face / 2) * kFace + row;
    const uint32_t c = tc * kTile + (face % 2) * kFace + j;
    if (r >= g.Rl || c >= g.Cl) return;  // narrowed away
    uint8_t *p = dst + w * g.s0 + z * g.s1 + (uint64_t)r * g.s2 + (uint64_t)c * g.s3;
    const uint8_t *tile_in = src + (QUEUE ? tile_offset(q, w, z, tr, tc) : tile * TB);
    uint32_t bits;
    if constexpr (M != 0) {
        constexpr int ROW_BYTES = 16 * (M + 1) / 8;
        constexpr int PER_BYTE = 8 / (M + 1);
        const uint32_t byte = tile_in[kExpSection + face_row * ROW_BYTES + j / PER_BYTE];
        const uint32_t e = is_a_format(SRC) ? (tile_in[face_row] & 0x1fu) + kHalfExponentRebase : tile_in[face_row];
        bits = dequantize_datum<M>((byte >> ((j % PER_BYTE) * (M + 1))) & ((2u << M) - 1u), e);
        if constexpr (std::is_same<DstT, half_t>::value) bits = f32_pattern_to_half(bits) << 16;
    } else if constexpr (SRC == kFloat32) {
        bits = ((const uint32_t *)tile_in)[face_row * 16 + j];
    } else {
        bits = (uint32_t)((const uint16_t *)tile_in)[face_row * 16 + j] << 16;
    }
    // strides are multiples of the element size (checked at the boundary): with an aligned base the element is one store
    if ((uintptr_t)dst % sizeof(DstT) == 0) {
        if (sizeof(DstT) == 4)
            *(uint32_t *)p = bits;
        else
            *(uint16_t *)p = (uint16_t)(bits >> 16);
        return;
    }
    if (sizeof(DstT) == 4) {
        p[0] = (uint8_t)bits;
        p[1] = (uint8_t)(bits >> 8);
    }
    p[sizeof(DstT) - 2] = (uint8_t)(bits >> 16);
    p[sizeof(DstT) - 1] = (uint8_t)(bits >> 24);
}

// One-byte elements (Int8 / RawUInt8 queues): the inverse permutation of bytes, one thread per face row of 16.
template <bool QUEUE>
__global__ __launch_bounds__(256) void untilize_bytes_blocks(const uint8_t *__restrict__ src, TensorGeom g, uint8_t *__restrict__ dst,
                                                             uint64_t nblocks, QueueLayout q)
{
    constexpr uint32_t TB = tile_bytes(kRaw8);
    const uint64_t blk = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (blk >= nblocks) return;
    const uint32_t tiles_c = g.C / kTile, tiles_r = g.R / kTile;
    const uint32_t face_row = blk % 64;
    const uint64_t tile = blk / 64;
    const uint32_t tc = tile % tiles_c;
    const uint64_t band = tile / tiles_c;
    const uint32_t tr = band % tiles_r;
    const uint64_t wz = band / tiles_r;
    const uint32_t z = wz % g.Z, w = wz / g.Z;
    const uint32_t face = face_row / kFace, row = face_row % kFace;
    const uint32_t r = tr * kTile + (face / 2) * kFace + row;
    const uint32_t c = tc * kTile + (face % 2) * kFace;
    if (r >= g.Rl) return;  // narrowed away
    uint8_t *p = dst + w * g.s0 + z * g.s1 + (uint64_t)r * g.s2 + (uint64_t)c * g.s3;
    const uint8_t *tile_in = src + (QUEUE ? tile_offset(q, w, z, tr, tc) : tile * TB);
#pragma unroll
    for (int j = 0; j < 16; ++j)
        if (c + j < g.Cl) p[j * g.s3] = tile_in[face_row * 16 + j];
}

hipError_t launch_bytes(const void *src, const TensorGeom &g, void *dst, const QueueLayout *q, hipStream_t stream)
{
    const uint64_t nblocks = (uint64_t)g.W * g.Z * (g.R / kTile) * (g.C / kTile) * 64;
    if (nblocks == 0) return hipSuccess;
    const uint64_t grid = (nblocks + 255) / 256;
    if (grid > 0x7fffffffull) return hipErrorInvalidValue;
    if (q)
        hipLaunchKernelGGL(untilize_bytes_blocks<true>, dim3((uint32_t)grid), dim3(256), 0, stream, (const uint8_t *)src, g, (uint8_t *)dst, nblocks, *q);
    else
        hipLaunchKernelGGL(untilize_bytes_blocks<false>, dim3((uint32_t)grid), dim3(256), 0, stream, (const uint8_t *)src, g, (uint8_t *)dst, nblocks, QueueLayout{});
    return hipGetLastError();
}

// Workgroups per CU of the row kernel.  On tensors of hundreds of MiB fewer workgroups in flight than LDS and registers
// admit stream faster (fewer concurrent streams into HBM), as long as enough bytes stay in flight: a workgroup loads
// `segment_bytes` of tiles at once and stores 32 KiB.  Measured at 1 GiB of results (us, 8 / 4 / 3 workgroups per CU):
// bf16 from Bfp8_b 277 / 261 / 258, fp32 from Bfp8_b 229 / 214 / 220, bf16 from Bfp4_b 228 / 216 / 225, fp32 from Bfp4_b
// 207 / 205 / 229, fp32 from Bfp2_b 188 / 197 / 203.  A small grid wants them all, to cover its ramp and its tail.
inline uint32_t unpack_resident(uint64_t workgroups, uint32_t segment_bytes)
{
    if (workgroups < TTBFP_RESIDENT_MIN_GRID) return 8;
    return segment_bytes >= 16384 ? 3 : segment_bytes >= 5120 ? 4 : 8;
}

template <uint8_t SRC, typename DstT, bool QUEUE>
hipError_t launch_kernel(const void *src, const TensorGeom &g, void *dst, const QueueLayout &q, hipStream_t stream)
{
    const uint32_t tiles_r = g.R / kTile, tiles_c = g.C / kTile;
    const uint64_t bands = (uint64_t)g.W * g.Z * tiles_r;
    if (bands == 0 || tiles_c == 0) return hipSuccess;
    // unit element stride; the row-major side aligned to its elements (the strides are, by the boundary's checks), the tiles to 16 bytes
    const bool aligned = g.s3 == sizeof(DstT) && ((uintptr_t)src % 16 == 0) && ((uintptr_t)dst % sizeof(DstT) == 0) &&
                         (!QUEUE || q.buffer_pitch % 16 == 0);
    constexpr int SEG_TILES = 64 * (16 / sizeof(DstT)) / kTile;
    const uint32_t segs = (tiles_c + SEG_TILES - 1) / SEG_TILES;
    const bool narrow_ok = g.Cl % (16 / sizeof(DstT)) == 0;  // whole 16-byte stores only
    if (aligned && bands * segs <= 0x7fffffffull && (!g.padded() || narrow_ok)) {
        // partial segments take the rolled load loop, one load per thread in flight, which needs every workgroup it can get
        const bool mostly_whole = tiles_c % SEG_TILES == 0 || tiles_c >= 4 * SEG_TILES;
        const uint32_t lds_cap = resident_cap_bytes(SEG_TILES * tile_bytes(SRC), unpack_resident(mostly_whole ? bands * segs : 0, SEG_TILES * tile_bytes(SRC)));
        // Results up to the size of the last-level cache (256 MiB) measured 5 % faster with plain stores (fp32 [8192, 8192]
        // from Bfp8_b: 53.7 against 57.6 us), larger ones 3 % faster with non-temporal stores (1 GiB: 215 against 224 us).
        const uint64_t result_bytes = (uint64_t)g.W * g.Z * g.Rl * g.Cl * sizeof(DstT);
        const uint32_t streaming = result_bytes > (256ull << 20);
        if (g.padded())
            hipLaunchKernelGGL((unpack_untilize_rows<SRC, DstT, QUEUE, true>), dim3((uint32_t)(bands * segs)), dim3(256), lds_cap, stream,
                               (const uint8_t *)src, g, (uint8_t *)dst, segs, streaming, q);
        else
            hipLaunchKernelGGL((unpack_untilize_rows<SRC, DstT, QUEUE, false>), dim3((uint32_t)(bands * segs)), dim3(256), lds_cap, stream,
                               (const uint8_t *)src, g, (uint8_t *)dst, segs, streaming, q);
    } else {
        const uint64_t nblocks = bands * tiles_c * 64;
        const uint64_t grid = nblocks / 16;  // 16 threads per face row, 256 per workgroup
        if (grid > 0x7fffffffull) return hipErrorInvalidValue;
        hipLaunchKernelGGL((unpack_untilize_blocks<SRC, DstT, QUEUE>), dim3((uint32_t)grid), dim3(256), 0, stream,
                           (const uint8_t *)src, g, (uint8_t *)dst, nblocks, q);
    }
    return hipGetLastError();
}

template <uint8_t SRC, typename DstT>
hipError_t launch(const void *src, const TensorGeom &g, void *dst, const QueueLayout *q, hipStream_t stream)
{
    if (q) return launch_kernel<SRC, DstT, true>(src, g, dst, *q, stream);
    return launch_kernel<SRC, DstT, false>(src, g, dst, QueueLayout{}, stream);
}

template <typename DstT>
hipError_t by_format(uint8_t src_fmt, const void *src, const TensorGeom &g, void *dst, const QueueLayout *q, hipStream_t s)
{
    switch (src_fmt) {
        case kBfp8_b: return launch<kBfp8_b, DstT>(src, g, dst, q, s);
        case kBfp4_b: return launch<kBfp4_b, DstT>(src, g, dst, q, s);
        case kBfp2_b: return launch<kBfp2_b, DstT>(src, g, dst, q, s);
        case kFloat16_b: return launch<kFloat16_b, DstT>(src, g, dst, q, s);
        case kFloat32:
            if constexpr (sizeof(DstT) == 4) return launch<kFloat32, DstT>(src, g, dst, q, s);
            return hipErrorInvalidValue;
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

hipError_t launch_unpack_untilize(const void *src, uint8_t src_fmt, const TensorGeom &g, uint8_t dst_fmt, void *dst,
                                  const QueueLayout *q, hipStream_t stream)
{
    if (src_fmt == kRaw8 || dst_fmt == kRaw8) return src_fmt == dst_fmt ? launch_bytes(src, g, dst, q, stream) : hipErrorInvalidValue;
    if (dst_fmt == kFloat32) return by_format<float>(src_fmt, src, g, dst, q, stream);
    if (dst_fmt == kFloat16_b) return by_format<uint16_t>(src_fmt, src, g, dst, q, stream);
    if (dst_fmt == kFloat16) {  // the A family reads back as IEEE half, and only the A family does
        switch (src_fmt) {
            case kBfp8: return launch<kBfp8, half_t>(src, g, dst, q, stream);
            case kBfp4: return launch<kBfp4, half_t>(src, g, dst, q, stream);
            case kBfp2: return launch<kBfp2, half_t>(src, g, dst, q, stream);
            case kFloat16: return launch<kFloat16, half_t>(src, g, dst, q, stream);
            default: return hipErrorInvalidValue;
        }
    }
    return hipErrorInvalidValue;
}

}  // namespace ttbfp
