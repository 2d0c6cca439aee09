// tilize + pack: row-major [w,z,r,c] fp32/bf16 -> 32x32 tiles of four 16x16 faces in Bfp8_b /
// Bfp4_b / Bfp2_b (or plain Float32 / Float16_b tiles).  This is the conversion behind
// tt::backend::tilize_tensor and push_input (pybuda/csrc/backend_api/backend_api.cpp:688-704).
//
// Streaming kernel, HBM bound.  One workgroup of four wavefronts converts a 32-row band segment
// that is one wave-load wide (64 lanes x 16 bytes = 256 fp32 or 512 bf16 columns = 8 or 16 tiles):
//   * every lane issues its eight 128-bit row loads up front (a wave reads 1 KiB contiguous per row);
//   * a 16-datum block lives in 4 (fp32) or 2 (bf16) neighbouring lanes, so the shared exponent is
//     an in-lane max followed by one or two DPP quad permutes;
//   * datums are assembled into 1..8-byte pieces and written into an LDS image of the packed tiles
//     (this is where the row-major -> face order regroup happens);
//   * the workgroup then streams the LDS image out with 128-bit stores: the tiles of a band segment
//     are contiguous in the packed tensor, so the write is one linear run of up to 17 KiB.
#include <type_traits>

#include "bfp_codec.hpp"
#include "launch.hpp"
#include "queue_layout.hpp"

#ifndef TTBFP_PACK_RESIDENT
#define TTBFP_PACK_RESIDENT 3  // workgroups of the row kernel per CU on large tensors (see resident_cap_bytes)
#endif

#ifndef TTBFP_RESIDENT_MIN_GRID
#define TTBFP_RESIDENT_MIN_GRID 8192  // smallest grid (workgroups) whose residency is capped
#endif

namespace ttbfp {

namespace {

template <typename T>
struct Chunk;  // the 16 bytes one lane loads
template <>
struct Chunk<float> {
    static constexpr int kElems = 4;
    __device__ static uint32_t bits(const uint4 &v, int j) { return j == 0 ? v.x : j == 1 ? v.y : j == 2 ? v.z : v.w; }
};
template <>
struct Chunk<uint16_t> {
    static constexpr int kElems = 8;
    __device__ static uint32_t bits(const uint4 &v, int j)
    {
        const uint32_t w = (j >> 1) == 0 ? v.x : (j >> 1) == 1 ? v.y : (j >> 1) == 2 ? v.z : v.w;
        return (j & 1) ? (w & 0xffff0000u) : (w << 16);
    }
};

template <>
struct Chunk<half_t> {
    static constexpr int kElems = 8;
    __device__ static uint32_t bits(const uint4 &v, int j)
    {
        const uint32_t w = (j >> 1) == 0 ? v.x : (j >> 1) == 1 ? v.y : (j >> 1) == 2 ? v.z : v.w;
        return half_to_f32_pattern((j & 1) ? (w >> 16) : (w & 0xffffu));
    }
};

template <int BYTES>
__device__ __forceinline__ void lds_store(uint8_t *p, uint64_t v)
{
    if (BYTES == 1) *p = (uint8_t)v;
    if (BYTES == 2) *(uint16_t *)p = (uint16_t)v;
    if (BYTES == 4) *(uint32_t *)p = (uint32_t)v;
    if (BYTES == 8) *(uint2 *)p = make_uint2((uint32_t)v, (uint32_t)(v >> 32));
}

// Fast path.  Requires: element stride == itemsize; base address and the three outer strides
// multiples of the element size (a sliced view of a row-major tensor: its 16-byte loads then start anywhere); dst
// 16-byte aligned.  1-D grid of bands x segments with the segment index
// varying fastest, so that the workgroups resident at any moment sweep contiguous memory on both
// sides instead of one column strip (which would camp on a few HBM channels).
// QUEUE: the tiles go to their slots of a queue's per-core buffers instead of one linear run; a
// tile stays one contiguous piece, so only the write-out changes.
// PAD: the memory holds g.Rl x g.Cl (g.Cl a multiple of the elements a lane loads); rows and chunks past that are read from
// the last row / chunk inside (so that every load stays unconditional) and then zeroed, or kept where g.rep_r says so.
template <typename SrcT, uint8_t DST, int ROUNDING, bool QUEUE, bool PAD>
__global__ __launch_bounds__(256) void tilize_pack_rows(const uint8_t *__restrict__ src, TensorGeom g,
                                                        uint8_t *__restrict__ dst, uint32_t segs, QueueLayout q)
{
    constexpr int EPL = Chunk<SrcT>::kElems;       // elements per lane
    constexpr int LPB = 16 / EPL;                  // lanes per 16-datum block
    constexpr int SEG_TILES = 64 * EPL / kTile;    // tiles one wave-load spans
    constexpr int M = mantissa_bits(DST);
    constexpr uint32_t TB = tile_bytes(DST);
    __shared__ __attribute__((aligned(16))) uint8_t image[SEG_TILES * TB];
    __shared__ uint64_t tile_dst[QUEUE ? SEG_TILES : 1];

    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t tiles_c = g.C / kTile, tiles_r = g.R / kTile;
    const uint32_t band = blockIdx.x / segs;  // (w * Z + z) * tiles_r + tile_row
    const uint32_t tr = band % tiles_r, wz = band / tiles_r;
    const uint32_t z = wz % g.Z, w = wz / g.Z;
    const uint32_t tile0 = (blockIdx.x % segs) * SEG_TILES;
    const uint32_t c0 = tile0 * kTile + lane * EPL;
    const bool live = c0 < g.C;

    // Lanes past the last column fetch the row's last chunk again instead of nothing (and store nothing below): loads
    // under a condition make the compiler wait for all outstanding loads at once (vmcnt(0)), two full trips to memory
    // before the first row is touched; unconditional ones are counted exactly, row i is converted while rows
    // i + 1 .. 7 are still in flight.
    uint4 v[8];
    if constexpr (PAD) {
        const bool in_cols = c0 < g.Cl;
        const uint8_t *col0 = src + w * g.s0 + z * g.s1 + (uint64_t)(in_cols ? c0 : g.Cl - EPL) * sizeof(SrcT);
        const uint32_t r0 = tr * kTile + wave * 8;
#pragma unroll
        for (int i = 0; i < 8; ++i) v[i] = load_stream_at<sizeof(SrcT)>(col0 + (uint64_t)min(r0 + i, g.Rl - 1) * g.s2);
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (!in_cols || (r0 + i >= g.Rl && !g.rep_r)) v[i] = make_uint4(0, 0, 0, 0);
    } else {
    const uint8_t *row0 = src + w * g.s0 + z * g.s1 + (uint64_t)(tr * kTile + wave * 8) * g.s2 +
                          (uint64_t)(live ? c0 : g.C - EPL) * sizeof(SrcT);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = load_stream_at<sizeof(SrcT)>(row0 + i * g.s2);
    }
    if constexpr (QUEUE) {
        if (threadIdx.x < SEG_TILES && tile0 + threadIdx.x < tiles_c) tile_dst[threadIdx.x] = tile_offset(q, w, z, tr, tile0 + threadIdx.x);
    }

    const uint32_t tile_in_seg = lane * EPL / kTile;
    const uint32_t cc = lane * EPL % kTile;
    const uint32_t col_in_face = cc % kFace;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const uint32_t rr = wave * 8 + i;
        const uint32_t face_row = ((rr / kFace) * 2 + cc / kFace) * kFace + rr % kFace;  // face*16 + row
        uint8_t *tile_img = image + tile_in_seg * TB;
        if constexpr (M != 0) {
            constexpr bool LEAN = std::is_same<SrcT, uint16_t>::value && DST == kBfp8_b && ROUNDING == 0;
            uint32_t e = 0;
            if constexpr (LEAN) {
                e = bf16_chunk_max_exponent(v[i]);
            } else {
#pragma unroll
                for (int j = 0; j < EPL; ++j) {
                    const uint32_t ej = biased_exponent(Chunk<SrcT>::bits(v[i], j));
                    e = ej > e ? ej : e;
                }
            }
            e = block_max<LPB>(e);
            uint64_t piece = 0;
            // The packed 16-bit path needs E == 0 or E >= 8 and the float path E == 0 or 8 <= E <= 250;
            // a block outside (values below 2^-119, or Inf/NaN) sends the whole wavefront down the
            // shift-and-mask path for this row.
            const bool lean = LEAN ? __builtin_amdgcn_ballot_w64(e - 1u < 7u) == 0
                                   : __builtin_amdgcn_ballot_w64(e != 0u && e - 8u > 242u) == 0;
            if (LEAN && lean) {
                const uint2 d = bf16_chunk_to_bfp8(v[i], e);
                piece = (uint64_t)d.x | ((uint64_t)d.y << 32);
            } else if (lean) {
                const float mult = quantize_multiplier<M, ROUNDING>(e);
#pragma unroll
                for (int j = 0; j < EPL; ++j)
                    piece |= (uint64_t)quantize_datum_scaled<M, ROUNDING>(Chunk<SrcT>::bits(v[i], j), mult) << (j * (M + 1));
            } else {
#pragma unroll
                for (int j = 0; j < EPL; ++j)
                    piece |= (uint64_t)quantize_datum<M, ROUNDING>(Chunk<SrcT>::bits(v[i], j), e) << (j * (M + 1));
            }
            constexpr int ROW_BYTES = 16 * (M + 1) / 8;
            constexpr int PIECE_BYTES = EPL * (M + 1) / 8;
            if (live) {
                lds_store<PIECE_BYTES>(tile_img + kExpSection + face_row * ROW_BYTES + col_in_face * (M + 1) / 8, piece);
                if (col_in_face == 0) tile_img[face_row] = (uint8_t)(is_a_format(DST) && e ? e - kHalfExponentRebase : e);
            }
        } else if constexpr (DST == kFloat32) {
            static_assert(sizeof(SrcT) == 4, "16-bit sources reach Float32 tiles through the general kernel only");
            if (live) *(uint4 *)(tile_img + (face_row * 16 + col_in_face) * 4) = v[i];
        } else {  // Float16_b tiles, or Float16 tiles from a half source
            if constexpr (sizeof(SrcT) == 2) {
                if (live) *(uint4 *)(tile_img + (face_row * 16 + col_in_face) * 2) = v[i];
            } else {
                uint32_t h[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const uint32_t b = Chunk<SrcT>::bits(v[i], j);
                    h[j] = ROUNDING ? f32_to_bf16_rne(b) : (b >> 16);
                }
                if (live)
                    *(uint2 *)(tile_img + (face_row * 16 + col_in_face) * 2) = make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
            }
        }
    }
    __syncthreads();

    const uint32_t seg_tiles = min((uint32_t)SEG_TILES, tiles_c - tile0);
    const uint32_t bytes = seg_tiles * TB;  // a multiple of 16 for every format
    if constexpr (QUEUE) {
        if (q.prefix) {  // a slot = 16-byte header, the tile, 16 bytes of padding: one contiguous run per tile, zeros at both ends
            constexpr uint32_t SLOT = TB + 32;
            for (uint32_t o = threadIdx.x * 16; o < seg_tiles * SLOT; o += 256 * 16) {
                const uint32_t tile = o / SLOT, within = o - tile * SLOT;
                const bool data = within - 16u < TB;
                const uint4 v = *(const uint4 *)(image + (data ? tile * TB + within - 16 : 0));
                store_stream(dst + tile_dst[tile] + within - 16, data ? v : make_uint4(0, 0, 0, 0));
            }
        } else {
            for (uint32_t o = threadIdx.x * 16; o < bytes; o += 256 * 16) {
                const uint32_t tile = o / TB;
                store_stream(dst + tile_dst[tile] + (o - tile * TB), *(const uint4 *)(image + o));
            }
        }
    } else {
        uint8_t *out = dst + ((uint64_t)band * tiles_c + tile0) * TB;
        for (uint32_t o = threadIdx.x * 16; o < bytes; o += 256 * 16) store_stream(out + o, *(const uint4 *)(image + o));
    }
}

// General path: any strides and alignments.  One thread converts one 16-datum block (face row).
template <typename SrcT, uint8_t DST, int ROUNDING, bool QUEUE>
__global__ __launch_bounds__(256) void tilize_pack_blocks(const uint8_t *__restrict__ src, TensorGeom g,
                                                          uint8_t *__restrict__ dst, uint64_t nblocks, QueueLayout q)
{
    constexpr int M = mantissa_bits(DST);
    constexpr uint32_t TB = tile_bytes(DST);
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
    // rows and columns past the memory's Rl x Cl: the last one inside where the replicate mode says so, else zeros
    const bool row_inside = r < g.Rl || g.rep_r;
    const uint8_t *p = src + w * g.s0 + z * g.s1 + (uint64_t)min(r, g.Rl - 1) * g.s2;
    uint32_t bits[16];
    uint16_t raw[16];  // the half itself, for Float16 tiles
    // strides are multiples of the element size (checked at the boundary); with an aligned base every element is one load,
    // else it is put together from bytes
    const bool whole = (uintptr_t)src % sizeof(SrcT) == 0;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const bool inside = row_inside && (c + j < g.Cl || g.rep_c);
        const uint8_t *e = p + (uint64_t)min(c + j, g.Cl - 1) * g.s3;
        uint32_t v;  // the element's bits, in the low 16 or all 32
        if (sizeof(SrcT) == 4)
            v = whole ? *(const uint32_t *)e : (uint32_t)e[0] | (uint32_t)e[1] << 8 | (uint32_t)e[2] << 16 | (uint32_t)e[3] << 24;
        else
            v = whole ? (uint32_t) * (const uint16_t *)e : (uint32_t)e[0] | (uint32_t)e[1] << 8;
        if (sizeof(SrcT) == 4)
            bits[j] = v;
        else if (std::is_same<SrcT, half_t>::value) {
            raw[j] = inside ? (uint16_t)v : (uint16_t)0;
            bits[j] = half_to_f32_pattern(raw[j]);
        } else
            bits[j] = v << 16;
        if (!inside) bits[j] = 0;
    }
    uint8_t *tile_out = dst + (QUEUE ? tile_offset(q, w, z, tr, tc) : tile * TB);
    if constexpr (QUEUE) {
        if (q.prefix && face_row < 2)  // header (face_row 0) and trailing pad (1) of the slot: zeros
            for (int k = 0; k < 16; ++k) (face_row ? tile_out + TB : tile_out - 16)[k] = 0;
    }
    if constexpr (M != 0) {
        uint32_t e = 0;
#pragma unroll
        for (int j = 0; j < 16; ++j) e = max(e, biased_exponent(bits[j]));
        constexpr int ROW_BYTES = 16 * (M + 1) / 8;
        constexpr int PER_BYTE = 8 / (M + 1);
        tile_out[face_row] = (uint8_t)(is_a_format(DST) && e ? e - kHalfExponentRebase : e);
#pragma unroll
        for (int k = 0; k < ROW_BYTES; ++k) {
            uint32_t byte = 0;
#pragma unroll
            for (int i = 0; i < PER_BYTE; ++i) byte |= quantize_datum<M, ROUNDING>(bits[k * PER_BYTE + i], e) << (i * (M + 1));
            tile_out[kExpSection + face_row * ROW_BYTES + k] = (uint8_t)byte;
        }
    } else if constexpr (DST == kFloat32) {
#pragma unroll
        for (int j = 0; j < 16; ++j) ((uint32_t *)tile_out)[face_row * 16 + j] = bits[j];
    } else if constexpr (std::is_same<SrcT, half_t>::value) {  // Float16 tiles: the half itself
#pragma unroll
        for (int j = 0; j < 16; ++j) ((uint16_t *)tile_out)[face_row * 16 + j] = raw[j];
    } else {
#pragma unroll
        for (int j = 0; j < 16; ++j)
            ((uint16_t *)tile_out)[face_row * 16 + j] =
                (ROUNDING && sizeof(SrcT) == 4) ? f32_to_bf16_rne(bits[j]) : (uint16_t)(bits[j] >> 16);
    }
}

// One-byte elements (Int8 / RawUInt8 queues): a permutation of bytes, one thread per face row of 16.  Index tensors and
// quantized constants, a few MB at most: no row kernel.
template <bool QUEUE>
__global__ __launch_bounds__(256) void tilize_bytes_blocks(const uint8_t *__restrict__ src, TensorGeom g, uint8_t *__restrict__ dst,
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
    const bool row_inside = r < g.Rl || g.rep_r;
    const uint8_t *p = src + w * g.s0 + z * g.s1 + (uint64_t)min(r, g.Rl - 1) * g.s2;
    uint8_t *tile_out = dst + (QUEUE ? tile_offset(q, w, z, tr, tc) : tile * TB);
    if constexpr (QUEUE) {
        if (q.prefix && face_row < 2)  // header (face_row 0) and trailing pad (1) of the slot: zeros
            for (int k = 0; k < 16; ++k) (face_row ? tile_out + TB : tile_out - 16)[k] = 0;
    }
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        const bool inside = row_inside && (c + j < g.Cl || g.rep_c);
        tile_out[face_row * 16 + j] = inside ? p[(uint64_t)min(c + j, g.Cl - 1) * g.s3] : (uint8_t)0;
    }
}

hipError_t launch_bytes(const void *src, const TensorGeom &g, void *dst, const QueueLayout *q, hipStream_t stream)
{
    const uint64_t nblocks = (uint64_t)g.W * g.Z * (g.R / kTile) * (g.C / kTile) * 64;
    if (nblocks == 0) return hipSuccess;
    const uint64_t grid = (nblocks + 255) / 256;
    if (grid > 0x7fffffffull) return hipErrorInvalidValue;
    if (q)
        hipLaunchKernelGGL(tilize_bytes_blocks<true>, dim3((uint32_t)grid), dim3(256), 0, stream, (const uint8_t *)src, g, (uint8_t *)dst, nblocks, *q);
    else
        hipLaunchKernelGGL(tilize_bytes_blocks<false>, dim3((uint32_t)grid), dim3(256), 0, stream, (const uint8_t *)src, g, (uint8_t *)dst, nblocks, QueueLayout{});
    return hipGetLastError();
}

// Workgroups per CU of the row kernel.  Each holds 32 KiB of loads in flight, and on tensors of hundreds of MiB three per
// CU stream faster than the eight that LDS and registers would admit (bf16 [8,1,8192,8192] -> Bfp8_b: 254 against 275 us;
// fp32 sources 7-8 % likewise); a small grid wants them all, to cover its ramp and its tail.
inline uint32_t pack_resident(uint64_t workgroups) { return workgroups >= TTBFP_RESIDENT_MIN_GRID ? TTBFP_PACK_RESIDENT : 8; }

// ROWS_OK = false: the pair has no fast kernel (a 16-bit source widened into Float32 tiles: the full-precision mode of the
// host layer, not a conversion of the hot path) and always takes the general one.
template <typename SrcT, uint8_t DST, int ROUNDING, bool QUEUE, bool ROWS_OK = true>
hipError_t launch_kernel(const void *src, const TensorGeom &g, void *dst, const QueueLayout &q, hipStream_t stream)
{
    const uint32_t tiles_r = g.R / kTile, tiles_c = g.C / kTile;
    const uint64_t bands = (uint64_t)g.W * g.Z * tiles_r;
    if (bands == 0 || tiles_c == 0) return hipSuccess;
    // unit element stride; the row-major side aligned to its elements (the strides are, by the boundary's checks), the tiles to 16 bytes
    const bool aligned = g.s3 == sizeof(SrcT) && ((uintptr_t)src % sizeof(SrcT) == 0) && ((uintptr_t)dst % 16 == 0) &&
                         (!QUEUE || q.buffer_pitch % 16 == 0);
    constexpr int SEG_TILES = 64 * Chunk<SrcT>::kElems / kTile;
    const uint32_t segs = (tiles_c + SEG_TILES - 1) / SEG_TILES;
    // padding on the fast path: whole chunks only, and a replicated column is a column of one element
    const bool pad_ok = g.Cl % Chunk<SrcT>::kElems == 0 && !(g.rep_c && g.Cl != g.C);
    bool launched = false;
    if constexpr (ROWS_OK) {
        if (aligned && bands * segs <= 0x7fffffffull && (!g.padded() || pad_ok)) {
            const uint32_t lds_cap = resident_cap_bytes(SEG_TILES * tile_bytes(DST), pack_resident(bands * segs));
            if (g.padded())
                hipLaunchKernelGGL((tilize_pack_rows<SrcT, DST, ROUNDING, QUEUE, true>), dim3((uint32_t)(bands * segs)), dim3(256), lds_cap, stream,
                                   (const uint8_t *)src, g, (uint8_t *)dst, segs, q);
            else
                hipLaunchKernelGGL((tilize_pack_rows<SrcT, DST, ROUNDING, QUEUE, false>), dim3((uint32_t)(bands * segs)), dim3(256), lds_cap, stream,
                                   (const uint8_t *)src, g, (uint8_t *)dst, segs, q);
            launched = true;
        }
    }
    if (!launched) {
        const uint64_t nblocks = bands * tiles_c * 64;
        const uint64_t grid = (nblocks + 255) / 256;
        if (grid > 0x7fffffffull) return hipErrorInvalidValue;
        hipLaunchKernelGGL((tilize_pack_blocks<SrcT, DST, ROUNDING, QUEUE>), dim3((uint32_t)grid), dim3(256), 0, stream,
                           (const uint8_t *)src, g, (uint8_t *)dst, nblocks, q);
    }
    return hipGetLastError();
}

template <typename SrcT, uint8_t DST, int ROUNDING, bool ROWS_OK = true>
hipError_t launch(const void *src, const TensorGeom &g, void *dst, const QueueLayout *q, hipStream_t stream)
{
    if (q) return launch_kernel<SrcT, DST, ROUNDING, true, ROWS_OK>(src, g, dst, *q, stream);
    return launch_kernel<SrcT, DST, ROUNDING, false, ROWS_OK>(src, g, dst, QueueLayout{}, stream);
}

// half sources feed the A family only (pybuda/pybuda/device_connector.py:188-192)
template <int ROUNDING>
hipError_t by_format_a(uint8_t dst_fmt, const void *src, const TensorGeom &g, void *dst, const QueueLayout *q, hipStream_t s)
{
    switch (dst_fmt) {
        case kBfp8: return launch<half_t, kBfp8, ROUNDING>(src, g, dst, q, s);
        case kBfp4: return launch<half_t, kBfp4, ROUNDING>(src, g, dst, q, s);
        case kBfp2: return launch<half_t, kBfp2, ROUNDING>(src, g, dst, q, s);
        case kFloat16: return launch<half_t, kFloat16, ROUNDING>(src, g, dst, q, s);
        default: return hipErrorInvalidValue;
    }
}

template <typename SrcT, int ROUNDING>
hipError_t by_format(uint8_t dst_fmt, const void *src, const TensorGeom &g, void *dst, const QueueLayout *q, hipStream_t s)
{
    switch (dst_fmt) {
        case kBfp8_b: return launch<SrcT, kBfp8_b, ROUNDING>(src, g, dst, q, s);
        case kBfp4_b: return launch<SrcT, kBfp4_b, ROUNDING>(src, g, dst, q, s);
        case kBfp2_b: return launch<SrcT, kBfp2_b, ROUNDING>(src, g, dst, q, s);
        case kFloat16_b: return launch<SrcT, kFloat16_b, ROUNDING>(src, g, dst, q, s);
        case kFloat32:
            if constexpr (sizeof(SrcT) == 4) return launch<SrcT, kFloat32, ROUNDING>(src, g, dst, q, s);
            return launch<SrcT, kFloat32, 0, false>(src, g, dst, q, s);  // exact widening, general kernel only
        default: return hipErrorInvalidValue;
    }
}

}  // namespace

hipError_t launch_tilize_pack(const void *src, uint8_t src_fmt, const TensorGeom &g, uint8_t dst_fmt, int rounding,
                              void *dst, const QueueLayout *q, hipStream_t stream)
{
    if (src_fmt == kFloat32)
        return rounding ? by_format<float, 1>(dst_fmt, src, g, dst, q, stream) : by_format<float, 0>(dst_fmt, src, g, dst, q, stream);
    if (src_fmt == kFloat16_b)
        return rounding ? by_format<uint16_t, 1>(dst_fmt, src, g, dst, q, stream)
                        : by_format<uint16_t, 0>(dst_fmt, src, g, dst, q, stream);
    if (src_fmt == kFloat16) return rounding ? by_format_a<1>(dst_fmt, src, g, dst, q, stream) : by_format_a<0>(dst_fmt, src, g, dst, q, stream);
    if (src_fmt == kRaw8 && dst_fmt == kRaw8) return launch_bytes(src, g, dst, q, stream);
    return hipErrorInvalidValue;
}

}  // namespace ttbfp
