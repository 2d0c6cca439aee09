// Y[M,N] = epilogue(X[M,K] (bf16) * dequant(W[K,N] in Bfp8_b tiles) + bias), fp32 accumulate.
// The device-side counterpart of the golden dequantize-then-matmul
// (pybuda/pybuda/op/eval/buda/matmul.py:233-249) for the operand formats the mixed-precision pass
// picks (weights Bfp8_b, activations Float16_b: pybuda/csrc/passes/amp.cpp:474-484).
//
// W stays packed in HBM (1.0625 bytes per weight) in exactly the layout the pack kernel writes:
// tiles [K/32][N/32], 64 exponent bytes + four 16x16 faces, a face row being 16 consecutive n of
// one k.  The MFMA B operand wants 8 consecutive k per lane, so a thread fetches an 8(n) x 8(k)
// patch of one face (eight 8-byte loads + the eight exponent bytes), turns every byte into bf16
// (exact: a 7-bit magnitude fits the bf16 significand) with v_cvt_f32_ubyteN + v_ldexp_f32, and
// writes eight k-contiguous 128-bit vectors into LDS.  X tiles are copied to LDS unchanged.
//
// Workgroup = WM x WN wavefronts, one per SIMD, each owning (BM/WM) x (BN/WN) of the BM x BN macro
// tile as 32x32 v_mfma_f32_32x32x16_bf16 blocks; K advances 64 at a time (a "slab" = 4 k steps of
// 16) through two LDS stages.  A lone wavefront issues one instruction at a time, so everything that
// is not an MFMA has to fit into the issue gaps between MFMAs (about five instructions per MFMA)
// and must be spread evenly: the loop is written as slots of {one MFMA + a small unit of side work}
// with the scheduler fenced at every slot boundary.
// One iteration runs from barrier to barrier and holds 4 k steps: the last k step of slab s (its
// operands were read before the barrier) and k steps 0..2 of slab s+1 - or, where a k step has so few MFMAs that
// its operands must be read two k steps ahead (Shape::AHEAD), the last two of slab s and the first two of slab s+1;
// either way an iteration reads all four k steps of slab s+1 and nothing else.  Stage s&1 is dead from the
// barrier on, so during the whole iteration
//   * X of slab s+2 goes from global memory straight into it (global_load_lds_dwordx4, no registers);
//   * W of slab s+2, fetched into registers one iteration earlier, is dequantized into it;
//   * W of slab s+3 is fetched into the other register set.
// LDS layouts (both conflict-free for the 128-bit operand reads):
//   A: [m][8 chunks of 8 k], 128-byte rows, chunk c stored at c ^ ((m ^ (m >> 3)) & 7): a wavefront's
//      direct load fills 8 whole rows, and 16 consecutive rows of one k chunk cover all 64 banks;
//   B: [k/8][n'][8 k] with n' = n ^ (((n >> 3) ^ (n >> 6)) & 7), which also spreads the vectors a
//      thread stores (consecutive n) over distinct banks.
// This kernel has no bounds tests: M % BM == 0, N % BN == 0, K % 32 == 0 and K >= 64.  N is the number of columns this
// launch computes, ldn the number of columns of the whole problem (the pitch of Y's rows and of W's tile rows): a
// problem whose N does not suit the tiles is cut into column ranges by the host, which offsets the W, Y and bias
// pointers to the range's first column.  A K that is an odd number of tile rows ends in half a slab, which is multiplied
// in a short phase of its own after the loop (no overlap: it is one tile row of W and 32 k of X).  Other shapes take
// gemm_bfp8b_general.hip.
#pragma once

#include <type_traits>

#include "bfp_codec.hpp"
#include "launch.hpp"

namespace ttbfp {

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int BK = 64;
constexpr int A_ROW = BK * 2;  // bytes per A row in LDS

// Measurement aid, never set in the library that ships (make -C tt-buda_amd/csrc ablate ABLATE=<bits> builds a copy of the
// library whose 256 x 256 kernel leaves parts of its work out, for bench.py --ablation to time): bit 0 no dequantization (the
// B stage is never written), bit 1 no X loads, bit 2 no W fetches (the dequantization then runs on whatever the registers
// hold, kept alive as opaque values), bit 3 no MFMAs, bit 4 the dequantization without its LDS stores.  The results of such
// a build are garbage; what it shows is what the rest of the kernel costs.
#ifndef TTBFP_ABLATE
#define TTBFP_ABLATE 0
#endif
constexpr uint32_t kW8Tile = tile_bytes(kBfp8_b);

// Where column n of a B stage sits inside its group of eight columns: slot (n & 7) ^ key(n / 8).  A 128-bit operand read
// takes 16 consecutive columns of one k chunk per pass and is free of bank conflicts under any key; the key is chosen for
// the stores of the dequantization.  Whole chunks (128-bit stores, one pass = column I of 16 groups): the keys of the eight
// even and of the eight odd groups must differ, which g ^ (g >> 3) gives.  Half chunks (HALF: 64-bit stores, one pass =
// columns I and I + 4 of the 8 groups of a 64-column stage, both halves): the keys of the four even and of the four odd
// groups must differ in their low two bits, which g ^ (g >> 2) gives.
template <bool HALF = false>
__device__ __forceinline__ uint32_t swizzle_key(uint32_t n) { return HALF ? ((n >> 3) ^ (n >> 5)) & 7u : ((n >> 3) ^ (n >> 6)) & 7u; }
template <bool HALF = false>
__device__ __forceinline__ uint32_t swizzle_n(uint32_t n) { return n ^ swizzle_key<HALF>(n); }

// One thread's share of a W slab: PW consecutive n x KH consecutive k of one face (KH = 8: a whole k chunk of the B
// stage; KH = 4: its lower or upper half, for tiles so narrow that a whole chunk per thread would leave threads idle).
template <int PW, int KH>
struct WPatch {
    uint32_t d[KH][PW / 4];  // d[j][c]: datums of k = j, columns 4c .. 4c+3
    uint2 e;                 // shared exponents of k = 0..3 (.x) and, with KH = 8, 4..7 (.y)
};

// Hides a value from the optimizer (no instruction is emitted).  Without it the 0x7f mask is folded
// into the byte extraction, which then no longer matches v_cvt_f32_ubyteN.
__device__ __forceinline__ uint32_t opaque(uint32_t v)
{
    asm("" : "+v"(v));
    return v;
}

template <int B>
__device__ __forceinline__ float byte_to_float(uint32_t w)
{
    return (float)((w >> (8 * B)) & 0xffu);  // v_cvt_f32_ubyteB
}

// compile-time loop: f(integral_constant<int, 0>{}) ... f(integral_constant<int, N - 1>{})
template <typename F, int... Is>
__device__ __forceinline__ void static_for_impl(F &&f, std::integer_sequence<int, Is...>)
{
    (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f)
{
    static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// Shape of one workgroup: BM x BN macro tile, WM x WN wavefronts (each owns BM/WM x BN/WN).
template <int BM_, int BN_, int WM_, int WN_, bool WDIRECT_ = false>
struct Shape {
    static constexpr int BM = BM_, BN = BN_, WM = WM_, WN = WN_;
    // the data sections of W's tiles travel by direct loads into raw areas of LDS (two-stage form; see the kernel)
    static constexpr bool WDIRECT = WDIRECT_;
    static constexpr uint32_t RAW_BYTES = WDIRECT_ ? (uint32_t)(2 * (BN_ / 32) * 1024) : 0u;  // the data of a slab's tiles
    static constexpr int NW = WM * WN, NT = 64 * NW;            // wavefronts, threads
    static constexpr int MB = BM / WM / 32, NB = BN / WN / 32;  // 32x32 blocks per wave in m and n
    static constexpr int XI = BM / 8 / NW;                      // direct X loads (8 rows each) per wave per slab
    static constexpr int PW = 8 * BN / NT >= 4 ? 8 * BN / NT : 4;  // W columns per thread per slab
    static constexpr int KH = BK * BN / NT / PW;                   // ... x KH k: 8, or 4 for narrow tiles
    static constexpr uint32_t A_BYTES = BM * A_ROW, B_BYTES = (BK / 8) * BN * 16;
    static constexpr uint32_t STAGE = A_BYTES + B_BYTES;
    static_assert(NW == 4 || NW == 8, "one or two wavefronts per SIMD");
    static_assert(MB * NB <= 16 && (NW == 4 || MB * NB <= 8), "the accumulators of a SIMD's wavefronts must fit its AGPRs");
    static_assert(PW == 4 || PW == 8, "a thread dequantizes 4 or 8 columns");
    static_assert(KH == 8 || (KH == 4 && PW == 4), "a thread dequantizes a whole k chunk, or half of one at four columns");
    static_assert(MB + NB <= 2 * MB * NB, "at most two operand reads per MFMA slot");
    // How many k steps ahead of its MFMAs a k step's operands are read from LDS.  One step is time enough where a k step has
    // four or more MFMAs (128 cycles and up); the two MFMAs of the narrowest tile are over before an LDS read comes back.
#ifndef TTBFP_AHEAD_MAX_MFMAS
#define TTBFP_AHEAD_MAX_MFMAS 2
#endif
    static constexpr int AHEAD = MB * NB <= TTBFP_AHEAD_MAX_MFMAS ? 2 : 1;
};

// ---- accumulators ------------------------------------------------------------------------------------
// The MB x NB accumulators of a wavefront (16 x 16 registers for a 128 x 128 wave tile) fill the AGPR
// half of the register file exactly.  Handed to the register allocator as ordinary values they get
// different homes in different code regions and are swapped through VGPRs or spilled inside the K
// loop, so they are kept out of its sight: accumulator i lives in a[16 i : 16 i + 15] by
// construction, the MFMAs are issued as inline assembly on those registers, and every such
// statement declares all AGPRs clobbered so that the compiler keeps nothing of its own there.
#define TTBFP_A10(n) "a" #n "0", "a" #n "1", "a" #n "2", "a" #n "3", "a" #n "4", "a" #n "5", "a" #n "6", "a" #n "7", "a" #n "8", "a" #n "9"
#define TTBFP_AGPRS_0_127                                                                                            \
    "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7", "a8", "a9", TTBFP_A10(1), TTBFP_A10(2), TTBFP_A10(3),            \
        TTBFP_A10(4), TTBFP_A10(5), TTBFP_A10(6), TTBFP_A10(7), TTBFP_A10(8), TTBFP_A10(9), TTBFP_A10(10),           \
        TTBFP_A10(11), "a120", "a121", "a122", "a123", "a124", "a125", "a126", "a127"
#define TTBFP_AGPRS_128_255                                                                                          \
    "a128", "a129", TTBFP_A10(13), TTBFP_A10(14), TTBFP_A10(15), TTBFP_A10(16), TTBFP_A10(17), TTBFP_A10(18),        \
        TTBFP_A10(19), TTBFP_A10(20), TTBFP_A10(21), TTBFP_A10(22), TTBFP_A10(23), TTBFP_A10(24), "a250", "a251",    \
        "a252", "a253", "a254", "a255"
// one statement on the accumulator registers; ALL = true: 16 accumulators (a0..a255), false: 8 (a0..a127)
#define TTBFP_ACC_ASM(ALL, TEXT, OUTS, INS)                                     \
    do {                                                                        \
        if constexpr (ALL)                                                      \
            asm volatile(TEXT : OUTS : INS : TTBFP_AGPRS_0_127, TTBFP_AGPRS_128_255); \
        else                                                                    \
            asm volatile(TEXT : OUTS : INS : TTBFP_AGPRS_0_127);                \
    } while (0)

// GUARD: an MFMA must not read a VGPR less than two wait states after a VALU instruction wrote it.
// The compiler inserts those for its own MFMAs but cannot see through this statement, and it does
// place register copies of the operands at block boundaries; the first MFMA of every k step (the one
// that can follow such a boundary) therefore carries the wait itself.
template <int IDX, bool GUARD, bool ALL>
__device__ __forceinline__ void mfma_accumulate(const bf16x8 &a, const bf16x8 &b)
{
    if constexpr ((TTBFP_ABLATE & 8) != 0) return;
#define TTBFP_MFMA_INS "v"(a), "v"(b), "n"(16 * IDX), "n"(16 * IDX + 15)
    if constexpr (GUARD)
        TTBFP_ACC_ASM(ALL, "s_nop 1\n\tv_mfma_f32_32x32x16_bf16 a[%c2:%c3], %0, %1, a[%c2:%c3]", , TTBFP_MFMA_INS);
    else
        TTBFP_ACC_ASM(ALL, "v_mfma_f32_32x32x16_bf16 a[%c2:%c3], %0, %1, a[%c2:%c3]", , TTBFP_MFMA_INS);
#undef TTBFP_MFMA_INS
}
template <int REG, bool ALL>
__device__ __forceinline__ void accumulator_clear()
{
    TTBFP_ACC_ASM(ALL, "v_accvgpr_write_b32 a%c0, 0", , "n"(REG));
}
template <int REG, bool ALL>
__device__ __forceinline__ float accumulator_read()
{
    float v;
    TTBFP_ACC_ASM(ALL, "v_accvgpr_read_b32 %0, a%c1", "=v"(v), "n"(REG));
    return v;
}
// the compiler does not know that the statements above are MFMAs: the wait between the last of them
// and the first read of its result (up to 18 cycles for a 16-pass MFMA) is spelled out
template <bool ALL>
__device__ __forceinline__ void accumulator_settle()
{
    TTBFP_ACC_ASM(ALL, "s_nop 15\n\ts_nop 15", , );
}

// 16 bytes per lane from global memory (uniform base + per-lane 32-bit offset + OFFSET) straight into
// LDS at M0 + OFFSET + lane * 16: the instruction offset applies to both addresses.  The four loads of a
// group, whose LDS destinations are 1 KiB apart, use one value of M0 and offsets 0, 1024, 2048, 3072, with the
// lane offsets prepared so that the global addresses come out right.  Every load writes M0 itself, in the same
// statement that uses it, and says so to the compiler (clobber): nothing the compiler may place between two
// statements - it is free to use M0 for its own purposes - can then send a transfer to the wrong LDS address.
// Issued as inline assembly on purpose: for the builtin the compiler cannot tell that the transfer
// and the surrounding LDS accesses never overlap and drains all outstanding loads (vmcnt(0)) before
// every following LDS instruction, which serializes the whole slab.  Completion is awaited
// explicitly with wait_direct_loads() before the barrier that publishes the stage.
// (M0 is a register the compiler reserves for itself: it warns that it will not save and restore it around the
// statement, which is not wanted here either - the clobber is there to tell it that its own copy of M0, if any, is gone.)
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
template <int OFFSET>
__device__ __forceinline__ void direct_load_16(uint64_t base, uint32_t lane_offset, uint32_t lds_base)
{
    static_assert(OFFSET >= 0 && OFFSET < 4096, "13-bit signed instruction offset");
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%c3"
                 :
                 : "v"(lane_offset), "s"(base), "s"(lds_base), "n"(OFFSET)
                 : "memory", "m0");
}
#pragma clang diagnostic pop
__device__ __forceinline__ void wait_direct_loads() { asm volatile("s_waitcnt vmcnt(0)" : : : "memory"); }
// all but the LAST most recently issued loads (loads complete in order)
template <int LAST>
__device__ __forceinline__ void wait_direct_loads_except()
{
    static_assert(LAST >= 0 && LAST < 64, "vmcnt is a 6-bit counter");
    asm volatile("s_waitcnt vmcnt(%c0)" : : "n"(LAST) : "memory");
}
// LDS stages of the panel form: three where they fit (the loads of a slab then have two iterations to
// land, which matters for the small tile, whose iteration is shorter than a trip to memory), else two
template <typename S>
constexpr int panel_stages()
{
    return 3u * S::STAGE <= 160u * 1024u ? 3 : 2;
}
__device__ __forceinline__ uint32_t lds_address(const void *p)
{
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void *)p;
}
__device__ __forceinline__ uint64_t uniform64(uint64_t v)
{
    // the builtin returns a signed int: without the unsigned casts the low half would be sign-extended
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)v);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (uint64_t)lo | ((uint64_t)hi << 32);
}

// LDS of the ring form: LA A stages, two B stages, LA raw areas (the arithmetic of the kernel's RAW_PITCH)
template <typename S, int LA>
constexpr uint32_t ring_lds_bytes()
{
    constexpr uint32_t run = (S::BN / kTile) * kW8Tile, cpw = 2 * run / 16 / S::NW, wi = (cpw + 63) / 64;
    return LA * S::A_BYTES + 2 * S::B_BYTES + LA * (2 * run + (wi * 64 - cpw) * 16);
}

// LDS of one pipeline: the rings, or two (packed W) or two to three (panel) stages
template <typename S, bool PANEL, int RING>
constexpr uint32_t pipeline_lds_bytes()
{
    if constexpr (RING > 0)
        return ring_lds_bytes<S, RING>();
    else
        return (PANEL ? panel_stages<S>() : 2) * S::STAGE + (PANEL ? 0u : 2 * S::RAW_BYTES);
}

// Bytes that the two pipelines of a workgroup exchange their partial sums through (0 with one pipeline)
template <typename S, int GROUPS>
constexpr uint32_t exchange_lds_bytes()
{
    return GROUPS == 2 ? (uint32_t)(S::MB * S::NB * S::NW * 16 * 64 * 4) : 0u;
}
// A Float16_b result leaves through LDS: the wavefronts lay the tile down row-major (16 bytes of padding per row keep the
// 2-byte stores of the two half-wavefronts, which are four rows apart, on different banks) and the whole workgroup then
// writes it out in 16-byte pieces, whole 128-byte lines at a time.
template <typename S>
constexpr uint32_t kImagePitch = S::BN * 2 + 16;
// LDS of a workgroup: what its pipelines need during the K loop, or the exchange area plus the image of the result tile
template <typename S, typename OutT, bool PANEL, int RING, int GROUPS>
constexpr uint32_t workgroup_lds_bytes()
{
    constexpr uint32_t pipes = GROUPS * pipeline_lds_bytes<S, PANEL, RING>();
    constexpr uint32_t image = sizeof(OutT) == 2 ? exchange_lds_bytes<S, GROUPS>() + S::BM * kImagePitch<S> : 0u;
    return pipes > image ? pipes : image;
}
// Two fp32 values to a pair of bf16, round to nearest even (lo in the lower half)
__device__ __forceinline__ uint32_t pack_bf16_rne(float lo, float hi)
{
    uint32_t r;
    asm("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(r) : "v"(lo), "v"(hi));
    return r;
}

// PANEL: Wp is not the packed weight but its bf16 image made by the panel pre-pass
// (gemm_bfp8b_panel.hip): for every (column of macro tiles, slab) the B_BYTES of the B stage exactly
// as the dequantization below would have left them in LDS.  The stage is then filled by direct loads
// like X, and the W fetches and the dequantization drop out of the loop.
//
// SPLITK: the grid's y dimension cuts K into gridDim.y equal runs of slabs; workgroup (tile, j) multiplies run j only
// and writes its fp32 partial tile into plane j of Y ([gridDim.y][M][N], no bias, no epilogue), for
// gemm_bfp8b_splitk.hip to add up.  For shapes whose tiles do not fill the CUs.
//
// RING (= LA, the depth of the rings; 0: off): the form for tiles whose iteration is shorter than a trip to memory (the
// 128-wide and 64-wide tiles on four wavefronts).  With two stages a slab's loads are issued and awaited inside one
// iteration, so every slab costs that trip.  Here X goes into a ring of LA A stages and the packed bytes of W - two tile
// rows of BN / 32 tiles, contiguous runs in HBM - by direct loads into a ring of LA raw areas, both LA - 2 iterations before
// anything needs them; the dequantization reads its patch out of the raw area (LDS reads, which the compiler counts apart from
// loads) into the B stage two iterations ahead as before.  All loads from memory are then direct loads in issue order,
// and the one wait per iteration names exactly how many of the youngest may stay in flight.
//
// GROUPS = 2: for launches of at most one workgroup per CU on four-wavefront tiles.  A lone wavefront per SIMD issues
// every instruction of its iteration one behind the other - some 170 per slab for the 128 x 64 tile, against 8 MFMAs - and
// that, not any unit's throughput, sets its pace.  The workgroup then holds two pipelines of S::NW wavefronts, each with
// LDS of its own, on the same macro tile: pipeline g multiplies the g-th half of K, and the two meet only at the barriers
// (both run the same number of iterations) and at the end, where the halves are added through LDS and each pipeline
// finishes half of the tile's 32 x 32 blocks.  A SIMD then has two wavefronts to issue from.
template <typename S, typename OutT, bool XCD_BLOCKS, bool PANEL = false, bool SPLITK = false, int RING = 0, int GROUPS = 1>
__global__ __launch_bounds__(S::NT * GROUPS) void gemm_bfp8b_kernel(uint32_t M, uint32_t N, uint32_t K, uint32_t ldn, int epilogue,
                                                           const uint16_t *__restrict__ X,
                                                           const uint8_t *__restrict__ Wp,
                                                           const uint16_t *__restrict__ bias, OutT *__restrict__ Y)
{
    constexpr int BM = S::BM, BN = S::BN, MB = S::MB, NB = S::NB, XI = S::XI, PW = S::PW, KH = S::KH;
    constexpr uint32_t A_BYTES = S::A_BYTES, STAGE = S::STAGE;
    extern __shared__ __attribute__((aligned(16))) uint8_t lds_all[];
    // (an odd number of blocks per wavefront is split unevenly at the end: pipeline 0 finishes the even ones, one more)
    static_assert(GROUPS == 1 || (GROUPS == 2 && S::NW == 4 && !PANEL && !SPLITK && MB * NB >= 2), "two pipelines: packed W, four wavefronts each");
    const uint32_t group = GROUPS == 1 ? 0u : (uint32_t)__builtin_amdgcn_readfirstlane(threadIdx.x / S::NT);  // pipeline of this wavefront
    uint8_t *const lds = lds_all + group * pipeline_lds_bytes<S, PANEL, RING>();

    const uint32_t tid = threadIdx.x % S::NT, lane = tid & 63;  // thread and wavefront inside the pipeline
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t wm = wave / S::WN, wn = wave % S::WN;
    // Macro tile of this workgroup.  Workgroups are dealt to the 8 XCDs round-robin and each XCD has
    // its own L2, so the tiles an XCD works on at a time should be neighbours: their X rows and W columns are then
    // fetched into that L2 once for all of them.  When the tile grid allows it (XCD_BLOCKS) the 32 tiles an XCD works on at
    // a time form a 4 (m) x 8 (n) block.  Any other grid is walked in panels of eight tile columns, down the rows inside a
    // panel, and every XCD takes one contiguous eighth of that walk (the launch rounds the grid up to a multiple of
    // eight; the workgroups past the end leave at once, before any barrier).
    uint32_t tile_m, tile_n;
    {
        const uint32_t gm = M / BM, gn = N / BN;
        const uint32_t id = blockIdx.x;
        if (XCD_BLOCKS) {
            const uint32_t block = (id / 256) * 8 + id % 8, j = (id / 8) % 32;  // block of this XCD, tile inside it
            tile_m = (block % (gm / 4)) * 4 + j / 8;
            tile_n = (block / (gm / 4)) * 8 + j % 8;
        } else if (SPLITK) {
            tile_m = id / gn;
            tile_n = id % gn;
        } else {
            const uint32_t tiles = gm * gn, share = (tiles + 7) / 8;
            const uint32_t v = (id % 8) * share + id / 8;  // place in the walk
            if (v >= tiles) return;
            const uint32_t panel = v / (gm * 8), r = v - panel * (gm * 8);
            const uint32_t width = gn - panel * 8 < 8 ? gn - panel * 8 : 8;
            tile_m = r / width;
            tile_n = panel * 8 + r % width;
        }
    }
    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;
    const uint32_t tiles_n = ldn / kTile;  // tiles in a tile row of W
    static_assert(!(SPLITK && PANEL) && (!SPLITK || sizeof(OutT) == 4), "k split: packed W, fp32 partial sums");
    static_assert(RING == 0 || (RING >= 3 && !PANEL && !SPLITK && S::NW == 4), "rings: three or more stages, packed W, four wavefronts");
    const uint32_t split = SPLITK ? blockIdx.y : group;
    const uint32_t nslabs = SPLITK ? K / BK / gridDim.y : K / BK / GROUPS;  // slabs split * nslabs .. + nslabs - 1
    if constexpr (SPLITK) Y += (uint64_t)split * M * N;

    // ---- X: direct loads.  Load i of this wave fills rows (wave XI + i) 8 .. + 7 of the stage; lane l
    // lands at row l / 8, stored chunk l % 8, so it must fetch the logical chunk that is stored there.
    // Address = uniform base of the wave's rows (advanced by one slab per iteration) + a per-lane
    // offset that is fixed for the whole K loop.
    const uint32_t lds_base = __builtin_amdgcn_readfirstlane(lds_address(lds));
    const uint64_t x_wave = uniform64((uint64_t)(uintptr_t)X + (uint64_t)(m0 + wave * XI * 8) * K * 2 + (uint64_t)split * nslabs * (BK * 2));
    uint32_t x_off[XI];  // the instruction offset 1024 (i % 4) of load i is taken out again here
#pragma unroll
    for (int i = 0; i < XI; ++i) {
        const uint32_t chunk = (lane & 7) ^ (lane >> 3) ^ ((wave * XI + i) & 7u);
        x_off[i] = (i * 8 + (lane >> 3)) * K * 2 + chunk * 16 - (i % 4) * 1024;
    }
    auto load_x = [&](uint32_t slab, uint32_t stage, auto ic) {
        constexpr int I = decltype(ic)::value;
        if constexpr ((TTBFP_ABLATE & 2) != 0) return;
        direct_load_16<(I % 4) * 1024>(x_wave + (uint64_t)slab * (BK * 2), x_off[I],
                                                   lds_base + stage * STAGE + (wave * XI + I / 4 * 4) * 8 * A_ROW);
    };

    // ---- B from a panel: the wave's share of the stage image, 1 KiB per direct load
    constexpr int BI = S::B_BYTES / S::NW / 1024;
    const uint64_t b_wave = uniform64((uint64_t)(uintptr_t)Wp + ((uint64_t)tile_n * nslabs) * S::B_BYTES + wave * (S::B_BYTES / S::NW));
    const uint32_t b_lane = lane * 16;
    auto load_b = [&](uint32_t slab, uint32_t stage, auto ic) {
        constexpr int I = decltype(ic)::value;
        direct_load_16<(I % 4) * 1024>(b_wave + (uint64_t)slab * S::B_BYTES + (I / 4) * 4096, b_lane,
                                                   lds_base + stage * STAGE + A_BYTES + wave * (S::B_BYTES / S::NW) + (I / 4) * 4096);
    };

    // ---- W: this thread's patch inside a slab: columns w_n .. w_n+PW-1, k chunk w_kc (8 k each)
    // (with KH = 4 two threads share a chunk: w_half says which four of its eight k this one holds)
    const uint32_t w_n = (tid % (BN / PW)) * PW, w_kc = tid / (BN / PW) / (8 / KH), w_half = KH == 8 ? 0 : (tid / (BN / PW)) & 1;
    const uint32_t w_face = ((w_kc >> 1) & 1) * 2 + ((w_n >> 4) & 1), w_kh = w_kc & 1;
    const uint32_t w_in_tile = w_face * 256 + w_kh * 128 + w_half * 64 + (w_n & 15);
    const uint32_t w_key = swizzle_key<KH == 4>(w_n);
    const uint32_t w_lds = A_BYTES + (w_kc * BN + (w_n & ~7u)) * 16 + w_half * 8;  // the 8-column group the patch lies in
    const uint64_t w_slab_bytes = (uint64_t)(BK / kTile) * tiles_n * kW8Tile;
    const uint8_t *w_src = Wp + ((uint64_t)(w_kc >> 2) * tiles_n + n0 / kTile + w_n / kTile) * kW8Tile + (uint64_t)split * nslabs * w_slab_bytes;

    // Two register sets, set q holding slabs of parity q: while one is dequantized into LDS the loads
    // of the following slab are in flight into the other, a whole iteration ahead of their use.
    WPatch<PW, KH> wp[2];
    if constexpr ((TTBFP_ABLATE & 4) != 0) {  // never fetched: values the optimizer cannot see through
#pragma unroll
        for (int q = 0; q < 2; ++q) {
            wp[q].e = make_uint2(opaque(0x78797a7bu), opaque(0x7a797877u));
#pragma unroll
            for (int j = 0; j < KH; ++j)
#pragma unroll
                for (int c = 0; c < PW / 4; ++c) wp[q].d[j][c] = opaque(0x01020304u * (j + 1) + lane);
        }
    }
    constexpr int WU = 1 + KH;  // fetch units per slab
    auto fetch_w = [&](uint32_t slab, auto pc, auto uc) {  // unit 0: exponents, units 1..KH: datum rows
        constexpr int P = decltype(pc)::value, U = decltype(uc)::value;
        if constexpr ((TTBFP_ABLATE & 4) != 0) return;
        const uint8_t *t = w_src + slab * w_slab_bytes;
        if constexpr (U == 0 && KH == 4) {
            wp[P].e.x = *(const uint32_t *)(t + w_face * 16 + w_kh * 8 + w_half * 4);
        } else if constexpr (U == 0) {
            wp[P].e = *(const uint2 *)(t + w_face * 16 + w_kh * 8);
        } else if constexpr (PW == 8) {
            const uint2 v = *(const uint2 *)(t + kExpSection + w_in_tile + (U - 1) * 16);
            wp[P].d[U - 1][0] = v.x;
            wp[P].d[U - 1][PW / 4 - 1] = v.y;
        } else {
            wp[P].d[U - 1][0] = *(const uint32_t *)(t + kExpSection + w_in_tile + (U - 1) * 16);
        }
    };

    // WDIRECT (two-stage form): a thread's patch is eight 4-byte pieces of eight different 16-byte face rows, so fetched
    // into registers a wavefront's load touches sixteen cache lines for 256 bytes, nine loads per slab.  Instead the
    // 1024-byte data section of every tile of the slab goes into a raw area of LDS by ONE direct load (64 lanes x 16
    // bytes, contiguous in memory), slab s + 3 during iteration s, and the threads pick their patches out of it with
    // 4-byte LDS reads at the start of iteration s + 1; only the exponent bytes still travel through registers.  Two raw
    // areas: the one slab s + 3 lands in was last read at the start of iteration s, before the barrier at its end.
    // Inside a tile's image the 16-byte rows are permuted, row c stored at c ^ key with key = 2 (tile column & 3) + (face & 1):
    // a patch read takes the same row of sixteen (tile, face) pairs, which would all sit on four banks otherwise; the
    // eight pairs of a half-wavefront get eight different keys.
    constexpr bool WDIRECT = S::WDIRECT && !PANEL && !SPLITK && RING == 0;
    constexpr uint32_t RAWD = S::RAW_BYTES, RAWD_BASE = 2 * STAGE;
    constexpr int WT = WDIRECT ? 2 * (BN / kTile) / S::NW : 1;  // tiles (direct loads) per wavefront and slab
    static_assert(!WDIRECT || (2 * (BN / kTile)) % S::NW == 0, "whole tiles per wavefront");
    static_assert(!WDIRECT || PW == 4, "a thread's patch: rows of one dword");
    uint32_t wd_off[WT];  // lane's offset from the first tile of the slab's first tile row: tile, data section, permuted row
#pragma unroll
    for (int i = 0; i < WT; ++i) {
        const uint32_t ti = wave * WT + i, tr = ti / (BN / kTile), tc = ti % (BN / kTile);
        wd_off[i] = (tr * tiles_n + tc) * kW8Tile + kExpSection + ((lane ^ (((tc & 3u) << 1) | ((lane >> 4) & 1u))) * 16);
    }
    const uint64_t wd_base = uniform64((uint64_t)(uintptr_t)Wp + (uint64_t)(n0 / kTile) * kW8Tile + (uint64_t)split * nslabs * w_slab_bytes);
    auto load_w_direct = [&](uint32_t slab, uint32_t area, auto ic) {
        constexpr int I = decltype(ic)::value;
        if constexpr ((TTBFP_ABLATE & 4) != 0) return;
        direct_load_16<0>(wd_base + (uint64_t)slab * w_slab_bytes, wd_off[I], lds_base + RAWD_BASE + area * RAWD + (wave * WT + I) * 1024);
    };
    // this thread's patch inside a raw area: tile (tile row of the slab, tile column), row group of eight, quarter of a row
    // (rows w_half * 4 + U - 1 of the group of eight; the permutation key and the half are folded into the address, the unit is XORed in)
    const uint32_t wd_patch = RAWD_BASE + ((w_kc >> 2) * (BN / kTile) + w_n / kTile) * 1024 + (w_face * 16 + w_kh * 8) * 16 + (w_n & 12u) +
                              ((((((w_n / kTile) & 3u) << 1) | (w_face & 1u)) ^ (w_half * 4)) << 4);
    auto read_w_direct = [&](uint32_t area, auto pc, auto uc) {  // unit U = 1 .. 8: row U - 1 of the patch
        constexpr int P = decltype(pc)::value, U = decltype(uc)::value;
        if constexpr ((TTBFP_ABLATE & 4) != 0) return;
        wp[P].d[U - 1][0] = *(const uint32_t *)(lds + area * RAWD + (wd_patch ^ ((U - 1) << 4)));
    };

    // ---- staging of a W register set into an LDS stage, cut into small units ----------------------
    int w_exp[KH];               // E - 133 of the patch's rows
    uint32_t w_mag[KH][PW / 4];  // datum words with the sign bits cleared
    uint32_t w_col[4];          // the column being assembled: four bf16 pairs
    auto stage_exponents = [&](auto pc) {
        constexpr int P = decltype(pc)::value;
#pragma unroll
        for (int j = 0; j < KH; ++j) w_exp[j] = (int)(((j < 4 ? wp[P].e.x : wp[P].e.y) >> (8 * (j & 3))) & 0xffu) - 133;
    };
    // The dequantization of a patch is cut into micro-steps of three to four instructions, one per
    // MFMA slot, whose operands were produced at least one slot earlier: a lone wavefront has nobody
    // to fill the issue gap behind an instruction that waits for its predecessor's result.
    // Group G = 2 I + H handles column I, rows 4 H .. 4 H + 3 (two bf16 pairs) in four micro-steps:
    //   0: mask (first column of a word only) and convert the four magnitudes;
    //   1: gather the sign bytes of both pairs, scale the first pair;
    //   2: scale the second pair, pack the first;
    //   3: pack the second pair, merge the signs, and with H == 1 store the column's eight k.
    // With KH = 4 a thread holds one half of every column: G = I, and the four k are stored as one 64-bit vector.
    constexpr int NU = 4 * (KH / 4) * PW;  // micro-steps per slab
    float q_f[4];
    uint32_t q_sgn[2], q_mag;
    auto dequant_step = [&](uint8_t *st, auto pc, auto uc) {
        constexpr int P = decltype(pc)::value, U = decltype(uc)::value;
        if constexpr ((TTBFP_ABLATE & 1) != 0) return;
        constexpr int G = U / 4, MS = U % 4, I = G / (KH / 4), H = G % (KH / 4), C = I / 4, B = I % 4, R = 4 * H;
        constexpr uint32_t SIGN_SEL = 0x000c000cu | ((uint32_t)(4 + B) << 24) | ((uint32_t)B << 8);
        if constexpr (MS == 0) {
            if constexpr (B == 0) {
#pragma unroll
                for (int j = 0; j < 4; ++j) w_mag[R + j][C] = opaque(wp[P].d[R + j][C] & 0x7f7f7f7fu);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) q_f[j] = byte_to_float<B>(w_mag[R + j][C]);
        } else if constexpr (MS == 1) {
            q_sgn[0] = __builtin_amdgcn_perm(wp[P].d[R + 1][C], wp[P].d[R][C], SIGN_SEL);
            q_sgn[1] = __builtin_amdgcn_perm(wp[P].d[R + 3][C], wp[P].d[R + 2][C], SIGN_SEL);
            q_f[0] = __builtin_amdgcn_ldexpf(q_f[0], w_exp[R]);
            q_f[1] = __builtin_amdgcn_ldexpf(q_f[1], w_exp[R + 1]);
        } else if constexpr (MS == 2) {
            q_f[2] = __builtin_amdgcn_ldexpf(q_f[2], w_exp[R + 2]);
            q_f[3] = __builtin_amdgcn_ldexpf(q_f[3], w_exp[R + 3]);
            q_mag = __builtin_amdgcn_perm(__float_as_uint(q_f[1]), __float_as_uint(q_f[0]), 0x07060302u);
        } else {
            const uint32_t mag1 = __builtin_amdgcn_perm(__float_as_uint(q_f[3]), __float_as_uint(q_f[2]), 0x07060302u);
            w_col[2 * H] = (q_sgn[0] & 0x80008000u) | q_mag;
            w_col[2 * H + 1] = (q_sgn[1] & 0x80008000u) | mag1;
            if constexpr ((TTBFP_ABLATE & 16) != 0) {  // computed, not stored
                asm volatile("" : : "v"(w_col[2 * H]), "v"(w_col[2 * H + 1]));
            } else if constexpr (KH == 4)  // this thread's four k of the column
                *(uint2 *)(st + w_lds + ((((w_n & 7u) + I) ^ w_key) * 16)) = make_uint2(w_col[0], w_col[1]);
            else if constexpr (H == 1)  // the column is complete: store its eight k as one 128-bit vector
                *(uint4 *)(st + w_lds + ((((w_n & 7u) + I) ^ w_key) * 16)) = make_uint4(w_col[0], w_col[1], w_col[2], w_col[3]);
        }
    };

    // ---- rings (RING): LDS = [LA A stages][two B stages][LA raw areas]; slab t uses A stage and raw area t % LA ---------
    constexpr int LA = RING > 0 ? RING : 2;
    constexpr uint32_t A_RING = LA * A_BYTES;
    constexpr uint32_t RUN_BYTES = (BN / kTile) * kW8Tile;           // the tiles of one tile row that the macro tile spans
    constexpr uint32_t RAW_CHUNKS = 2 * RUN_BYTES / 16;              // 16-byte pieces of a slab's two runs
    constexpr uint32_t CPW = RAW_CHUNKS / S::NW;                     // pieces per wavefront
    constexpr int WI = (CPW + 63) / 64;                              // direct loads per wavefront and slab
    // the last load of a wavefront reaches past its share: into the next wavefront's (the same bytes, fetched twice) and,
    // for the last wavefront, past the end of the area, which therefore carries that much padding
    constexpr uint32_t RAW_PITCH = 2 * RUN_BYTES + (WI * 64 - CPW) * 16;
    static_assert(RAW_CHUNKS % S::NW == 0 && RAW_PITCH % 16 == 0, "raw area: whole pieces per wavefront");
    constexpr uint32_t RAW_BASE = A_RING + 2 * S::B_BYTES;
    static_assert(RING == 0 || (PW == 4 && KH == 4), "the permutation of the raw rows is written for patches of four rows of one dword");
    uint32_t raw_off[WI];  // offset of this lane's piece from the first tile of the slab (pieces past the end: the last one again)
#pragma unroll
    for (int i = 0; i < WI; ++i) {
        const uint32_t c = wave * CPW + i * 64 + lane, cc = c < RAW_CHUNKS ? c : RAW_CHUNKS - 1;
        const uint32_t run = cc / (RUN_BYTES / 16), within = cc % (RUN_BYTES / 16);
        // inside a tile's data section the 16-byte face rows are permuted (row c lands at c ^ key, key = (face & 1) + 2 (tile
        // column & 1)): the patch reads of a half-wavefront - one row of two faces of two tiles, both halves of a k chunk -
        // then fall on 32 different banks instead of 8
        const uint32_t tile = within / (kW8Tile / 16), piece = within % (kW8Tile / 16);
        const uint32_t row = piece - kExpSection / 16;  // of the data section, if piece is past the exponents
        const uint32_t src = piece < kExpSection / 16 ? piece : kExpSection / 16 + (row ^ (((row >> 4) & 1u) | ((tile & 1u) << 1)));
        raw_off[i] = run * tiles_n * kW8Tile + (tile * (kW8Tile / 16) + src) * 16;
    }
    const uint64_t raw_wave = uniform64((uint64_t)(uintptr_t)Wp + (uint64_t)(n0 / kTile) * kW8Tile + (uint64_t)split * nslabs * w_slab_bytes);
    auto load_x_ring = [&](uint32_t slab, uint32_t slot, auto ic) {
        constexpr int I = decltype(ic)::value;
        direct_load_16<(I % 4) * 1024>(x_wave + (uint64_t)slab * (BK * 2), x_off[I], lds_base + slot * A_BYTES + (wave * XI + I / 4 * 4) * 8 * A_ROW);
    };
    auto load_raw = [&](uint32_t slab, uint32_t slot, auto ic) {
        constexpr int I = decltype(ic)::value;
        direct_load_16<0>(raw_wave + (uint64_t)slab * w_slab_bytes, raw_off[I], lds_base + RAW_BASE + slot * RAW_PITCH + (wave * CPW + I * 64) * 16);
    };
    // this thread's patch out of a raw area into register set 0: the same units as fetch_w
    const uint32_t raw_patch = (w_kc >> 2) * RUN_BYTES + (w_n / kTile) * kW8Tile;
    const uint32_t raw_key = ((w_face & 1u) | (((w_n / kTile) & 1u) << 1)) << 4;  // the row permutation above, as a byte offset
    auto fetch_w_ring = [&](uint32_t slot, auto uc) {
        constexpr int U = decltype(uc)::value;
        const uint8_t *t = lds + RAW_BASE + slot * RAW_PITCH + raw_patch;
        if constexpr (U == 0 && KH == 4) {
            wp[0].e.x = *(const uint32_t *)(t + w_face * 16 + w_kh * 8 + w_half * 4);
        } else if constexpr (U == 0) {
            wp[0].e = *(const uint2 *)(t + w_face * 16 + w_kh * 8);
        } else if constexpr (PW == 8) {
            const uint2 v = *(const uint2 *)(t + kExpSection + w_in_tile + (U - 1) * 16);
            wp[0].d[U - 1][0] = v.x;
            wp[0].d[U - 1][PW / 4 - 1] = v.y;
        } else {
            wp[0].d[U - 1][0] = *(const uint32_t *)(t + kExpSection + w_in_tile + (raw_key ^ ((U - 1) * 16)));
        }
    };

    // ---- operand fragment addresses of this lane (within a stage) ---------------------------------
    // A: row m = wm (BM/WM) + 32 mb + (lane & 31), logical chunk 2 ks + (lane >> 5).  The stored chunk is
    // chunk ^ key(m); key(m) = ((lane & 7) ^ ((lane >> 3) & 3)) ^ 4 (mb & 1), so the four values of
    // 2 ks + 4 (mb & 1) give four lane offsets and everything else is an immediate.
    const uint32_t a_row = (wm * (BM / S::WM) + (lane & 31)) * A_ROW;
    const uint32_t a_chunk = (lane >> 5) ^ (lane & 7) ^ ((lane >> 3) & 3);
    uint32_t a_off[4];
    // (a wavefront whose first 32-row block has an odd index in the tile - odd MB, odd wm - sees the two keys swapped)
    const uint32_t a_swap = MB % 2 ? 2 * (wm & 1) : 0;
#pragma unroll
    for (int v = 0; v < 4; ++v) a_off[v] = a_row + ((a_chunk ^ (2 * ((v + a_swap) & 3))) * 16);
    uint32_t b_off[NB];
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
        b_off[nb] = A_BYTES + ((lane >> 5) * BN + swizzle_n<KH == 4>(wn * (BN / S::WN) + nb * 32 + (lane & 31))) * 16;

    // Operand buffers: k step j of a slab is multiplied out of buffer j % NBUF, which is filled AHEAD k steps earlier.
    // A group of MFMA slots (four per iteration) holds the MFMAs of one k step and the operand reads of another:
    // group G reads k step G of the slab at hand and multiplies k step MUL(G) = (G - AHEAD) mod 4 - of the same slab
    // when G >= AHEAD, of the slab before (read during the previous iteration) otherwise.
    constexpr int AHEAD = S::AHEAD, NBUF = 2 * AHEAD;
    bf16x8 fa[NBUF][MB], fb[NBUF][NB];
    // operand read U (0 .. MB+NB-1) of k step KS into fragment buffer BUF
    // (sta: where the A stage begins; stb: A_BYTES before the B stage - in the two-stage forms both are the stage itself)
    auto read_one2 = [&](const uint8_t *sta, const uint8_t *stb, auto uc, auto ksc, auto bufc) {
        constexpr int U = decltype(uc)::value, KS = decltype(ksc)::value, BUF = decltype(bufc)::value;
        if constexpr (U < MB)
            fa[BUF][U] = *(const bf16x8 *)(sta + a_off[(KS + 2 * (U & 1)) & 3] + U * 32 * A_ROW);
        else if constexpr (U < MB + NB)
            fb[BUF][U - MB] = *(const bf16x8 *)(stb + b_off[U - MB] + KS * 2 * BN * 16);
    };
    auto read_one = [&](const uint8_t *st, auto uc, auto ksc, auto bufc) { read_one2(st, st, uc, ksc, bufc); };
    // the operand reads of MFMA slot U: read U, and where a k step has fewer MFMAs than operands also read U + MB NB
    auto read_frag2 = [&](const uint8_t *sta, const uint8_t *stb, auto uc, auto ksc, auto bufc) {
        constexpr int U = decltype(uc)::value;
        read_one2(sta, stb, uc, ksc, bufc);
        if constexpr (U < MB * NB) read_one2(sta, stb, std::integral_constant<int, U + MB * NB>{}, ksc, bufc);
    };
    auto read_frag = [&](const uint8_t *st, auto uc, auto ksc, auto bufc) { read_frag2(st, st, uc, ksc, bufc); };

    constexpr bool ALL_AGPRS = MB * NB > 8;
    static_for<MB * NB * 16>([&](auto rc) { accumulator_clear<decltype(rc)::value, ALL_AGPRS>(); });

    constexpr int MF = MB * NB;    // MFMAs per k step of 16
    constexpr int SLOTS = 4 * MF;  // MFMA slots per iteration
    using std::integral_constant;

    // the MFMAs of one k step on fragment buffer BUF; f(U) is the side work of slot U
    auto k_step = [&](auto bufc, auto &&side) {
        constexpr int BUF = decltype(bufc)::value;
        static_for<MF>([&](auto uc) {
            constexpr int U = decltype(uc)::value;
            mfma_accumulate<U, U == 0, ALL_AGPRS>(fa[BUF][U / NB], fb[BUF][U % NB]);  // accumulator (U / NB, U % NB)
            side(uc);
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    // Slots of the side work inside an iteration.  The nine W fetches come first and the first two
    // groups of micro-steps touch every register of the set being staged right away; the X loads
    // follow only after that, because the compiler counts outstanding loads without knowing of the
    // direct loads, and a wait it emits for a W register would then also wait for X loads issued before it.
    constexpr int TOUCHED = 1 + 4 * (SLOTS - 1) / NU + 1;  // first slot after micro-step 4
    constexpr int X_FIRST = SLOTS >= 32 && TOUCHED < 9 ? 9 : TOUCHED;
    constexpr int X_STEP = (SLOTS / 2 - X_FIRST) / XI > 1 ? (SLOTS / 2 - X_FIRST) / XI : 1;
    static_assert(X_FIRST + (XI - 1) * X_STEP < SLOTS, "every X load needs a slot");
    static_assert(WU <= SLOTS, "every W fetch needs a slot");
    constexpr int XW_STEP = (SLOTS - 1 - WT) / XI >= 2 ? 2 : 1;  // slots between the X loads of the WDIRECT form
    static_assert(!WDIRECT || 1 + WT + (XI - 1) * XW_STEP < SLOTS, "every direct load needs a slot");

    // One iteration (P = s & 1): the last AHEAD k steps of slab s, then the first 4 - AHEAD of slab s+1 (stage P^1).
    // With STAGING, slab s+2 is assembled in stage P meanwhile and a barrier publishes it at the end.
    auto iteration = [&](uint32_t s, auto pc, auto stagec) {
        constexpr int P = decltype(pc)::value;
        constexpr bool STAGING = decltype(stagec)::value;
        const uint8_t *cur = lds + (P ^ 1) * STAGE;  // slab s+1
        uint8_t *dst = lds + P * STAGE;              // slab s+2
        // slab whose W is fetched during this iteration; past the end the last slab is fetched again rather than branching
        const uint32_t w_slab = s + 3 < nslabs ? s + 3 : nslabs - 1;
        static_for<4>([&](auto gc) {
            constexpr int G = decltype(gc)::value;  // group G: MFMAs of k step (G - AHEAD) mod 4, operands of k step G are read
            k_step(integral_constant<int, ((G + 4 - AHEAD) % 4) % NBUF>{}, [&](auto uc) {
                constexpr int U = decltype(uc)::value, T = G * MF + U;
                if constexpr (U < MB + NB) read_frag(cur, uc, integral_constant<int, G>{}, integral_constant<int, G % NBUF>{});
                if constexpr (STAGING && WDIRECT) {
                    if constexpr (T == 0) {
                        // the patch of slab s + 2 out of its raw area (it landed before the barrier that ended iteration s - 1),
                        // the exponents of slab s + 3 into the other register set
                        static_for<KH>([&](auto jc) { read_w_direct(P, pc, integral_constant<int, 1 + decltype(jc)::value>{}); });
                        fetch_w(w_slab, integral_constant<int, P ^ 1>{}, integral_constant<int, 0>{});
                        stage_exponents(pc);
                    }
                    static_for<WT>([&](auto ic) {  // the data of slab s + 3 into the raw area slab s + 1 was read from an iteration ago
                        if constexpr (1 + decltype(ic)::value == T) load_w_direct(w_slab, P ^ 1, ic);
                    });
                    static_for<NU>([&](auto kc) {  // micro-steps spread evenly over slots 2 .. SLOTS - 1: the patch reads have had a slot to land
                        if constexpr (2 + decltype(kc)::value * (SLOTS - 2) / NU == T) dequant_step(dst, pc, kc);
                    });
                    static_for<XI>([&](auto ic) {
                        if constexpr (1 + WT + decltype(ic)::value * XW_STEP == T) load_x(s + 2, P, ic);
                    });
                } else if constexpr (STAGING) {
                    if constexpr (T < WU) fetch_w(w_slab, integral_constant<int, P ^ 1>{}, integral_constant<int, T>{});
                    if constexpr (T == 0) stage_exponents(pc);
                    static_for<NU>([&](auto kc) {  // micro-steps spread evenly over slots 1 .. SLOTS - 1
                        if constexpr (1 + decltype(kc)::value * (SLOTS - 1) / NU == T) dequant_step(dst, pc, kc);
                    });
                    static_for<XI>([&](auto ic) {
                        if constexpr (X_FIRST + decltype(ic)::value * X_STEP == T) load_x(s + 2, P, ic);
                    });
                }
            });
        });
        if constexpr (STAGING) {
            wait_direct_loads();
            __syncthreads();  // stage P is complete; every wave holds the operands of the last AHEAD k steps of slab s+1
        }
    };

    // The panel form of an iteration: the same four k steps on stage `cur`; both operands of slab s + NSTAGE go
    // by direct loads into stage `dst`, the one slab s has just left.  At its end slab s + 2 must have landed,
    // while the loads issued during this iteration (NSTAGE == 3) may stay in flight.
    constexpr int NSTAGE = PANEL ? panel_stages<S>() : 2;
    auto iteration_panel = [&](uint32_t s, uint32_t cur_stage, uint32_t dst_stage, auto stagec) {
        constexpr bool STAGING = decltype(stagec)::value;
        const uint8_t *cur = lds + cur_stage * STAGE;
        static_for<4>([&](auto gc) {
            constexpr int G = decltype(gc)::value;
            k_step(integral_constant<int, ((G + 4 - AHEAD) % 4) % NBUF>{}, [&](auto uc) {
                constexpr int U = decltype(uc)::value, T = G * MF + U;
                if constexpr (U < MB + NB) read_frag(cur, uc, integral_constant<int, G>{}, integral_constant<int, G % NBUF>{});
                if constexpr (STAGING) {
                    static_for<XI>([&](auto ic) {
                        if constexpr (1 + decltype(ic)::value == T) load_x(s + NSTAGE, dst_stage, ic);
                    });
                    static_for<BI>([&](auto ic) {
                        if constexpr (1 + XI + decltype(ic)::value == T) load_b(s + NSTAGE, dst_stage, ic);
                    });
                }
            });
        });
        if constexpr (STAGING)
            wait_direct_loads_except<(NSTAGE - 2) * (XI + BI)>();
        else
            wait_direct_loads();
        __syncthreads();
    };

    // The ring form of an iteration (P = s & 1): the same four k steps, A operands out of slab s + 1's A stage, B out of
    // B stage P ^ 1.  Meanwhile slab s + 2 is dequantized out of its raw area into B stage P (the patch is read in the first
    // slot, the micro-steps follow from the third on), X of slab s + LA goes into the A stage slab s has just left and the
    // raw bytes of slab s + LA + 1 into the area slab s + 1 left one iteration ago.  At the end X of slab s + 2 and the raw
    // bytes of slab s + 3 must have landed: they were issued LA - 2 iterations ago, so the loads of the iterations since
    // then - (LA - 2) (XI + WI) of them, the youngest - may stay in flight.
    constexpr int RING_FIRST = 2;  // first slot with micro-steps: the patch reads of slot 0 have had a slot to land
    auto slot_of = [&](uint32_t slab) { return slab % LA; };
    auto iteration_ring = [&](uint32_t s, auto pc, auto stagec) {
        constexpr int P = decltype(pc)::value;
        constexpr bool STAGING = decltype(stagec)::value;  // false: no slab s + 2 to dequantize
        const uint8_t *cur_a = lds + slot_of(s + 1) * A_BYTES;
        const uint8_t *cur_b = lds + A_RING + (P ^ 1) * S::B_BYTES - A_BYTES;
        uint8_t *dst_b = lds + A_RING + P * S::B_BYTES - A_BYTES;
        const uint32_t x_slab = s + LA < nslabs ? s + LA : nslabs - 1, raw_slab = s + LA + 1 < nslabs ? s + LA + 1 : nslabs - 1;
        const uint32_t a_dst = slot_of(s), raw_dst = slot_of(s + 1), raw_src = slot_of(s + 2);
        static_for<4>([&](auto gc) {
            constexpr int G = decltype(gc)::value;
            k_step(integral_constant<int, ((G + 4 - AHEAD) % 4) % NBUF>{}, [&](auto uc) {
                constexpr int U = decltype(uc)::value, T = G * MF + U;
                if constexpr (U < MB + NB) read_frag2(cur_a, cur_b, uc, integral_constant<int, G>{}, integral_constant<int, G % NBUF>{});
                if constexpr (STAGING) {
                    if constexpr (T == 0) static_for<WU>([&](auto fc) { fetch_w_ring(raw_src, fc); });
                    if constexpr (T == RING_FIRST - 1) stage_exponents(integral_constant<int, 0>{});
                    static_for<NU>([&](auto kc) {
                        if constexpr (RING_FIRST + decltype(kc)::value * (SLOTS - RING_FIRST) / NU == T) dequant_step(dst_b, integral_constant<int, 0>{}, kc);
                    });
                }
                static_for<XI>([&](auto ic) {
                    if constexpr (1 + decltype(ic)::value * ((SLOTS - 2) / (XI + WI)) == T) load_x_ring(x_slab, a_dst, ic);
                });
                static_for<WI>([&](auto ic) {
                    if constexpr (1 + (XI + decltype(ic)::value) * ((SLOTS - 2) / (XI + WI)) == T) load_raw(raw_slab, raw_dst, ic);
                });
            });
        });
        wait_direct_loads_except<(LA - 2) * (XI + WI)>();
        __syncthreads();
    };

    // prologue: slabs 0 and 1 into the two stages, W of slab 2 into register set 0, first operands
    constexpr integral_constant<int, 0> P0{};
    constexpr integral_constant<int, 1> P1{};
    constexpr integral_constant<bool, true> STAGE_ON{};
    constexpr integral_constant<bool, false> STAGE_OFF{};
    const uint32_t last = nslabs - 1;
    if constexpr (RING > 0) {
        static_assert((SLOTS - 2) / (XI + WI) >= 1 && (LA - 2) * (XI + WI) < 64, "every direct load needs a slot; vmcnt is a 6-bit counter");
        // X and the raw bytes of slabs 0 .. LA - 1 (past the end: the last slab again, unused)
        static_for<LA>([&](auto sc) {
            constexpr uint32_t SL = decltype(sc)::value;
            static_for<XI>([&](auto ic) { load_x_ring(last < SL ? last : SL, SL, ic); });
            static_for<WI>([&](auto ic) { load_raw(last < SL ? last : SL, SL, ic); });
        });
        wait_direct_loads();
        __syncthreads();
        // slabs 0 and 1 dequantized into the two B stages
        static_for<2>([&](auto sc) {
            constexpr uint32_t SL = decltype(sc)::value;
            static_for<WU>([&](auto fc) { fetch_w_ring(SL % LA, fc); });
            stage_exponents(P0);
            static_for<NU>([&](auto kc) { dequant_step(lds + A_RING + SL * S::B_BYTES - A_BYTES, P0, kc); });
        });
        __syncthreads();
        // raw area 0 is free again: slab LA (the main loop goes on with slab LA + 1 in its first iteration)
        static_for<WI>([&](auto ic) { load_raw(last < LA ? last : LA, 0, ic); });
        // the first 4 - AHEAD k steps of slab 0 (all four are read); the barrier after them frees B stage 0 for slab 2
        const uint8_t *b0 = lds + A_RING - A_BYTES;
        static_for<AHEAD>([&](auto kc) {
            static_for<MB + NB>([&](auto uc) { read_one2(lds, b0, uc, kc, integral_constant<int, decltype(kc)::value % NBUF>{}); });
        });
        static_for<4 - AHEAD>([&](auto gc) {
            constexpr int G = decltype(gc)::value;
            k_step(integral_constant<int, G % NBUF>{}, [&](auto uc) {
                if constexpr (decltype(uc)::value < MB + NB)
                    read_frag2(lds, b0, uc, integral_constant<int, G + AHEAD>{}, integral_constant<int, (G + AHEAD) % NBUF>{});
            });
        });
        __syncthreads();
        uint32_t s = 0;
        for (; s + 3 < nslabs; s += 2) {
            iteration_ring(s, P0, STAGE_ON);
            iteration_ring(s + 1, P1, STAGE_ON);
        }
        if (nslabs - s == 3) {
            iteration_ring(s, P0, STAGE_ON);
            iteration_ring(s + 1, P1, STAGE_OFF);
        } else if (nslabs - s == 2) {
            iteration_ring(s, P0, STAGE_OFF);
        }
        wait_direct_loads();  // nothing may still be on its way into LDS when the workgroup ends
    } else {
    if constexpr (PANEL) {
        static_assert(1 + XI + BI < SLOTS, "every direct load needs a slot");
        static_for<NSTAGE>([&](auto sc) {  // slabs 0 .. NSTAGE-1 (past the end: the last slab again, unused)
            constexpr uint32_t SL = decltype(sc)::value;
            static_for<XI>([&](auto ic) { load_x(last < SL ? last : SL, SL, ic); });
            static_for<BI>([&](auto ic) { load_b(last < SL ? last : SL, SL, ic); });
        });
        wait_direct_loads_except<(NSTAGE - 2) * (XI + BI)>();  // slabs 0 and 1 are needed first
    } else {
    static_for<XI>([&](auto ic) { load_x(0, 0, ic); });
    static_for<WU>([&](auto uc) { fetch_w(0, P0, uc); });
    static_for<WU>([&](auto uc) { fetch_w(last < 1 ? last : 1, P1, uc); });
    stage_exponents(P0);
    static_for<NU>([&](auto kc) { dequant_step(lds, P0, kc); });
    static_for<XI>([&](auto ic) { load_x(last < 1 ? last : 1, 1, ic); });
    stage_exponents(P1);
    static_for<NU>([&](auto kc) { dequant_step(lds + STAGE, P1, kc); });
    if constexpr (WDIRECT) {  // slab 2: its exponents into register set 0, its data into raw area 0
        fetch_w(last < 2 ? last : 2, P0, integral_constant<int, 0>{});
        static_for<WT>([&](auto ic) { load_w_direct(last < 2 ? last : 2, 0, ic); });
    } else {
        static_for<WU>([&](auto uc) { fetch_w(last < 2 ? last : 2, P0, uc); });
    }
    }
    wait_direct_loads();
    __syncthreads();
    // the first 4 - AHEAD k steps of slab 0 (all four are read); the barrier after them frees stage 0 for slab 2
    static_for<AHEAD>([&](auto kc) {
        static_for<MB + NB>([&](auto uc) { read_one(lds, uc, kc, integral_constant<int, decltype(kc)::value % NBUF>{}); });
    });
    static_for<4 - AHEAD>([&](auto gc) {
        constexpr int G = decltype(gc)::value;
        k_step(integral_constant<int, G % NBUF>{}, [&](auto uc) {
            if constexpr (decltype(uc)::value < MB + NB)
                read_frag(lds, uc, integral_constant<int, G + AHEAD>{}, integral_constant<int, (G + AHEAD) % NBUF>{});
        });
    });
    __syncthreads();

    // iterations s = 0 .. nslabs-2; the ones with s + 2 < nslabs stage a slab
    uint32_t s = 0;
    if constexpr (PANEL) {
        uint32_t stage = 0;  // s % NSTAGE
        auto next = [&](uint32_t st) { return st + 1 == NSTAGE ? 0u : st + 1; };
        for (; s + NSTAGE < nslabs; ++s, stage = next(stage)) iteration_panel(s, next(stage), stage, STAGE_ON);
        for (; s + 1 < nslabs; ++s, stage = next(stage)) iteration_panel(s, next(stage), stage, STAGE_OFF);
    } else {
    for (; s + 3 < nslabs; s += 2) {
        iteration(s, P0, STAGE_ON);
        iteration(s + 1, P1, STAGE_ON);
    }
    if (nslabs - s == 3) {
        iteration(s, P0, STAGE_ON);
        iteration(s + 1, P1, STAGE_OFF);
    } else if (nslabs - s == 2) {
        iteration(s, P0, STAGE_OFF);
    }
    }
    }
    static_for<AHEAD>([&](auto jc) {  // the last AHEAD k steps of the last slab
        k_step(integral_constant<int, (4 - AHEAD + decltype(jc)::value) % NBUF>{}, [&](auto) {});
    });

    // ---- half a slab at the end of K (K an odd number of tile rows): k rows K - 32 .. K - 1 ------------------------------
    // Stage 0 of the first pipeline takes the 32 k of X (the chunks of its upper half are filled with copies and never
    // read) and the one tile row of W that is left; two k steps multiply them.  Nothing here overlaps: it runs once.
    if constexpr (!PANEL && !SPLITK) {
        if (K % BK) {  // uniform
            __syncthreads();  // every wavefront has read its last operands out of the stages
            if (group == 0) {
                const uint32_t tail_slab = K / BK;
                const uint64_t x_rows = uniform64((uint64_t)(uintptr_t)X + (uint64_t)(m0 + wave * XI * 8) * K * 2 + (uint64_t)tail_slab * (BK * 2));
                static_for<XI>([&](auto ic) {
                    constexpr int I = decltype(ic)::value;
                    const uint32_t chunk = (lane & 7) ^ (lane >> 3) ^ ((wave * XI + I) & 7u);  // the logical chunk this lane's piece stands for
                    const uint32_t off = (I * 8 + (lane >> 3)) * K * 2 + (chunk & 3u) * 16 - (I % 4) * 1024;  // chunks 4 .. 7 lie past the row: chunk - 4 again
                    direct_load_16<(I % 4) * 1024>(x_rows, off, lds_base + (wave * XI + I / 4 * 4) * 8 * A_ROW);
                });
                uint8_t *const b_stage = RING > 0 ? lds + A_RING - A_BYTES : lds;
                if ((w_kc >> 2) == 0) {  // the threads whose patch lies in the slab's first tile row; the second does not exist
                    const uint32_t w_tail_slab = tail_slab - split * nslabs;  // w_src starts at this pipeline's first slab
                    static_for<WU>([&](auto uc) { fetch_w(w_tail_slab, P0, uc); });
                    stage_exponents(P0);
                    static_for<NU>([&](auto kc) { dequant_step(b_stage, P0, kc); });
                }
                wait_direct_loads();
            }
            __syncthreads();
            if (group == 0) {
                uint8_t *const b_stage = RING > 0 ? lds + A_RING - A_BYTES : lds;
                static_for<2>([&](auto kc) {
                    static_for<MB + NB>([&](auto uc) { read_one2(lds, b_stage, uc, kc, kc); });
                });
                static_for<2>([&](auto kc) { k_step(kc, [&](auto) {}); });
            }
        }
    }

    // D layout of the 32x32 MFMA: register r of lane l holds row 8*(r/4) + 4*(l/32) + r%4, column l%32
    accumulator_settle<ALL_AGPRS>();
    // two pipelines: block BLK is finished by pipeline BLK % 2, which gets the other one's partial sums through LDS
    // ([block][wavefront][register][lane] floats over the start of the workgroup's LDS, which nobody reads any more)
    float *const exchange = (float *)lds_all;
    auto exchange_at = [&](int blk, int r) { return exchange + ((blk * S::NW + wave) * 16 + r) * 64 + lane; };
    if constexpr (GROUPS == 2) {
        static_assert(exchange_lds_bytes<S, GROUPS>() <= 2 * pipeline_lds_bytes<S, PANEL, RING>(), "the exchange fits the workgroup's LDS");
        __syncthreads();  // both pipelines have read their last operands
        static_for<MB * NB>([&](auto bc) {
            constexpr int BLK = decltype(bc)::value;
            if ((BLK & 1) != (int)group)
                static_for<16>([&](auto rc) { *exchange_at(BLK, decltype(rc)::value) = accumulator_read<16 * BLK + decltype(rc)::value, ALL_AGPRS>(); });
        });
        __syncthreads();
    }
    constexpr bool STAGED = sizeof(OutT) == 2;  // a bf16 result is assembled in LDS and written out in whole lines
    constexpr uint32_t PITCH = kImagePitch<S>;
    uint8_t *const image = lds_all + exchange_lds_bytes<S, GROUPS>();
    if constexpr (STAGED && GROUPS == 1) __syncthreads();  // every wavefront has read its last operands (two pipelines: the barriers above)
    // The activation is chosen once for the whole tile, not per element: straight-line code lets the compiler interleave the
    // independent chains of a lane's values (a reciprocal and an exponential each) instead of finishing them one by one.
    auto finish_blocks = [&](auto actc) {
    constexpr int ACTIVATION = decltype(actc)::value;
    static_for<MB * NB>([&](auto bc) {
        constexpr int BLK = decltype(bc)::value, mb = BLK / NB, nb = BLK % NB;
        if (GROUPS == 2 && (BLK & 1) != (int)group) return;
        const uint32_t col_in_tile = wn * (BN / S::WN) + nb * 32 + (lane & 31);
        const uint32_t row_in_tile = wm * (BM / S::WM) + mb * 32 + (lane >> 5) * 4;
        const float bv = bias ? load_bias(bias, n0 + col_in_tile, epilogue & kEpilogueBiasF32) : 0.0f;
        // The block's sixteen values leave the accumulators first (statements the compiler keeps in order), then bias and
        // activation are applied to all of them in ordinary code: sixteen independent chains to interleave.
        float v[16];
        static_for<16>([&](auto rc) { v[decltype(rc)::value] = accumulator_read<16 * BLK + decltype(rc)::value, ALL_AGPRS>(); });
        if constexpr (GROUPS == 2) {
#pragma unroll
            for (int r = 0; r < 16; ++r) v[r] += *exchange_at(BLK, r);
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) v[r] = apply_epilogue(ACTIVATION, v[r] + bv);
        if constexpr (STAGED) {
            uint8_t *ip = image + row_in_tile * PITCH + col_in_tile * 2;
#pragma unroll
            for (int r0 = 0; r0 < 16; r0 += 2) {
                const uint32_t rr0 = (r0 >> 2) * 8 + (r0 & 3), rr1 = rr0 + 1;  // rows inside the block, before the lane's 4-row offset
                const uint32_t pair = pack_bf16_rne(v[r0], v[r0 + 1]);
                *(uint16_t *)(ip + rr0 * PITCH) = (uint16_t)pair;
                *(uint16_t *)(ip + rr1 * PITCH) = (uint16_t)(pair >> 16);
            }
        } else {
            OutT *yp = Y + (uint64_t)(m0 + row_in_tile) * ldn + n0 + col_in_tile;
#pragma unroll
            for (int r = 0; r < 16; ++r) yp[(uint64_t)((r >> 2) * 8 + (r & 3)) * ldn] = v[r];
        }
    });
    };
    if constexpr ((TTBFP_ABLATE & 64) == 0)
    switch (epilogue & kEpilogueMask) {  // uniform
        case 1: finish_blocks(integral_constant<int, 1>{}); break;
        case 2: finish_blocks(integral_constant<int, 2>{}); break;
        default: finish_blocks(integral_constant<int, 0>{}); break;
    }
    if constexpr (STAGED) {
        __syncthreads();
        constexpr int LPR = BN * 2 / 16;                // lanes per row of the tile: 16 bytes each
        constexpr int RPP = S::NT * GROUPS / LPR;       // rows per pass of the whole workgroup
        static_assert(BM % RPP == 0, "whole passes");
        const uint32_t row = threadIdx.x / LPR, piece = threadIdx.x % LPR;
        const uint8_t *from = image + row * PITCH + piece * 16;
        uint8_t *to = (uint8_t *)Y + ((uint64_t)(m0 + row) * ldn + n0) * 2 + piece * 16;
        const uint64_t step = (uint64_t)RPP * ldn * 2;
        if constexpr ((TTBFP_ABLATE & 32) == 0)
        static_for<BM / RPP>([&](auto pc) {
            constexpr int PASS = decltype(pc)::value;
            *(uint4 *)(to + PASS * step) = *(const uint4 *)(from + PASS * RPP * PITCH);
        });
    }
}

template <typename S, typename OutT, bool XCD_BLOCKS, bool PANEL, int GROUPS = 1>
hipError_t launch_tile(uint32_t M, uint32_t N, uint32_t K, uint32_t ldn, const void *x, const void *w, const void *bias, int epilogue,
                       void *y, hipStream_t stream)
{
    constexpr uint32_t smem = workgroup_lds_bytes<S, OutT, PANEL, 0, GROUPS>();
    static_assert(smem <= 160 * 1024, "LDS of a CU");
    if (GROUPS > 1 && (K / BK) % GROUPS) return hipErrorInvalidValue;
    auto kernel = gemm_bfp8b_kernel<S, OutT, XCD_BLOCKS, PANEL, false, 0, GROUPS>;
    if (hipError_t e = allow_dynamic_lds(kernel, smem); e != hipSuccess) return e;
    const uint64_t tiles = (uint64_t)(N / S::BN) * (M / S::BM);
    if (tiles > 0x7ffffff0ull) return hipErrorInvalidValue;
    const uint32_t grid = XCD_BLOCKS ? (uint32_t)tiles : (uint32_t)((tiles + 7) / 8 * 8);  // the walk in eighths: see the kernel
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(S::NT * GROUPS), smem, stream, M, N, K, ldn, epilogue, (const uint16_t *)x,
                       (const uint8_t *)w, (const uint16_t *)bias, (OutT *)y);
    return hipGetLastError();
}

template <typename S, typename OutT, bool XCD_BLOCKS, int LA, int GROUPS = 1>
hipError_t launch_tile_ring(uint32_t M, uint32_t N, uint32_t K, uint32_t ldn, const void *x, const void *w, const void *bias, int epilogue,
                            void *y, hipStream_t stream)
{
    constexpr uint32_t smem = workgroup_lds_bytes<S, OutT, false, LA, GROUPS>();
    static_assert(smem <= 160 * 1024, "LDS of a CU");
    if (GROUPS > 1 && (K / BK) % GROUPS) return hipErrorInvalidValue;
    auto kernel = gemm_bfp8b_kernel<S, OutT, XCD_BLOCKS, false, false, LA, GROUPS>;
    if (hipError_t e = allow_dynamic_lds(kernel, smem); e != hipSuccess) return e;
    const uint64_t tiles = (uint64_t)(N / S::BN) * (M / S::BM);
    if (tiles > 0x7ffffff0ull) return hipErrorInvalidValue;
    const uint32_t grid = XCD_BLOCKS ? (uint32_t)tiles : (uint32_t)((tiles + 7) / 8 * 8);
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(S::NT * GROUPS), smem, stream, M, N, K, ldn, epilogue, (const uint16_t *)x,
                       (const uint8_t *)w, (const uint16_t *)bias, (OutT *)y);
    return hipGetLastError();
}

template <typename S, typename OutT, int LA, int GROUPS = 1>
hipError_t launch_shape_ring(uint32_t M, uint32_t N, uint32_t K, uint32_t ldn, const void *x, const void *w, const void *bias, int epilogue,
                             void *y, hipStream_t stream)
{
    const uint32_t gm = M / S::BM, gn = N / S::BN;
    if (gm % 4 == 0 && gn % 8 == 0 && ((gm / 4) * (gn / 8)) % 8 == 0)
        return launch_tile_ring<S, OutT, true, LA, GROUPS>(M, N, K, ldn, x, w, bias, epilogue, y, stream);
    return launch_tile_ring<S, OutT, false, LA, GROUPS>(M, N, K, ldn, x, w, bias, epilogue, y, stream);
}

// k split: `splits` workgroups per tile, fp32 partial planes [splits][M][N] at `partials`
template <typename S>
hipError_t launch_tile_splitk(uint32_t M, uint32_t N, uint32_t K, uint32_t splits, const void *x, const void *w, float *partials,
                              hipStream_t stream)
{
    constexpr uint32_t smem = 2 * S::STAGE;
    auto kernel = gemm_bfp8b_kernel<S, float, false, false, true>;
    if (hipError_t e = allow_dynamic_lds(kernel, smem); e != hipSuccess) return e;
    const uint64_t tiles = (uint64_t)(N / S::BN) * (M / S::BM);
    if (tiles > 0x7fffffffull || splits == 0 || splits > 65535 || K % BK || (K / BK) % splits) return hipErrorInvalidValue;
    hipLaunchKernelGGL(kernel, dim3((uint32_t)tiles, splits), dim3(S::NT), smem, stream, M, N, K, N, 0, (const uint16_t *)x,
                       (const uint8_t *)w, (const uint16_t *)nullptr, partials);
    return hipGetLastError();
}

// true if the shape fits the macro-tiled kernel with shape S
template <typename S>
bool fits(uint32_t M, uint32_t N, uint32_t K)
{
    return M % S::BM == 0 && N % S::BN == 0 && K % kTile == 0 && K >= BK && K <= (1u << 24);  // 32-bit X offsets inside a wave's rows
}

template <typename S, typename OutT, bool PANEL = false, int GROUPS = 1>
hipError_t launch_shape(uint32_t M, uint32_t N, uint32_t K, uint32_t ldn, const void *x, const void *w, const void *bias, int epilogue,
                        void *y, hipStream_t stream)
{
    if (PANEL && (K % BK || ldn != N)) return hipErrorInvalidValue;  // the panel is made for whole slabs of the whole weight
    // 4 x 8 blocks of tiles per XCD need a whole number of rounds of 8 blocks
    const uint32_t gm = M / S::BM, gn = N / S::BN;
    if (gm % 4 == 0 && gn % 8 == 0 && ((gm / 4) * (gn / 8)) % 8 == 0)
        return launch_tile<S, OutT, true, PANEL, GROUPS>(M, N, K, ldn, x, w, bias, epilogue, y, stream);
    return launch_tile<S, OutT, false, PANEL, GROUPS>(M, N, K, ldn, x, w, bias, epilogue, y, stream);
}

}  // namespace

// The macro-tile shapes in use.  Each (shape, output type) pair is compiled in a translation unit
// of its own (gemm_bfp8b_<shape>_<type>.hip) so that the build can run them in parallel.
#ifndef TTBFP_BIG_WDIRECT
#define TTBFP_BIG_WDIRECT true
#endif
#ifndef TTBFP_BIG_SHAPE
#define TTBFP_BIG_SHAPE Shape<256, 256, 2, 4, TTBFP_BIG_WDIRECT>
#endif
using BigShape = TTBFP_BIG_SHAPE;
using SmallShape = Shape<128, 128, 2, 2>;
// Half as wide: twice the workgroups for shapes whose 128 x 128 tiles leave CUs idle, and half the weights to dequantize
// per workgroup and slab (a thread holds four k of four columns); three of them fit a CU.
using SlimShape = Shape<128, 64, 2, 2>;
// Three tile rows of 128 in one: M = 3072 (24 tile rows of 128) at N = 4096 gives 8 x 32 = 256 workgroups, one per CU, where
// 256 x 256 tiles give 192.  Eight wavefronts, wave tile 96 x 64 (five operand reads for the six MFMAs of a k step; as 192 x 32
// it would be seven: 3072 x 4096 x 4096 94-97 against 98-103 us).
using TallShape = Shape<384, 128, 4, 2>;
// One and a half tile rows of 128, half the width: M = 3072 at N = 1024 gives 16 x 16 = 256 workgroups, one per CU, where 128 x 128
// tiles give 192.  Four wavefronts 2 x 2 (wave tile 96 x 32), two pipelines per workgroup: a thread dequantizes 16 weights
// per slab for the wavefront's 12 MFMAs, where the 128 x 128 tile has 32 for 16.
using LeanShape = Shape<192, 64, 2, 2>;

// true if the problem can be cut into macro tiles of shape S
template <typename S>
inline bool gemm_fits(uint32_t M, uint32_t N, uint32_t K)
{
    return fits<S>(M, N, K);
}

// defined by the per-shape translation units; y_is_fp32 selects the Float32 (else Float16_b) output
#define TTBFP_DECLARE_GEMM(NAME)                                                                                        \
    hipError_t launch_gemm_bfp8b_##NAME(uint32_t M, uint32_t N, uint32_t K, uint32_t ldn, const void *x, const void *w, const void *bias, \
                                        int epilogue, void *y, hipStream_t stream)
TTBFP_DECLARE_GEMM(big_f32);
TTBFP_DECLARE_GEMM(big_bf16);
TTBFP_DECLARE_GEMM(small_f32);
TTBFP_DECLARE_GEMM(small_bf16);
TTBFP_DECLARE_GEMM(slim_f32);
TTBFP_DECLARE_GEMM(slim_bf16);
TTBFP_DECLARE_GEMM(tall_f32);
TTBFP_DECLARE_GEMM(tall_bf16);
TTBFP_DECLARE_GEMM(ring_slim_f32);  // SlimShape in the ring form
TTBFP_DECLARE_GEMM(ring_slim_bf16);
TTBFP_DECLARE_GEMM(duo_slim_f32);  // SlimShape in the ring form, two pipelines per workgroup (K a multiple of 128)
TTBFP_DECLARE_GEMM(duo_slim_bf16);
TTBFP_DECLARE_GEMM(duo_small_f32);  // SmallShape on two stages, two pipelines per workgroup
TTBFP_DECLARE_GEMM(duo_small_bf16);
TTBFP_DECLARE_GEMM(duo_lean_f32);  // LeanShape on two stages, two pipelines per workgroup
TTBFP_DECLARE_GEMM(duo_lean_bf16);
TTBFP_DECLARE_GEMM(panel_f32);   // BigShape on a bf16 panel of W instead of the packed tiles
TTBFP_DECLARE_GEMM(panel_bf16);
TTBFP_DECLARE_GEMM(panel_small_f32);  // SmallShape on a panel made for 128-wide tiles
TTBFP_DECLARE_GEMM(panel_small_bf16);
#define TTBFP_DEFINE_PANEL_GEMM(NAME, SHAPE, OUT_T)                                                                    \
    TTBFP_DECLARE_GEMM(NAME) { return launch_shape<SHAPE, OUT_T, true>(M, N, K, ldn, x, w, bias, epilogue, y, stream); }
#define TTBFP_DEFINE_RING_GEMM(NAME, SHAPE, OUT_T, LA)                                                                 \
    TTBFP_DECLARE_GEMM(NAME) { return launch_shape_ring<SHAPE, OUT_T, LA>(M, N, K, ldn, x, w, bias, epilogue, y, stream); }
#define TTBFP_DEFINE_DUO_GEMM(NAME, SHAPE, OUT_T, LA)                                                                  \
    TTBFP_DECLARE_GEMM(NAME) { return launch_shape_ring<SHAPE, OUT_T, LA, 2>(M, N, K, ldn, x, w, bias, epilogue, y, stream); }
#define TTBFP_DEFINE_DUO_STAGED_GEMM(NAME, SHAPE, OUT_T)                                                               \
    TTBFP_DECLARE_GEMM(NAME) { return launch_shape<SHAPE, OUT_T, false, 2>(M, N, K, ldn, x, w, bias, epilogue, y, stream); }
#define TTBFP_DEFINE_GEMM(NAME, SHAPE, OUT_T)                                                                          \
    TTBFP_DECLARE_GEMM(NAME) { return launch_shape<SHAPE, OUT_T>(M, N, K, ldn, x, w, bias, epilogue, y, stream); }

}  // namespace ttbfp
