// Bfp8_b-weight GEMM, macro tile SlimShape in the ring form, Float32 output: see gemm_bfp8b_kernel.hpp.
#include "gemm_bfp8b_kernel.hpp"

#ifndef TTBFP_RING_DEPTH
#define TTBFP_RING_DEPTH 4  // measured at 512 x 4096 x 4096: 3 stages 42 us, 4 38 us, 5 40 us (two stages: 49 us)
#endif

namespace ttbfp {
TTBFP_DEFINE_RING_GEMM(ring_slim_f32, SlimShape, float, TTBFP_RING_DEPTH)
}  // namespace ttbfp
