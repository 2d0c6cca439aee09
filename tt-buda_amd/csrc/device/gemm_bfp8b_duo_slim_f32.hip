// Bfp8_b-weight GEMM, macro tile SlimShape in the ring form with two pipelines per workgroup, Float32 output: see gemm_bfp8b_kernel.hpp.
#include "gemm_bfp8b_kernel.hpp"

#ifndef TTBFP_DUO_RING_DEPTH
#define TTBFP_DUO_RING_DEPTH 3  // two pipelines of this depth fill the LDS of a CU
#endif

namespace ttbfp {
TTBFP_DEFINE_DUO_GEMM(duo_slim_f32, SlimShape, float, TTBFP_DUO_RING_DEPTH)
}  // namespace ttbfp
