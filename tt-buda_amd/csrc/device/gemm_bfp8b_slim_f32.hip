// Bfp8_b-weight GEMM, macro tile SlimShape (128 x 64), Float32 output: see gemm_bfp8b_kernel.hpp.
#include "gemm_bfp8b_kernel.hpp"

namespace ttbfp {
TTBFP_DEFINE_GEMM(slim_f32, SlimShape, float)
}  // namespace ttbfp
