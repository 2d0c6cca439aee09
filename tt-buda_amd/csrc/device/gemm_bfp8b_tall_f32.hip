// Bfp8_b-weight GEMM, macro tile TallShape, Float32 output: see gemm_bfp8b_kernel.hpp.
#include "gemm_bfp8b_kernel.hpp"

namespace ttbfp {
TTBFP_DEFINE_GEMM(tall_f32, TallShape, float)
}  // namespace ttbfp
