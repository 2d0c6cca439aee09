// Bfp8_b-weight GEMM, macro tile TallShape, Float16_b output: see gemm_bfp8b_kernel.hpp.
#include "gemm_bfp8b_kernel.hpp"

namespace ttbfp {
TTBFP_DEFINE_GEMM(tall_bf16, TallShape, uint16_t)
}  // namespace ttbfp
