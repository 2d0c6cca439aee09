// Bfp8_b-weight GEMM, macro tile LeanShape on two stages with two pipelines per workgroup, Float16_b output: see gemm_bfp8b_kernel.hpp.
#include "gemm_bfp8b_kernel.hpp"

namespace ttbfp {
TTBFP_DEFINE_DUO_STAGED_GEMM(duo_lean_bf16, LeanShape, uint16_t)
}  // namespace ttbfp
