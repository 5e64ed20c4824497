// int8 contraction kernel, tile shape 128 x 32 (wavefronts 4 x 1): see gemm_i8_kernel.hpp
#include "gemm_i8_kernel.hpp"

namespace mlel {
MLEL_DEFINE_GEMM_TILE(5, 128, 32, 4, 1)
}  // namespace mlel
