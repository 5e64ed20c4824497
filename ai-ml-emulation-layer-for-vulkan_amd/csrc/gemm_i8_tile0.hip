// int8 contraction kernel, tile shape 128 x 128 (wavefronts 2 x 2): see gemm_i8_kernel.hpp
#include "gemm_i8_kernel.hpp"

namespace mlel {
MLEL_DEFINE_GEMM_TILE(0, 128, 128, 2, 2)
}  // namespace mlel
