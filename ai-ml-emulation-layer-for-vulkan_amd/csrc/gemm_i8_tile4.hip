// int8 contraction kernel, tile shape 64 x 64 (wavefronts 2 x 2): see gemm_i8_kernel.hpp
#include "gemm_i8_kernel.hpp"

namespace mlel {
MLEL_DEFINE_GEMM_TILE(4, 64, 64, 2, 2)
}  // namespace mlel
