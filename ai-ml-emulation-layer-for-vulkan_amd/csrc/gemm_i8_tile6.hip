// int8 contraction kernel, tile shape 256 x 256 (wavefronts 2 x 4): see gemm_i8_kernel.hpp
#include "gemm_i8_kernel.hpp"

namespace mlel {
MLEL_DEFINE_GEMM_TILE(6, 256, 256, 2, 4)
}  // namespace mlel
