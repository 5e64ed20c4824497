// int8 contraction kernel, tile shape 64 x 128 (wavefronts 1 x 4): see gemm_i8_kernel.hpp
#include "gemm_i8_kernel.hpp"

namespace mlel {
MLEL_DEFINE_GEMM_TILE(3, 64, 128, 1, 4)
}  // namespace mlel
