// The f16 instantiations of the 256 x 256 tile on the 16 x 16 x 32 instruction (gemm_mfma_pipe16.hpp).
#define HODU_MI16_DEFINE_HERE 1
#include "gemm_mfma_launch.hpp"
