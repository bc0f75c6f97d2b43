// Test input (tests/test_isa_hazards_cpu.py): the f8e4m3-weight forms of the 16 x 16 x 32 tile kernels alone, so that
// their generated code can be read without compiling the whole translation unit they ship in (gemm_mfma_w8a16.hip,
// minutes).  Same headers, same configurations as gemm_mfma_launch.hpp instantiates.
#include "gemm_mfma_pipe16.hpp"

namespace hodu {
namespace mfma {
#define F8W_CONFIG(LB) PipeConfig<CK_BF16, OUT_BF16, 256, 256, 2, 2, LM_K, LB, SK_F8, 2>
template int launch_pipe16_f8w<F8W_CONFIG(LM_K)>(hodu_rocm_ctx *, const void *, const void *, void *, const DevProduct &);
template int launch_pipe16_f8w<F8W_CONFIG(LM_MN)>(hodu_rocm_ctx *, const void *, const void *, void *, const DevProduct &);
template int launch_pipe16r_f8w<F8W_CONFIG(LM_K)>(hodu_rocm_ctx *, const void *, const void *, void *, const DevProduct &);
template int launch_pipe16r_f8w<F8W_CONFIG(LM_MN)>(hodu_rocm_ctx *, const void *, const void *, void *, const DevProduct &);
}  // namespace mfma
}  // namespace hodu
