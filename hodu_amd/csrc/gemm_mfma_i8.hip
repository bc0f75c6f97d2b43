// i8 x i8 -> i32 on v_mfma_i32_16x16x64_i8: exact integer arithmetic, wrap-around i32 accumulate.
#include "gemm_mfma_launch.hpp"
namespace hodu {
int launch_mfma_i8(hodu_rocm_ctx *ctx, const void *a, const void *b, void *c, const DevProduct &g) {
    static const char *const names[mfma::kVariants] = HODU_MFMA_NAMES("mfma_i32_i8i8");
    return mfma::launch_kind<mfma::CK_I8, mfma::SK_SAME, mfma::SK_SAME, mfma::OUT_I32>(ctx, a, b, c, g, names);
}
}  // namespace hodu
