#include "gemm_mfma_launch.hpp"
namespace hodu {
int launch_mfma_f32(hodu_rocm_ctx *ctx, const void *a, const void *b, void *c, const DevProduct &g) {
    static const char *const names[mfma::kVariants] = HODU_MFMA_NAMES("mfma_f32");
    return mfma::launch_kind<mfma::CK_F32, mfma::SK_SAME, mfma::SK_SAME, mfma::OUT_F32>(ctx, a, b, c, g, names);
}
}  // namespace hodu
