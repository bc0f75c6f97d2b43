#include "gemm_mfma_launch.hpp"
namespace hodu {
int launch_mfma_bf16(hodu_rocm_ctx *ctx, const void *a, const void *b, void *c, const DevProduct &g) {
    static const char *const names[mfma::kVariants] = HODU_MFMA_NAMES("mfma_bf16");
    return mfma::launch_kind<mfma::CK_BF16, mfma::SK_SAME, mfma::SK_SAME, mfma::OUT_BF16>(ctx, a, b, c, g, names);
}
}  // namespace hodu
