// bf16 activations x f8e4m3 weights -> bf16: the weight's to_dtype(bf16) happens between the global
// load and the LDS store.
#include "gemm_mfma_launch.hpp"
namespace hodu {
int launch_mfma_w8a16(hodu_rocm_ctx *ctx, const void *a, const void *b, void *c, const DevProduct &g) {
    static const char *const names[mfma::kVariants] = HODU_MFMA_NAMES("mfma_bf16_f8w");
    return mfma::launch_kind<mfma::CK_BF16, mfma::SK_SAME, mfma::SK_F8, mfma::OUT_BF16>(ctx, a, b, c, g, names);
}
}  // namespace hodu
