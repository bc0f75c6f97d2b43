// i8 x i8 -> i8 and u8 x u8 -> u8 on the i8 matrix instruction: hodu's 8-bit integer matmul / dot wrap around
// (crates/hodu_cpu_kernels/kernels/ops_matrix.c:355, :359, :717, :721: the accumulator has the operands' type), which
// is the low byte of the exact i32 sum the matrix core delivers.  (One file per output type: they compile side by side.)
#include "gemm_mfma_launch.hpp"
namespace hodu {
int launch_mfma_i8_out(hodu_rocm_ctx *ctx, const void *a, const void *b, void *c, const DevProduct &g) {
    static const char *const names[mfma::kVariants] = HODU_MFMA_NAMES("mfma_i8");
    return mfma::launch_kind<mfma::CK_I8, mfma::SK_SAME, mfma::SK_SAME, mfma::OUT_I8>(ctx, a, b, c, g, names);
}
}  // namespace hodu
