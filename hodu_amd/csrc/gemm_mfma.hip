// Routes a product to the MFMA tile kernel of its dtype, if there is one.
#include "common.hpp"
namespace hodu {
int launch_mfma_bf16(hodu_rocm_ctx *, const void *, const void *, void *, const DevProduct &);
int launch_mfma_f16(hodu_rocm_ctx *, const void *, const void *, void *, const DevProduct &);
int launch_mfma_w8a16(hodu_rocm_ctx *, const void *, const void *, void *, const DevProduct &);
int launch_mfma_i8(hodu_rocm_ctx *, const void *, const void *, void *, const DevProduct &);
int launch_mfma_f32(hodu_rocm_ctx *, const void *, const void *, void *, const DevProduct &);
int launch_mfma_i8_out(hodu_rocm_ctx *, const void *, const void *, void *, const DevProduct &);
int launch_mfma_u8_out(hodu_rocm_ctx *, const void *, const void *, void *, const DevProduct &);
int launch_mfma_f8(hodu_rocm_ctx *, int dtype, const void *, const void *, void *, const DevProduct &);

int launch_mfma(hodu_rocm_ctx *ctx, int kind, int dtype, const void *a, const void *b, void *c, const DevProduct &g) {
    if (g.K == 0) return HODU_ROCM_UNSUPPORTED;  // nothing to multiply: the generic kernel writes the zeros
    if (kind == PK_BF16_F8W) return launch_mfma_w8a16(ctx, a, b, c, g);
    if (kind == PK_I32_I8I8) return launch_mfma_i8(ctx, a, b, c, g);
    switch (dtype) {
    case HODU_BF16: return launch_mfma_bf16(ctx, a, b, c, g);
    case HODU_F16: return launch_mfma_f16(ctx, a, b, c, g);
    case HODU_F32: return launch_mfma_f32(ctx, a, b, c, g);
    case HODU_I8: return launch_mfma_i8_out(ctx, a, b, c, g);
    case HODU_U8: return launch_mfma_u8_out(ctx, a, b, c, g);
    case HODU_F8E4M3:
    case HODU_F8E5M2: return launch_mfma_f8(ctx, dtype, a, b, c, g);
    default: return HODU_ROCM_UNSUPPORTED;
    }
}
}  // namespace hodu
