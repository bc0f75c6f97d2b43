// f8e4m3 x f8e4m3 -> f8e4m3 and f8e5m2 x f8e5m2 -> f8e5m2 on the 8-bit matrix instruction (gemm_mfma_pipe_f8.hpp):
// applicability and launch.
#include "gemm_mfma_pipe_f8.hpp"
#include "gemm_mfma_pipe_f8_16.hpp"
namespace hodu {
int launch_mfma_f8(hodu_rocm_ctx *ctx, int dtype, const void *a, const void *b, void *c, const DevProduct &g) {
    using namespace mfma;
    // both operands k-dense with every 16-byte chunk aligned, K a whole number of 128-byte stages;
    // anything else stays with the generic kernel
    const int la = pick_mode(a, g.a_off, g.a_m, g.a_k, g.M, g.K, 1, 16, 16, g, g.a_bs);
    const int lb = pick_mode(b, g.b_off, g.b_n, g.b_k, g.N, g.K, 1, 16, 16, g, g.b_bs);
    const int forced = ctx->force_tile;
    if (la != LM_K || lb != LM_K || g.K % P_ROW_BYTES != 0 || (forced >= 0 && forced < 10)) return HODU_ROCM_UNSUPPORTED;
    if (!pipe_offsets_fit(g.a_m, 1) || !pipe_offsets_fit(g.b_n, 1)) return HODU_ROCM_UNSUPPORTED;
    const long cus = ctx->props.multiProcessorCount;
    auto tiles = [&](long bm, long bn) { return g.batches * ((g.M + bm - 1) / bm) * ((g.N + bn - 1) / bn); };
    const bool big = forced >= 10 ? forced != 12 : tiles(256, 256) >= cus;
    const int stages = (int)(g.K / P_ROW_BYTES);
    const long elems = g.batches * (long)g.M * g.N;
    int splits = 1;
    if (ctx->force_splits >= 1) splits = pick_splits(1, cus, stages, elems, ctx->force_splits);
    else if (!big) splits = pick_splits(tiles(128, 128), cus, stages, elems, -1);
    const bool e5m2 = dtype == HODU_F8E5M2;
    // the 256 x 256 tile of an uncut product: four wavefronts on the 16 x 16 x 128 form of the instruction (hook value 15
    // pins it, 11 the eight wavefronts on the 32 x 32 x 64 form)
    if (big && splits == 1 && (forced < 0 || forced == 15)) {
        ctx->last_kernel = e5m2 ? "mfma_f8e5m2_pipe256x256mi16_KK" : "mfma_f8e4m3_pipe256x256mi16_KK";
        if (e5m2) return launch_pipe_f8x16<PipeF8x16Config<OUT_F8E5M2, 256, 256>>(ctx, a, b, c, g);
        return launch_pipe_f8x16<PipeF8x16Config<OUT_F8E4M3, 256, 256>>(ctx, a, b, c, g);
    }
    if (forced == 15) return HODU_ROCM_UNSUPPORTED;
    const char *base = e5m2 ? (big ? "mfma_f8e5m2_pipe256x256_KK" : "mfma_f8e5m2_pipe128x128_KK")
                            : (big ? "mfma_f8e4m3_pipe256x256_KK" : "mfma_f8e4m3_pipe128x128_KK");
    if (splits > 1) {
        snprintf(ctx->kernel_name, sizeof(ctx->kernel_name), "%s_splitk%d", base, splits);
        ctx->last_kernel = ctx->kernel_name;
    } else {
        ctx->last_kernel = base;
    }
    if (e5m2) {
        if (big) return launch_pipe_f8<PipeF8Config<OUT_F8E5M2, 256, 256, 25, false, 4>>(ctx, a, b, c, g, splits);
        return launch_pipe_f8<PipeF8Config<OUT_F8E5M2, 128, 128>>(ctx, a, b, c, g, splits);
    }
    if (big) return launch_pipe_f8<PipeF8Config<OUT_F8E4M3, 256, 256, 25, false, 4>>(ctx, a, b, c, g, splits);
    return launch_pipe_f8<PipeF8Config<OUT_F8E4M3, 128, 128>>(ctx, a, b, c, g, splits);
}
}  // namespace hodu
