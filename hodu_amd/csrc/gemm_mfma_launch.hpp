// Variant selection and launch for one compute kind of the MFMA tile kernels.
#pragma once

#include <cstring>

#include "gemm_mfma.hpp"
#include "gemm_mfma_pipe.hpp"
#include "gemm_mfma_pipe16.hpp"

namespace hodu {
namespace mfma {

// The 256 x 256 tile on the 16 x 16 x 32 instruction (both generations, four layout pairs, two 16-bit types) is compiled
// in translation units of its own, gemm_mfma_mi16_{bf16,f16}.hip, so that the build's longest compile stays short:
// everywhere else these launchers are only declared.
#ifdef HODU_MI16_DEFINE_HERE
#define HODU_MI16_LINKAGE
#else
#define HODU_MI16_LINKAGE extern
#endif
#define HODU_MI16_ONE(CK, OUT, LA, LB)                                                                                     \
    HODU_MI16_LINKAGE template int launch_pipe16<PipeConfig<CK, OUT, 256, 256, 2, 2, LA, LB, SK_SAME, 2>>(                   \
        hodu_rocm_ctx *, const void *, const void *, void *, const DevProduct &);                                            \
    HODU_MI16_LINKAGE template int launch_pipe16r<PipeConfig<CK, OUT, 256, 256, 2, 2, LA, LB, SK_SAME, 2>>(                  \
        hodu_rocm_ctx *, const void *, const void *, void *, const DevProduct &);
#define HODU_MI16_ALL(CK, OUT)                                                                                             \
    HODU_MI16_ONE(CK, OUT, LM_K, LM_K) HODU_MI16_ONE(CK, OUT, LM_K, LM_MN) HODU_MI16_ONE(CK, OUT, LM_MN, LM_K)               \
    HODU_MI16_ONE(CK, OUT, LM_MN, LM_MN)
#if !defined(HODU_MI16_DEFINE_HERE) || HODU_MI16_DEFINE_HERE == 0
HODU_MI16_ALL(CK_BF16, OUT_BF16)
#endif
#if !defined(HODU_MI16_DEFINE_HERE) || HODU_MI16_DEFINE_HERE == 1
HODU_MI16_ALL(CK_F16, OUT_F16)
#endif

// One compute kind: {KK, KM, MK, MM} x {256x256 with 4 wavefronts, 128x128, 64x64}, {KK, KM} x 256x256
// with 8 wavefronts, a scalar-load 64x64 kernel, and -- when both operands are stored in the compute
// type -- the software-pipelined kernels of gemm_mfma_pipe.hpp: KK at four tile shapes and, for the
// 16-bit types, KM / MK / MM at the three larger ones.  The tile is the largest that still yields at
// least one workgroup per compute unit.
constexpr int kVariants = 36;
template <int CK, int SKA, int SKB, int OUT>
int launch_kind(hodu_rocm_ctx *ctx, const void *a, const void *b, void *c, const DevProduct &g,
                const char *const names[kVariants]) {
    constexpr int ES = Compute<CK>::ES, EPC = 16 / ES;
    constexpr int SA = SKA == SK_F8 ? 1 : ES, SB = SKB == SK_F8 ? 1 : ES;
    constexpr int ROWVEC = ES == 4 ? 4 : 8;
    const int la = pick_mode(a, g.a_off, g.a_m, g.a_k, g.M, g.K, SA, EPC, ROWVEC, g, g.a_bs);
    const int lb = pick_mode(b, g.b_off, g.b_n, g.b_k, g.N, g.K, SB, EPC, ROWVEC, g, g.b_bs);
    const long cus = ctx->props.multiProcessorCount;
    auto tiles = [&](long bm, long bn) { return g.batches * ((g.M + bm - 1) / bm) * ((g.N + bn - 1) / bn); };
    if (la >= LM_SCALAR || lb >= LM_SCALAR) {
        // an operand whose rows or columns do not start on vector boundaries is loaded element by element; the other
        // one keeps its vector loads (a [K, 2] right operand must not slow down the [M, K] matrix beside it)
        const int gs = pick_splits(tiles(64, 64), cus, (int)(((long)g.K * ES + 127) / 128), g.batches * (long)g.M * g.N,
                                   ctx->force_splits);
        // large products: 128 x 128 tiles (a quarter of the LDS traffic per flop), where they fill the chip
        const bool big = SKA == SK_SAME && SKB == SK_SAME && ctx->force_tile < 0 && g.M >= 256 && g.N >= 256 &&
                         tiles(128, 128) >= cus;
        if (big) {  // "<prefix>_64x64_scalar" -> "<prefix>_128x128_scalar"
            const char *cut = strstr(names[16], "_64x64_scalar");
            snprintf(ctx->kernel_name, sizeof(ctx->kernel_name), "%.*s_128x128_scalar", (int)(cut ? cut - names[16] : 0), names[16]);
            ctx->last_kernel = ctx->kernel_name;
        } else if (gs > 1) {
            snprintf(ctx->kernel_name, sizeof(ctx->kernel_name), "%s_splitk%d", names[16], gs);
            ctx->last_kernel = ctx->kernel_name;
        } else {
            ctx->last_kernel = names[16];
        }
        if constexpr (SKA == SK_SAME && SKB == SK_SAME) {
#define HODU_IRREGULAR(LA, LB)                                                                                         \
    if (la == LA && lb == LB) {                                                                                        \
        if (big) return launch_config<Config<CK, SKA, SKB, OUT, 128, 128, 2, 2, LA, LB>>(ctx, a, b, c, g, 1);           \
        return launch_config<Config<CK, SKA, SKB, OUT, 64, 64, 2, 2, LA, LB>>(ctx, a, b, c, g, gs);                     \
    }
            HODU_IRREGULAR(LM_K, LM_SCALAR) HODU_IRREGULAR(LM_MN, LM_SCALAR) HODU_IRREGULAR(LM_MNU, LM_SCALAR)
            HODU_IRREGULAR(LM_SCALAR, LM_K) HODU_IRREGULAR(LM_SCALAR, LM_MN) HODU_IRREGULAR(LM_SCALAR, LM_MNU)
            HODU_IRREGULAR(LM_K, LM_MNU) HODU_IRREGULAR(LM_MN, LM_MNU) HODU_IRREGULAR(LM_MNU, LM_K)
            HODU_IRREGULAR(LM_MNU, LM_MN) HODU_IRREGULAR(LM_MNU, LM_MNU)
            HODU_IRREGULAR(LM_SCALAR, LM_SCALAR)
#undef HODU_IRREGULAR
        }
        // (f8e4m3 weight bytes: element loads for both)
        return launch_config<Config<CK, SKA, SKB, OUT, 64, 64, 2, 2, LM_SCALAR, LM_SCALAR>>(ctx, a, b, c, g, gs);
    }
    // size: 0 = 256x256 / 8 wavefronts, 1 = 256x256 / 4 wavefronts, 2 = 128x128, 3 = 64x64
    const int forced = ctx->force_tile;
    int size = forced >= 0 ? forced % 10 : tiles(256, 256) >= cus ? 0 : tiles(128, 128) >= cus ? 2 : 3;
    if (forced < 0) {
        // many small matrices (a batch of 128 x 128 or 16 x 16 products) fill the chip with tiles that are mostly
        // padding: step down while the smaller tile wastes markedly less (fraction of a tile's outputs that exist)
        auto used = [&](long bm) {
            return (double)g.M * g.N / ((double)((g.M + bm - 1) / bm * bm) * (double)((g.N + bm - 1) / bm * bm));
        };
        if (size == 0 && used(256) < 0.75 * used(128)) size = 2;
        // (the 64 x 64 kernels are the plainest ones: only when they waste less than half as much; bf16
        // [64, 512, 512] x [64, 512, 64] measured 11.3 us with 128 x 128 tiles against 14.3 us with 64 x 64)
        if (size == 2 && used(128) < 0.5 * used(64)) size = 3;
    }
    // 16-bit operands of one type: the 256 x 256 tile on four wavefronts (one per SIMD, 128 x 128 outputs each) reads
    // a third fewer fragment bytes out of LDS than on eight and measured 2 % ahead (config 5 down 335 against 341 us,
    // up 368 against 376); with f8e4m3 weights, whose widening wants a second wavefront on the SIMD to hide behind,
    // eight stay ahead (349 against 355 us), and so they do on the 32 x 32 x 16 kernels when element-wise steps ride on
    // the store (config 2 with the attention scale: 38 against 44 us)
    if constexpr (SKA == SK_SAME && SKB == SK_SAME && ES == 2) {
        if (forced < 0 && size == 0 && g.epi.n == 0) size = 1;
    }
    // A product too small to fill the machine with 128x128 tiles is cut along K instead of shrinking the tile
    // further (pipelined kernels only): same HBM traffic, four times fewer bytes through LDS per flop.
    const int stages = (int)((long)g.K * ES / 128);
    const long elems = g.batches * (long)g.M * g.N;
    bool pipe_ok = false;  // one of the pipelined kernels will take this product
    if constexpr (SKA == SK_SAME && SKB == SK_SAME) pipe_ok = pipe_eligible<CK>(la, lb, g) && (forced < 0 || forced >= 10);
    if constexpr (SKA == SK_SAME && SKB == SK_F8) pipe_ok = pipe_f8_eligible(la, lb, b, g) && (forced < 0 || forced >= 10);
    int splits = 1;
    if (!pipe_ok) {
    } else if (forced < 0 && size == 3) {
        splits = pick_splits(tiles(128, 128), cus, stages, elems, ctx->force_splits);
        if (splits > 1) size = 2;
        if constexpr (SKA == SK_SAME && SKB == SK_SAME) {
            // Cutting K costs a second kernel and the partial sums' trip through memory, which a short K does not
            // earn back.  Measured (bf16, one workgroup per CU or fewer; microseconds): a 128 x 128 workgroup takes
            // 5 + 0.42 per stage, a 64 x 64 one (both operands k-dense) 4.5 + 0.25 per stage, the second pass
            // 3 + 8 bytes per output and range at 4 TB/s.  [1024, 1024] x [1024, 1024]^T: 18.3 us cut four ways,
            // 11.8 on 128 x 128 tiles as it is, 8.1 on 64 x 64 tiles; [512, 4096] x [4096, 512]: 15.3 cut eight ways,
            // 19.3 / 30.1 uncut.  f32 (a stage is 32 k, and the f32 matrix instruction is eight times slower per
            // k): 2.05 and 0.65 per stage; [1024, 1024] x [1024, 1024]^T 31.5 us cut four ways, 24.5 on 64 x 64 tiles.
            if (ctx->force_splits < 0 && tiles(128, 128) < cus) {
                constexpr double S128 = ES == 4 ? 2.05 : 0.42, S64 = ES == 4 ? 0.65 : 0.25;
                const bool kk = la == LM_K && lb == LM_K;
                const double t_cut = splits > 1 ? 8.0 + S128 * ((stages + splits - 1) / splits) + (double)elems * splits * 8 / 4e6 : 1e30;
                const double t_128 = g.M >= 64 && g.N >= 64 ? 5.0 + S128 * stages : 1e30;
                const double waves64 = (double)tiles(64, 64) / cus;
                const double t_64 = kk ? 4.5 + S64 * stages * (waves64 > 1 ? waves64 : 1) : 1e30;
                if (t_64 <= t_cut && t_64 <= t_128) {
                    size = 3;
                    splits = 1;
                } else if (t_128 <= t_cut) {
                    size = 2;
                    splits = 1;
                }
            }
        }
    } else if (ctx->force_splits >= 1 && (size < 3 || size == 4)) {
        splits = pick_splits(1, cus, stages, elems, ctx->force_splits);
    }
    if (size == 4 && !pipe_ok) size = 2;  // 256x128 exists as a pipelined kernel only
    auto named = [&](const char *base, int sp) -> const char * {
        if (sp <= 1) return base;
        snprintf(ctx->kernel_name, sizeof(ctx->kernel_name), "%s_splitk%d", base, sp);
        return ctx->kernel_name;
    };
    const int combo = (la == LM_MN ? 2 : 0) + (lb == LM_MN ? 1 : 0);
    if constexpr (SKA == SK_SAME && SKB == SK_SAME && ES == 2 && CK != CK_I8) {
        // 16-bit operands on the 256 x 256 tile of four wavefronts: the 16 x 16 x 32 instruction, which
        // leaves the power-limited part a higher clock than the 32 x 32 x 16 one (hook value 15 pins it, 11 the other)
        // (with element-wise steps on the store as well: config 5 up with bias and ReLU 375 against 420 us on eight
        // wavefronts of the 32 x 32 x 16 kernel, config 2 with the attention scale 36.5-38.5 against 38.5-39.3)
        const bool fused = size == 0 && g.epi.n != 0;
        if (pipe_ok && splits == 1 && size == 6 && pipe16r_stages_ok(g.K, ES)) {
            snprintf(ctx->kernel_name, sizeof(ctx->kernel_name), "%s_r", names[32 + combo]);
            ctx->last_kernel = ctx->kernel_name;
            if (combo == 0) return launch_pipe16r<PipeConfig<CK, OUT, 256, 256, 2, 2, LM_K, LM_K, SK_SAME, 2>>(ctx, a, b, c, g);
            if (combo == 1) return launch_pipe16r<PipeConfig<CK, OUT, 256, 256, 2, 2, LM_K, LM_MN, SK_SAME, 2>>(ctx, a, b, c, g);
            if (combo == 2) return launch_pipe16r<PipeConfig<CK, OUT, 256, 256, 2, 2, LM_MN, LM_K, SK_SAME, 2>>(ctx, a, b, c, g);
            return launch_pipe16r<PipeConfig<CK, OUT, 256, 256, 2, 2, LM_MN, LM_MN, SK_SAME, 2>>(ctx, a, b, c, g);
        }
        if (pipe_ok && splits == 1 && ((forced < 0 && (size == 1 || fused)) || size == 5)) {
            ctx->last_kernel = names[32 + combo];
            if (combo == 0) return launch_pipe16<PipeConfig<CK, OUT, 256, 256, 2, 2, LM_K, LM_K, SK_SAME, 2>>(ctx, a, b, c, g);
            if (combo == 1) return launch_pipe16<PipeConfig<CK, OUT, 256, 256, 2, 2, LM_K, LM_MN, SK_SAME, 2>>(ctx, a, b, c, g);
            if (combo == 2) return launch_pipe16<PipeConfig<CK, OUT, 256, 256, 2, 2, LM_MN, LM_K, SK_SAME, 2>>(ctx, a, b, c, g);
            return launch_pipe16<PipeConfig<CK, OUT, 256, 256, 2, 2, LM_MN, LM_MN, SK_SAME, 2>>(ctx, a, b, c, g);
        }
    }
    if constexpr (SKA == SK_SAME && SKB == SK_F8) {
        // f8e4m3 weights, k-dense or row-dense: the same tile and instruction with the widening in front of the MFMA
        if (pipe_ok && combo <= 1 && splits == 1 && size == 6) {
            snprintf(ctx->kernel_name, sizeof(ctx->kernel_name), "%s_r", names[32 + combo]);
            ctx->last_kernel = ctx->kernel_name;
            if (combo == 0) return launch_pipe16r_f8w<PipeConfig<CK, OUT, 256, 256, 2, 2, LM_K, LM_K, SK_F8, 2>>(ctx, a, b, c, g);
            return launch_pipe16r_f8w<PipeConfig<CK, OUT, 256, 256, 2, 2, LM_K, LM_MN, SK_F8, 2>>(ctx, a, b, c, g);
        }
        if (pipe_ok && combo <= 1 && splits == 1 && ((forced < 0 && size == 0) || size == 5)) {
            ctx->last_kernel = names[32 + combo];
            if (combo == 0) return launch_pipe16_f8w<PipeConfig<CK, OUT, 256, 256, 2, 2, LM_K, LM_K, SK_F8, 2>>(ctx, a, b, c, g);
            return launch_pipe16_f8w<PipeConfig<CK, OUT, 256, 256, 2, 2, LM_K, LM_MN, SK_F8, 2>>(ctx, a, b, c, g);
        }
    }
    if (size == 5 || size == 6) return HODU_ROCM_UNSUPPORTED;
    if constexpr (SKA == SK_SAME && SKB == SK_SAME) {
        // testing hook values 10..13 pin the pipelined kernel's tile, 0..3 the general kernel's
        if (pipe_ok && size == 4 && combo <= 1) {
            ctx->last_kernel = named(names[30 + combo], splits);
            if (combo == 0) return launch_pipe<PipeConfig<CK, OUT, 256, 128, 2, 2, LM_K, LM_K, SK_SAME, 3>>(ctx, a, b, c, g, splits);
            if constexpr (ES <= 2)
                return launch_pipe<PipeConfig<CK, OUT, 256, 128, 2, 2, LM_K, LM_MN, SK_SAME, 3>>(ctx, a, b, c, g, splits);
        }
        if (pipe_ok && size < 4 && (combo == 0 || size < 3)) {
            ctx->last_kernel = named(combo == 0 ? names[17 + size] : names[21 + (combo - 1) * 3 + size], splits);
#define HODU_PIPE_CASE(SZ, BM, BN, WM, WN, LA, LB) \
    if (size == SZ) return launch_pipe<PipeConfig<CK, OUT, BM, BN, WM, WN, LA, LB>>(ctx, a, b, c, g, splits);
#define HODU_PIPE_CASE4(SZ, BM, BN, WM, WN, LA, LB) \
    if (size == SZ) return launch_pipe<PipeConfig<CK, OUT, BM, BN, WM, WN, LA, LB, SK_SAME, 4>>(ctx, a, b, c, g, splits);
#define HODU_PIPE_COMBO(CB, LA, LB)                       \
    if (combo == CB) {                                    \
        HODU_PIPE_CASE(0, 256, 256, 2, 4, LA, LB)         \
        HODU_PIPE_CASE(1, 256, 256, 2, 2, LA, LB)         \
        HODU_PIPE_CASE4(2, 128, 128, 2, 2, LA, LB)        \
    }
            HODU_PIPE_COMBO(0, LM_K, LM_K)
            if constexpr (ES <= 2) {
                HODU_PIPE_COMBO(1, LM_K, LM_MN)
                HODU_PIPE_COMBO(2, LM_MN, LM_K)
                HODU_PIPE_COMBO(3, LM_MN, LM_MN)
            }
            if (combo == 0) return launch_pipe<PipeConfig<CK, OUT, 64, 64, 2, 2, LM_K, LM_K, SK_SAME, 4>>(ctx, a, b, c, g, 1);
#undef HODU_PIPE_COMBO
#undef HODU_PIPE_CASE4
#undef HODU_PIPE_CASE
        }
    }
    if constexpr (SKA == SK_SAME && SKB == SK_F8) {
        if (pipe_ok && size == 4 && combo <= 1) {
            ctx->last_kernel = named(names[30 + combo], splits);
            if (combo == 0) return launch_pipe<PipeConfig<CK, OUT, 256, 128, 2, 2, LM_K, LM_K, SK_F8, 3>>(ctx, a, b, c, g, splits);
            return launch_pipe<PipeConfig<CK, OUT, 256, 128, 2, 2, LM_K, LM_MN, SK_F8, 3>>(ctx, a, b, c, g, splits);
        }
        if (pipe_ok && size < 3) {
            ctx->last_kernel = named(combo == 0 ? names[17 + size] : names[21 + size], splits);
#define HODU_PIPE_F8(SZ, BM, BN, WM, WN, NST)                                                                     \
    if (size == SZ && combo == 0)                                                                                 \
        return launch_pipe<PipeConfig<CK, OUT, BM, BN, WM, WN, LM_K, LM_K, SK_F8, NST>>(ctx, a, b, c, g, splits);  \
    if (size == SZ && combo == 1)                                                                                 \
        return launch_pipe<PipeConfig<CK, OUT, BM, BN, WM, WN, LM_K, LM_MN, SK_F8, NST>>(ctx, a, b, c, g, splits);
            HODU_PIPE_F8(0, 256, 256, 2, 4, 2)
            HODU_PIPE_F8(1, 256, 256, 2, 2, 2)
            HODU_PIPE_F8(2, 128, 128, 2, 2, 4)
#undef HODU_PIPE_F8
        }
    }
    // a row-dense LEFT operand needs 32 staging registers more than the 8-wavefront variant has
    // (two wavefronts share a SIMD's register file): those layouts use the 4-wavefront variant
    if (size == 0 && la == LM_MN) size = 1;
    // the general kernel, too, is cut along K where its tiles would leave most of the chip idle (an f32 product
    // with a row-dense operand and few rows, a small square one): same rule as for the pipelined kernels
    const int ksteps = (int)(((long)g.K * ES + 127) / 128);
    int gsplits = 1;
    if (forced < 0 && size == 3 && la != LM_SCALAR && lb != LM_SCALAR && g.M >= 128 && g.N >= 128) {
        // as above: 128 x 128 tiles cut along K before 64 x 64 tiles, if that still fills half the chip (and the
        // product has the rows to fill such a tile: with 32 or 64 rows the small tiles measured 25 % faster)
        const int s128 = pick_splits(tiles(128, 128), cus, ksteps, elems, ctx->force_splits);
        if (s128 > 1 && tiles(128, 128) * s128 * 2 >= cus) {
            size = 2;
            gsplits = s128;
        }
    }
    if (gsplits == 1) {
        const int bm = size <= 1 ? 256 : size == 2 ? 128 : 64;
        gsplits = pick_splits(tiles(bm, bm), cus, ksteps, elems, ctx->force_splits);
    }
    ctx->last_kernel = named(names[size * 4 + combo], gsplits);
#define HODU_MFMA_CASE(SZ, CB, BM, BN, WM, WN, LA, LB)                                                     \
    if (size == SZ && combo == CB) return launch_config<Config<CK, SKA, SKB, OUT, BM, BN, WM, WN, LA, LB>>(ctx, a, b, c, g, gsplits);
#define HODU_MFMA_SIZE(SZ, BM, BN, WM, WN)               \
    HODU_MFMA_CASE(SZ, 0, BM, BN, WM, WN, LM_K, LM_K)    \
    HODU_MFMA_CASE(SZ, 1, BM, BN, WM, WN, LM_K, LM_MN)   \
    HODU_MFMA_CASE(SZ, 2, BM, BN, WM, WN, LM_MN, LM_K)   \
    HODU_MFMA_CASE(SZ, 3, BM, BN, WM, WN, LM_MN, LM_MN)
    HODU_MFMA_CASE(0, 0, 256, 256, 2, 4, LM_K, LM_K)
    HODU_MFMA_CASE(0, 1, 256, 256, 2, 4, LM_K, LM_MN)
    HODU_MFMA_SIZE(1, 256, 256, 2, 2)
    HODU_MFMA_SIZE(2, 128, 128, 2, 2)
    HODU_MFMA_SIZE(3, 64, 64, 2, 2)
#undef HODU_MFMA_SIZE
#undef HODU_MFMA_CASE
    return fail(HODU_ROCM_UNSUPPORTED, "no MFMA variant");
}

#define HODU_MFMA_NAMES(P)                                                                                       \
    {P "_256x256w8_KK", P "_256x256w8_KM", P "_256x256w8_MK", P "_256x256w8_MM", P "_256x256_KK", P "_256x256_KM", \
     P "_256x256_MK",   P "_256x256_MM",   P "_128x128_KK",   P "_128x128_KM",   P "_128x128_MK", P "_128x128_MM", \
     P "_64x64_KK",     P "_64x64_KM",     P "_64x64_MK",     P "_64x64_MM",     P "_64x64_scalar",                \
     P "_pipe256x256w8_KK", P "_pipe256x256_KK", P "_pipe128x128_KK", P "_pipe64x64_KK",                           \
     P "_pipe256x256w8_KM", P "_pipe256x256_KM", P "_pipe128x128_KM",                                              \
     P "_pipe256x256w8_MK", P "_pipe256x256_MK", P "_pipe128x128_MK",                                              \
     P "_pipe256x256w8_MM", P "_pipe256x256_MM", P "_pipe128x128_MM",                                              \
     P "_pipe256x128_KK", P "_pipe256x128_KM", P "_pipe256x256mi16_KK", P "_pipe256x256mi16_KM",                \
     P "_pipe256x256mi16_MK", P "_pipe256x256mi16_MM"}

}  // namespace mfma
}  // namespace hodu
