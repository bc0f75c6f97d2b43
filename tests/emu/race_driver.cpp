// Test infrastructure: a native driver for the CPU build under ThreadSanitizer (tests/test_emu_races_cpu.py builds and
// runs it).  In the CPU build a wavefront is a host thread, so a workgroup's wavefronts race on LDS exactly where the
// kernel lacks a barrier (or a wait for an LDS-DMA that another wavefront's read depends on): ThreadSanitizer sees every
// access of the kernels' unmodified source and reports such a pair.  The lanes of one wavefront are contexts on one
// thread and cannot race with each other.
//
// The driver runs products and the one-kernel attention through the C ABI with the testing hook pinning one tile kernel after the other, under the
// earliest and the latest model of LDS-DMA arrival (a refill that comes too early for a slower reader shows under the
// first, a wait that comes too late under the second), checks each result against the integer product (operands are
// small integers: every partial sum is exact), and exits non-zero on a wrong result; ThreadSanitizer makes the exit
// code non-zero on a report.
//
// That the detector has teeth is shown by three hand-offs of 1 KB from wavefront 0 to wavefront 1 through LDS, chosen
// by the first argument: "handoff" (load, wait, barrier, read: clean, part of the default run too), "missing-barrier"
// and "late-wait" (load, barrier, wait), which must each end in a report.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "hodu_rocm_debug.h"
#include "hodu_rocm_kernels.h"

extern "C" void emu_dma_lazy(int model);

namespace {
uint16_t bf16_of(int v) {
    const float f = (float)v;
    uint32_t bits;
    memcpy(&bits, &f, 4);
    return (uint16_t)((bits + 0x7FFFu + ((bits >> 16) & 1u)) >> 16);  // to nearest, ties to even
}
float f32_of(uint16_t h) {
    const uint32_t bits = (uint32_t)h << 16;
    float f;
    memcpy(&f, &bits, 4);
    return f;
}
uint8_t e4m3_of(int v) {  // |v| <= 8: exact in OCP e4m3
    if (v == 0) return 0;
    const unsigned sign = v < 0 ? 0x80u : 0u;
    unsigned a = (unsigned)(v < 0 ? -v : v), e = 0;
    while ((a >> (e + 1)) != 0) e++;
    const unsigned mant = ((a << 3) >> e) & 7u;
    return (uint8_t)(sign | ((e + 7) << 3) | mant);
}
uint32_t lcg(uint32_t &s) { return s = s * 1664525u + 1013904223u; }

// wavefront 0 fetches 1 KB into LDS by LDS-DMA, wavefront 1 copies it out
template <bool BARRIER, bool WAIT_FIRST> __global__ void handoff_kernel(const char *src, char *dst) {
    HODU_DYNAMIC_LDS(smem);
    const unsigned lane = threadIdx.x % 64, wave = threadIdx.x / 64;
    if (wave == 0) {
        hodu::mfma::dma16_raw(src + 16 * lane, (unsigned)(uintptr_t)smem);
        if (WAIT_FIRST) __builtin_amdgcn_s_waitcnt(0);
    }
    if (BARRIER) __syncthreads();
    if (wave == 0 && !WAIT_FIRST) __builtin_amdgcn_s_waitcnt(0);
    if (wave == 1) memcpy(dst + 16 * lane, smem + 16 * lane, 16);
}

int handoff(hodu_rocm_ctx *ctx, bool barrier, bool wait_first) {
    std::vector<unsigned char> in(1024), out(1024);
    for (int i = 0; i < 1024; i++) in[i] = (unsigned char)(i * 7 + 3);
    void *src = nullptr, *dst = nullptr;
    if (hodu_rocm_alloc(ctx, 1024, &src) || hodu_rocm_alloc(ctx, 1024, &dst)) return 1;
    hodu_rocm_memcpy_h2d(ctx, src, in.data(), 1024);
    auto kernel = barrier ? (wait_first ? handoff_kernel<true, true> : handoff_kernel<true, false>) : handoff_kernel<false, true>;
    hipLaunchKernelGGL(kernel, dim3(1), dim3(128), 1024, nullptr, (const char *)src, (char *)dst);
    hodu_rocm_memcpy_d2h(ctx, out.data(), dst, 1024);
    hodu_rocm_free(ctx, src);
    hodu_rocm_free(ctx, dst);
    return barrier && wait_first && in != out;  // only the clean hand-off promises the bytes
}

struct Case { const char *what; int hook, splits, m, n, k; bool f8_weights, rhs_row_dense; };

int run(hodu_rocm_ctx *ctx, const Case &c) {
    std::vector<int> a((size_t)c.m * c.k), b((size_t)c.n * c.k);
    uint32_t seed = 12345u + (uint32_t)c.hook * 7u + (uint32_t)c.k;
    for (auto &v : a) v = (int)(lcg(seed) >> 28) - 8;
    for (auto &v : b) v = (int)(lcg(seed) >> 29) - 4;
    std::vector<uint16_t> ha(a.size());
    for (size_t i = 0; i < a.size(); i++) ha[i] = bf16_of(a[i]);
    // right operand stored [N, K] (k-dense) or [K, N] (row-dense)
    std::vector<uint16_t> hb16(b.size());
    std::vector<uint8_t> hb8(b.size());
    for (int n = 0; n < c.n; n++)
        for (int k = 0; k < c.k; k++) {
            const size_t at = c.rhs_row_dense ? (size_t)k * c.n + n : (size_t)n * c.k + k;
            hb16[at] = bf16_of(b[(size_t)n * c.k + k]);
            hb8[at] = e4m3_of(b[(size_t)n * c.k + k]);
        }
    void *da = nullptr, *db = nullptr, *dc = nullptr;
    const size_t b_bytes = c.f8_weights ? hb8.size() : 2 * hb16.size();
    if (hodu_rocm_alloc(ctx, 2 * ha.size(), &da) || hodu_rocm_alloc(ctx, b_bytes, &db) || hodu_rocm_alloc(ctx, 2 * (size_t)c.m * c.n, &dc)) return 1;
    hodu_rocm_memcpy_h2d(ctx, da, ha.data(), 2 * ha.size());
    hodu_rocm_memcpy_h2d(ctx, db, c.f8_weights ? (const void *)hb8.data() : (const void *)hb16.data(), b_bytes);
    hodu_rocm_memset(ctx, dc, 0xFF, 2 * (size_t)c.m * c.n);
    const size_t md[9] = {(size_t)c.m, (size_t)c.k, (size_t)c.n, (size_t)c.k, 1, c.rhs_row_dense ? (size_t)c.n : 1,
                          c.rhs_row_dense ? 1 : (size_t)c.k, 0, 0};
    hodu_rocm_debug_force_tile(ctx, c.hook);
    hodu_rocm_debug_force_splitk(ctx, c.splits);
    const int rc = c.f8_weights ? hodu_rocm_dot_bf16_f8e4m3w(ctx, da, db, dc, md, 9) : hodu_rocm_dot_bf16(ctx, da, db, dc, md, 9);
    int bad = 0;
    if (rc != 0) {
        fprintf(stderr, "%s: status %d: %s\n", c.what, rc, hodu_rocm_last_error(ctx));
        bad = 1;
    } else {
        std::vector<uint16_t> out((size_t)c.m * c.n);
        hodu_rocm_memcpy_d2h(ctx, out.data(), dc, 2 * out.size());
        for (int i = 0; i < c.m && !bad; i++)
            for (int j = 0; j < c.n; j++) {
                long want = 0;
                for (int k = 0; k < c.k; k++) want += (long)a[(size_t)i * c.k + k] * b[(size_t)j * c.k + k];
                if (f32_of(out[(size_t)i * c.n + j]) != f32_of(bf16_of((int)want))) {
                    fprintf(stderr, "%s: output [%d, %d] is %g, the product is %ld\n", c.what, i, j, f32_of(out[(size_t)i * c.n + j]), want);
                    bad = 1;
                    break;
                }
            }
    }
    printf("%-44s %-44s %s\n", c.what, hodu_rocm_last_kernel(ctx), bad ? "WRONG" : "ok");
    fflush(stdout);
    hodu_rocm_free(ctx, da);
    hodu_rocm_free(ctx, db);
    hodu_rocm_free(ctx, dc);
    return bad;
}
// the one-kernel attention (eight wavefronts share K / V blocks in LDS and meet in pairs at the end), with and without an
// attn_mask, against a plain float loop
int attention(hodu_rocm_ctx *ctx, int d, int sq, int sk, bool causal, bool masked) {
    const int heads = 2;
    std::vector<uint16_t> q((size_t)heads * sq * d), k((size_t)heads * sk * d), v((size_t)heads * sk * d);
    std::vector<uint8_t> keep((size_t)sk);
    uint32_t seed = 777u + (uint32_t)(d + sq + sk);
    for (auto &x : q) x = bf16_of((int)(lcg(seed) >> 29) - 4);
    for (auto &x : k) x = bf16_of((int)(lcg(seed) >> 30) - 2);
    for (auto &x : v) x = bf16_of((int)(lcg(seed) >> 28) - 8);
    for (int j = 0; j < sk; j++) keep[j] = j == 0 || (lcg(seed) >> 30) != 0;
    void *dq, *dk, *dv, *dm, *dout;
    if (hodu_rocm_alloc(ctx, 2 * q.size(), &dq) || hodu_rocm_alloc(ctx, 2 * k.size(), &dk) || hodu_rocm_alloc(ctx, 2 * v.size(), &dv) ||
        hodu_rocm_alloc(ctx, keep.size(), &dm) || hodu_rocm_alloc(ctx, 2 * q.size(), &dout))
        return 1;
    hodu_rocm_memcpy_h2d(ctx, dq, q.data(), 2 * q.size());
    hodu_rocm_memcpy_h2d(ctx, dk, k.data(), 2 * k.size());
    hodu_rocm_memcpy_h2d(ctx, dv, v.data(), 2 * v.size());
    hodu_rocm_memcpy_h2d(ctx, dm, keep.data(), keep.size());
    const size_t md[] = {1, (size_t)heads, (size_t)sq, (size_t)sk, (size_t)d, (size_t)sq * d, (size_t)d, 1, (size_t)sk * d, (size_t)d, 1,
                         (size_t)sk * d, (size_t)d, 1, 0, 0, 0};
    const float scale = 0.125f;  // exact in bf16
    const uint16_t scale_bits = 0x3E00;
    const size_t mask_layout[] = {3, 0, 0, 1, 0};  // one [Sk] mask for every head and row
    hodu_rocm_debug_force_tile(ctx, -1);
    const int rc = masked ? hodu_rocm_attention_masked(ctx, HODU_BF16, dq, dk, dv, dout, md, 17, &scale_bits, causal, dm, HODU_U8, mask_layout, 5)
                          : hodu_rocm_attention(ctx, HODU_BF16, dq, dk, dv, dout, md, 17, &scale_bits, causal);
    int bad = 0;
    if (rc != 0) {
        fprintf(stderr, "attention: status %d: %s\n", rc, hodu_rocm_last_error(ctx));
        bad = 1;
    } else {
        std::vector<uint16_t> out(q.size());
        hodu_rocm_memcpy_d2h(ctx, out.data(), dout, 2 * out.size());
        std::vector<double> p((size_t)sk);
        for (int h = 0; h < heads && !bad; h++)
            for (int i = 0; i < sq && !bad; i++) {
                double top = -1e300, sum = 0;
                for (int j = 0; j < sk; j++) {
                    double s = 0;
                    for (int c = 0; c < d; c++) s += (double)f32_of(q[((size_t)h * sq + i) * d + c]) * f32_of(k[((size_t)h * sk + j) * d + c]);
                    s *= scale;
                    const bool filled = (masked && !keep[j]) || (causal && j > i);
                    p[j] = filled ? (masked ? -65536.0 : -1e300) : s;
                    top = p[j] > top ? p[j] : top;
                }
                for (int j = 0; j < sk; j++) sum += (p[j] = std::exp(p[j] - top));
                for (int c = 0; c < d; c++) {
                    double want = 0, size = 0;
                    for (int j = 0; j < sk; j++) {
                        want += p[j] / sum * f32_of(v[((size_t)h * sk + j) * d + c]);
                        size += p[j] / sum * std::fabs(f32_of(v[((size_t)h * sk + j) * d + c]));
                    }
                    const double got = f32_of(out[((size_t)h * sq + i) * d + c]);
                    if (!(std::fabs(got - want) <= 2e-2 * size + 1e-3)) {
                        fprintf(stderr, "attention head %d row %d column %d: %g, the function gives %g\n", h, i, c, got, want);
                        bad = 1;
                        break;
                    }
                }
            }
    }
    printf("%-44s %-44s %s\n", masked ? "attention with a mask" : "attention", hodu_rocm_last_kernel(ctx), bad ? "WRONG" : "ok");
    fflush(stdout);
    for (void *b : {dq, dk, dv, dm, dout}) hodu_rocm_free(ctx, b);
    return bad;
}
}  // namespace

int main(int argc, char **argv) {
    hodu_rocm_ctx *ctx = nullptr;
    if (hodu_rocm_ctx_create(0, &ctx) != 0) return 2;
    if (argc > 1) {
        const std::string which = argv[1];
        emu_dma_lazy(1);
        const int bad = which == "handoff" ? handoff(ctx, true, true) : which == "missing-barrier" ? handoff(ctx, false, true)
                      : which == "late-wait" ? handoff(ctx, true, false) : 2;
        hodu_rocm_ctx_destroy(ctx);
        return bad;
    }
    // operands are small integers: every partial sum is exact in f32, so the stored value is the rounded exact product
    const Case cases[] = {
        {"general tile kernel 256x256", 1, -1, 264, 136, 200, false, false},
        {"general tile kernel 128x128, row-dense rhs", 2, -1, 136, 136, 200, false, true},
        {"pipelined 32x32x16, 256x256", 11, -1, 264, 136, 256, false, false},
        {"pipelined 32x32x16, 128x128", 12, -1, 136, 136, 192, false, false},
        {"pipelined, K cut three ways", 11, 3, 136, 136, 448, false, false},
        {"pipelined, f8e4m3 weights", 11, -1, 264, 136, 256, true, false},
        {"16x16x32 tile", 15, -1, 264, 136, 192, false, false},
        {"16x16x32 tile, row-dense rhs", 15, -1, 264, 136, 192, false, true},
        {"16x16x32 tile, f8e4m3 weights", 15, -1, 264, 136, 256, true, false},
        {"16x16x32 tile, f8e4m3 weights row-dense", 15, -1, 264, 144, 192, true, true},
        {"respaced 16x16x32 tile", 16, -1, 264, 136, 256, false, false},
        {"respaced 16x16x32 tile, row-dense rhs", 16, -1, 264, 136, 256, false, true},
        {"respaced 16x16x32 tile, f8e4m3 weights", 16, -1, 264, 136, 384, true, false},
        {"respaced 16x16x32 tile, f8e4m3 weights row-dense", 16, -1, 264, 144, 256, true, true},
        {"few rows, one pass", 35, -1, 16, 264, 1024, false, false},
        {"few rows, one pass, f8e4m3 weights", 36, -1, 12, 264, 1024, true, false},
    };
    int bad = 0;
    for (int model = 0; model < 2; model++) {
        emu_dma_lazy(model);
        printf("LDS-DMA arrival model %d\n", model);
        for (const Case &c : cases) bad |= run(ctx, c);
        bad |= handoff(ctx, true, true);
        bad |= attention(ctx, 128, 200, 300, true, false);
        bad |= attention(ctx, 64, 130, 200, false, false);
        bad |= attention(ctx, 128, 130, 200, true, true);
        bad |= attention(ctx, 64, 200, 300, false, true);
    }
    hodu_rocm_ctx_destroy(ctx);
    return bad;
}
