/*
 * hodu_oracle.c -- CPU restatement of hodu's matmul / dot / to_dtype / contiguous arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker for the HIP kernels: it is built into
 * oracle/liboracle.so and may be loaded only by tests/, by __graft_entry__.smoke() and by the
 * cpu_baseline leg of bench.py.  Nothing in the product path (the C-ABI library or the host
 * layer above it) links, loads or calls it.
 *
 * It follows the *behaviour* of the reference C kernels, restated as one generic walker plus
 * per-dtype scalar arithmetic (the reference instantiates a macro per dtype):
 *
 *   matmul   crates/hodu_cpu_kernels/kernels/ops_matrix.c:46-193 (native types),
 *            :196-339 (bf16/f16/f8 "exotic" types), metadata layout :16-29
 *   dot      crates/hodu_cpu_kernels/kernels/ops_matrix.c:399-549, :556-701, metadata :371-380
 *   cast     crates/hodu_cpu_kernels/kernels/ops_cast.c:34-103 and the table :108-388
 *   gather   crates/hodu_cpu_kernels/kernels/ops_memory.c:19-84
 *   add      crates/hodu_cpu_kernels/kernels/ops_binary.c:208-262 (bf16/f16/f8: widen, add in f32, narrow with the
 *            type's own routine) and the native-type macro :60-118; metadata :214-222
 *   sum      crates/hodu_cpu_kernels/kernels/ops_reduce.c:47-118 (generic macro: one output at a time, the reduced
 *            dims walked innermost first, accumulator in the storage type -- bf16 / f16 / f8 re-round after every
 *            add, :127-130), :133-237 (f32; a lane-wise SIMD order only when the last, dense dim alone is reduced)
 *   softmax  crates/hodu_core/src/tensor/ops/normalization.rs:4-21 (max(keep_dim), sub, exp, sum(keep_dim), div) with
 *            the causal masked_fill(-inf) of crates/hodu_nn/src/modules/attention.rs:40-48, :73-86 (mask j > i) and
 *            the attn_mask masked_fill of :50-56 with get_neg_inf (:88-96)
 *   mul_scalar, relu
 *            crates/hodu_cpu_kernels/kernels/ops_unary.c:138-200, :352-386 (scalar arrives in the storage type),
 *            :648-697, :1233, :1319, :1404, :1484 ((x > 0) ? x : 0 in f32)
 *   scalars  kernels/t_bf16.h:27-55, t_f16.h:27-84, t_f8e4m3.h:27-85, t_f8e5m2.h:27-84
 *   helpers  kernels/utils.h:16-38 (is_contiguous, get_strided_index)
 *
 * Two modes:
 *   ASIS  bit-faithful to the reference: every branch of the reference (threaded, blocked,
 *         strided, batched) adds the products of one output element in ascending k, so a single
 *         sequential-k loop reproduces all of them.  bf16/f16/f8 accumulate IN THE NARROW TYPE
 *         with a conversion after every multiply and every add (ops_matrix.c:212-213).
 *         Integers wrap in their own width.  f8e4m3 decodes exponent 15 as inf/NaN
 *         (t_f8e4m3.h:34-38).
 *   SPEC  the comparator named by the parity bar for bf16/f16/fp8: inputs widened exactly to
 *         f32 (f8e4m3 decoded as OCP E4M3FN, max 448, as the gfx950 hardware does), products
 *         accumulated in f32 in ascending k.  Also returns an f64-accumulated value and
 *         sum_k |a*b| so a test can put a floor under the relative-error denominator.
 *
 * Pinning (see tests/test_oracle_*.py): ASIS is compared bit for bit with oracle/_ref (the real
 * reference C compiled from /root/reference) and with the committed fixtures tests/golden/ that
 * were produced from it; with the literal vectors of the reference's own kernel tests; integer
 * results with numpy int64 matmul; SPEC with float64 matmul and torch's float8/bfloat16 tables.
 *
 * The element-wise functions (add, mul_scalar, relu) are compared bit for bit with oracle/_ref on random bit
 * patterns of every dtype, with the literal vectors of the reference's tests (tests/ops_binary.rs:68-73,
 * tests/ops_unary.rs:143-147, :503-507) and, for bf16, with an independent numpy f32 sum whose low 16 bits are cut.
 *
 * sum: ASIS is compared bit for bit with oracle/_ref on every dtype and layout, except f32 / f64 sums over the last
 * dense dim alone, where the reference adds lane-wise (SIMD width of the build) and only a tolerance applies: the
 * bits of that one case are parity unpinned.  Integer sums against numpy; SPEC against float64.
 *
 * softmax: the comparator computes the function itself in f32 and f64 on exactly widened inputs (one rounding, none in
 * between); it is held against a float64 numpy softmax, against sum-to-one and shift invariance, and -- for f32 --
 * against the five-kernel chain run through oracle/_ref (hodu_cpu_max / sub / exp / sum / div), which it matches to
 * rounding.  The reference's bf16 / f16 chain rounds after every kernel and accumulates the sum in the narrow type;
 * as for the products, the GPU is gated against the f32 comparator, not against that chain.  The masked form is
 * held against the softmax of each row's unmasked entries (what it must equal whenever a row has one), against the
 * unmasked function for a mask of ones, against the explicit fill-then-softmax in numpy, and -- for f32 -- against the
 * reference's five-kernel chain run on a numpy masked_fill of the scores.  The conversion of -65504 to bf16 (-65536 by
 * round-to-nearest) is the Rust `half` crate's, not under /root/reference: parity unpinned; it only shows in the
 * maximum of a row masked entirely, whose result (uniform) does not depend on it.
 *
 * Parity unpinned: float->integer casts of out-of-range or NaN inputs are undefined behaviour
 * in the reference C ((T)x) and are not checked.  The stored code of an f8 x f8 -> f8 product: the reference
 * narrows an accumulator that it re-rounded to f8 after every k with float_to_f8e4m3 (t_f8e4m3.h:52-85); the device
 * rounds the f32 sum once, to nearest even, saturating.  No fixture of the reference holds an f8 product, so the
 * device's f8 outputs are checked against the SPEC value narrowed by an independent round-to-nearest-even encoder
 * (bit for bit on exactly representable sums, tests/test_gpu_exact.py), not against the reference's bytes.  (The
 * library's optional reference-sum mode, hodu_rocm_ctx_set_reference_sums, IS held to the reference's bytes: against
 * the asis products here and against oracle/_ref, tests/test_emu_reference_sums_cpu.py.)
 */
#include <math.h>
#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* dtype ids: crates/hodu_core/src/types/dtype.rs:6-28 */
enum {
    DT_BOOL = 0, DT_F8E4M3 = 1, DT_F8E5M2 = 2, DT_BF16 = 3, DT_F16 = 4, DT_F32 = 5, DT_F64 = 6,
    DT_U8 = 7, DT_U16 = 8, DT_U32 = 9, DT_U64 = 10, DT_I8 = 11, DT_I16 = 12, DT_I32 = 13, DT_I64 = 14,
    DT_COUNT = 15
};

enum { F8_DECODE_HODU = 0, F8_DECODE_OCP = 1 };

static const size_t k_dtype_size[DT_COUNT] = {1, 1, 1, 2, 2, 4, 8, 1, 2, 4, 8, 1, 2, 4, 8};

size_t oracle_dtype_size(int dt) { return (dt >= 0 && dt < DT_COUNT) ? k_dtype_size[dt] : 0; }

/* ------------------------------------------------------------------------------------------ */
/* scalar conversions                                                                           */
/* ------------------------------------------------------------------------------------------ */

static inline float bits_to_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static inline uint32_t f32_to_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

/* t_bf16.h:27-39 -- widening is a 16-bit shift, narrowing TRUNCATES (no rounding). */
static inline float bf16_widen(uint16_t h) { return bits_to_f32((uint32_t)h << 16); }
static inline uint16_t bf16_truncate(float f) { return (uint16_t)(f32_to_bits(f) >> 16); }

/* t_f16.h:27-48 */
static inline float f16_widen(uint16_t h) {
    uint32_t s = (h >> 15) & 1u, e = (h >> 10) & 0x1Fu, m = h & 0x3FFu;
    float v;
    if (e == 0x1F) {
        if (m != 0) return NAN;
        v = INFINITY;
    } else if (e == 0) {
        if (m == 0) return s ? -0.0f : 0.0f;
        v = ldexpf((float)m / 1024.0f, -14);
    } else {
        v = ldexpf(1.0f + (float)m / 1024.0f, (int)e - 15);
    }
    return s ? -v : v;
}

/* t_f16.h:50-84 -- not IEEE rounding: values below 2^-14 flush to signed zero, the mantissa is
 * rounded half-up and clamped (no carry into the exponent). */
static inline uint16_t f16_narrow(float val) {
    if (val == 0.0f) return 0;
    if (isnan(val)) return 0x7E00;
    uint32_t sign = val < 0 ? 1u : 0u;
    val = fabsf(val);
    if (isinf(val) || val > 65504.0f) return (uint16_t)((sign << 15) | 0x7C00u);
    if (val < 0.00006103515625f) return (uint16_t)(sign << 15);
    int e;
    float m = frexpf(val, &e);
    e += 14;
    if (e <= 0) { m = ldexpf(m, e); e = 0; }
    else if (e >= 31) return (uint16_t)((sign << 15) | 0x7C00u);
    int mb = (int)((m * 2.0f - 1.0f) * 1024.0f + 0.5f);
    if (mb > 1023) mb = 1023;
    return (uint16_t)((sign << 15) | ((uint32_t)e << 10) | (uint32_t)mb);
}

/* t_f8e4m3.h:27-50 -- hodu's CPU decoder treats exponent 15 as inf (mant 0) / NaN. */
static inline float f8e4m3_widen_hodu(uint8_t b) {
    uint32_t s = (b >> 7) & 1u, e = (b >> 3) & 0xFu, m = b & 7u;
    float v;
    if (e == 15) {
        if (m != 0) return NAN;
        v = INFINITY;
    } else if (e == 0) {
        if (m == 0) return s ? -0.0f : 0.0f;
        v = ldexpf((float)m / 8.0f, -6);
    } else {
        v = ldexpf(1.0f + (float)m / 8.0f, (int)e - 7);
    }
    return s ? -v : v;
}

/* OCP 8-bit floating point, E4M3 ("FN"): exponent 15 is an ordinary binade up to 448;
 * only S.1111.111 is NaN; no infinities.  This is what hodu's Rust F8E4M3 type and the gfx950
 * conversion / MFMA instructions implement. */
static inline float f8e4m3_widen_ocp(uint8_t b) {
    uint32_t s = (b >> 7) & 1u, e = (b >> 3) & 0xFu, m = b & 7u;
    float v;
    if (e == 15 && m == 7) return NAN;
    if (e == 0) {
        if (m == 0) return s ? -0.0f : 0.0f;
        v = ldexpf((float)m / 8.0f, -6);
    } else {
        v = ldexpf(1.0f + (float)m / 8.0f, (int)e - 7);
    }
    return s ? -v : v;
}

/* t_f8e4m3.h:52-85.  The expression (sign<<7)|(exp<<3)|mant_bits is evaluated in 32-bit
 * arithmetic and truncated to a byte on return; in the sub-normal branch mant_bits can be
 * negative, which the truncation turns into high bits.  Kept as is. */
static inline uint8_t f8e4m3_narrow(float val) {
    if (val == 0.0f) return 0;
    if (isnan(val)) return 0x7F;
    uint32_t sign = val < 0 ? 1u : 0u;
    val = fabsf(val);
    if (isinf(val) || val > 448.0f) return (uint8_t)((sign << 7) | 0x7Fu);
    if (val < 0.001953125f) return (uint8_t)(sign << 7);
    int e;
    float m = frexpf(val, &e);
    e += 6;
    if (e <= 0) { m = ldexpf(m, e); e = 0; }
    else if (e >= 15) return (uint8_t)((sign << 7) | 0x7Fu);
    int mb = (int)((m * 2.0f - 1.0f) * 8.0f + 0.5f);
    if (mb > 7) mb = 7;
    return (uint8_t)((sign << 7) | (uint32_t)(e << 3) | (uint32_t)mb);
}

/* t_f8e5m2.h:27-50 */
static inline float f8e5m2_widen(uint8_t b) {
    uint32_t s = (b >> 7) & 1u, e = (b >> 2) & 0x1Fu, m = b & 3u;
    float v;
    if (e == 31) {
        if (m != 0) return NAN;
        v = INFINITY;
    } else if (e == 0) {
        if (m == 0) return s ? -0.0f : 0.0f;
        v = ldexpf((float)m / 4.0f, -14);
    } else {
        v = ldexpf(1.0f + (float)m / 4.0f, (int)e - 15);
    }
    return s ? -v : v;
}

/* t_f8e5m2.h:52-84 */
static inline uint8_t f8e5m2_narrow(float val) {
    if (val == 0.0f) return 0;
    if (isnan(val)) return 0x7F;
    uint32_t sign = val < 0 ? 1u : 0u;
    val = fabsf(val);
    if (isinf(val) || val > 57344.0f) return (uint8_t)((sign << 7) | 0x7Fu);
    if (val < 0.0000152587890625f) return (uint8_t)(sign << 7);
    int e;
    float m = frexpf(val, &e);
    e += 14;
    if (e <= 0) { m = ldexpf(m, e); e = 0; }
    else if (e >= 31) return (uint8_t)((sign << 7) | 0x7Fu);
    int mb = (int)((m * 2.0f - 1.0f) * 4.0f + 0.5f);
    if (mb > 3) mb = 3;
    return (uint8_t)((sign << 7) | (uint32_t)(e << 2) | (uint32_t)mb);
}

/* exported scalar probes (tables in the tests are built with these) */
float oracle_f8e4m3_to_f32(uint8_t b, int decode) {
    return decode == F8_DECODE_OCP ? f8e4m3_widen_ocp(b) : f8e4m3_widen_hodu(b);
}
uint8_t oracle_f32_to_f8e4m3(float f) { return f8e4m3_narrow(f); }
float oracle_f8e5m2_to_f32(uint8_t b) { return f8e5m2_widen(b); }
uint8_t oracle_f32_to_f8e5m2(float f) { return f8e5m2_narrow(f); }
float oracle_f16_to_f32(uint16_t h) { return f16_widen(h); }
uint16_t oracle_f32_to_f16(float f) { return f16_narrow(f); }
float oracle_bf16_to_f32(uint16_t h) { return bf16_widen(h); }
uint16_t oracle_f32_to_bf16(float f) { return bf16_truncate(f); }

/* ------------------------------------------------------------------------------------------ */
/* layout helpers                                                                               */
/* ------------------------------------------------------------------------------------------ */

/* utils.h:16-27 -- dims of extent 1 do not constrain their stride. */
int oracle_is_contiguous(size_t nd, const size_t *dims, const size_t *strides) {
    size_t expect = 1;
    for (size_t r = nd; r-- > 0;) {
        if (dims[r] > 1 && strides[r] != expect) return 0;
        expect *= dims[r];
    }
    return 1;
}

/* utils.h:29-38 -- row-major unravel of a flat index, then dot with the strides. */
static inline size_t strided_pos(size_t flat, size_t nd, const size_t *dims, const size_t *strides) {
    size_t pos = 0;
    for (size_t r = nd; r-- > 0;) {
        pos += (flat % dims[r]) * strides[r];
        flat /= dims[r];
    }
    return pos;
}

/* thread_utils.h:46-58 -- thread count the reference would use (reported by the bench). */
size_t oracle_reference_threads(size_t work, size_t min_per_thread, size_t online) {
    if (work < 2 * min_per_thread) return 1;
    size_t want = work / min_per_thread;
    return want < online ? want : online;
}

/* One product space: `batches` independent (M x K) * (K x N) problems, each with its own base
 * offsets, sharing the four matrix strides (all in elements). */
typedef struct {
    size_t batches, M, K, N;
    size_t a_m, a_k, b_k, b_n;
    size_t *a_base, *b_base; /* [batches] */
} product_space;

static void product_space_free(product_space *ps) { free(ps->a_base); free(ps->b_base); }

/* ops_matrix.c:76-93 (unpack) and :152-185 (batch index -> operand offsets: an operand whose
 * batch extent is 1 stays at index 0; operands may have fewer batch dims than the output). */
static int product_space_from_matmul(const size_t *md, product_space *ps) {
    const size_t l_nd = md[1], r_nd = md[2], b_nd = md[3];
    if (l_nd < 2 || r_nd < 2 || b_nd > 16) return -1;
    const size_t *l_shape = md + 4, *r_shape = l_shape + l_nd, *b_shape = r_shape + r_nd;
    const size_t *l_str = b_shape + b_nd, *r_str = l_str + l_nd;
    const size_t *tail = r_str + r_nd;
    const size_t l_off = tail[0], r_off = tail[1];
    ps->M = tail[2]; ps->K = tail[3]; ps->N = tail[4];
    ps->a_m = l_str[l_nd - 2]; ps->a_k = l_str[l_nd - 1];
    ps->b_k = r_str[r_nd - 2]; ps->b_n = r_str[r_nd - 1];
    size_t nb = 1;
    for (size_t d = 0; d < b_nd; d++) nb *= b_shape[d];
    ps->batches = nb;
    ps->a_base = (size_t *)malloc(sizeof(size_t) * (nb ? nb : 1));
    ps->b_base = (size_t *)malloc(sizeof(size_t) * (nb ? nb : 1));
    const size_t l_bnd = l_nd - 2, r_bnd = r_nd - 2;
    for (size_t b = 0; b < nb; b++) {
        size_t idx[16], t = b;
        for (size_t d = b_nd; d-- > 0;) { idx[d] = t % b_shape[d]; t /= b_shape[d]; }
        size_t ao = l_off, bo = r_off;
        for (size_t d = 0; d < l_bnd; d++) {
            size_t i = (l_shape[d] == 1) ? 0 : idx[b_nd - l_bnd + d];
            ao += i * l_str[d];
        }
        for (size_t d = 0; d < r_bnd; d++) {
            size_t i = (r_shape[d] == 1) ? 0 : idx[b_nd - r_bnd + d];
            bo += i * r_str[d];
        }
        ps->a_base[b] = ao; ps->b_base[b] = bo;
    }
    return 0;
}

/* ops_matrix.c:429-437 */
static int product_space_from_dot(const size_t *md, product_space *ps) {
    ps->M = md[0]; ps->K = md[1]; ps->N = md[2];
    ps->a_m = md[3]; ps->a_k = md[4]; ps->b_k = md[5]; ps->b_n = md[6];
    ps->batches = 1;
    ps->a_base = (size_t *)malloc(sizeof(size_t));
    ps->b_base = (size_t *)malloc(sizeof(size_t));
    ps->a_base[0] = md[7]; ps->b_base[0] = md[8];
    return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* ASIS products                                                                                */
/* ------------------------------------------------------------------------------------------ */

/* Native types: `sum += a * b` in the element type.  Integer sums are done in the unsigned type
 * of the same width so that wrap-around is defined; the bit pattern equals what the reference's
 * signed arithmetic produces on two's-complement hardware. */
#define ASIS_NATIVE(NAME, T, ACC)                                                              \
    static void NAME(const void *ap, const void *bp, void *op, const product_space *ps) {      \
        const T *a = (const T *)ap, *b = (const T *)bp;                                        \
        T *o = (T *)op;                                                                        \
        const size_t MN = ps->M * ps->N;                                                       \
        _Pragma("omp parallel for collapse(2) schedule(static)")                               \
        for (size_t bt = 0; bt < ps->batches; bt++)                                            \
            for (size_t i = 0; i < ps->M; i++) {                                               \
                const T *arow = a + ps->a_base[bt] + i * ps->a_m;                              \
                const T *bmat = b + ps->b_base[bt];                                            \
                for (size_t j = 0; j < ps->N; j++) {                                           \
                    ACC acc = 0;                                                               \
                    for (size_t k = 0; k < ps->K; k++)                                         \
                        acc = (ACC)(acc + (ACC)((ACC)arow[k * ps->a_k] *                       \
                                                (ACC)bmat[k * ps->b_k + j * ps->b_n]));        \
                    o[bt * MN + i * ps->N + j] = (T)acc;                                       \
                }                                                                              \
            }                                                                                  \
    }

ASIS_NATIVE(asis_f32, float, float)
ASIS_NATIVE(asis_f64, double, double)
ASIS_NATIVE(asis_u8, uint8_t, uint8_t)
ASIS_NATIVE(asis_u16, uint16_t, uint16_t)
ASIS_NATIVE(asis_u32, uint32_t, uint32_t)
ASIS_NATIVE(asis_u64, uint64_t, uint64_t)
ASIS_NATIVE(asis_i8, int8_t, uint8_t)
ASIS_NATIVE(asis_i16, int16_t, uint16_t)
ASIS_NATIVE(asis_i32, int32_t, uint32_t)
ASIS_NATIVE(asis_i64, int64_t, uint64_t)

/* Narrow floats: widen both factors, multiply in f32, narrow; widen the running sum, add in
 * f32, narrow -- two narrowing conversions per k. */
#define ASIS_NARROW(NAME, T, WIDEN, NARROW)                                                    \
    static void NAME(const void *ap, const void *bp, void *op, const product_space *ps) {      \
        const T *a = (const T *)ap, *b = (const T *)bp;                                        \
        T *o = (T *)op;                                                                        \
        const size_t MN = ps->M * ps->N;                                                       \
        _Pragma("omp parallel for collapse(2) schedule(static)")                               \
        for (size_t bt = 0; bt < ps->batches; bt++)                                            \
            for (size_t i = 0; i < ps->M; i++) {                                               \
                const T *arow = a + ps->a_base[bt] + i * ps->a_m;                              \
                const T *bmat = b + ps->b_base[bt];                                            \
                for (size_t j = 0; j < ps->N; j++) {                                           \
                    T acc = 0;                                                                 \
                    for (size_t k = 0; k < ps->K; k++) {                                       \
                        T p = NARROW(WIDEN(arow[k * ps->a_k]) *                                \
                                     WIDEN(bmat[k * ps->b_k + j * ps->b_n]));                  \
                        acc = NARROW(WIDEN(acc) + WIDEN(p));                                   \
                    }                                                                          \
                    o[bt * MN + i * ps->N + j] = acc;                                          \
                }                                                                              \
            }                                                                                  \
    }

ASIS_NARROW(asis_bf16, uint16_t, bf16_widen, bf16_truncate)
ASIS_NARROW(asis_f16, uint16_t, f16_widen, f16_narrow)
ASIS_NARROW(asis_f8e4m3, uint8_t, f8e4m3_widen_hodu, f8e4m3_narrow)
ASIS_NARROW(asis_f8e5m2, uint8_t, f8e5m2_widen, f8e5m2_narrow)

typedef void (*asis_fn)(const void *, const void *, void *, const product_space *);

static asis_fn asis_for(int dt) {
    switch (dt) {
    case DT_F8E4M3: return asis_f8e4m3;
    case DT_F8E5M2: return asis_f8e5m2;
    case DT_BF16: return asis_bf16;
    case DT_F16: return asis_f16;
    case DT_F32: return asis_f32;
    case DT_F64: return asis_f64;
    case DT_U8: return asis_u8;
    case DT_U16: return asis_u16;
    case DT_U32: return asis_u32;
    case DT_U64: return asis_u64;
    case DT_I8: return asis_i8;
    case DT_I16: return asis_i16;
    case DT_I32: return asis_i32;
    case DT_I64: return asis_i64;
    default: return NULL; /* bool has no matmul: utils/valid.rs:260-264 */
    }
}

/* hodu_cpu_matmul_<dt>: out has metadata[0] elements of dtype dt. */
int oracle_matmul_asis(int dt, const void *lhs, const void *rhs, void *out, const size_t *md) {
    asis_fn fn = asis_for(dt);
    product_space ps;
    if (!fn || product_space_from_matmul(md, &ps)) return -1;
    fn(lhs, rhs, out, &ps);
    product_space_free(&ps);
    return 0;
}

/* hodu_cpu_dot_<dt> */
int oracle_dot_asis(int dt, const void *lhs, const void *rhs, void *out, const size_t *md) {
    asis_fn fn = asis_for(dt);
    product_space ps;
    if (!fn || product_space_from_dot(md, &ps)) return -1;
    fn(lhs, rhs, out, &ps);
    product_space_free(&ps);
    return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* SPEC products                                                                                */
/* ------------------------------------------------------------------------------------------ */

static inline float widen_any(int dt, const void *p, size_t i, int f8_decode) {
    switch (dt) {
    case DT_F8E4M3: {
        uint8_t b = ((const uint8_t *)p)[i];
        return f8_decode == F8_DECODE_OCP ? f8e4m3_widen_ocp(b) : f8e4m3_widen_hodu(b);
    }
    case DT_F8E5M2: return f8e5m2_widen(((const uint8_t *)p)[i]);
    case DT_BF16: return bf16_widen(((const uint16_t *)p)[i]);
    case DT_F16: return f16_widen(((const uint16_t *)p)[i]);
    case DT_F32: return ((const float *)p)[i];
    case DT_I8: return (float)((const int8_t *)p)[i];
    case DT_U8: return (float)((const uint8_t *)p)[i];
    default: return NAN;
    }
}

/* Mixed-storage product in f32: lhs stored as l_dt, rhs stored as r_dt (e.g. bf16 activations
 * times f8e4m3 weights == to_dtype(bf16) of the weights followed by matmul, because widening
 * f8 -> bf16 -> f32 is exact).  out32: sequential-k f32 sums; out64 / outabs (optional):
 * sum and sum of magnitudes accumulated in f64. */
static int spec_run(int l_dt, int r_dt, int f8_decode, const void *lhs, const void *rhs,
                    float *out32, double *out64, double *outabs, const product_space *ps) {
    const size_t M = ps->M, K = ps->K, N = ps->N, MN = M * N;
    float *A = (float *)malloc(sizeof(float) * (M * K + 1));
    float *B = (float *)malloc(sizeof(float) * (K * N + 1));
    if (!A || !B) { free(A); free(B); return -2; }
    for (size_t bt = 0; bt < ps->batches; bt++) {
        _Pragma("omp parallel for schedule(static)")
        for (size_t i = 0; i < M; i++)
            for (size_t k = 0; k < K; k++)
                A[i * K + k] = widen_any(l_dt, lhs, ps->a_base[bt] + i * ps->a_m + k * ps->a_k, f8_decode);
        _Pragma("omp parallel for schedule(static)")
        for (size_t k = 0; k < K; k++)
            for (size_t j = 0; j < N; j++)
                B[k * N + j] = widen_any(r_dt, rhs, ps->b_base[bt] + k * ps->b_k + j * ps->b_n, f8_decode);
        _Pragma("omp parallel for schedule(static)")
        for (size_t i = 0; i < M; i++) {
            float *o = out32 + bt * MN + i * N;
            for (size_t j = 0; j < N; j++) o[j] = 0.0f;
            /* i-k-j order: each o[j] still receives its products in ascending k */
            for (size_t k = 0; k < K; k++) {
                const float av = A[i * K + k];
                const float *brow = B + k * N;
                for (size_t j = 0; j < N; j++) o[j] += av * brow[j];
            }
            if (out64 || outabs) {
                /* same i-k-j order in f64: row-wise passes over B keep the oracle fast */
                double *s = (double *)calloc(2 * (N + 1), sizeof(double));
                double *sa = s + N + 1;
                for (size_t k = 0; k < K; k++) {
                    const double av = (double)A[i * K + k];
                    const float *brow = B + k * N;
                    for (size_t j = 0; j < N; j++) {
                        const double p = av * (double)brow[j];
                        s[j] += p;
                        sa[j] += fabs(p);
                    }
                }
                for (size_t j = 0; j < N; j++) {
                    if (out64) out64[bt * MN + i * N + j] = s[j];
                    if (outabs) outabs[bt * MN + i * N + j] = sa[j];
                }
                free(s);
            }
        }
    }
    free(A); free(B);
    return 0;
}

int oracle_matmul_spec(int l_dt, int r_dt, int f8_decode, const void *lhs, const void *rhs,
                       float *out32, double *out64, double *outabs, const size_t *md) {
    product_space ps;
    if (product_space_from_matmul(md, &ps)) return -1;
    int rc = spec_run(l_dt, r_dt, f8_decode, lhs, rhs, out32, out64, outabs, &ps);
    product_space_free(&ps);
    return rc;
}

int oracle_dot_spec(int l_dt, int r_dt, int f8_decode, const void *lhs, const void *rhs,
                    float *out32, double *out64, double *outabs, const size_t *md) {
    product_space ps;
    if (product_space_from_dot(md, &ps)) return -1;
    int rc = spec_run(l_dt, r_dt, f8_decode, lhs, rhs, out32, out64, outabs, &ps);
    product_space_free(&ps);
    return rc;
}

/* ------------------------------------------------------------------------------------------ */
/* casts and strided gather                                                                     */
/* ------------------------------------------------------------------------------------------ */

/* The reference converts through exactly one intermediate, chosen by the SOURCE type
 * (ops_cast.c:108-388): narrow floats and f32 go through `float`; f64 stays `double` except on
 * the way to a narrow float ((float)x first); integers convert directly, except to narrow floats
 * ((float)x first); bool is first normalised to 0/1. */
typedef struct { int kind; float f; double d; int64_t s; uint64_t u; } wide_value;
enum { WV_F32, WV_F64, WV_SINT, WV_UINT };

static inline wide_value load_wide(int dt, const void *p, size_t i, int f8_decode) {
    wide_value w; w.kind = WV_F32; w.f = 0; w.d = 0; w.s = 0; w.u = 0;
    switch (dt) {
    case DT_BOOL: w.kind = WV_UINT; w.u = ((const uint8_t *)p)[i] != 0; break;
    case DT_F8E4M3: w.f = widen_any(dt, p, i, f8_decode); break;
    case DT_F8E5M2: case DT_BF16: case DT_F16: case DT_F32: w.f = widen_any(dt, p, i, 0); break;
    case DT_F64: w.kind = WV_F64; w.d = ((const double *)p)[i]; break;
    case DT_U8: w.kind = WV_UINT; w.u = ((const uint8_t *)p)[i]; break;
    case DT_U16: w.kind = WV_UINT; w.u = ((const uint16_t *)p)[i]; break;
    case DT_U32: w.kind = WV_UINT; w.u = ((const uint32_t *)p)[i]; break;
    case DT_U64: w.kind = WV_UINT; w.u = ((const uint64_t *)p)[i]; break;
    case DT_I8: w.kind = WV_SINT; w.s = ((const int8_t *)p)[i]; break;
    case DT_I16: w.kind = WV_SINT; w.s = ((const int16_t *)p)[i]; break;
    case DT_I32: w.kind = WV_SINT; w.s = ((const int32_t *)p)[i]; break;
    case DT_I64: w.kind = WV_SINT; w.s = ((const int64_t *)p)[i]; break;
    default: break;
    }
    return w;
}

static inline float wide_as_f32(wide_value w) {
    switch (w.kind) {
    case WV_F32: return w.f;
    case WV_F64: return (float)w.d;
    case WV_SINT: return (float)w.s;
    default: return (float)w.u;
    }
}

/* (T)x for an integer destination; float sources truncate toward zero. */
#define STORE_INT(T)                                                                           \
    do {                                                                                       \
        T v;                                                                                   \
        switch (w.kind) {                                                                      \
        case WV_F32: v = (T)w.f; break;                                                        \
        case WV_F64: v = (T)w.d; break;                                                        \
        case WV_SINT: v = (T)w.s; break;                                                       \
        default: v = (T)w.u; break;                                                            \
        }                                                                                      \
        ((T *)p)[i] = v;                                                                       \
    } while (0)

static inline void store_wide(int dt, void *p, size_t i, wide_value w) {
    switch (dt) {
    case DT_BOOL: {
        uint8_t v;
        switch (w.kind) {
        case WV_F32: v = (w.f != 0.0f); break;
        case WV_F64: v = (w.d != 0.0); break;
        case WV_SINT: v = (w.s != 0); break;
        default: v = (w.u != 0); break;
        }
        ((uint8_t *)p)[i] = v;
        break;
    }
    case DT_F8E4M3: ((uint8_t *)p)[i] = f8e4m3_narrow(wide_as_f32(w)); break;
    case DT_F8E5M2: ((uint8_t *)p)[i] = f8e5m2_narrow(wide_as_f32(w)); break;
    case DT_BF16: ((uint16_t *)p)[i] = bf16_truncate(wide_as_f32(w)); break;
    case DT_F16: ((uint16_t *)p)[i] = f16_narrow(wide_as_f32(w)); break;
    case DT_F32: ((float *)p)[i] = wide_as_f32(w); break;
    case DT_F64:
        ((double *)p)[i] = w.kind == WV_F32 ? (double)w.f : w.kind == WV_F64 ? w.d
                           : w.kind == WV_SINT ? (double)w.s : (double)w.u;
        break;
    case DT_U8: STORE_INT(uint8_t); break;
    case DT_U16: STORE_INT(uint16_t); break;
    case DT_U32: STORE_INT(uint32_t); break;
    case DT_U64: STORE_INT(uint64_t); break;
    case DT_I8: STORE_INT(int8_t); break;
    case DT_I16: STORE_INT(int16_t); break;
    case DT_I32: STORE_INT(int32_t); break;
    case DT_I64: STORE_INT(int64_t); break;
    default: break;
    }
}

/* hodu_cpu_cast_<src>_to_<dst>; metadata = [num_els, nd, shape.., strides.., offset]
 * (ops_cast.c:55-63).  Same-type casts copy the element unchanged except bool -> bool, which
 * normalises to 0/1 (ops_cast.c:108). */
int oracle_cast(int src, int dst, int f8_decode, const void *in, void *out, const size_t *md) {
    if (src < 0 || src >= DT_COUNT || dst < 0 || dst >= DT_COUNT) return -1;
    const size_t n = md[0], nd = md[1];
    const size_t *dims = md + 2, *strides = md + 2 + nd;
    const size_t off = nd > 0 ? md[2 + 2 * nd] : 0;
    const int dense = oracle_is_contiguous(nd, dims, strides);
    _Pragma("omp parallel for schedule(static)")
    for (size_t i = 0; i < n; i++) {
        size_t pos = off + (dense ? i : strided_pos(i, nd, dims, strides));
        if (src == dst && src != DT_BOOL) {
            memcpy((char *)out + i * k_dtype_size[dst], (const char *)in + pos * k_dtype_size[src],
                   k_dtype_size[dst]);
        } else {
            store_wide(dst, out, i, load_wide(src, in, pos, f8_decode));
        }
    }
    return 0;
}

/* hodu_cpu_contiguous_<dt> (ops_memory.c:36-84) */
int oracle_contiguous(int dt, const void *in, void *out, const size_t *md) {
    if (dt < 0 || dt >= DT_COUNT) return -1;
    const size_t n = md[0], nd = md[1], es = k_dtype_size[dt];
    const size_t *dims = md + 2, *strides = md + 2 + nd;
    const size_t off = nd > 0 ? md[2 + 2 * nd] : 0;
    if (oracle_is_contiguous(nd, dims, strides)) {
        memcpy(out, (const char *)in + off * es, n * es);
        return 0;
    }
    _Pragma("omp parallel for schedule(static)")
    for (size_t i = 0; i < n; i++) {
        size_t pos = off + strided_pos(i, nd, dims, strides);
        memcpy((char *)out + i * es, (const char *)in + pos * es, es);
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* element-wise kernels that the callers of the product run on its output                       */
/* ------------------------------------------------------------------------------------------ */
enum { EW_ADD = 1, EW_MUL = 2, EW_RELU = 3 };

/* one element of `op` in the arithmetic of dtype dt; a, b, out point at single elements.
 * Narrow floats: ops_binary.c:228-232 / ops_unary.c:359-371 (float x = TO_FLOAT(..); out = FROM_FLOAT(FUNC)).
 * Native types: the expression is evaluated in TYPE (`TYPE x = ...; out[i] = x + y`), which for the integer types
 * means C's promotion to int followed by conversion back -- modular arithmetic on two's-complement machines. */
static int ew_one(int dt, int op, const void *a, const void *b, void *out) {
#define EW_NARROW(T, WIDEN, NARROW)                                                    \
    {                                                                                  \
        const float x = WIDEN(*(const T *)a);                                          \
        float r;                                                                       \
        if (op == EW_RELU) r = (x > 0.0f) ? x : 0.0f;                                  \
        else {                                                                         \
            const float y = WIDEN(*(const T *)b);                                      \
            r = op == EW_ADD ? x + y : x * y;                                          \
        }                                                                              \
        *(T *)out = NARROW(r);                                                         \
        return 0;                                                                      \
    }
#define EW_FLOAT(T)                                                                    \
    {                                                                                  \
        const T x = *(const T *)a;                                                     \
        if (op == EW_RELU) *(T *)out = (x > (T)0) ? x : (T)0;                          \
        else *(T *)out = op == EW_ADD ? x + *(const T *)b : x * *(const T *)b;         \
        return 0;                                                                      \
    }
#define EW_INT(T, U)                                                                   \
    {                                                                                  \
        if (op == EW_RELU) return -1; /* the reference has no relu for integer types */\
        const U x = (U) * (const T *)a, y = (U) * (const T *)b;                        \
        *(T *)out = (T)(U)(op == EW_ADD ? x + y : x * y);                              \
        return 0;                                                                      \
    }
    switch (dt) {
    case DT_BF16: EW_NARROW(uint16_t, bf16_widen, bf16_truncate)
    case DT_F16: EW_NARROW(uint16_t, f16_widen, f16_narrow)
    case DT_F8E4M3: EW_NARROW(uint8_t, f8e4m3_widen_hodu, f8e4m3_narrow)
    case DT_F8E5M2: EW_NARROW(uint8_t, f8e5m2_widen, f8e5m2_narrow)
    case DT_F32: EW_FLOAT(float)
    case DT_F64: EW_FLOAT(double)
    case DT_U8: EW_INT(uint8_t, uint8_t)
    case DT_U16: EW_INT(uint16_t, uint16_t)
    case DT_U32: EW_INT(uint32_t, uint32_t)
    case DT_U64: EW_INT(uint64_t, uint64_t)
    case DT_I8: EW_INT(int8_t, uint8_t)
    case DT_I16: EW_INT(int16_t, uint16_t)
    case DT_I32: EW_INT(int32_t, uint32_t)
    case DT_I64: EW_INT(int64_t, uint64_t)
    default: return -1;
    }
#undef EW_NARROW
#undef EW_FLOAT
#undef EW_INT
}

/* hodu_cpu_add_<dt>(lhs, rhs, out, metadata); metadata = [num_els, nd, lhs_shape.., rhs_shape.., lhs_strides..,
 * rhs_strides.., lhs_offset, rhs_offset] (ops_binary.c:214-222, op_metadatas.rs:36-73).  All four
 * contiguous / strided branches of the reference compute the same element positions. */
int oracle_add(int dt, const void *lhs, const void *rhs, void *out, const size_t *md) {
    if (dt < 0 || dt >= DT_COUNT) return -1;
    const size_t n = md[0], nd = md[1], es = k_dtype_size[dt];
    const size_t *ls = md + 2, *rs = md + 2 + nd, *lst = md + 2 + 2 * nd, *rst = md + 2 + 3 * nd;
    const size_t lo = md[2 + 4 * nd], ro = md[2 + 4 * nd + 1];
    const int ld = oracle_is_contiguous(nd, ls, lst), rd = oracle_is_contiguous(nd, rs, rst);
    int bad = 0;
    _Pragma("omp parallel for schedule(static) reduction(|:bad)")
    for (size_t i = 0; i < n; i++) {
        const size_t li = lo + (ld ? i : strided_pos(i, nd, ls, lst));
        const size_t ri = ro + (rd ? i : strided_pos(i, nd, rs, rst));
        bad |= ew_one(dt, EW_ADD, (const char *)lhs + li * es, (const char *)rhs + ri * es, (char *)out + i * es) != 0;
    }
    return bad ? -1 : 0;
}

/* hodu_cpu_mul_scalar_<dt>(in, out, metadata, scalar) and hodu_cpu_relu_<dt>(in, out, metadata); metadata =
 * [num_els, nd, shape.., strides.., offset] (ops_unary.c:64-76).  `scalar` points at one element of dtype dt. */
static int ew_unary(int dt, int op, const void *in, void *out, const size_t *md, const void *scalar) {
    if (dt < 0 || dt >= DT_COUNT) return -1;
    const size_t n = md[0], nd = md[1], es = k_dtype_size[dt];
    const size_t *dims = md + 2, *strides = md + 2 + nd;
    const size_t off = nd > 0 ? md[2 + 2 * nd] : 0;
    const int dense = oracle_is_contiguous(nd, dims, strides);
    int bad = 0;
    _Pragma("omp parallel for schedule(static) reduction(|:bad)")
    for (size_t i = 0; i < n; i++) {
        const size_t pos = off + (dense ? i : strided_pos(i, nd, dims, strides));
        bad |= ew_one(dt, op, (const char *)in + pos * es, scalar, (char *)out + i * es) != 0;
    }
    return bad ? -1 : 0;
}
int oracle_mul_scalar(int dt, const void *in, void *out, const size_t *md, const void *scalar) {
    return ew_unary(dt, EW_MUL, in, out, md, scalar);
}
int oracle_relu(int dt, const void *in, void *out, const size_t *md) { return ew_unary(dt, EW_RELU, in, out, md, NULL); }

/* ------------------------------------------------------------------------------------------ */
/* sum over dims (ops_reduce.c)                                                                  */
/* ------------------------------------------------------------------------------------------ */
typedef struct {
    size_t nd, out_nd, n_red, reduce_size, n_out, offset;
    const size_t *dims, *strides, *out_shape, *red;
    int keep;
} reduce_space;

static void reduce_space_from(const size_t *md, reduce_space *r) {
    r->nd = md[0];
    r->dims = md + 1;
    r->strides = md + 1 + r->nd;
    r->offset = md[1 + 2 * r->nd];
    r->out_nd = md[2 + 2 * r->nd];
    r->out_shape = md + 3 + 2 * r->nd;
    r->n_red = md[3 + 2 * r->nd + r->out_nd];
    r->red = md + 4 + 2 * r->nd + r->out_nd;
    r->keep = md[4 + 2 * r->nd + r->out_nd + r->n_red] != 0;
    r->reduce_size = md[5 + 2 * r->nd + r->out_nd + r->n_red];
    r->n_out = 1;
    for (size_t i = 0; i < r->out_nd; i++) r->n_out *= r->out_shape[i];
}

/* input position of reduced index `ri` for output `oi` (ops_reduce.c:68-110) */
static size_t reduce_pos(const reduce_space *r, size_t oi, size_t ri) {
    size_t oidx[16], iidx[16];
    for (size_t d = r->out_nd; d-- > 0;) { oidx[d] = oi % r->out_shape[d]; oi /= r->out_shape[d]; }
    if (r->keep) {
        for (size_t i = 0; i < r->nd; i++) iidx[i] = oidx[i];
    } else {
        size_t o = 0;
        for (size_t d = 0; d < r->nd; d++) {
            int is_red = 0;
            for (size_t k = 0; k < r->n_red; k++) is_red |= r->red[k] == d;
            if (is_red) iidx[d] = 0;
            else { iidx[d] = o < r->out_nd ? oidx[o] : 0; o++; }
        }
    }
    for (size_t k = r->n_red; k-- > 0;) { iidx[r->red[k]] = ri % r->dims[r->red[k]]; ri /= r->dims[r->red[k]]; }
    size_t pos = r->offset;
    for (size_t d = 0; d < r->nd; d++) pos += iidx[d] * r->strides[d];
    return pos;
}

/* hodu_cpu_sum_<dt>: accumulator in the storage type, reduced elements added in reduced-index order */
int oracle_sum_asis(int dt, const void *in, void *out, const size_t *md) {
    if (dt <= DT_BOOL || dt >= DT_COUNT) return -1;
    reduce_space r;
    reduce_space_from(md, &r);
    const size_t es = k_dtype_size[dt];
    _Pragma("omp parallel for schedule(static)")
    for (size_t o = 0; o < r.n_out; o++) {
        unsigned char acc[8] = {0};
        for (size_t i = 0; i < r.reduce_size; i++) {
            unsigned char next[8];
            ew_one(dt, EW_ADD, acc, (const char *)in + reduce_pos(&r, o, i) * es, next);
            memcpy(acc, next, es);
        }
        memcpy((char *)out + o * es, acc, es);
    }
    return 0;
}

/* comparator for the floating dtypes: elements widened exactly (f8e4m3 by `f8_decode`), summed in f32 in the same
 * order; also the f64 sum and the sum of magnitudes (floor of the relative-error denominator) */
int oracle_sum_spec(int dt, int f8_decode, const void *in, const size_t *md, float *out32, double *out64, double *out_abs) {
    if (dt <= DT_BOOL || dt >= DT_COUNT) return -1;
    reduce_space r;
    reduce_space_from(md, &r);
    _Pragma("omp parallel for schedule(static)")
    for (size_t o = 0; o < r.n_out; o++) {
        float s32 = 0.0f;
        double s64 = 0.0, sabs = 0.0;
        for (size_t i = 0; i < r.reduce_size; i++) {
            const size_t pos = reduce_pos(&r, o, i);
            const float v = dt == DT_F64 ? (float)((const double *)in)[pos] : widen_any(dt, in, pos, f8_decode);
            const double d = dt == DT_F64 ? ((const double *)in)[pos] : (double)v;
            s32 += v;
            s64 += d;
            sabs += fabs(d);
        }
        if (out32) out32[o] = s32;
        if (out64) out64[o] = s64;
        if (out_abs) out_abs[o] = sabs;
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* softmax along one dim (normalization.rs:4-21), comparator form                                */
/* ------------------------------------------------------------------------------------------ */
/* md: reduce_metadata of the input with the softmax dim as the single reduced dim.  out32 / out64: the function in
 * f32 (expf, f32 sum in index order) and in f64, contiguous in the input's shape.  causal: entries j > i of every
 * [.., Sq, Sk] matrix (softmax dim last) are -inf before the softmax (attention.rs:40-48). */
int oracle_softmax_spec(int dt, const void *in, const size_t *md, int causal, float *out32, double *out64) {
    if (dt != DT_BF16 && dt != DT_F16 && dt != DT_F32 && dt != DT_F64) return -1;
    reduce_space r;
    reduce_space_from(md, &r);
    if (r.n_red != 1) return -1;
    const size_t dim = r.red[0], len = r.dims[dim];
    if (causal && (dim + 1 != r.nd || r.nd < 2)) return -1;
    const size_t sq = r.nd >= 2 ? r.dims[r.nd - 2] : 1;
    size_t inner = 1;  /* contiguous output: elements between consecutive entries of the softmax dim */
    for (size_t d = dim + 1; d < r.nd; d++) inner *= r.dims[d];
    _Pragma("omp parallel for schedule(static)")
    for (size_t o = 0; o < r.n_out; o++) {
        /* n_out counts the kept positions (keep_dim or not): o = outer * inner + in_pos */
        const size_t outer = o / inner, in_pos = o % inner;
        const size_t limit = causal ? ((o % sq) + 1 < len ? (o % sq) + 1 : len) : len;
        double m64 = -INFINITY;
        float m32 = -INFINITY;
        for (size_t j = 0; j < limit; j++) {
            const size_t pos = reduce_pos(&r, o, j);
            const double v = dt == DT_F64 ? ((const double *)in)[pos] : (double)widen_any(dt, in, pos, F8_DECODE_OCP);
            if (v > m64) m64 = v;
            if ((float)v > m32) m32 = (float)v;
        }
        double s64 = 0.0;
        float s32 = 0.0f;
        for (size_t j = 0; j < limit; j++) {
            const size_t pos = reduce_pos(&r, o, j);
            const double v = dt == DT_F64 ? ((const double *)in)[pos] : (double)widen_any(dt, in, pos, F8_DECODE_OCP);
            s64 += exp(v - m64);
            s32 += expf((float)v - m32);
        }
        for (size_t j = 0; j < len; j++) {
            const size_t pos = reduce_pos(&r, o, j);
            const double v = dt == DT_F64 ? ((const double *)in)[pos] : (double)widen_any(dt, in, pos, F8_DECODE_OCP);
            const size_t q = (outer * len + j) * inner + in_pos;
            if (out64) out64[q] = j < limit ? exp(v - m64) / s64 : 0.0;
            if (out32) out32[q] = j < limit ? expf((float)v - m32) / s32 : 0.0f;
        }
    }
    return 0;
}

/* The same with scaled_dot_product_attention's attn_mask (crates/hodu_nn/src/modules/attention.rs:40-56): the causal
 * mask (j > i) and the attention mask (mask element == 0; `mask.eq_scalar(0)`) are both applied by masked_fill with
 * get_neg_inf(dtype) (attention.rs:88-96: -inf for f32 / f64, -65504 for f16 / bf16), the scalar converted to the
 * tensor's dtype by full_like (tensor/ops/selection.rs:20-24; round to nearest: -65504 in f16, -65536 in bf16), and the
 * softmax runs over ALL entries of the row, filled ones included.  So a masked entry of a row that has an unmasked one
 * comes out as exp(fill - max) = 0; a row masked entirely comes out uniform (1 / len) in the 16-bit types and NaN in
 * f32 / f64 (-inf - -inf).  mask: one byte per element; mask_strides: nd element strides over the INPUT's shape (0
 * where the mask is broadcast), softmax dim last. */
int oracle_softmax_masked_spec(int dt, const void *in, const size_t *md, int causal, const unsigned char *mask,
                               const size_t *mask_strides, size_t mask_off, float *out32, double *out64) {
    if (dt != DT_BF16 && dt != DT_F16 && dt != DT_F32 && dt != DT_F64) return -1;
    reduce_space r;
    reduce_space_from(md, &r);
    if (r.n_red != 1 || r.red[0] + 1 != r.nd) return -1;
    const size_t len = r.dims[r.nd - 1];
    const size_t sq = r.nd >= 2 ? r.dims[r.nd - 2] : 1;
    const double fill = dt == DT_F16 ? -65504.0 : dt == DT_BF16 ? -65536.0 : -INFINITY;
    _Pragma("omp parallel for schedule(static)")
    for (size_t o = 0; o < r.n_out; o++) {
        /* o counts the rows in row-major order of the leading dims */
        size_t mrow = mask_off, rem = o;
        for (size_t d = r.nd - 1; d-- > 0;) {
            mrow += (rem % r.dims[d]) * mask_strides[d];
            rem /= r.dims[d];
        }
        const size_t limit = causal ? ((o % sq) + 1 < len ? (o % sq) + 1 : len) : len;
        double m64 = -INFINITY, s64 = 0.0;
        float m32 = -INFINITY, s32 = 0.0f;
        for (int pass = 0; pass < 3; pass++)
            for (size_t j = 0; j < len; j++) {
                const size_t pos = reduce_pos(&r, o, j);
                const int open = j < limit && mask[mrow + j * mask_strides[r.nd - 1]] != 0;
                const double v = !open ? fill : dt == DT_F64 ? ((const double *)in)[pos] : (double)widen_any(dt, in, pos, F8_DECODE_OCP);
                if (pass == 0) {
                    if (v > m64) m64 = v;
                    if ((float)v > m32) m32 = (float)v;
                } else if (pass == 1) {
                    s64 += exp(v - m64);
                    s32 += expf((float)v - m32);
                } else {
                    if (out64) out64[o * len + j] = exp(v - m64) / s64;
                    if (out32) out32[o * len + j] = expf((float)v - m32) / s32;
                }
            }
    }
    return 0;
}

/* ------------------------------------------------------------------------------------------ */
/* single-thread timing entry points for the cpu_baseline (the reference runs batched / strided */
/* matmul and M < 512 dot on ONE thread: ops_matrix.c:144-192, :455, thread_utils.h:46-50)      */
/* ------------------------------------------------------------------------------------------ */
void oracle_set_threads(int n) {
#ifdef _OPENMP
    extern void omp_set_num_threads(int);
    omp_set_num_threads(n > 0 ? n : 1);
#else
    (void)n;
#endif
}
