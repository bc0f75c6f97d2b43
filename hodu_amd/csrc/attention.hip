// softmax(Q K^T * scale [+ causal mask]) V as ONE kernel that never writes the scores.
//
// hodu_nn's scaled_dot_product_attention (crates/hodu_nn/src/modules/attention.rs:25-70) is, in the reference, a
// batched matmul, mul_scalar, (mask construction + masked_fill,) the five kernels of Tensor::softmax
// (crates/hodu_core/src/tensor/ops/normalization.rs:4-21) and a second batched matmul; the [.., Sq, Sk] scores cross
// memory eight times.  Here a workgroup owns 128 query rows of one head and walks the keys in blocks of 64.  Its
// eight wavefronts are 4 groups of 32 query rows x 2 halves of every key block: a wavefront computes S = Q K^T for
// its 32 rows and 32 keys on the matrix cores, keeps a reference maximum and the row sum of the online softmax of
// ITS keys in registers, converts P = exp(S - m) in registers to the operand layout of the second product and
// adds P V to its own accumulators on the matrix cores.  The two wavefronts of a row group meet once, at the end,
// through LDS: O = (O1 w1 + O2 w2) / (l1 w1 + l2 w2) with w = exp(m - max(m1, m2)), one division and one rounding.
// Spreading a query block over eight wavefronts instead of four halves the time a workgroup needs per key block,
// which is what a causal launch with few heads waits for.  Head dim 128, bf16 or f16, K-dense rows, a positive
// scale; everything else takes the three-launch path (product with fused scale, hodu_rocm_softmax, product).
//
// Pipeline: K and V blocks go from memory straight into LDS (global_load_lds, no registers in between), K one block
// ahead of V, each into a ring of two; a wavefront computes the scores of block i + 1 on the matrix cores while its
// vector ALU runs the softmax of block i (the two are independent, so the compiler interleaves them), then P V of
// block i; one barrier per block.  The exponent reference of a row follows its running maximum lazily (see
// row_max), so the accumulators are rescaled on the first block and then almost never.
//
// Layouts (the MFMAs run with swapped operands, as in the GEMM kernels, so that a lane owns ONE query row):
//   * 32x32x16 MFMA, mma(first, second, acc): both operands hold, in lane (lr, lh) = (lane % 32, lane / 32), the 8
//     consecutive k (8 * lh .. 8 * lh + 7 of the 16-k slice) of their row lr; acc[4 * q + e] of that lane is
//     (second's row lr) x (first's row 8 * q + 4 * lh + e);
//   * S: first = K block rows (keys) from LDS (k-dense rows of 128 bytes, two halves of the 256-byte head row,
//     chunks XOR-swizzled by (row >> 1) & 7), second = the wavefront's Q rows, loaded once into registers;
//   * O: first = V^T (rows = head dim, k = keys) through LDS transpose reads of the [key][head dim] block (chunks
//     XOR-swizzled by (key & 3) << 2), second = P in operand layout.  A lane's S values for a 16-key slice are
//     keys {4 * lh + e} and {8 + 4 * lh + e}; the operand needs keys 8 * lh .. 8 * lh + 7: the two lanes of a row
//     trade one packed register pair (v_permlane32_swap).
//
// Arithmetic: scores and probabilities in f32 (no rounding of the scores to the storage type, unlike the
// three-launch path and the reference), exp(scale * (s - m)) as one fused multiply-add into a base-2 exponential, P
// (at most 2^8) rounded to the storage type only as the second product's operand, O accumulated in f32 and rounded
// once.  The scale is the scalar in the storage type, widened.
//
// With an attn_mask (attention.rs:50-56; the instantiations with a mask operand -- everything they add is behind
// `if constexpr`, so the plain instantiations' code does not change): a lane reads the mask bytes of its row's 16 keys of a block in place, through the mask's own
// strides (0 where it is broadcast), and a masked score becomes fill / scale, fill being what the reference's
// masked_fill writes over the SCALED scores in a 16-bit type (get_neg_inf, attention.rs:88-96, through full_like's
// rounding: -65504 in f16, -65536 in bf16) -- a finite value, so a row masked entirely comes out as the reference's
// uniform average of V over all keys, and any open key zeroes the masked ones (exp(fill - max) = 0 in f32).  The
// causal mask is filled the same way there, so with a mask the kernel walks every key block: a row whose open causal
// keys are all masked averages over the future keys too.  Keys past Sk stay at -inf: they do not exist.
#include <type_traits>

#include "common.hpp"
#include "device_types.hpp"
#include "gemm_mfma_pipe.hpp"
#include "gfx950_insn.hpp"

namespace hodu {
namespace {

using mfma::bitcast;
using mfma::Compute32;
using mfma::kd_slot;
using mfma::lds_get;
using mfma::lds_get_tr;

constexpr int AT_BQ = 128;       // query rows per workgroup (4 groups of 32)
constexpr int AT_BK = 64;        // keys per step (2 halves of 32, one per wavefront of a row group)
constexpr int AT_NT = 512;       // 8 wavefronts: wave & 3 = row group, wave >> 2 = key half
// per head dim D (64 or 128):
//   K block: D / 64 halves of [64 keys][128 bytes], chunks XOR-swizzled by (key >> 1) & 7;
//   V block: [64 keys][2 D bytes], chunks XOR-swizzled so that the four key rows one LDS transpose read touches fall
//   into different banks: by (key & 3) << 2 for 256-byte rows, by ((key >> 1) & 1) << 2 for 128-byte rows (whose keys k and k + 2 would share banks);
//   two blocks of each: the next is written while this one is read.  The same memory carries, at the end, the
//   second key half's (m, l, O) of every row: 4 row groups x (2 + D / 2) floats x 64 lanes.
template <int D> struct AtGeom {
    static_assert(D == 64 || D == 128, "head dim");
    static constexpr int KSTEPS = D / 16, OT = D / 32, NP = D / 64;  // MFMA k steps of S, output tiles, DMAs per wavefront
    static constexpr int K_BYTES = AT_BK * D * 2, V_BYTES = AT_BK * D * 2, ROW = D * 2;
    static constexpr int MERGE = 4 * (2 + D / 2) * 64 * 4;
    static constexpr int LDS = MERGE > 2 * (K_BYTES + V_BYTES) ? MERGE : 2 * (K_BYTES + V_BYTES);
    static __device__ __forceinline__ int vswz(int key) { return D == 128 ? (key & 3) << 2 : ((key >> 1) & 1) << 2; }
};

struct DevAttention {
    int sq, sk;
    long q_row, k_row, v_row;     // element strides between rows (last dim stride 1)
    int nb;                       // batch dims handled in the kernel
    int bshape[kKernelBatchDims];
    long q_bs[kKernelBatchDims], k_bs[kKernelBatchDims], v_bs[kKernelBatchDims];
    long q_off, k_off, v_off;
    long batches;
    float scale_log2e;  // scale * log2(e): the softmax runs on base-2 exponentials
    int causal;
    int q_blocks;
};

struct DevMask {
    const uint8_t *ptr;
    long bs[kKernelBatchDims];  // element (= byte) strides over the batch dims, 0 where the mask is broadcast
    long row, key, off;         // strides along Sq and Sk, offset
    float fill_raw;             // the reference's fill value divided by the scale
};
struct NoMask {};

template <int CK> struct Narrow;
template <> struct Narrow<mfma::CK_BF16> {
    static __device__ __forceinline__ uint32_t pack(float lo, float hi) {  // one v_cvt_pk_bf16_f32
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, bf16x2));
    }
};
template <> struct Narrow<mfma::CK_F16> {
    static __device__ __forceinline__ uint32_t pack(float lo, float hi) {
        typedef float f32x2 __attribute__((ext_vector_type(2)));
        typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
        return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{lo, hi}, f16x2));
    }
};

// the value the other lane of the row (lane ^ 32) holds
__device__ __forceinline__ float partner(float v) {
    const unsigned u = __float_as_uint(v);
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    // r[0]: lanes 32..63 now hold what lanes 0..31 had; r[1]: lanes 0..31 now hold what lanes 32..63 had
    return __uint_as_float((threadIdx.x & 32) ? r[0] : r[1]);
}

template <int CK, int D, class MK>
__global__ __launch_bounds__(AT_NT, 1) void attention_fwd_kernel(const uint16_t *__restrict__ Q, const uint16_t *__restrict__ K,
                                                               const uint16_t *__restrict__ V, uint16_t *__restrict__ O,
                                                               DevAttention a, MK mk) {
    constexpr bool MASKED = !std::is_same<MK, NoMask>::value;
    typedef Compute32<CK> Cmp;
    typedef typename Cmp::acc_t acc_t;
    typedef AtGeom<D> G;
    constexpr int AT_D = D, AT_KSTEPS = G::KSTEPS, AT_K_BYTES = G::K_BYTES, AT_V_BYTES = G::V_BYTES;
    HODU_DYNAMIC_LDS(smem);
    const unsigned lds0 = (unsigned)(uintptr_t)smem;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, lr = lane & 31, lh = lane >> 5;
    const int qg = wave & 3, kh = wave >> 2;
    // the last query block of every head first: with the causal mask it walks the most keys, and the workgroups that
    // finish the launch should be the short ones
    const long batch = blockIdx.x % a.batches;
    const int q0 = (a.q_blocks - 1 - (int)(blockIdx.x / a.batches)) * AT_BQ;
    long qo = a.q_off, ko = a.k_off, vo = a.v_off;
    [[maybe_unused]] long mo = 0;
    if constexpr (MASKED) mo = mk.off;
    {
        long b = batch;
#pragma unroll
        for (int d = kKernelBatchDims - 1; d >= 0; d--)
            if (d < a.nb) {
                const long i = b % a.bshape[d];
                b /= a.bshape[d];
                qo += i * a.q_bs[d]; ko += i * a.k_bs[d]; vo += i * a.v_bs[d];
                if constexpr (MASKED) mo += i * mk.bs[d];
            }
    }

    // keys this workgroup needs: with the causal mask nothing beyond its last query row
    int k_end = a.sk;
    if (!MASKED && a.causal) {
        const int last = q0 + AT_BQ < a.sq ? q0 + AT_BQ : a.sq;
        k_end = last < a.sk ? last : a.sk;
    }
    const int n_blocks = (k_end + AT_BK - 1) / AT_BK;  // >= 1: Sk >= 1

    // ---- global -> LDS without registers in between (global_load_lds_dwordx4: a wavefront's 64 lanes fill 1 KB of
    // consecutive LDS, so the lane that owns an LDS slot fetches the chunk the swizzle puts there).  D / 8 such
    // instructions per K block and per V block, D / 64 of each per wavefront ----
    const uint16_t *k_src[G::NP], *v_src[G::NP];  // the lane's source in block 0
    int k_srow[G::NP], v_srow[G::NP];             // its key row within the block
    unsigned k_dst[G::NP], v_dst[G::NP];          // LDS byte offset of the instruction within the block's buffer
#pragma unroll
    for (int p = 0; p < G::NP; p++) {
        const int i = wave + 8 * p;
        // K: halves of [64 rows][128 bytes]; instruction i fills rows (i % 8) * 8 .. + 7 of half i / 8
        k_srow[p] = (i & 7) * 8 + (lane >> 3);
        k_src[p] = K + ko + (long)k_srow[p] * a.k_row + (i >> 3) * 64 + ((lane & 7) ^ ((k_srow[p] >> 1) & 7)) * 8;
        k_dst[p] = i * 1024;
        // V: [64 keys][2 D bytes]; instruction i fills 1024 / (2 D) keys, a lane one 16-byte chunk of one of them
        constexpr int CPR = G::ROW / 16;  // chunks per key row
        v_srow[p] = i * (64 / CPR) + lane / CPR;
        v_src[p] = V + vo + (long)v_srow[p] * a.v_row + ((lane % CPR) ^ G::vswz(v_srow[p])) * 8;
        v_dst[p] = i * 1024;
    }
    auto dma_k = [&](int kb, int buf) {
#pragma unroll
        for (int p = 0; p < G::NP; p++) {
            int key = kb * AT_BK + k_srow[p];
            key = key < a.sk ? key : a.sk - 1;  // ragged tail: clamped, masked below
            mfma::dma16_raw(reinterpret_cast<const char *>(k_src[p] + (long)(key - k_srow[p]) * a.k_row),
                            __builtin_amdgcn_readfirstlane(lds0 + buf * AT_K_BYTES + k_dst[p]));
        }
    };
    auto dma_v = [&](int kb, int buf) {
#pragma unroll
        for (int p = 0; p < G::NP; p++) {
            int key = kb * AT_BK + v_srow[p];
            key = key < a.sk ? key : a.sk - 1;
            mfma::dma16_raw(reinterpret_cast<const char *>(v_src[p] + (long)(key - v_srow[p]) * a.v_row),
                            __builtin_amdgcn_readfirstlane(lds0 + 2 * AT_K_BYTES + buf * AT_V_BYTES + v_dst[p]));
        }
    };
    // the same for a block that lies wholly inside the keys: one wavefront-uniform offset
    auto dma_k_full = [&](int kb, int buf) {
        const long step = (long)kb * AT_BK * a.k_row;
#pragma unroll
        for (int p = 0; p < G::NP; p++)
            mfma::dma16_raw(reinterpret_cast<const char *>(k_src[p] + step),
                            __builtin_amdgcn_readfirstlane(lds0 + buf * AT_K_BYTES + k_dst[p]));
    };
    auto dma_v_full = [&](int kb, int buf) {
        const long step = (long)kb * AT_BK * a.v_row;
#pragma unroll
        for (int p = 0; p < G::NP; p++)
            mfma::dma16_raw(reinterpret_cast<const char *>(v_src[p] + step),
                            __builtin_amdgcn_readfirstlane(lds0 + 2 * AT_K_BYTES + buf * AT_V_BYTES + v_dst[p]));
    };
    // K runs one block ahead of V: the scores of block kb + 1 are computed while block kb goes through the softmax
    dma_k(0, 0);
    dma_v(0, 0);
    if (n_blocks > 1) dma_k(1, 1);

    // Q fragments of the wavefront's 32 rows stay in registers: lane (lr, lh) holds, per 16-wide slice of the head
    // dim, the 8 elements at 16 * ks + 8 * lh of row lr (rows past Sq are clamped; their results are not stored)
    const int my_row = q0 + qg * 32 + lr;
    const int q_row = my_row < a.sq ? my_row : a.sq - 1;
    u32x4_t qf[AT_KSTEPS];
#pragma unroll
    for (int ks = 0; ks < AT_KSTEPS; ks++)
        qf[ks] = *reinterpret_cast<const u32x4_t *>(Q + qo + (long)q_row * a.q_row + 16 * ks + 8 * lh);

    acc_t o_acc[AT_D / 32];
#pragma unroll
    for (int j = 0; j < AT_D / 32; j++)
#pragma unroll
        for (int e = 0; e < 16; e++) o_acc[j][e] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;  // the maximum is kept on the raw scores (the scale is positive)

    // fragment addresses within a buffer
    int k_frag[AT_KSTEPS];  // K block, the wavefront's 32 keys
#pragma unroll
    for (int ks = 0; ks < AT_KSTEPS; ks++)
        k_frag[ks] = (ks >> 2) * (AT_BK * 128) + (kh * 32 + lr) * 128 + (kd_slot(lr, 2 * (ks & 3) + lh) << 4);
    int v_mn[AT_D / 32];    // V block through transpose reads: head-dim tile j, first 16-key slice of the wavefront
    {
        const int s16 = lane & 15, kq = s16 >> 2, sub = s16 & 3;
        const int col_bytes = ((lane >> 4) & 1) * 32 + sub * 8;
#pragma unroll
        for (int j = 0; j < AT_D / 32; j++) {
            const int bytes = j * 64 + col_bytes, c = bytes >> 4;
            v_mn[j] = (kh * 32 + lh * 8 + kq) * (AT_D * 2) + ((c ^ G::vswz(kq)) << 4) + (bytes & 8);
        }
    }
    const int wave_row0 = q0 + qg * 32;  // the wavefront's first query row
    // the wavefront has nothing to do in a block whose 32 keys of its half lie past the end, or past the mask of all
    // its 32 rows; the tile needs the per-element mask at the ragged end of the keys and where it meets the diagonal
    // (with an attn_mask every block takes the per-element path and the causal mask skips nothing: see the top)
    auto idle_in = [&](int kb) {
        const int key0 = kb * AT_BK + kh * 32;
        return kb >= n_blocks || key0 >= a.sk || (!MASKED && a.causal && key0 > wave_row0 + 31);
    };
    auto edge_in = [&](int kb) {
        const int key0 = kb * AT_BK + kh * 32;
        return MASKED || key0 + 32 > a.sk || (a.causal && key0 + 31 > wave_row0);
    };

    // ---- the phases ----
    auto read_k = [&](u32x4_t (&kf)[AT_KSTEPS], int buf, int from = 0, int to = G::KSTEPS) {
        const char *k_lds = smem + buf * AT_K_BYTES;
#pragma unroll
        for (int ks = from; ks < to; ks++) kf[ks] = lds_get(k_lds, k_frag[ks]);
    };
    auto read_v = [&](u32x2_t (&vf)[AT_D / 32][2], int buf, int sl) {  // one 16-key slice
        const char *v_lds = smem + 2 * AT_K_BYTES + buf * AT_V_BYTES;
#pragma unroll
        for (int j = 0; j < AT_D / 32; j++) {
            vf[j][0] = lds_get_tr<2>(v_lds, v_mn[j] + (sl * 16) * (AT_D * 2));
            vf[j][1] = lds_get_tr<2>(v_lds, v_mn[j] + (sl * 16 + 4) * (AT_D * 2));
        }
    };
    // S = Q K^T: steps [from, to) of the chain over the head dim
    auto scores = [&](const u32x4_t (&kf)[AT_KSTEPS], acc_t &sc, int from, int to) {
#pragma unroll
        for (int ks = from; ks < to; ks++) Cmp::mma(kf[ks], qf[ks], sc);
    };
    auto zero = [&](acc_t &sc) {
#pragma unroll
        for (int e = 0; e < 16; e++) sc[e] = 0.f;
    };
    // the attn_mask bytes of the lane's 16 keys of block kb (a row past Sq reads the last row's, a key past Sk the last
    // key's); fetched one block ahead, so that the loads are in flight during a whole iteration
    struct NoBytes {};
    typedef typename std::conditional<MASKED, uint8_t[16], NoBytes>::type mask_bytes_t;
    auto load_mask = [&](int kb, mask_bytes_t &open) {
        if constexpr (MASKED) {
            const int key0 = kb * AT_BK + kh * 32;
            const uint8_t *mrow = mk.ptr + mo + (long)q_row * mk.row;
#pragma unroll
            for (int q = 0; q < 4; q++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int key = key0 + 8 * q + 4 * lh + e;
                    open[4 * q + e] = mrow[(long)(key < a.sk ? key : a.sk - 1) * mk.key];
                }
        }
    };
    auto mask = [&](acc_t &sc, int kb, const mask_bytes_t &open) {
        const int key0 = kb * AT_BK + kh * 32;
        if constexpr (MASKED) {
#pragma unroll
            for (int q = 0; q < 4; q++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    const int key = key0 + 8 * q + 4 * lh + e;
                    const bool filled = open[4 * q + e] == 0 || (a.causal && key > my_row);
                    sc[4 * q + e] = key >= a.sk ? -INFINITY : filled ? mk.fill_raw : sc[4 * q + e];
                }
        } else {
            const int limit = a.causal && my_row < a.sk - 1 ? my_row : a.sk - 1;  // last key the row attends
#pragma unroll
            for (int q = 0; q < 4; q++)
#pragma unroll
                for (int e = 0; e < 4; e++) sc[4 * q + e] = key0 + 8 * q + 4 * lh + e > limit ? -INFINITY : sc[4 * q + e];
        }
    };
    // The reference value m_run of a row (exponents are taken relative to it) follows the running maximum lazily: it
    // moves only when a block's maximum exceeds it by more than 8 in the base-2 exponent, so P stays below 2^8 --
    // harmless in f32 sums and in the 16-bit operand, whose precision is relative -- and the 64 accumulator
    // registers are rescaled on the first block and then almost never, instead of whenever one of the wavefront's
    // 32 rows meets a new maximum (which with 32 rows is nearly every block).  The result is the same quotient.
    // Returns true if some row's accumulators need the rescale.
    float rescale, neg_mc;
    auto row_max = [&](const acc_t &sc) {
        float m_blk = sc[0];
#pragma unroll
        for (int e = 1; e < 16; e++) m_blk = __builtin_fmaxf(m_blk, sc[e]);
        m_blk = __builtin_fmaxf(m_blk, partner(m_blk));
        // true from -inf (first unmasked key); false for -inf - -inf = NaN (nothing unmasked yet)
        const bool up = (m_blk - m_run) * a.scale_log2e > 8.f;
        const float m_new = up ? m_blk : m_run;
        // a row of the second key half may not have met an unmasked key yet: its reference is still -inf, and
        // exp2(-inf) = 0 keeps its sums at zero instead of producing inf - inf
        const float m_use = m_new == -INFINITY ? 0.f : m_new;
        rescale = up ? __builtin_amdgcn_exp2f((m_run - m_use) * a.scale_log2e) : 1.0f;  // 0 from m_run = -inf
        neg_mc = -m_use * a.scale_log2e;
        m_run = m_new;
        return __builtin_amdgcn_ballot_w64(up) != 0;
    };
    // (in place, through the assembler: written as C++ the conditional product makes the compiler keep two copies of
    // the 64 accumulator registers around the branch and move one onto the other in every iteration)
    auto rescale_o = [&]() {
#pragma unroll
        for (int j = 0; j < AT_D / 32; j++)
            mfma::scale16_in_place(o_acc[j], rescale);
    };
    // P of one 16-key slice (groups q = 2 sl and 2 sl + 1) in operand layout; adds the slice's row sums to l_blk
    auto probs = [&](const acc_t &sc, int sl, float &l_blk) {
        uint32_t pk[4];  // [2 * (q - 2 sl) + pair]: keys 8 * q + 4 * lh + {0, 1} and {2, 3}
#pragma unroll
        for (int qq = 0; qq < 2; qq++) {
            float p[4];
#pragma unroll
            for (int e = 0; e < 4; e++) {
                // exp(scale * (s - m)) as one fused multiply-add and a base-2 exponential; 0 for masked keys
                p[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[4 * (2 * sl + qq) + e], a.scale_log2e, neg_mc));
                l_blk += p[e];
            }
            pk[2 * qq] = Narrow<CK>::pack(p[0], p[1]);
            pk[2 * qq + 1] = Narrow<CK>::pack(p[2], p[3]);
        }
        // lane lh = 0 keeps group 2 sl and receives the partner's; lane lh = 1 receives the partner's group 2 sl + 1
        // and keeps its own: one swap per packed register
        const auto w0 = __builtin_amdgcn_permlane32_swap(pk[0], pk[2], false, false);
        const auto w1 = __builtin_amdgcn_permlane32_swap(pk[1], pk[3], false, false);
        return u32x4_t{w0[0], w1[0], w0[1], w1[1]};
    };
    auto pv = [&](const u32x2_t (&vf)[AT_D / 32][2], const u32x4_t &pf) {  // O += P V for one slice
#pragma unroll
        for (int j = 0; j < AT_D / 32; j++) Cmp::mma(u32x4_t{vf[j][0].x, vf[j][0].y, vf[j][1].x, vf[j][1].y}, pf, o_acc[j]);
    };
    // (l_run is the lane's share of the row sum; the two lanes of a row add up at the end)
    auto finish_row_sum = [&](float l_blk) { l_run = l_run * rescale + l_blk; };

    // ---- prologue: the first block's scores ----
    __builtin_amdgcn_s_waitcnt(mfma::waitcnt_vm_lgkm0(0));
    // (the Q registers are pinned so that the compiler's wait-count tracking knows, on every path into the loop,
    // that their loads have returned; otherwise it waits for them, i.e. for every load in flight, inside the loop)
#pragma unroll
    for (int ks = 0; ks < AT_KSTEPS; ks++) asm volatile("" : "+v"(qf[ks]));
    __syncthreads();
    acc_t s_cur;
    zero(s_cur);
    {
        u32x4_t kf[AT_KSTEPS];
        read_k(kf, 0);
        scores(kf, s_cur, 0, AT_KSTEPS);  // (the second key half's result is not used where its block 0 is idle)
    }
    __syncthreads();  // K buffer 0 may be overwritten

    // The leading blocks of a wavefront need neither the mask nor a test for idleness (both only ever begin to
    // apply, towards the diagonal and the ragged end).  They run in a loop of their own, whose body is two straight
    // blocks around the rarely taken rescale: the matrix cores compute the next block's scores while the vector ALU
    // runs this block's softmax.  The remaining blocks take the general body.  Every wavefront meets one barrier per
    // block either way.
    int n_fast = 0;
    auto loads_whole = [&](int kb) {  // what block kb's iteration loads lies wholly inside the keys
        return (kb + 2 >= n_blocks || (kb + 3) * AT_BK <= a.sk) && (kb + 1 >= n_blocks || (kb + 2) * AT_BK <= a.sk);
    };
    while (n_fast < n_blocks && !idle_in(n_fast) && !idle_in(n_fast + 1) && !edge_in(n_fast) && loads_whole(n_fast)) n_fast++;
    auto next_loads = [&](int kb) {
        // K of the block after next into the buffer S(kb) was read from (behind a barrier), V of the next block into
        // the buffer P V of the previous block was read from (behind the same barrier)
        if (kb + 2 < n_blocks) dma_k(kb + 2, kb & 1);
        if (kb + 1 < n_blocks) dma_v(kb + 1, (kb + 1) & 1);
    };
    auto publish = [&]() {
        __builtin_amdgcn_s_waitcnt(mfma::waitcnt_vm_lgkm0(0));  // this wavefront's part of the next loads has landed
        __syncthreads();  // everybody's has; what this iteration read may be overwritten
    };
    // one fast iteration for a block of parity P (a literal at both call sites, so that ring slots become immediate
    // offsets of the LDS instructions instead of an address add per read): S(kb) in s_in, S(kb + 1) into s_out
    auto fast_block = [&](int kb, const int P, acc_t &s_in, acc_t &s_out) {
        if (kb + 2 < n_blocks) dma_k_full(kb + 2, P);
        if (kb + 1 < n_blocks) dma_v_full(kb + 1, 1 - P);
        u32x4_t kf[AT_KSTEPS];
        u32x2_t vf0[AT_D / 32][2], vf1[AT_D / 32][2];
        constexpr int HALF = AT_KSTEPS / 2, HEAD = D == 128 ? 3 : 2;  // MFMAs issued ahead of the row maximum
        read_k(kf, 1 - P, 0, HALF);
        read_v(vf0, P, 0);
        __builtin_amdgcn_sched_barrier(0);
        read_k(kf, 1 - P, HALF, AT_KSTEPS);
        zero(s_out);
        scores(kf, s_out, 0, HEAD);
        if (row_max(s_in)) rescale_o();
        scores(kf, s_out, HEAD, AT_KSTEPS);
        float l_blk = 0.f;
        const u32x4_t pf0 = probs(s_in, 0, l_blk);
        read_v(vf1, P, 1);
        pv(vf0, pf0);
        const u32x4_t pf1 = probs(s_in, 1, l_blk);
        pv(vf1, pf1);
        finish_row_sum(l_blk);
        publish();
    };
    int kb = 0;
    {
        acc_t s_odd;  // the scores ping-pong between two register sets instead of being copied
        for (; kb + 1 < n_fast; kb += 2) {
            fast_block(kb, 0, s_cur, s_odd);
            fast_block(kb + 1, 1, s_odd, s_cur);
        }
    }
    mask_bytes_t open_cur, open_next;
    load_mask(kb, open_cur);  // (kb = 0 here with a mask: its blocks all take this loop; block 0 exists)
    for (; kb < n_blocks; kb++) {
        next_loads(kb);
        if (kb + 1 < n_blocks) load_mask(kb + 1, open_next);
        acc_t s_next;
        zero(s_next);
        if (!idle_in(kb + 1)) {
            u32x4_t kf[AT_KSTEPS];
            read_k(kf, (kb + 1) & 1);
            scores(kf, s_next, 0, AT_KSTEPS);
        }
        if (!idle_in(kb)) {
            u32x2_t vf0[AT_D / 32][2], vf1[AT_D / 32][2];
            read_v(vf0, kb & 1, 0);
            read_v(vf1, kb & 1, 1);
            mask(s_cur, kb, open_cur);
            if (row_max(s_cur)) rescale_o();
            float l_blk = 0.f;
            const u32x4_t pf0 = probs(s_cur, 0, l_blk);
            pv(vf0, pf0);
            const u32x4_t pf1 = probs(s_cur, 1, l_blk);
            pv(vf1, pf1);
            finish_row_sum(l_blk);
        }
        s_cur = s_next;
        if constexpr (MASKED) {
#pragma unroll
            for (int i = 0; i < 16; i++) open_cur[i] = open_next[i];
        }
        publish();
    }

    // ---- the two key halves of a row group meet: the second half hands (m, l, O) over through LDS, one float per
    // lane and register so that a wavefront's store covers 64 consecutive words (every K / V read is behind the
    // loop's last barrier) ----
    float *mg = reinterpret_cast<float *>(smem) + qg * ((2 + AT_D / 2) * 64) + lane;
    l_run += partner(l_run);
    if (kh == 1) {
        mg[0] = m_run;
        mg[64] = l_run;
#pragma unroll
        for (int j = 0; j < AT_D / 32; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) mg[(2 + 16 * j + e) * 64] = o_acc[j][e];
    }
    __syncthreads();
    if (kh == 1) return;
    {
        // the first half has seen key 0, which no row masks (an attn_mask fills it with a finite value): its reference
        // is finite; the second half's may be -inf (w2 = 0).  Any common reference gives the same quotient.
        const float m2 = mg[0], l2 = mg[64];
        const float m = __builtin_fmaxf(m2, m_run);
        const float w1 = __builtin_amdgcn_exp2f((m_run - m) * a.scale_log2e), w2 = __builtin_amdgcn_exp2f((m2 - m) * a.scale_log2e);
        l_run = l_run * w1 + l2 * w2;
#pragma unroll
        for (int j = 0; j < AT_D / 32; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) o_acc[j][e] = o_acc[j][e] * w1 + mg[(2 + 16 * j + e) * 64] * w2;
    }

    // ---- O / l, one rounding, 8-byte stores: lane (lr, lh) holds row lr, head-dim columns 32 j + 8 q + 4 lh + e ----
    if (my_row >= a.sq) return;
    const float inv = 1.0f / l_run;
    uint16_t *orow = O + (batch * (long)a.sq + my_row) * AT_D;
#pragma unroll
    for (int j = 0; j < AT_D / 32; j++)
#pragma unroll
        for (int q = 0; q < 4; q++) {
            u32x2_t w;
            w.x = Narrow<CK>::pack(o_acc[j][4 * q] * inv, o_acc[j][4 * q + 1] * inv);
            w.y = Narrow<CK>::pack(o_acc[j][4 * q + 2] * inv, o_acc[j][4 * q + 3] * inv);
            *reinterpret_cast<u32x2_t *>(orow + 32 * j + 8 * q + 4 * lh) = w;
        }
}

}  // namespace

// returns HODU_ROCM_UNSUPPORTED (no error text) when the fused kernel does not take the call
int launch_attention(hodu_rocm_ctx *ctx, int dtype, const void *q, const void *k, const void *v, void *out,
                     const AttentionArgs &g, const AttentionMask *mask) {
    if (dtype != HODU_BF16 && dtype != HODU_F16) return HODU_ROCM_UNSUPPORTED;
    if ((g.d != 64 && g.d != 128) || g.sq < 1 || g.sk < 1 || g.batches < 1) return HODU_ROCM_UNSUPPORTED;
    // the row maximum is taken before the scale is applied: the scale must be positive (and finite)
    if (!(g.scale > 0.f) || !(g.scale < INFINITY)) return HODU_ROCM_UNSUPPORTED;
    if (g.nb > kKernelBatchDims) return HODU_ROCM_UNSUPPORTED;
    // 16-byte loads of 8 elements: rows, offsets, batch strides and bases aligned to 8 elements / 16 bytes
    auto al = [](long e) { return e % 8 == 0; };
    if (!al(g.q_row) || !al(g.k_row) || !al(g.v_row) || !al(g.q_off) || !al(g.k_off) || !al(g.v_off)) return HODU_ROCM_UNSUPPORTED;
    for (int d = 0; d < g.nb; d++)
        if (!al(g.q_bs[d]) || !al(g.k_bs[d]) || !al(g.v_bs[d])) return HODU_ROCM_UNSUPPORTED;
    if ((uintptr_t)q % 16 || (uintptr_t)k % 16 || (uintptr_t)v % 16 || (uintptr_t)out % 16) return HODU_ROCM_UNSUPPORTED;
    DevAttention a{};
    a.sq = (int)g.sq; a.sk = (int)g.sk;
    a.q_row = g.q_row; a.k_row = g.k_row; a.v_row = g.v_row;
    a.nb = g.nb;
    for (int d = 0; d < kKernelBatchDims; d++) {
        a.bshape[d] = d < g.nb ? (int)g.bshape[d] : 1;
        a.q_bs[d] = d < g.nb ? g.q_bs[d] : 0;
        a.k_bs[d] = d < g.nb ? g.k_bs[d] : 0;
        a.v_bs[d] = d < g.nb ? g.v_bs[d] : 0;
    }
    a.q_off = g.q_off; a.k_off = g.k_off; a.v_off = g.v_off;
    a.batches = g.batches;
    a.scale_log2e = g.scale * 1.44269504088896340736f;
    a.causal = g.causal ? 1 : 0;
    a.q_blocks = (int)((g.sq + AT_BQ - 1) / AT_BQ);
    const long blocks = g.batches * a.q_blocks;
    if (blocks > 0x7FFFFFFFL) return HODU_ROCM_UNSUPPORTED;
    if (mask) {
        DevMask mk{};
        mk.ptr = (const uint8_t *)mask->ptr;
        for (int d = 0; d < kKernelBatchDims; d++) mk.bs[d] = d < g.nb ? mask->bs[d] : 0;
        mk.row = mask->row; mk.key = mask->key; mk.off = mask->off;
        // what masked_fill writes over the scaled scores (get_neg_inf through full_like's rounding), before the scale
        mk.fill_raw = (dtype == HODU_BF16 ? -65536.f : -65504.f) / g.scale;
        auto launch_masked = [&](auto kernel, int lds, const char *name) -> int {
            if (int rc = ensure_dynamic_lds(ctx, reinterpret_cast<const void *>(kernel), lds)) return rc;
            ctx->last_kernel = name;
            hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(AT_NT), lds, ctx->stream, (const uint16_t *)q, (const uint16_t *)k,
                               (const uint16_t *)v, (uint16_t *)out, a, mk);
            return HODU_ROCM_OK;
        };
        int rc;
        if (g.d == 128)
            rc = dtype == HODU_BF16 ? launch_masked(attention_fwd_kernel<mfma::CK_BF16, 128, DevMask>, AtGeom<128>::LDS, "attention_masked_fwd_bf16")
                                    : launch_masked(attention_fwd_kernel<mfma::CK_F16, 128, DevMask>, AtGeom<128>::LDS, "attention_masked_fwd_f16");
        else
            rc = dtype == HODU_BF16 ? launch_masked(attention_fwd_kernel<mfma::CK_BF16, 64, DevMask>, AtGeom<64>::LDS, "attention_masked_fwd_bf16_d64")
                                    : launch_masked(attention_fwd_kernel<mfma::CK_F16, 64, DevMask>, AtGeom<64>::LDS, "attention_masked_fwd_f16_d64");
        if (rc != HODU_ROCM_OK) return rc;
        HODU_HIP(hipGetLastError());
        return HODU_ROCM_OK;
    }
    auto launch = [&](auto kernel, int lds, const char *name) -> int {
        if (int rc = ensure_dynamic_lds(ctx, reinterpret_cast<const void *>(kernel), lds)) return rc;
        ctx->last_kernel = name;
        hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(AT_NT), lds, ctx->stream, (const uint16_t *)q, (const uint16_t *)k,
                           (const uint16_t *)v, (uint16_t *)out, a, NoMask{});
        return HODU_ROCM_OK;
    };
    int rc;
    if (g.d == 128)
        rc = dtype == HODU_BF16 ? launch(attention_fwd_kernel<mfma::CK_BF16, 128, NoMask>, AtGeom<128>::LDS, "attention_fwd_bf16")
                                : launch(attention_fwd_kernel<mfma::CK_F16, 128, NoMask>, AtGeom<128>::LDS, "attention_fwd_f16");
    else
        rc = dtype == HODU_BF16 ? launch(attention_fwd_kernel<mfma::CK_BF16, 64, NoMask>, AtGeom<64>::LDS, "attention_fwd_bf16_d64")
                                : launch(attention_fwd_kernel<mfma::CK_F16, 64, NoMask>, AtGeom<64>::LDS, "attention_fwd_f16_d64");
    if (rc != HODU_ROCM_OK) return rc;
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}

}  // namespace hodu
