// softmax(Q K^T * scale [+ causal mask]) V as ONE kernel that never writes the scores.
//
// hodu_nn's scaled_dot_product_attention (crates/hodu_nn/src/modules/attention.rs:25-70) is, in the reference, a
// batched matmul, mul_scalar, (mask construction + masked_fill,) the five kernels of Tensor::softmax
// (crates/hodu_core/src/tensor/ops/normalization.rs:4-21) and a second batched matmul; the [.., Sq, Sk] scores cross
// memory eight times.  Here a workgroup owns 128 query rows of one head (a wavefront 32 of them) and walks the keys
// in blocks of 64: S = Q K^T on the matrix cores, the running row maximum and row sum of the online softmax in
// registers, P = exp(S - max) converted in registers to the operand layout of the second product, O += P V on the
// matrix cores, one division and one rounding at the end.  Head dim 128, bf16 or f16, K-dense rows; everything else
// takes the three-launch path (product with fused scale, hodu_rocm_softmax, product).
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
// three-launch path and the reference), P rounded to the storage type only as the second product's operand, O
// accumulated in f32 and rounded once.  The scale is the scalar in the storage type, widened.
#include "common.hpp"
#include "device_types.hpp"
#include "gemm_mfma_pipe.hpp"

namespace hodu {
namespace {

using mfma::bitcast;
using mfma::Compute32;
using mfma::kd_slot;
using mfma::lds_get;
using mfma::lds_get_tr;

constexpr int AT_D = 128;        // head dim
constexpr int AT_BQ = 128;       // query rows per workgroup (32 per wavefront)
constexpr int AT_BK = 64;        // keys per step
constexpr int AT_KSTEPS = AT_D / 16;
constexpr int AT_K_BYTES = AT_BK * AT_D * 2;  // 16 KB: K block, two halves of [64 rows][128 bytes]
constexpr int AT_V_BYTES = AT_BK * AT_D * 2;  // 16 KB: V block, [64 keys][256 bytes]
constexpr int AT_BUF = AT_K_BYTES + AT_V_BYTES;  // one K block and one V block
constexpr int AT_LDS = 2 * AT_BUF;              // two of them: the next block is written while this one is read

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

template <int CK>
__global__ __launch_bounds__(256, 2) void attention_fwd_kernel(const uint16_t *__restrict__ Q, const uint16_t *__restrict__ K,
                                                              const uint16_t *__restrict__ V, uint16_t *__restrict__ O,
                                                              DevAttention a) {
    typedef Compute32<CK> Cmp;
    typedef typename Cmp::acc_t acc_t;
    extern __shared__ __align__(16) char smem[];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, lr = lane & 31, lh = lane >> 5;
    // the last query block of every head first: with the causal mask it walks the most keys, and the workgroups that
    // finish the launch should be the short ones
    const long batch = blockIdx.x % a.batches;
    const int q0 = (a.q_blocks - 1 - (int)(blockIdx.x / a.batches)) * AT_BQ;
    long qo = a.q_off, ko = a.k_off, vo = a.v_off;
    {
        long b = batch;
#pragma unroll
        for (int d = kKernelBatchDims - 1; d >= 0; d--)
            if (d < a.nb) {
                const long i = b % a.bshape[d];
                b /= a.bshape[d];
                qo += i * a.q_bs[d]; ko += i * a.k_bs[d]; vo += i * a.v_bs[d];
            }
    }

    // Q fragments of the wavefront's 32 rows stay in registers: lane (lr, lh) holds, per 16-wide slice of the head
    // dim, the 8 elements at 16 * ks + 8 * lh of row lr (rows past Sq are clamped; their results are not stored)
    const int my_row = q0 + wave * 32 + lr;
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
    float m_run = -INFINITY, l_run = 0.f;

    // keys this workgroup needs: with the causal mask nothing beyond its last query row
    int k_end = a.sk;
    if (a.causal) {
        const int last = q0 + AT_BQ < a.sq ? q0 + AT_BQ : a.sq;
        k_end = last < a.sk ? last : a.sk;
    }
    const int n_blocks = (k_end + AT_BK - 1) / AT_BK;

    // global -> register staging of one K block and one V block: 1024 16-byte chunks each, 4 per thread
    u32x4_t kst[4], vst[4];
    auto fetch = [&](int kb) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int c = tid + 256 * i;           // chunk id: key row = c / 16, chunk of the 256-byte row = c % 16
            int key = kb * AT_BK + (c >> 4);
            key = key < a.sk ? key : a.sk - 1;     // ragged tail: clamped, masked below
            kst[i] = *reinterpret_cast<const u32x4_t *>(K + ko + (long)key * a.k_row + (c & 15) * 8);
            vst[i] = *reinterpret_cast<const u32x4_t *>(V + vo + (long)key * a.v_row + (c & 15) * 8);
        }
    };
    // fragment addresses
    int k_frag[AT_KSTEPS];  // K block, tile 0; tile t adds t * 32 * 128
#pragma unroll
    for (int ks = 0; ks < AT_KSTEPS; ks++)
        k_frag[ks] = (ks >> 2) * (AT_BK * 128) + lr * 128 + (kd_slot(lr, 2 * (ks & 3) + lh) << 4);
    int v_mn[AT_D / 32];    // V block through transpose reads: head-dim tile j, 16-key slice 0
    {
        const int s16 = lane & 15, kq = s16 >> 2, sub = s16 & 3;
        const int col_bytes = ((lane >> 4) & 1) * 32 + sub * 8;
#pragma unroll
        for (int j = 0; j < AT_D / 32; j++) {
            const int bytes = j * 64 + col_bytes, c = bytes >> 4;
            v_mn[j] = (lh * 8 + kq) * (AT_D * 2) + ((c ^ (kq << 2)) << 4) + (bytes & 8);
        }
    }

    auto commit_to = [&](char *buf) {
        char *k_lds = buf, *v_lds = buf + AT_K_BYTES;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int c = tid + 256 * i, row = c >> 4, g = c & 15;
            // K: half g / 8 of the row, chunk g % 8 at its swizzled slot
            *reinterpret_cast<u32x4_t *>(k_lds + (g >> 3) * (AT_BK * 128) + row * 128 + (kd_slot(row, g & 7) << 4)) = kst[i];
            // V: [key][256 bytes], chunk g at slot g ^ ((key & 3) << 2)
            *reinterpret_cast<u32x4_t *>(v_lds + row * (AT_D * 2) + ((g ^ ((row & 3) << 2)) << 4)) = vst[i];
        }
    };

    if (n_blocks > 0) {
        fetch(0);
        commit_to(smem);
        if (n_blocks > 1) fetch(1);
    }
    __syncthreads();
    const int wave_row0 = q0 + wave * 32;  // the wavefront's first query row
    for (int kb = 0; kb < n_blocks; kb++) {
        const char *k_lds = smem + (kb & 1) * AT_BUF, *v_lds = k_lds + AT_K_BYTES;

        // ---- S = Q K^T: two 32-key tiles, their accumulation chains interleaved ----
        acc_t s_acc[AT_BK / 32];
#pragma unroll
        for (int t = 0; t < AT_BK / 32; t++)
#pragma unroll
            for (int e = 0; e < 16; e++) s_acc[t][e] = 0.f;
#pragma unroll
        for (int ks = 0; ks < AT_KSTEPS; ks++)
#pragma unroll
            for (int t = 0; t < AT_BK / 32; t++) Cmp::mma(lds_get(k_lds, k_frag[ks] + t * 32 * 128), qf[ks], s_acc[t]);

        // the next block's K and V have had the S phase to arrive: into the other buffer (nobody reads it: the
        // barrier at the end of the previous iteration came after its last read), then fetch the one after
        if (kb + 1 < n_blocks) {
            commit_to(smem + ((kb + 1) & 1) * AT_BUF);
            if (kb + 2 < n_blocks) fetch(kb + 2);
        }

        // ---- scale (base-2 logits), mask, running maximum ----
        // a block needs the per-element mask only at the ragged end of the keys or where it meets the diagonal
        const bool edge = (kb + 1) * AT_BK > a.sk || (a.causal && (kb + 1) * AT_BK - 1 > wave_row0);
        float m_blk = -INFINITY;
#pragma unroll
        for (int t = 0; t < AT_BK / 32; t++)
#pragma unroll
            for (int q = 0; q < 4; q++)
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    float sv = s_acc[t][4 * q + e] * a.scale_log2e;
                    if (edge) {
                        const int key = kb * AT_BK + t * 32 + 8 * q + 4 * lh + e;
                        if (key >= a.sk || (a.causal && key > my_row)) sv = -INFINITY;
                    }
                    s_acc[t][4 * q + e] = sv;
                    m_blk = sv > m_blk ? sv : m_blk;
                }
        const float m_other = partner(m_blk);
        m_blk = m_other > m_blk ? m_other : m_blk;
        const float m_new = m_blk > m_run ? m_blk : m_run;
        // every row has at least key 0 unmasked in its first block, so m_new is finite from the first block on
        const float rescale = __builtin_amdgcn_exp2f(m_run - m_new);  // 0 on the first block (m_run = -inf)
        m_run = m_new;
        float l_blk = 0.f;
        uint32_t p_pack[AT_BK / 32][8];  // [tile][2 * q + pair]: keys 8 * q + 4 * lh + {0, 1} and {2, 3}
#pragma unroll
        for (int t = 0; t < AT_BK / 32; t++)
#pragma unroll
            for (int q = 0; q < 4; q++) {
                float p[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    p[e] = __builtin_amdgcn_exp2f(s_acc[t][4 * q + e] - m_new);  // exp2(-inf) = 0 for masked keys
                    l_blk += p[e];
                }
                p_pack[t][2 * q] = Narrow<CK>::pack(p[0], p[1]);
                p_pack[t][2 * q + 1] = Narrow<CK>::pack(p[2], p[3]);
            }
        l_blk += partner(l_blk);
        l_run = l_run * rescale + l_blk;
        // the running maximum settles after a few blocks: the accumulators are rescaled only while some row's moves
        if (__builtin_amdgcn_ballot_w64(rescale != 1.0f) != 0) {
#pragma unroll
            for (int j = 0; j < AT_D / 32; j++)
#pragma unroll
                for (int e = 0; e < 16; e++) o_acc[j][e] *= rescale;
        }

        // ---- O += P V: four 16-key slices ----
#pragma unroll
        for (int sl = 0; sl < AT_BK / 16; sl++) {
            const int t = sl >> 1, qe = 2 * (sl & 1);  // the slice's keys are groups q = qe and qe + 1 of tile t
            // lane lh = 0 keeps group qe and receives the partner's group qe; lane lh = 1 receives the partner's
            // group qe + 1 and keeps its own: one swap per packed register
            const auto w0 = __builtin_amdgcn_permlane32_swap(p_pack[t][2 * qe], p_pack[t][2 * qe + 2], false, false);
            const auto w1 = __builtin_amdgcn_permlane32_swap(p_pack[t][2 * qe + 1], p_pack[t][2 * qe + 3], false, false);
            const u32x4_t pf = {w0[0], w1[0], w0[1], w1[1]};
#pragma unroll
            for (int j = 0; j < AT_D / 32; j++) {
                const u32x2_t lo = lds_get_tr<2>(v_lds, v_mn[j] + (sl * 16) * (AT_D * 2));
                const u32x2_t hi = lds_get_tr<2>(v_lds, v_mn[j] + (sl * 16 + 4) * (AT_D * 2));
                Cmp::mma(u32x4_t{lo.x, lo.y, hi.x, hi.y}, pf, o_acc[j]);
            }
        }
        __syncthreads();  // this block's buffer may be overwritten, the next one's is complete
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
                     const AttentionArgs &g) {
    if (dtype != HODU_BF16 && dtype != HODU_F16) return HODU_ROCM_UNSUPPORTED;
    if (g.d != AT_D || g.sq < 1 || g.sk < 1 || g.batches < 1) return HODU_ROCM_UNSUPPORTED;
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
    static bool configured = false;  // benign race: the attribute calls are idempotent
    if (!configured) {
        HODU_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(attention_fwd_kernel<mfma::CK_BF16>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, AT_LDS));
        HODU_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(attention_fwd_kernel<mfma::CK_F16>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, AT_LDS));
        configured = true;
    }
    if (dtype == HODU_BF16) {
        ctx->last_kernel = "attention_fwd_bf16";
        hipLaunchKernelGGL(attention_fwd_kernel<mfma::CK_BF16>, dim3((unsigned)blocks), dim3(256), AT_LDS, ctx->stream,
                           (const uint16_t *)q, (const uint16_t *)k, (const uint16_t *)v, (uint16_t *)out, a);
    } else {
        ctx->last_kernel = "attention_fwd_f16";
        hipLaunchKernelGGL(attention_fwd_kernel<mfma::CK_F16>, dim3((unsigned)blocks), dim3(256), AT_LDS, ctx->stream,
                           (const uint16_t *)q, (const uint16_t *)k, (const uint16_t *)v, (uint16_t *)out, a);
    }
    HODU_HIP(hipGetLastError());
    return HODU_ROCM_OK;
}

}  // namespace hodu
