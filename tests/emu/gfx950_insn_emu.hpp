// Test infrastructure: CPU stand-ins for the instruction wrappers of hodu_amd/csrc/gfx950_insn.hpp and for the gfx950
// builtins the kernels use, so that their unmodified source runs in the CPU build (tests/emu/hip/hip_runtime.h).  A translation unit gets this file through -include, ahead of everything else.
//
// What is modelled, as this repository understands the hardware (the kernels that have run on a GPU and pass their
// tests there are the evidence for the model; a kernel that has not is checked against the model, not against the
// hardware):
//   * v_mfma_f32_16x16x32_{bf16,f16}: lane (r = lane % 16, g = lane / 16) supplies k = 8 g .. 8 g + 7 of row r of the
//     first operand and of column r of the second; it then holds D[4 g + e][r], e = 0..3, added to its accumulator;
//   * v_mfma_f32_32x32x16_{bf16,f16}: lane (r = lane % 32, h = lane / 32) supplies k = 8 h .. 8 h + 7 of row / column r;
//     it then holds D[8 (e / 4) + 4 h + e % 4][r], e = 0..15;
//   * the other shapes alike, with the k a lane supplies: one (f32 32 x 32 x 2 and 16 x 16 x 4; f64 16 x 16 x 4, which
//     holds D[4 e + g][r] instead), 16 bytes (i8 32 x 32 x 32 and 16 x 16 x 64), 32 bytes (the 8-bit float forms
//     32 x 32 x 64 and 16 x 16 x 128 with unit scales);
//     all sum in the accumulator's type with k ascending (the hardware's order inside one instruction is not
//     architected; the tests that compare bit for bit use operands whose products and partial sums are exact);
//   * v_dot2_f32_bf16, v_readlane, v_mov with the DPP controls quad_perm / row_mirror / row_half_mirror, ballot,
//     v_permlane32_swap;
//   * global_load_lds_dwordx4: lane l copies 16 bytes from (base + lane offset + immediate) to LDS at M0 + immediate
//     + 16 l: the immediate moves both addresses.  M0 is a per-wavefront register, kept per lane here (every lane
//     writes the same value); a DMA before any M0 write aborts;
//   * when a DMA's bytes arrive is the hardware's business between the issue and the s_waitcnt vmcnt(n) that leaves at
//     most n of the wavefront's loads outstanding.  Two models, chosen by emu_dma_lazy(): at issue (0, the default),
//     and as late as allowed (1) -- queued per lane and written by the s_waitcnt that retires them, oldest first; what
//     is still queued when the kernel returns is dropped.  A kernel must give the same result under both.  A third
//     setting (2) is there to show that the second model can fail a kernel: every wait leaves one load more
//     outstanding than it asks for, as if the kernel's counts were one too lax;
//   * ds_read_b64_tr_b16: of 16 lanes that execute together, lane s supplies the address of 8 bytes; lane i receives
//     16-bit element i % 4 of the data of lanes i / 4, 4 + i / 4, 8 + i / 4, 12 + i / 4.  ds_read_b64_tr_b8: byte i % 8
//     of the data of lanes i / 8, 2 + i / 8, .., 14 + i / 8;
//   * v_cvt_scalef32_pk_bf16_fp8 with a unit scale: the two f8e4m3 (OCP: no infinities, 0x7F / 0xFF are NaN) of the
//     low or high half of a word, widened exactly;
//   * v_perm_b32 with byte selectors 0..7, v_cvt_pk_f32_fp8;
//   * buffer accesses with a raw resource: base + byte offset, dropped (stores) or zero (loads) beyond the size.
// LDS is one 160 KiB array; an "LDS address" is the low 32 bits of a host pointer into it and is turned back into a
// pointer by its distance from the array's start, so the kernels' own address arithmetic runs unchanged, and an address
// outside the array aborts with a message instead of writing somewhere.
#pragma once
#define HODU_GFX950_INSN_PROVIDED

#include <hip/hip_runtime.h>

#include <cstdlib>
#include <vector>

namespace emu {
int &dma_lazy();     // the model of LDS-DMA arrival: 0 at issue, 1 as late as allowed, 2 later than allowed by one
inline char *lds_at(unsigned addr32, unsigned bytes) {
    const unsigned off = addr32 - (unsigned)(uintptr_t)lds_base();
    if (off > kLdsBytes - bytes) {
        fprintf(stderr, "emu: LDS access of %u bytes at %u from the start of a %u-byte LDS\n", bytes, off, kLdsBytes);
        abort();
    }
    return lds_base() + off;
}
// M0, the flag that it has been written and the queue of loads in flight live in the lane (hip_runtime.h: Lane)
#define EMU_M0 (emu::t_lane->m0)
#define EMU_M0_WRITTEN (emu::t_lane->m0_written)
#define EMU_DMA_QUEUE (emu::t_lane->dma_queue)

inline unsigned lane_id() { return flat_tid() % kWave; }
inline void dma16_now(const char *src, unsigned lds_addr) { memcpy(lds_at(lds_addr, 16), src, 16); }
inline void dma16(const char *src, unsigned wave_lds_addr) {
    if (!EMU_M0_WRITTEN) {
        fprintf(stderr, "emu: LDS-DMA before any M0 write\n");
        abort();
    }
    const unsigned dst = wave_lds_addr + 16 * lane_id();
    (void)lds_at(dst, 16);  // the address is checked at issue under both models
    if (dma_lazy()) EMU_DMA_QUEUE.push_back({src, dst});
    else dma16_now(src, dst);
}
// s_waitcnt: vmcnt is bits 3:0 and 15:14 of the immediate
inline void waitcnt(int imm) {
    const size_t vm = (size_t)((imm & 15) | (((imm >> 14) & 3) << 4)) + (dma_lazy() == 2 ? 1 : 0);
    auto &queue = EMU_DMA_QUEUE;
    if (queue.size() > vm) {
        const size_t retire = queue.size() - vm;
        for (size_t i = 0; i < retire; i++) dma16_now(queue[i].src, queue[i].lds_addr);
        queue.erase(queue.begin(), queue.begin() + (long)retire);
    }
}

// One wavefront-wide exchange: every lane deposits `mine`, all wait, every lane reads what it needs.  Deposits
// alternate between two sets of slots, so the next exchange's deposits cannot overwrite what a slower lane still
// reads and one wait per exchange is enough.  All 64 lanes must be running.
constexpr int kWideBytes = 64;
template <class T> inline const unsigned char (*wave_deposit(const T &mine))[kWideBytes] {
    static_assert(sizeof(T) <= kWideBytes, "exchange slot");
    Block *b = current();
    const unsigned tid = flat_tid(), w = tid / kWave, lane = tid % kWave;
    auto slots = b->wide[t_lane->wide_phase++ & 1][w];
    memcpy(slots[lane], &mine, sizeof(T));
    wave_meet();
    return slots;
}

inline float widen_bf16(uint16_t h) { return __uint_as_float((unsigned)h << 16); }
inline float widen_f16(uint16_t h) { return (float)__builtin_bit_cast(_Float16, h); }

typedef unsigned vu32x4 __attribute__((ext_vector_type(4)));
typedef float vf32x4 __attribute__((ext_vector_type(4)));
typedef float vf32x16 __attribute__((ext_vector_type(16)));

// D (ROWS x ROWS) += A (ROWS x K) * B (K x ROWS) for every MFMA shape used here: a lane supplies KPL consecutive k
// (OPB bytes) of row / column r = lane % ROWS, starting at k = KPL * (lane / ROWS); it then holds column r of D rows
//   4 g + e                    (16 x 16: e = 0..3, g = lane / 16)
//   8 (e / 4) + 4 g + e % 4    (32 x 32: e = 0..15, g = lane / 32)
//   4 e + g                    (the f64 16 x 16 x 4 form: its registers step through the rows by four)
// The sums themselves are in emu_models.cpp (compiled with optimisation; this header is not): products of the two
// lanes' operand elements in the accumulate type, k ascending.
enum MfmaKind { kMfmaBf16, kMfmaF16, kMfmaF32, kMfmaF64, kMfmaI8, kMfmaF8E4M3, kMfmaF8E5M2 };
// slots: what the 64 lanes deposited (first operand at byte 0, second at byte opb); acc: this lane's registers
void mfma_sums(int rows, int kpl, int opb, MfmaKind kind, bool f64_rows, const unsigned char (*slots)[64], unsigned lane, void *acc);

template <int ROWS, int KPL, int OPB, MfmaKind KIND, bool F64ROWS = false, class Acc>
inline void mfma_model(const void *a, const void *b, Acc &c) {
    static_assert(2 * OPB <= kWideBytes, "both operands in one exchange slot");
    struct Ops { unsigned char a[OPB], b[OPB]; };
    Ops mine;
    memcpy(mine.a, a, OPB);
    memcpy(mine.b, b, OPB);
    const auto slots = wave_deposit(mine);
    mfma_sums(ROWS, KPL, OPB, KIND, F64ROWS, slots, lane_id(), &c);
}
template <int ROWS, MfmaKind KIND, class Acc> inline void mfma_8k(const vu32x4 &a, const vu32x4 &b, Acc &c) {
    mfma_model<ROWS, 8, 16, KIND>(&a, &b, c);
}
template <int ROWS, class Acc> inline Acc mfma_f32(float a, float b, Acc c) {
    mfma_model<ROWS, 1, 4, kMfmaF32>(&a, &b, c);
    return c;
}
template <class Acc> inline Acc mfma_f64_16(double a, double b, Acc c) {
    mfma_model<16, 1, 8, kMfmaF64, true>(&a, &b, c);
    return c;
}
template <int ROWS, class Vec, class Acc> inline Acc mfma_i8(const Vec &a, const Vec &b, Acc c) {
    static_assert(sizeof(Vec) == 16, "16 bytes of k per lane");
    mfma_model<ROWS, 16, 16, kMfmaI8>(&a, &b, c);
    return c;
}
// the 8-bit float forms (v_mfma_scale_f32_*_f8f6f4 with unit scales): 32 bytes of k per lane; FMT 0 = e4m3, 1 = e5m2
template <int ROWS, int FMT, class Vec, class Acc> inline void mfma_f8(const Vec &a, const Vec &b, Acc &c) {
    static_assert(sizeof(Vec) == 32, "32 bytes of k per lane");
    mfma_model<ROWS, 32, 32, FMT == 0 ? kMfmaF8E4M3 : kMfmaF8E5M2>(&a, &b, c);
}

// v_dot2_f32_bf16: c + a.x * b.x + a.y * b.y
inline float fdot2_bf16(unsigned a, unsigned b, float c) {
    return c + widen_bf16((uint16_t)(a & 0xFFFF)) * widen_bf16((uint16_t)(b & 0xFFFF)) + widen_bf16((uint16_t)(a >> 16)) * widen_bf16((uint16_t)(b >> 16));
}
// what every lane of the wavefront holds in `v`, by lane
inline const unsigned char (*wave_values(unsigned v))[kWideBytes] { return wave_deposit(v); }
inline unsigned slot_u32(const unsigned char (*slots)[kWideBytes], unsigned lane) {
    unsigned v;
    memcpy(&v, slots[lane], 4);
    return v;
}
inline int readlane(int v, int lane) { return (int)slot_u32(wave_values((unsigned)v), (unsigned)lane & 63u); }
// v_mov_b32 with a DPP control, all rows and banks enabled: the controls these kernels use
inline int update_dpp(int old, int src, int ctrl, int row_mask, int bank_mask, bool bound_ctrl) {
    (void)old; (void)bound_ctrl;
    if (row_mask != 0xF || bank_mask != 0xF) (void)no_such_instruction("DPP with a row or bank mask");
    const auto slots = wave_values((unsigned)src);
    const unsigned l = lane_id();
    unsigned from;
    if (ctrl >= 0 && ctrl <= 0xFF) from = (l & ~3u) + (((unsigned)ctrl >> (2 * (l & 3u))) & 3u);  // quad_perm
    else if (ctrl == 0x140) from = (l & ~15u) + (15u - (l & 15u));                                 // row_mirror
    else if (ctrl == 0x141) from = (l & ~7u) + (7u - (l & 7u));                                    // row_half_mirror
    else { (void)no_such_instruction("DPP control"); from = l; }
    return (int)slot_u32(slots, from);
}
inline unsigned long long ballot(bool pred) {
    const auto slots = wave_values(pred ? 1u : 0u);
    unsigned long long m = 0;
    for (unsigned l = 0; l < 64; l++) m |= (unsigned long long)(slot_u32(slots, l) & 1u) << l;
    return m;
}
// v_permlane32_swap: lanes 0..31 of `hi_src` change places with lanes 32..63 of `lo_src`; returns {lo_src', hi_src'}
typedef unsigned vu32x2 __attribute__((ext_vector_type(2)));
inline vu32x2 permlane32_swap(unsigned a, unsigned b) {
    struct Pair { unsigned a, b; };
    const auto slots = wave_deposit(Pair{a, b});
    const unsigned l = lane_id();
    Pair other;
    memcpy(&other, slots[l ^ 32u], sizeof(Pair));
    // vdst (a) keeps its lower half and takes the partner's src (b) lower half in its upper lanes; src the reverse
    return l < 32 ? vu32x2{a, other.a} : vu32x2{other.b, b};
}

template <int ELEM_BYTES, class R> inline R ds_read_tr(const void *lds_ptr) {
    struct Slot { unsigned char d[8]; };
    Slot mine;
    memcpy(&mine, lds_at((unsigned)(uintptr_t)lds_ptr, 8), 8);
    const auto slots = wave_deposit(mine);
    const unsigned lane = lane_id(), group = lane & ~15u, i = lane & 15u;
    unsigned char res[8];
    if (ELEM_BYTES == 2) {
        for (unsigned e = 0; e < 4; e++) memcpy(res + 2 * e, slots[group + 4 * e + i / 4] + 2 * (i % 4), 2);
    } else {
        for (unsigned e = 0; e < 8; e++) res[e] = slots[group + 2 * e + i / 8][i % 8];
    }
    R out;
    memcpy(&out, res, 8);
    return out;
}

// f8e4m3 (OCP) -> bf16 bits, exact
inline uint16_t f8e4m3_to_bf16_bits(uint8_t v) {
    const unsigned sign = (v & 0x80u) << 8, e = (v >> 3) & 15, m = v & 7;
    if (e == 15 && m == 7) return (uint16_t)(sign | 0x7FC0u);
    if (e == 0) {
        if (m == 0) return (uint16_t)sign;
        // subnormal: m * 2^-9; normalise
        int shift = 0;
        unsigned mm = m;
        while (!(mm & 8)) { mm <<= 1; shift++; }
        return (uint16_t)(sign | ((unsigned)(127 - 6 - shift) << 7) | ((mm & 7) << 4));
    }
    return (uint16_t)(sign | ((e - 7 + 127) << 7) | (m << 4));
}
typedef __bf16 vbf16x2 __attribute__((ext_vector_type(2)));
inline vbf16x2 cvt_pk_bf16_fp8(unsigned word, float scale, bool hi) {
    if (scale != 1.0f) (void)no_such_instruction("cvt_scalef32_pk_bf16_fp8 with a scale");
    const unsigned half = hi ? word >> 16 : word & 0xFFFFu;
    const unsigned both = (unsigned)f8e4m3_to_bf16_bits((uint8_t)(half & 0xFF)) | ((unsigned)f8e4m3_to_bf16_bits((uint8_t)(half >> 8)) << 16);
    return __builtin_bit_cast(vbf16x2, both);
}

// v_perm_b32: result byte i is byte sel[i] of the eight bytes {s1 (0..3), s0 (4..7)}; selectors above 7 (sign fills and
// constants) are not used by these kernels
inline unsigned perm_b32(unsigned s0, unsigned s1, unsigned sel) {
    const uint64_t both = ((uint64_t)s0 << 32) | s1;
    unsigned out = 0;
    for (int i = 0; i < 4; i++) {
        const unsigned pick = (sel >> (8 * i)) & 0xFF;
        if (pick > 7) (void)no_such_instruction("perm with a selector above 7");
        out |= (unsigned)((both >> (8 * (pick & 7))) & 0xFF) << (8 * i);
    }
    return out;
}
typedef float vf32x2 __attribute__((ext_vector_type(2)));
inline vf32x2 cvt_pk_f32_fp8(unsigned word, bool hi) {
    const unsigned half = hi ? word >> 16 : word & 0xFFFFu;
    return vf32x2{f8_decode<4, 3>(half & 0xFF), f8_decode<4, 3>(half >> 8)};
}

struct BufferRsrc { char *base; unsigned bytes; };
inline BufferRsrc make_rsrc(void *base, unsigned bytes) { return BufferRsrc{(char *)base, bytes}; }
inline void buffer_store16(const vu32x4 &v, const BufferRsrc &r, unsigned off) {
    if (off <= r.bytes - 16 && r.bytes >= 16) memcpy(r.base + off, &v, 16);
}
inline vu32x4 buffer_load16(const BufferRsrc &r, unsigned off) {
    vu32x4 v{0, 0, 0, 0};
    if (off <= r.bytes - 16 && r.bytes >= 16) memcpy(&v, r.base + off, 16);
    return v;
}

// a value of whatever type the expression wants: for builtins no kernel that runs here reaches
struct Any {
    const char *what;
    template <class T> operator T() const { (void)no_such_instruction(what); return T{}; }
};
}  // namespace emu

#define __amdgpu_buffer_rsrc_t emu::BufferRsrc
#define __builtin_amdgcn_make_buffer_rsrc(base, stride, bytes, flags) emu::make_rsrc(base, bytes)
#define __builtin_amdgcn_raw_buffer_store_b128(v, r, off, soff, aux) emu::buffer_store16(v, r, off)
#define __builtin_amdgcn_raw_buffer_load_b128(r, off, soff, aux) emu::buffer_load16(r, off)
#define __HIP_MEMORY_SCOPE_AGENT 0
#define __hip_atomic_fetch_add(p, v, order, scope) __atomic_fetch_add(p, v, order)
#define __hip_atomic_store(p, v, order, scope) __atomic_store_n(p, v, order)

#define __builtin_amdgcn_readfirstlane(x) (x)
#define __builtin_amdgcn_s_waitcnt(imm) emu::waitcnt(imm)
#define __builtin_amdgcn_sched_barrier(x) ((void)0)
#define __builtin_amdgcn_s_barrier() __syncthreads()
#define __builtin_amdgcn_s_memrealtime() 0ull
#define __builtin_amdgcn_ds_read_tr16_b64_v4i16(p) (emu::ds_read_tr<2, short __attribute__((ext_vector_type(4)))>((const void *)(p)))
#define __builtin_amdgcn_ds_read_tr8_b64_v2i32(p) (emu::ds_read_tr<1, int __attribute__((ext_vector_type(2)))>((const void *)(p)))
#define __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, scale, hi) emu::cvt_pk_bf16_fp8(w, scale, hi)
#define __builtin_amdgcn_global_load_lds(g, l, size, off, aux) \
    (EMU_M0_WRITTEN = true, emu::dma16((const char *)(g), (unsigned)(uintptr_t)(l)))
#define EMU_MFMA(ROWS, WIDEN, a, b, c) \
    ([&] { auto acc_ = (c); emu::mfma_8k<ROWS, WIDEN>(__builtin_bit_cast(emu::vu32x4, a), __builtin_bit_cast(emu::vu32x4, b), acc_); return acc_; }())
#define __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, x, y, z) EMU_MFMA(16, emu::kMfmaBf16, a, b, c)
#define __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, x, y, z) EMU_MFMA(16, emu::kMfmaF16, a, b, c)
#define __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, x, y, z) EMU_MFMA(32, emu::kMfmaBf16, a, b, c)
#define __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, x, y, z) EMU_MFMA(32, emu::kMfmaF16, a, b, c)
#define __builtin_amdgcn_perm(s0, s1, sel) (emu::perm_b32(s0, s1, sel))
#define __builtin_amdgcn_cvt_pk_f32_fp8(word, hi) (emu::cvt_pk_f32_fp8((unsigned)(word), hi))
#define __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, x, y, z) (emu::mfma_f32<32>(a, b, c))
#define __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, x, y, z) (emu::mfma_f32<16>(a, b, c))
#define __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, x, y, z) (emu::mfma_f64_16(a, b, c))
#define __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, x, y, z) (emu::mfma_i8<32>(a, b, c))
#define __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, x, y, z) (emu::mfma_i8<16>(a, b, c))
#define __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, c, fa, fb, sa, scale_a, sb, scale_b) \
    ([&] { auto acc_ = (c); if ((fa) != (fb) || (fa) > 1 || (scale_a) != 0x7F7F7F7F || (scale_b) != 0x7F7F7F7F) (void)emu::no_such_instruction("scaled MFMA beyond unit scales of one 8-bit format"); \
           if ((fa) == 0) emu::mfma_f8<32, 0>(a, b, acc_); else emu::mfma_f8<32, 1>(a, b, acc_); return acc_; }())
#define __builtin_amdgcn_fdot2_f32_bf16(a, b, c, clamp) (emu::fdot2_bf16(__builtin_bit_cast(unsigned, a), __builtin_bit_cast(unsigned, b), c))
#define __builtin_amdgcn_readlane(v, lane) (emu::readlane(v, lane))
#define __builtin_amdgcn_update_dpp(old, src, ctrl, rm, bm, bc) (emu::update_dpp(old, src, ctrl, rm, bm, bc))
#define __builtin_amdgcn_ballot_w64(p) (emu::ballot(p))
#define __builtin_amdgcn_exp2f(x) (exp2f(x))
#define __builtin_amdgcn_permlane32_swap(a, b, fi, bc) (emu::permlane32_swap(a, b))
#define __builtin_amdgcn_s_memtime() 0ull

namespace hodu {
namespace mfma {

typedef float f32x4_acc_t __attribute__((ext_vector_type(4)));
typedef unsigned emu_u32x4 __attribute__((ext_vector_type(4)));

inline void mfma16x16x32_bf16(const emu_u32x4 &a, const emu_u32x4 &b, f32x4_acc_t &c) { emu::mfma_8k<16, emu::kMfmaBf16>(a, b, c); }
inline void mfma16x16x32_f16(const emu_u32x4 &a, const emu_u32x4 &b, f32x4_acc_t &c) { emu::mfma_8k<16, emu::kMfmaF16>(a, b, c); }
typedef int emu_i32x8 __attribute__((ext_vector_type(8)));
template <int FMT> inline void mfma16x16x128_f8(const emu_i32x8 &a, const emu_i32x8 &b, f32x4_acc_t &c) { emu::mfma_f8<16, FMT>(a, b, c); }
inline void mfma_results_settle() {}

inline void emu_set_m0(unsigned v) { EMU_M0 = v; EMU_M0_WRITTEN = true; }
inline void dma16_raw(const char *gptr, unsigned lds_addr) { emu_set_m0(lds_addr); emu::dma16(gptr, EMU_M0); }
inline void dma16_sbase(const char *sbase, unsigned voff, unsigned lds_addr) { emu_set_m0(lds_addr); emu::dma16(sbase + voff, EMU_M0); }
template <int IMM> inline void dma16_imm(const char *sbase, unsigned voff) {
    static_assert(IMM >= 0 && IMM < 4096, "the instruction's offset field as these kernels use it: 12 bits, not negative");
    emu::dma16(sbase + voff + IMM, EMU_M0 + (unsigned)IMM);
}
template <int LIT> inline void m0_set(unsigned base) { emu_set_m0(base + (unsigned)LIT); }
inline void m0_wait_state() {}
template <class V16> inline void scale16_in_place(V16 &v, float s) {
    for (int e = 0; e < 16; e++) v[e] *= s;
}
// the lanes of a wavefront run one after the other here: where the kernels count on their executing together, they meet
inline void wave_lds_fence() { emu::wave_meet(); }

}  // namespace mfma
}  // namespace hodu
