// The gfx950 instructions these kernels write out in assembly, one small function each: the matrix instruction with
// a tied accumulator, the LDS-DMA load in its three addressing forms, the M0 writes that go with it, and the wait
// states the hardware wants and the compiler cannot insert for instructions it does not see.
//
// Kept apart from the kernels so that a CPU build of the kernels for tests (tests/emu) can put stand-ins with the
// same names in their place: it defines HODU_GFX950_INSN_PROVIDED before this file is reached.  The product never
// does.
#pragma once
#ifndef HODU_GFX950_INSN_PROVIDED

#include "device_types.hpp"

namespace hodu {
namespace mfma {

typedef float f32x4_acc_t __attribute__((ext_vector_type(4)));

// v_mfma_f32_16x16x32_{bf16,f16} with the accumulator tied to itself and held in the accumulation registers: left to
// the register allocator, a kernel with 64 four-register accumulators and 128 fragment registers came out with the
// accumulators rotating through copies inside the loop (twice the time).  What the compiler then no longer knows about
// the instruction: an accumulator is next touched 64 MFMAs later (or, behind the loop, after a barrier), and its other
// operands come from LDS reads the compiler waits for as for any use of a register.
__device__ __forceinline__ void mfma16x16x32_bf16(const u32x4_t &a, const u32x4_t &b, f32x4_acc_t &c) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma16x16x32_f16(const u32x4_t &a, const u32x4_t &b, f32x4_acc_t &c) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}

// v_mfma_scale_f32_16x16x128_f8f6f4 with unit scales (scale bytes 0x7F = 2^0), both operands of one 8-bit float format
// (FMT 0 = e4m3, 1 = e5m2: the instruction's cbsz / blgp fields), the accumulator tied as above -- left to the register
// allocator, kernels with this many small accumulators came out with copies inside the loop; an accumulator is next
// touched 64 MFMAs later, the other operands come from LDS reads the compiler waits for as for any use of a register.
template <int FMT> __device__ __forceinline__ void mfma16x16x128_f8(const i32x8_t &a, const i32x8_t &b, f32x4_acc_t &c) {
    const int unit = 0x7F7F7F7F;
    if constexpr (FMT == 0)
        asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %3 op_sel_hi:[0,0,0]" : "+a"(c) : "v"(a), "v"(b), "v"(unit));
    else
        asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %3 op_sel_hi:[0,0,0] cbsz:1 blgp:1"
                     : "+a"(c) : "v"(a), "v"(b), "v"(unit));
}

// Kernels that write their MFMAs out in assembly hide them from the compiler's hazard recogniser, which therefore
// inserts nothing between the last matrix instruction and the first read of an accumulator behind the loop.  The
// hardware wants idle wait states there -- up to 18 when a 16-pass instruction's result is read by a vector
// instruction, fewer for the 4- and 8-pass instructions used here -- and does not interlock: these are they.
// The statement orders memory accesses, not registers: the compiler may, and in some kernels does, schedule reads of
// accumulators in front of it -- of those the epilogue needs first, which the loop's last slice wrote some sixty
// matrix instructions earlier.  (Naming the last-written accumulators as operands of the statement does not help:
// the register allocator then copies them to other registers in front of it, which is the read to be avoided.)
// tests/test_isa_hazards_cpu.py holds the generated code to the rule itself: no instruction names a register the
// final two matrix instructions wrote until 18 wait states have passed.
__device__ __forceinline__ void mfma_results_settle() { asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory"); }

// LDS-DMA: 16 bytes per lane from global memory straight into LDS at M0 + lane * 16 (+ the immediate offset, which
// moves the global and the LDS address alike).  Issued through inline assembly so that the compiler's own wait-count
// bookkeeping (which would put an s_waitcnt vmcnt(0) in front of the next LDS read) stays out of the way; completion
// is awaited explicitly before the barrier that publishes the stage.
//   dma16_raw    a full 64-bit address per lane
//   dma16_sbase  a wave-uniform 64-bit base (scalar registers) + a 32-bit byte offset per lane: the form whose
//                per-instruction cost is one M0 write -- no vector arithmetic, no readfirstlane
//   dma16_imm    the same with M0 written beforehand (m0_set) and an immediate offset, so that one M0 value serves
//                several instructions
__device__ __forceinline__ void dma16_raw(const char *gptr, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_addr), "v"(gptr) : "memory");
}
__device__ __forceinline__ void dma16_sbase(const char *sbase, unsigned voff, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_addr), "v"(voff), "s"(sbase) : "memory");
}
template <int IMM> __device__ __forceinline__ void dma16_imm(const char *sbase, unsigned voff) {
    asm volatile("global_load_lds_dwordx4 %0, %1 offset:%2" ::"v"(voff), "s"(sbase), "n"(IMM) : "memory");
}
// M0 = base + literal.  M0 stays as written until the next call: nothing else in these loops reads or writes it (LDS
// reads need no M0 on this target).  An instruction has to separate the write from the DMA that uses it: the MFMA
// that follows in a loop, m0_wait_state() where there is none.
template <int LIT> __device__ __forceinline__ void m0_set(unsigned base) {
    asm volatile("s_add_u32 m0, %0, %1" ::"s"(base), "n"(LIT) : "scc");
}
__device__ __forceinline__ void m0_wait_state() { asm volatile("s_nop 0"); }

// v[e] *= s for the 16 registers of an accumulator, in place.  Through the assembler because, written as C++ inside a
// conditional, the product makes the compiler keep two copies of the accumulators around the branch and move one onto
// the other in every iteration.
template <class V16> __device__ __forceinline__ void scale16_in_place(V16 &v, float s) {
    asm volatile("v_mul_f32 %0, %16, %0\n\tv_mul_f32 %1, %16, %1\n\tv_mul_f32 %2, %16, %2\n\tv_mul_f32 %3, %16, %3\n\t"
                 "v_mul_f32 %4, %16, %4\n\tv_mul_f32 %5, %16, %5\n\tv_mul_f32 %6, %16, %6\n\tv_mul_f32 %7, %16, %7\n\t"
                 "v_mul_f32 %8, %16, %8\n\tv_mul_f32 %9, %16, %9\n\tv_mul_f32 %10, %16, %10\n\tv_mul_f32 %11, %16, %11\n\t"
                 "v_mul_f32 %12, %16, %12\n\tv_mul_f32 %13, %16, %13\n\tv_mul_f32 %14, %16, %14\n\tv_mul_f32 %15, %16, %15"
                 : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]), "+v"(v[8]),
                   "+v"(v[9]), "+v"(v[10]), "+v"(v[11]), "+v"(v[12]), "+v"(v[13]), "+v"(v[14]), "+v"(v[15])
                 : "v"(s));
}

// Between a wavefront's LDS writes and its own reads of what other lanes of it wrote (or the other way round): the
// lanes of a wavefront execute together and one wavefront's LDS operations complete in order, so no instruction is
// needed -- only the compiler must not move the accesses across this point.
__device__ __forceinline__ void wave_lds_fence() { asm volatile("" ::: "memory"); }

}  // namespace mfma
}  // namespace hodu

#endif  // HODU_GFX950_INSN_PROVIDED
