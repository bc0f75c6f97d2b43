// Device-scope exchange of partial sums between the workgroups of one launch: 16-byte buffer accesses with the sc1
// bit, an arrival counter, and the argument why that is a release / acquire pair on gfx942 / gfx950.  Used by the
// M <= 16 kernel that cuts K across workgroups (skinny.hip) and by the pipelined tile kernels when they are cut along
// K (gemm_mfma_pipe.hpp): in both the workgroup that arrives last adds the slices in slice order, so the result does
// not depend on who was last.
#pragma once

#include "device_types.hpp"

namespace hodu {

// How partial sums cross from one workgroup to another inside one launch (the workgroups run on different XCDs,
// each with an L2 of its own that is not kept coherent with the others for ordinary accesses):
//   * every partial sum is written and read with 16-byte buffer accesses that carry the sc1 bit, the encoding the
//     gfx942 / gfx950 memory model gives an agent-scope atomic store / load: the store writes through the XCD's L2
//     to memory, the load is served from the point all XCDs share and cannot hit a stale line this XCD kept from
//     an earlier launch.  They are compiler builtins, so the wait-count bookkeeping of every load is the
//     compiler's own;
//   * release: each thread waits for its own stores (s_waitcnt vmcnt(0): a write-through store is acknowledged once
//     it is visible at agent scope), the workgroup barrier follows, and only then does thread 0 increment the
//     counter.  A release FENCE at agent scope would add a write-back of the whole L2 (buffer_wbl2), which exists
//     for dirty lines of ordinary stores; there are none to publish here -- everything published was written
//     through -- and it measured 7 us per launch;
//   * acquire: the workgroup that finds slices - 1 in the counter has, by the counter's atomicity, been preceded by
//     every other slice's increment and therefore by their completed stores; it passes its own barrier and reads
//     with the sc1 loads above, which do not depend on an invalidate of this XCD's caches (buffer_inv, the other
//     half of an acquire fence, is for ordinary loads).
// The counter itself is a relaxed agent-scope read-modify-write, executed where all XCDs see it.
constexpr int AUX_SC1 = 16;  // cache-policy bit of the raw buffer builtins that sets sc1 on gfx942 / gfx950
__device__ __forceinline__ __amdgpu_buffer_rsrc_t agent_buffer(void *base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(base, 0, bytes, 0x00020000);  // raw buffer: no stride, 32-bit format
}
template <typename V>
__device__ __forceinline__ void store16_agent(__amdgpu_buffer_rsrc_t r, unsigned byte_off, const V &v) {
    static_assert(sizeof(V) == 16, "one 16-byte access");
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, v), r, byte_off, 0, AUX_SC1);
}
template <typename V>
__device__ __forceinline__ V load16_agent(__amdgpu_buffer_rsrc_t r, unsigned byte_off) {
    static_assert(sizeof(V) == 16, "one 16-byte access");
    return __builtin_bit_cast(V, __builtin_amdgcn_raw_buffer_load_b128(r, byte_off, 0, AUX_SC1));
}


// Counts this workgroup in on `counter` (every thread's partial sums stored and waited for beforehand) and tells
// all its threads whether it was the last of `expected`; `flag` is a word of LDS.  The last one finds the others'
// sums visible to its sc1 loads.  It must put the counter back to zero (arrival_reset) once it has read them.
__device__ __forceinline__ bool arrive_and_check_last(int *counter, int expected, int *flag, int tid) {
    __builtin_amdgcn_s_waitcnt(0);  // vmcnt(0) expcnt(0) lgkmcnt(0): this thread's stores are visible at agent scope
    __syncthreads();
    if (tid == 0) {
        const int before = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        *flag = before == expected - 1;
    }
    __syncthreads();
    return *flag != 0;
}
__device__ __forceinline__ void arrival_reset(int *counter, int tid) {
    if (tid == 0) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace hodu
