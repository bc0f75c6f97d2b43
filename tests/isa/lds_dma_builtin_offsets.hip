// Test input (tests/test_isa_hazards_cpu.py reads the assembly the compiler generates for it; it is never run): two
// LDS-DMA loads through the compiler's own builtin, whose fourth argument is documented as an offset applied to both
// the global and the LDS address, from one global base to one LDS base with offsets of 1 and 2 KB.
#include <hip/hip_runtime.h>

extern "C" __global__ void two_offsets_one_base(const char *g, int *out) {
    extern __shared__ __attribute__((aligned(16))) char smem[];
    const __attribute__((address_space(1))) void *src = (const __attribute__((address_space(1))) void *)(g + threadIdx.x * 16);
    __attribute__((address_space(3))) void *dst = (__attribute__((address_space(3))) void *)smem;
    __builtin_amdgcn_global_load_lds(src, dst, 16, 1024, 0);
    __builtin_amdgcn_global_load_lds(src, dst, 16, 2048, 0);
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    out[threadIdx.x] = reinterpret_cast<int *>(smem)[threadIdx.x + 256];
}
