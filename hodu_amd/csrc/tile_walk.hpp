// Linear workgroup id -> (batch, tile row, tile column) of the MFMA tile kernels, in 32-bit unsigned arithmetic: a
// grid has fewer than 2^31 workgroups (the launchers check), and the 64-bit signed divisions this replaces took
// 0.65 of the 1.0 microsecond between a workgroup's first instruction and its first load.
// Plain C++ (also compiled for the host by tests/test_tile_walk_cpu.py, which holds it against the 64-bit formula).
#pragma once

#if defined(__HIPCC__)
#define HODU_TILE_WALK_HD __host__ __device__ __forceinline__
#else
#define HODU_TILE_WALK_HD inline
#endif

namespace hodu {

// ids that land on one XCD (id % 8) get neighbouring tiles -- XCD x owns ids x, x + 8, ... and with them a
// contiguous range of the walk -- and tiles are walked in groups of 8 tile-rows, column by column inside a group,
// so that the A and B panels a group shares stay in that XCD's L2
HODU_TILE_WALK_HD void tile_walk(unsigned pid, unsigned total, unsigned tiles_m, unsigned tiles_n, unsigned &batch,
                                 unsigned &tm, unsigned &tn) {
    if ((total & 7u) == 0u) pid = (pid & 7u) * (total >> 3) + (pid >> 3);
    const unsigned per_batch = tiles_m * tiles_n;
    batch = pid / per_batch;
    const unsigned t = pid - batch * per_batch;
    const unsigned width = 8u * tiles_n;
    const unsigned group = t / width, r = t - group * width;
    const unsigned first_m = group * 8u;
    const unsigned left = tiles_m - first_m, gsize = left < 8u ? left : 8u;
    tn = r / gsize;
    tm = first_m + (r - tn * gsize);
}

}  // namespace hodu
