// Tile order shared by the prefill kernels.
#pragma once
#include <hip/hip_runtime.h>

namespace qproj {

// Workgroup -> tile.  Consecutive workgroup ids are dealt round-robin to the 8 XCDs, each with its
// own L2: every XCD gets one contiguous stretch of the tile order, and the order walks groups of 8
// token tiles x all column tiles column by column, so the workgroups an XCD runs at the same time
// share activation tiles AND weight tiles instead of streaming the whole weight matrix once per
// row of tiles.
// `pid` is the workgroup's index inside the tile space (a launch that carries several matrices starts each
// at a multiple of 8 workgroups, so that pid % 8 is still the XCD).
__device__ __forceinline__ void tile_of_workgroup(int tiles_n, int tiles_m, int pid, int &tn, int &tm) {
    constexpr int kXcds = 8, kGroupM = 8;
    const int total = tiles_n * tiles_m;
    const int x = pid % kXcds, base = total / kXcds, rem = total % kXcds;
    const int q = x * base + min(x, rem) + pid / kXcds;
    const int span = kGroupM * tiles_n, group = q / span, local = q - group * span;
    const int first_m = group * kGroupM, gsz = min(tiles_m - first_m, kGroupM);
    tm = first_m + local % gsz;
    tn = local / gsz;
}

__device__ __forceinline__ void tile_of_workgroup(int tiles_n, int tiles_m, int &tn, int &tm) {
    tile_of_workgroup(tiles_n, tiles_m, (int)blockIdx.x, tn, tm);
}

}  // namespace qproj
