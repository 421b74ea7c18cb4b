// fkd_launch.hpp -- host-side launchers of the ahead-of-time compiled kernels (grid geometry, host-side alignment
// check, hipLaunchKernel).  Launch geometry being replaced: FK/core/execution_model/executors.h:242-351.
#pragma once

#include "fkd_kernels.hpp"
#include "registry.hpp"

namespace fkd {

// ---- host-side launchers -------------------------------------------------------------------------------

// Launch with pointers to the arguments: the runtime then makes the only copy of the (up to 8 KB) parameter block,
// straight into its kernel-argument buffer; the <<< >>> form would first copy it by value onto this thread's stack.
template <class Kernel, class... Args>
inline hipError_t launch_by_pointer(Kernel kernel, dim3 grid, dim3 block, hipStream_t stream, const Args&... args) {
    void* ptrs[] = {const_cast<void*>(static_cast<const void*>(&args))...};
    return hipLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, ptrs, 0, stream);
}

inline const char* aligned_name(bool aligned) { return aligned ? "rows" : "rows_unaligned"; }

// Launches with few workgroups (a single 1080p image is 1 080 of them at two rows per thread, about four per compute unit,
// so some units get five and some four) take half the rows per thread: twice the workgroups spread evenly, which on such
// launches outweighs the shorter run of independent loads per thread (1080p chains 5 - 9 % faster, 4K chains 3 % slower,
// hence the limit: below eight workgroups per compute unit of this chip).
constexpr unsigned kRowsSmallGrid = 2048;

template <class Chain, int V, int ROWS>
hipError_t launch_rows_with(const typename Chain::Params& p, hipStream_t stream, LaunchInfo* info, bool aligned) {
    const unsigned gx = (p.active_w + kRowsBX * V - 1) / (kRowsBX * V);
    const unsigned gy = (p.active_h + kRowsBY * ROWS - 1) / (kRowsBY * ROWS);
    dim3 grid(gx, gy, p.active_z);
    const dim3 block(kRowsBX, kRowsBY, 1);
    TileGeom g{0u, 0u, 0u, 0u};
    if constexpr (rows_in_bands<Chain>()) {
        // gathering reads, larger launches: a one-dimensional grid whose workgroups the kernel renumbers into one band per XCD
        if ((unsigned long long)gx * gy > 0x7fffff00ull) return hipErrorInvalidConfiguration;
        if (gx * gy >= kRowsBandBlocks) {
            grid = dim3(rows_band_chunk(gx * gy) * 8u, 1, p.active_z);
            g = TileGeom{gx, gy, gx * gy * p.active_z, division_magic(gx, gx * gy)};
        }
    }
    if (info) *info = LaunchInfo{aligned_name(aligned), {grid.x, grid.y, grid.z}, {block.x, block.y, 1}, 0};
    if (grid.x == 0 || grid.y == 0 || grid.z == 0) return hipSuccess;
    if (grid.y > 65535u || grid.z > 65535u) return hipErrorInvalidConfiguration;
    if (aligned) return launch_by_pointer(&k_rows<Chain, V, ROWS, true>, grid, block, stream, p, g);
    return launch_by_pointer(&k_rows<Chain, V, ROWS, false>, grid, block, stream, p, g);
}

template <class Chain>
hipError_t launch_rows(const typename Chain::Params& p, hipStream_t stream, LaunchInfo* info) {
    constexpr int V = RowsConfig<Chain>::V, ROWS = RowsConfig<Chain>::ROWS;
    // Wide (dwordx3/x4) accesses need every row start dword aligned; checked here, once per launch, on the host.
    const bool aligned = Chain::Read::rows_aligned(p.read, 0) && Chain::Write::rows_aligned(p.write);
    if constexpr (ROWS > 1) {
        const unsigned long long gx = (p.active_w + kRowsBX * V - 1) / (kRowsBX * V);
        const unsigned long long gy = (p.active_h + kRowsBY * ROWS - 1) / (kRowsBY * ROWS);
        if (gx * gy * p.active_z < kRowsSmallGrid) return launch_rows_with<Chain, V, ROWS / 2>(p, stream, info, aligned);
    }
    return launch_rows_with<Chain, V, ROWS>(p, stream, info, aligned);
}

template <class Chain>
hipError_t launch_gather(const typename Chain::Params& p, hipStream_t stream, LaunchInfo* info) {
    constexpr int XI = FKD_GATHER_XI, YI = FKD_GATHER_YI;
    constexpr int TW = kGatherBX * XI, TH = kGatherBY * YI;
    if constexpr (strip_capable<Chain>()) {
        // Narrow outputs (batches of small planes): the strip form, whose workgroups own 8 whole rows of a plane.
        // (an output without columns has no workgroup in the tile form's grid: it falls through and launches nothing)
        if (p.active_w != 0 && p.active_w <= unsigned(kStripMaxWidth) && (p.reserved & 1u) != 0 && fklhip::strip_enabled()) {
            const dim3 grid((p.active_h + kStripRows - 1) / kStripRows, 1, p.active_z), block(kGatherBX, kStripThreads / kGatherBX, 1);
            if (info) *info = LaunchInfo{"strip", {grid.x, 1, grid.z}, {block.x, block.y, 1}, unsigned(kStripMaxWidth * 16 + (kStripThreads / 64) * 4)};
            if (grid.x == 0 || grid.z == 0) return hipSuccess;
            if (grid.z > 65535u) return hipErrorInvalidConfiguration;
            return launch_by_pointer(&k_strip<Chain>, grid, block, stream, p, strip_first_late_workgroup((unsigned long long)grid.x * grid.z));
        }
    }
    TileGeom g;
    g.tiles_x = (p.active_w + TW - 1) / TW;
    g.tiles_y = (p.active_h + TH - 1) / TH;
    g.n_tiles = g.tiles_x * g.tiles_y * p.active_z;
    g.tiles_x_magic = division_magic(g.tiles_x, g.tiles_x * g.tiles_y);
    const unsigned chunk = (g.tiles_x * g.tiles_y + 7u) / 8u;
    const dim3 grid(chunk * 8u, 1, p.active_z), block(kGatherBX, kGatherBY, 1);
    if (info) *info = LaunchInfo{"gather", {grid.x, 1, grid.z}, {block.x, block.y, 1}, 0};
    if (g.n_tiles == 0) return hipSuccess;
    if (grid.z > 65535u) return hipErrorInvalidConfiguration;
    return launch_by_pointer(&k_gather<Chain, XI, YI>, grid, block, stream, p, g);
}

// Several chains in one launch: the grid of the rows kernel over the largest extent, alignment decided per plane on
// the device.
template <class D>
hipError_t launch_divergent(const typename D::Params& p, hipStream_t stream, LaunchInfo* info) {
    constexpr int V = RowsConfig<D>::V, ROWS = RowsConfig<D>::ROWS;
    const unsigned gx = (p.active_w + kRowsBX * V - 1) / (kRowsBX * V);
    const unsigned gy = (p.active_h + kRowsBY * ROWS - 1) / (kRowsBY * ROWS);
    const dim3 grid(gx, gy, p.active_z), block(kRowsBX, kRowsBY, 1);
    if (info) *info = LaunchInfo{"divergent", {grid.x, grid.y, grid.z}, {block.x, block.y, 1}, 0};
    if (grid.x == 0 || grid.y == 0 || grid.z == 0) return hipSuccess;
    if (grid.y > 65535u || grid.z > unsigned(D::kMaxPlanes)) return hipErrorInvalidConfiguration;
    return launch_by_pointer(&k_divergent<D>, grid, block, stream, p);
}

template <class Chain>
hipError_t launch_chain(const typename Chain::Params& p, hipStream_t stream, LaunchInfo* info) {
    if constexpr (IsDivergent<Chain>::value) return launch_divergent<Chain>(p, stream, info);
    else if constexpr (is_gather_chain<Chain>()) return launch_gather<Chain>(p, stream, info);
    else return launch_rows<Chain>(p, stream, info);
}

} // namespace fkd
