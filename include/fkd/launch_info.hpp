// fkd/launch_info.hpp -- what a launcher reports about the launch it made, and the geometry it hands to the kernels:
// shared by the launchers of the ahead-of-time kernels, the launcher of the run-time compiled ones and the kernels
// themselves (plain C++, no HIP).
#pragma once

namespace fkd {

struct LaunchInfo {
    const char* kernel;   // "rows", "rows_unaligned" or "gather"
    unsigned grid[3], block[3];
    unsigned lds_bytes;
};

// ---- the geometry a launcher hands to kernels that renumber their workgroups ----

// A run-time compiled kernel takes a TileGeom whichever form its launch has.  A launch of the strip form of the bilinear
// kernel has no tiles: its TileGeom has tiles_x == 0 and carries in n_tiles what strip_first_late_workgroup() says about it.
struct TileGeom {
    unsigned tiles_x, tiles_y, n_tiles;
    // floor(2^32 / tiles_x) + 1 when (t * magic) >> 32 == t / tiles_x for every tile number t of a plane, else 0: the
    // division then costs two scalar multiplications instead of a float reciprocal on the vector unit.
    unsigned tiles_x_magic;
};
// The magic for dividing numbers below `limit` by d, or 0 when there is none.
inline unsigned division_magic(unsigned d, unsigned limit) {
    if (d == 0) return 0;
    const unsigned long long m = (1ull << 32) / d + 1;        // m * d - 2^32 is in (0, d]; exact while n * d < 2^32
    return (m < (1ull << 32) && (unsigned long long)limit * d < (1ull << 32)) ? unsigned(m) : 0u;
}

// Rows kernel, bands form of grid: launches of kRowsBandBlocks blocks per plane or more are one-dimensional, 8 *
// rows_band_chunk(blocks) workgroups per plane (see rows_in_bands in the kernels' header).
inline constexpr unsigned rows_band_chunk(unsigned blocks) { return (blocks + 7u) / 8u; }
constexpr unsigned kRowsBandBlocks = 4096;

// Strip form of the bilinear kernel: a launch of at most kStripOneRoundWorkgroups workgroups (eight per compute unit: every
// workgroup resident from the start) runs with wave priorities; the kernel is told the number of the first workgroup that
// counts as started late, or 0 for a launch whose waves keep the default priority (see the kernels' header).
constexpr unsigned kStripOneRoundWorkgroups = 2048, kComputeUnits = 256, kStripLateWorkgroup = 4;
inline unsigned strip_first_late_workgroup(unsigned long long workgroups) {
    return workgroups <= kStripOneRoundWorkgroups ? kStripLateWorkgroup * kComputeUnits : 0u;
}

// What the launcher of a run-time compiled kernel needs to know about it; the kernel's module publishes one.
struct JitMeta {
    unsigned gather;          // 1: gather kernel geometry, 0: rows kernel geometry
    unsigned params_bytes;    // sizeof(Chain::Params)
    unsigned v, rows;         // rows kernel: elements per thread along x, rows per thread
    unsigned xi, yi, by;      // gather kernel: pixels per lane along x, rows per wave, waves per workgroup
    unsigned max_planes;      // most planes (grid z) a launch may have, 0: no limit of the kernel's own
    unsigned strip_width;     // gather kernel: outputs up to this width are launched in strip form (TileGeom::tiles_x == 0), 0: never
    unsigned bands;           // rows kernel: 1 when launches of kRowsBandBlocks blocks per plane or more take the bands form of grid
};

} // namespace fkd
