// fkd/launch_info.hpp -- what a launcher reports about the launch it made (plain C++, no HIP).
#pragma once

namespace fkd {

struct LaunchInfo {
    const char* kernel;   // "rows", "rows_unaligned" or "gather"
    unsigned grid[3], block[3];
    unsigned lds_bytes;
};

} // namespace fkd
