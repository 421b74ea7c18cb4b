#ifndef FK_AMD_ACTIVE_THREADS_H
#define FK_AMD_ACTIVE_THREADS_H
#include <fused_kernel/core/utils/utils.h>
namespace fk {
// Output geometry of a chain: one work item per (x, y) of each of z planes.
// Interface counterpart: FK/core/execution_model/active_threads.h.
struct ActiveThreads {
    uint x, y, z;
    constexpr ActiveThreads(const uint& vx = 1, const uint& vy = 1, const uint& vz = 1) : x(vx), y(vy), z(vz) {}
};
} // namespace fk
#endif
