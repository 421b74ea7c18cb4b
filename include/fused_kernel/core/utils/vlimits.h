// fk::maxValue<T> and fk::minValue<T>: the largest and the lowest value an element type can hold; for a vector type,
// that value in every channel.  Interface counterpart: FK/core/utils/vlimits.h (same two names, used as constants).
#ifndef FK_AMD_VLIMITS_H
#define FK_AMD_VLIMITS_H

#include <limits>

#include <fused_kernel/core/utils/vector_utils.h>

namespace fk {
namespace amd {
enum class Extreme { Lowest, Largest };
// One function for scalars and vectors: a vector broadcasts the bound of its channel type.
template <typename T, Extreme WHICH> constexpr T extreme_of() {
    if constexpr (validCUDAVec<T>) {
        return make_set<T>(extreme_of<VBase<T>, WHICH>());
    } else {
        static_assert(std::numeric_limits<T>::is_specialized, "fk::maxValue / fk::minValue: not an arithmetic element type");
        if constexpr (WHICH == Extreme::Largest) return std::numeric_limits<T>::max();
        else return std::numeric_limits<T>::lowest();
    }
}
} // namespace amd

template <typename T> inline constexpr T maxValue = amd::extreme_of<T, amd::Extreme::Largest>();
template <typename T> inline constexpr T minValue = amd::extreme_of<T, amd::Extreme::Lowest>();
} // namespace fk

#endif
