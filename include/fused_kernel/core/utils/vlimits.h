// maxValue<T> / minValue<T>: numeric limits of an element type, every channel for vector types.
// Interface counterpart: FK/core/utils/vlimits.h.
#ifndef FK_AMD_VLIMITS_H
#define FK_AMD_VLIMITS_H
#include <limits>
#include <fused_kernel/core/utils/vector_utils.h>
namespace fk {
template <typename T, typename Enabler = void> constexpr T maxValue{};
template <typename T> constexpr T maxValue<T, std::enable_if_t<!validCUDAVec<T> && !std::is_aggregate_v<T>>> = std::numeric_limits<T>::max();
template <typename T> constexpr T maxValue<T, std::enable_if_t<validCUDAVec<T>>> = make_set<T>(maxValue<VBase<T>>);
template <typename T, typename Enabler = void> constexpr T minValue{};
template <typename T> constexpr T minValue<T, std::enable_if_t<!validCUDAVec<T> && !std::is_aggregate_v<T>>> = std::numeric_limits<T>::lowest();
template <typename T> constexpr T minValue<T, std::enable_if_t<validCUDAVec<T>>> = make_set<T>(minValue<VBase<T>>);
} // namespace fk
#endif
