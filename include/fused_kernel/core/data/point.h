#ifndef FK_AMD_POINT_H
#define FK_AMD_POINT_H
#include <fused_kernel/core/utils/utils.h>
#include <fused_kernel/core/data/nd.h>
namespace fk {
// Thread / pixel index.  Interface counterpart: FK/core/data/point.h.
template <typename T, ND D> struct Point_;
template <typename T> struct Point_<T, ND::_1D> { T x; };
template <typename T> struct Point_<T, ND::_2D> { T x; T y; };
template <typename T> struct Point_<T, ND::_3D> { T x; T y; T z; };
using Point = Point_<int, ND::_3D>;
} // namespace fk
#endif
