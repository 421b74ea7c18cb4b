#ifndef FK_AMD_RECT_H
#define FK_AMD_RECT_H
#include <fused_kernel/core/data/size.h>
#include <fused_kernel/core/data/point.h>
namespace fk {
// Crop rectangle: unsigned origin, signed extent.  Interface counterpart: FK/core/data/rect.h.
template <typename P, typename S = P> struct Rect_ {
    P x{0}, y{0};
    S width{0}, height{0};
    constexpr Rect_(const Point point, const Size size) : x(point.x), y(point.y), width(size.width), height(size.height) {}
    constexpr Rect_(const P x_, const P y_, const S width_, const S height_) : x(x_), y(y_), width(width_), height(height_) {}
    constexpr Rect_() {}
};
using Rect = Rect_<uint, int>;
} // namespace fk
#endif
