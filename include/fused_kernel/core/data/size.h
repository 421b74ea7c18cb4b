#ifndef FK_AMD_SIZE_H
#define FK_AMD_SIZE_H
#include <fused_kernel/core/utils/utils.h>
namespace fk {
// Interface counterpart: FK/core/data/size.h.
template <typename T> struct Size_ {
    constexpr Size_(T width_, T height_) : width(width_), height(height_) {}
    constexpr Size_() {}
    T width{0};
    T height{0};
};
using Size = Size_<int>;
} // namespace fk
#endif
