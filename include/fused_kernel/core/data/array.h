#ifndef FK_AMD_ARRAY_H
#define FK_AMD_ARRAY_H
#include <array>
#include <cstddef>
#include <fused_kernel/core/utils/utils.h>
namespace fk {
// Fixed-size POD array usable inside parameter structs.  Interface counterpart: FK/core/data/array.h:24-41.
template <typename T, size_t SIZE> struct Array {
    static constexpr size_t size{SIZE};
    T values[SIZE];
    constexpr const T& operator[](const int index) const { return values[index]; }
    constexpr T& operator[](const int index) { return values[index]; }
    constexpr const T& operator[](const size_t index) const { return values[index]; }
    constexpr T& operator[](const size_t index) { return values[index]; }
};

// N copies of one value (FK/core/data/array.h:223-230).
template <size_t BATCH, typename T> constexpr std::array<T, BATCH> make_set_std_array(const T& value) {
    std::array<T, BATCH> a{};
    for (size_t i = 0; i < BATCH; ++i) a[i] = value;
    return a;
}
} // namespace fk
#endif
