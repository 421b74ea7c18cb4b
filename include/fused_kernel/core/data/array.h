#ifndef FK_AMD_ARRAY_H
#define FK_AMD_ARRAY_H
#include <array>
#include <cstddef>
#include <type_traits>
#include <utility>
#include <fused_kernel/core/utils/utils.h>
#include <fused_kernel/core/utils/vector_utils.h>
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

// A pixel's channels as an indexable value: `at[i]` / `[i]`, built from a channel vector (or from a scalar, which has one
// channel) and convertible back.  Interface counterpart: FK/core/data/array.h:42-221; here one template with an array
// member serves every size, the channel vectors being read and written through their named members.
template <typename T, size_t SIZE> struct ArrayVector {
    enum { size = SIZE };
    T at[SIZE > 0 ? SIZE : 1];
    constexpr ArrayVector() : at{} {}
    constexpr ArrayVector(const T& fill) : at{} { for (size_t i = 0; i < SIZE; ++i) at[i] = fill; }
    template <typename... Ts, typename = std::enable_if_t<(sizeof...(Ts) == SIZE) && (SIZE > 1) && (std::is_convertible_v<Ts, T> && ...)>>
    constexpr ArrayVector(const Ts&... values) : at{static_cast<T>(values)...} {}
    template <typename V, typename = std::enable_if_t<VectorTraits<V>::is_vector && std::is_same_v<VBase<V>, T> && size_t(cn<V>) == SIZE>, typename = void>
    constexpr ArrayVector(const V& v) : at{} { *this = v; }
    template <typename V, typename = std::enable_if_t<VectorTraits<V>::is_vector && std::is_same_v<VBase<V>, T> && size_t(cn<V>) == SIZE>>
    constexpr ArrayVector& operator=(const V& v) {
        at[0] = v.x;
        if constexpr (SIZE > 1) at[1] = v.y;
        if constexpr (SIZE > 2) at[2] = v.z;
        if constexpr (SIZE > 3) at[3] = v.w;
        return *this;
    }
    constexpr T operator[](const size_t& index) const { return at[index]; }
    constexpr T& operator[](const size_t& index) { return at[index]; }
    constexpr T operator()(const int& index) const { return at[index]; }
};
template <typename V> using ToArray = ArrayVector<VBase<V>, size_t(cn<V>)>;
template <typename V> constexpr ToArray<V> toArray(const V& value) { return ToArray<V>(value); }
template <typename T, size_t SIZE> constexpr VectorType_t<T, int(SIZE)> toVector(const ArrayVector<T, SIZE>& a) {
    static_assert(SIZE >= 1 && SIZE <= 4, "channel vectors have one to four channels");
    if constexpr (SIZE == 1) return VectorType_t<T, 1>{a.at[0]};
    else if constexpr (SIZE == 2) return VectorType_t<T, 2>{a.at[0], a.at[1]};
    else if constexpr (SIZE == 3) return VectorType_t<T, 3>{a.at[0], a.at[1], a.at[2]};
    else return VectorType_t<T, 4>{a.at[0], a.at[1], a.at[2], a.at[3]};
}

// Element-wise helpers over std::array, fk::Array and ArrayVector (FK/core/data/array.h:232-284).
namespace array_detail {
template <typename A> struct extent;
template <typename T, size_t N> struct extent<std::array<T, N>> : std::integral_constant<size_t, N> {};
template <typename T, size_t N> struct extent<Array<T, N>> : std::integral_constant<size_t, N> {};
template <typename T, size_t N> struct extent<ArrayVector<T, N>> : std::integral_constant<size_t, N> {};
template <typename R, size_t N> struct result_of { using type = std::array<R, N>; };
} // namespace array_detail
template <typename A> constexpr size_t arraySize = array_detail::extent<std::decay_t<A>>::value;

// {f(a[0]), f(a[1]), ...}: an std::array for std::array input, an ArrayVector for ArrayVector input.
template <typename T, size_t N, typename F> constexpr auto transformArray(const std::array<T, N>& a, F&& f) {
    return [&]<size_t... I>(std::index_sequence<I...>) {
        return std::array<std::decay_t<decltype(f(a[0]))>, N>{f(a[I])...};
    }(std::make_index_sequence<N>{});
}
template <typename T, size_t N, typename F> constexpr auto transformArray(const Array<T, N>& a, F&& f) {
    return [&]<size_t... I>(std::index_sequence<I...>) {
        return Array<std::decay_t<decltype(f(a[size_t(0)]))>, N>{{f(a[I])...}};
    }(std::make_index_sequence<N>{});
}
template <typename T, size_t N, typename F> constexpr auto transformArray(const ArrayVector<T, N>& a, F&& f) {
    return [&]<size_t... I>(std::index_sequence<I...>) {
        return ArrayVector<std::decay_t<decltype(f(a.at[0]))>, N>(f(a.at[I])...);
    }(std::make_index_sequence<N>{});
}
template <size_t N> constexpr ArrayVector<size_t, N> makeIndexArray() {
    ArrayVector<size_t, N> a;
    for (size_t i = 0; i < N; ++i) a.at[i] = i;
    return a;
}
template <typename T, typename A> constexpr bool allValuesAre(const T& value, const A& a) {
    bool all = true;
    for (size_t i = 0; i < arraySize<A>; ++i) all = all && (a[i] == value);
    return all;
}
} // namespace fk
#endif
