// Traits and builders for the channel vector types: cn<V>, VBase<V>, VectorType_t<T,N>, make_<V>(...),
// make_set<V>(v), channel access, and the channel-wise arithmetic operators host code may use on parameters.
// Interface counterpart: FK/core/utils/vector_utils.h.
#ifndef FK_AMD_VECTOR_UTILS_H
#define FK_AMD_VECTOR_UTILS_H

#include <cmath>
#include <utility>
#include <type_traits>

#include <fused_kernel/core/data/vector_types.h>

namespace fk {

template <typename T, int N> struct VectorType { };
#define FK_AMD_VT(T, Upper)                                       \
    template <> struct VectorType<T, 1> { using type = T; using type_v = Upper##1; };        \
    template <> struct VectorType<T, 2> { using type = Upper##2; using type_v = Upper##2; }; \
    template <> struct VectorType<T, 3> { using type = Upper##3; using type_v = Upper##3; }; \
    template <> struct VectorType<T, 4> { using type = Upper##4; using type_v = Upper##4; };
FK_AMD_VT(bool, Bool) FK_AMD_VT(signed char, Char) FK_AMD_VT(unsigned char, Uchar) FK_AMD_VT(short, Short)
FK_AMD_VT(unsigned short, Ushort) FK_AMD_VT(int, Int) FK_AMD_VT(unsigned int, Uint) FK_AMD_VT(long, Long)
FK_AMD_VT(unsigned long, Ulong) FK_AMD_VT(long long, Longlong) FK_AMD_VT(unsigned long long, Ulonglong)
FK_AMD_VT(float, Float) FK_AMD_VT(double, Double)
#undef FK_AMD_VT
template <> struct VectorType<char, 1> { using type = char; using type_v = Char1; };
template <> struct VectorType<char, 2> { using type = Char2; using type_v = Char2; };
template <> struct VectorType<char, 3> { using type = Char3; using type_v = Char3; };
template <> struct VectorType<char, 4> { using type = Char4; using type_v = Char4; };

template <typename T, int N> using VectorType_t = typename VectorType<T, N>::type;

template <typename V> struct VectorTraits { using base = V; static constexpr int cn = 1; static constexpr bool is_vector = false; };
#define FK_AMD_TRAITS(T, Upper)                                                                                     \
    template <> struct VectorTraits<Upper##1> { using base = T; static constexpr int cn = 1; static constexpr bool is_vector = true; }; \
    template <> struct VectorTraits<Upper##2> { using base = T; static constexpr int cn = 2; static constexpr bool is_vector = true; }; \
    template <> struct VectorTraits<Upper##3> { using base = T; static constexpr int cn = 3; static constexpr bool is_vector = true; }; \
    template <> struct VectorTraits<Upper##4> { using base = T; static constexpr int cn = 4; static constexpr bool is_vector = true; };
FK_AMD_TRAITS(bool, Bool) FK_AMD_TRAITS(signed char, Char) FK_AMD_TRAITS(unsigned char, Uchar) FK_AMD_TRAITS(short, Short)
FK_AMD_TRAITS(unsigned short, Ushort) FK_AMD_TRAITS(int, Int) FK_AMD_TRAITS(unsigned int, Uint) FK_AMD_TRAITS(long, Long)
FK_AMD_TRAITS(unsigned long, Ulong) FK_AMD_TRAITS(long long, Longlong) FK_AMD_TRAITS(unsigned long long, Ulonglong)
FK_AMD_TRAITS(float, Float) FK_AMD_TRAITS(double, Double)
#undef FK_AMD_TRAITS

template <typename V> using VBase = typename VectorTraits<std::remove_cv_t<V>>::base;
template <typename V> constexpr int cn = VectorTraits<std::remove_cv_t<V>>::cn;
template <typename V> constexpr bool validCUDAVec = VectorTraits<std::remove_cv_t<V>>::is_vector;
template <typename V> constexpr bool isVector = VectorTraits<std::remove_cv_t<V>>::is_vector;

template <int N> using float_ = VectorType_t<float, N>;
template <int N> using uchar_ = VectorType_t<uchar, N>;
template <int N> using int_ = VectorType_t<int, N>;
template <int N> using uint_ = VectorType_t<uint, N>;
template <int N> using double_ = VectorType_t<double, N>;

template <int I, typename V> constexpr auto vectorAt(const V& v) {
    if constexpr (!isVector<V>) { static_assert(I == 0); return v; }
    else if constexpr (I == 0) return v.x;
    else if constexpr (I == 1) return v.y;
    else if constexpr (I == 2) return v.z;
    else return v.w;
}

// make_<float3>(a, b, c); fewer values than channels leave the remaining channels zero (aggregate initialisation, as
// in the reference, FK/core/utils/vector_utils.h:251-277)
template <typename V, typename... Args> constexpr V make_(const Args&... args) {
    if constexpr (isVector<V>) {
        static_assert(sizeof...(Args) >= 1 && sizeof...(Args) <= cn<V>, "make_<V> takes at most cn<V> values");
        return V{static_cast<VBase<V>>(args)...};
    } else {
        static_assert(sizeof...(Args) == 1, "passing more than one argument for a non vector type");
        return (static_cast<V>(args), ...);
    }
}
// make_set<float3>(v): every channel = v
template <typename V, typename S> constexpr V make_set(const S& s) {
    using B = VBase<V>;
    if constexpr (!isVector<V>) return static_cast<V>(s);
    else if constexpr (cn<V> == 1) return V{static_cast<B>(s)};
    else if constexpr (cn<V> == 2) return V{static_cast<B>(s), static_cast<B>(s)};
    else if constexpr (cn<V> == 3) return V{static_cast<B>(s), static_cast<B>(s), static_cast<B>(s)};
    else return V{static_cast<B>(s), static_cast<B>(s), static_cast<B>(s), static_cast<B>(s)};
}

namespace vec_detail {
template <typename A, typename B, typename F> constexpr auto zip(const A& a, const B& b, F f) {
    constexpr int N = isVector<A> ? cn<A> : cn<B>;
    using R = decltype(f(vectorAt<0>(a), vectorAt<0>(b)));
    using O = VectorType_t<R, N>;
    auto pick = [](const auto& v, auto idx) {
        if constexpr (isVector<std::decay_t<decltype(v)>>) return vectorAt<decltype(idx)::value>(v); else return v;
    };
    if constexpr (N == 1) return O{f(pick(a, std::integral_constant<int, 0>{}), pick(b, std::integral_constant<int, 0>{}))};
    else if constexpr (N == 2) return O{f(pick(a, std::integral_constant<int, 0>{}), pick(b, std::integral_constant<int, 0>{})),
                                        f(pick(a, std::integral_constant<int, 1>{}), pick(b, std::integral_constant<int, 1>{}))};
    else if constexpr (N == 3) return O{f(pick(a, std::integral_constant<int, 0>{}), pick(b, std::integral_constant<int, 0>{})),
                                        f(pick(a, std::integral_constant<int, 1>{}), pick(b, std::integral_constant<int, 1>{})),
                                        f(pick(a, std::integral_constant<int, 2>{}), pick(b, std::integral_constant<int, 2>{}))};
    else return O{f(pick(a, std::integral_constant<int, 0>{}), pick(b, std::integral_constant<int, 0>{})),
                  f(pick(a, std::integral_constant<int, 1>{}), pick(b, std::integral_constant<int, 1>{})),
                  f(pick(a, std::integral_constant<int, 2>{}), pick(b, std::integral_constant<int, 2>{})),
                  f(pick(a, std::integral_constant<int, 3>{}), pick(b, std::integral_constant<int, 3>{}))};
}
template <typename A, typename B>
constexpr bool vec_operands = (isVector<A> || isVector<B>) && (!isVector<A> || !isVector<B> || cn<A> == cn<B>) &&
                              (isVector<A> || std::is_arithmetic_v<A>) && (isVector<B> || std::is_arithmetic_v<B>);
} // namespace vec_detail

} // namespace fk

// Channel-wise operators, visible without a using-directive like the reference's.
#define FK_AMD_VEC_OP(op)                                                                                          \
    template <typename A, typename B, std::enable_if_t<fk::vec_detail::vec_operands<A, B>, int> = 0>               \
    constexpr auto operator op(const A& a, const B& b) {                                                           \
        return fk::vec_detail::zip(a, b, [](auto x, auto y) { return x op y; });                                   \
    }
FK_AMD_VEC_OP(+) FK_AMD_VEC_OP(-) FK_AMD_VEC_OP(*) FK_AMD_VEC_OP(/)
#undef FK_AMD_VEC_OP
// Comparisons and logical operators are channel-wise too and yield a boolN, which converts to bool as "all channels".
#define FK_AMD_VEC_CMP(op)                                                                                         \
    template <typename A, typename B, std::enable_if_t<fk::vec_detail::vec_operands<A, B>, int> = 0>               \
    constexpr auto operator op(const A& a, const B& b) {                                                           \
        constexpr int N = fk::isVector<A> ? fk::cn<A> : fk::cn<B>;                                                 \
        using O = typename fk::VectorType<bool, N>::type_v;                                                        \
        const auto r = fk::vec_detail::zip(a, b, [](auto x, auto y) -> bool { return x op y; });                   \
        if constexpr (N == 1) return O{fk::vectorAt<0>(r)}; else return r;                                         \
    }
FK_AMD_VEC_CMP(==) FK_AMD_VEC_CMP(!=) FK_AMD_VEC_CMP(<) FK_AMD_VEC_CMP(>) FK_AMD_VEC_CMP(<=) FK_AMD_VEC_CMP(>=)
FK_AMD_VEC_CMP(&&) FK_AMD_VEC_CMP(||)
#undef FK_AMD_VEC_CMP

#endif
