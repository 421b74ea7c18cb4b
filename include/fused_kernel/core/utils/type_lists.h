// Type-list utilities.  Interface counterpart: FK/core/utils/type_lists.h (the subset the fused path and its tests use:
// TypeList, one_of_v, EquivalentType_t, TypeListCat_t, TypeAt_t, TypeIndex_v, InsertType*_t, FirstType_t, LastType_t).
#ifndef FK_AMD_TYPE_LISTS_H
#define FK_AMD_TYPE_LISTS_H
#include <cstddef>
#include <tuple>
#include <type_traits>
#include <utility>
#include <fused_kernel/core/execution_model/operation_model/operation_model.h>
namespace fk {
template <typename... Lists> struct TypeListCat;
template <typename... A> struct TypeListCat<TypeList<A...>> { using type = TypeList<A...>; };
template <typename... A, typename... B, typename... Rest> struct TypeListCat<TypeList<A...>, TypeList<B...>, Rest...> {
    using type = typename TypeListCat<TypeList<A..., B...>, Rest...>::type;
};
template <typename... Lists> using TypeListCat_t = typename TypeListCat<Lists...>::type;

template <size_t I, typename TL> struct TypeAt;
template <size_t I, typename... Ts> struct TypeAt<I, TypeList<Ts...>> { using type = std::tuple_element_t<I, std::tuple<Ts...>>; };
template <size_t I, typename TL> using TypeAt_t = typename TypeAt<I, TL>::type;

template <typename T, typename TL> struct TypeIndex;
template <typename T, typename... Ts> struct TypeIndex<T, TypeList<T, Ts...>> { static constexpr size_t value = 0; };
template <typename T, typename U, typename... Ts> struct TypeIndex<T, TypeList<U, Ts...>> { static constexpr size_t value = 1 + TypeIndex<T, TypeList<Ts...>>::value; };
template <typename T, typename TL> constexpr size_t TypeIndex_v = TypeIndex<T, TL>::value;

// A list with one more type: at the back, at the front, or so that it ends up at position I.
template <typename TL, typename T> using InsertTypeBack_t = TypeListCat_t<TL, TypeList<T>>;
template <typename T, typename TL> using InsertTypeFront_t = TypeListCat_t<TypeList<T>, TL>;
template <size_t I, typename T, typename TL, typename Seq = std::make_index_sequence<TL::size + 1>> struct InsertType;
template <size_t I, typename T, typename TL, size_t... K> struct InsertType<I, T, TL, std::index_sequence<K...>> {
    static_assert(I <= TL::size, "the position is past the end of the list");
    template <size_t P> struct pick { using type = TypeAt_t<(P < I ? P : P - 1), TL>; };
    template <size_t P> using slot = typename std::conditional_t<P == I, std::type_identity<T>, pick<P>>::type;
    using type = TypeList<slot<K>...>;
};
template <size_t I, typename T, typename TL> using InsertType_t = typename InsertType<I, T, TL>::type;

template <typename... Ts> using FirstType_t = std::tuple_element_t<0, std::tuple<Ts...>>;
template <typename... Ts> using LastType_t = std::tuple_element_t<sizeof...(Ts) - 1, std::tuple<Ts...>>;
} // namespace fk
#endif
