#ifndef FK_AMD_TUPLE_H
#define FK_AMD_TUPLE_H
#include <tuple>
#include <utility>
namespace fk {
// Host code only ever builds tuples of IOps on the CPU side of the launch, so the standard tuple does the job
// of the reference's device-safe one (FK/core/data/tuple.h).
template <typename... Ts> using Tuple = std::tuple<Ts...>;
using std::get;
using std::make_tuple;
using std::forward_as_tuple;
using std::tuple_cat;
using std::apply;

// An ordered list of IOps that forms one chain (read ... write): the unit DivergentBatchTransformDPP launches several
// of.  Interface counterpart: FK/core/data/tuple.h:359-378.
template <typename... IOpTypes> struct InstantiableOperationSequence {
    Tuple<IOpTypes...> iOps;
};
template <typename... IOpTypes> using IOpSequence = InstantiableOperationSequence<IOpTypes...>;
template <typename... IOpTypes> constexpr auto buildOperationSequence(const IOpTypes&... instantiableOperationInstances) {
    return InstantiableOperationSequence<IOpTypes...>{{instantiableOperationInstances...}};
}
template <typename... IOpTypes> constexpr auto buildOperationSequence_tup(const Tuple<IOpTypes...>& instantiableOperationInstances) {
    return std::apply([](const auto&... args) { return buildOperationSequence(args...); }, instantiableOperationInstances);
}
// The last of a parameter pack, and the pack with one more value put in front of its last one (as a tuple).
template <typename... Ts> constexpr decltype(auto) ppLast(const Ts&... ts) { return std::get<sizeof...(Ts) - 1>(std::forward_as_tuple(ts...)); }
template <typename T, typename... Ts> constexpr auto insert_before_last(const T& value, const Ts&... ts) {
    constexpr size_t N = sizeof...(Ts);
    static_assert(N >= 1);
    const auto all = std::forward_as_tuple(ts...);
    return [&]<size_t... Is>(std::index_sequence<Is...>) {
        return Tuple<std::decay_t<std::tuple_element_t<Is, Tuple<Ts...>>>..., T, std::decay_t<std::tuple_element_t<N - 1, Tuple<Ts...>>>>{
            std::get<Is>(all)..., value, std::get<N - 1>(all)};
    }(std::make_index_sequence<N - 1>{});
}
} // namespace fk
#endif
