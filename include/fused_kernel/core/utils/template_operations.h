// Folds over packs of compile-time booleans and a position search in an integer sequence.
// Interface counterpart: FK/core/utils/template_operations.h:20-63.
#ifndef FK_AMD_TEMPLATE_OPERATIONS_H
#define FK_AMD_TEMPLATE_OPERATIONS_H
#include <utility>
namespace fk {
template <bool... results> constexpr bool and_v = (results && ...);
template <bool... results> constexpr bool or_v = (results || ...);

// Find<T, e>::in(sequence): position of e in the sequence, -1 when it is not there; one_of(sequence): whether it is.
template <typename T, T Element> struct Find {
    template <T... Seq> static constexpr int in(std::integer_sequence<T, Seq...>) {
        int at = -1, i = 0;
        ((at = (at < 0 && Seq == Element) ? i : at, ++i), ...);
        return at;
    }
    template <T... Seq> static constexpr bool one_of(std::integer_sequence<T, Seq...> s) { return in(s) >= 0; }
};
} // namespace fk
#endif
