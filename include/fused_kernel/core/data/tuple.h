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
} // namespace fk
#endif
