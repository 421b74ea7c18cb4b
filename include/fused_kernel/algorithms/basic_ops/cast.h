// Cast<I,O>: per-channel static_cast.  Interface counterpart: FK/algorithms/basic_ops/cast.h:22-33.
#ifndef FK_AMD_CAST_H
#define FK_AMD_CAST_H
#include <fused_kernel/core/execution_model/operation_model/operation_model.h>
namespace fk {
template <typename I, typename O> struct Cast : UnaryOperation<I, O, Cast<I, O>> {
    using Parent = UnaryOperation<I, O, Cast<I, O>>;
    FK_STATIC_STRUCT(Cast, Cast)
};
namespace amd {
template <typename I, typename O> struct Lower<Cast<I, O>> {
    static constexpr bool available = true;
    using type = fkd::Cast<dev_t<I>, dev_t<O>>;
    static typename type::Params params(const OperationData<Cast<I, O>>&) { return {}; }
};
} // namespace amd
} // namespace fk
#endif
