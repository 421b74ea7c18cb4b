// SaturateCast<I,O>: OpenCV-style saturating conversion (float -> integer: NaN -> 0, round half to even, clamp).
// Interface counterpart: FK/algorithms/image_processing/saturate.h:25-36.
#ifndef FK_AMD_SATURATE_H
#define FK_AMD_SATURATE_H
#include <fused_kernel/core/execution_model/operation_model/operation_model.h>
namespace fk {
template <typename I, typename O> struct SaturateCast : UnaryOperation<I, O, SaturateCast<I, O>> {
    using Parent = UnaryOperation<I, O, SaturateCast<I, O>>;
    FK_STATIC_STRUCT(SaturateCast, SaturateCast)
    static_assert(cn<I> == cn<O>, "SaturateCast needs the same number of channels on both sides");
};
namespace amd {
template <typename I, typename O> struct Lower<SaturateCast<I, O>> {
    static constexpr bool available = true;
    using type = fkd::SaturateCast<dev_t<I>, dev_t<O>>;
    static typename type::Params params(const OperationData<SaturateCast<I, O>>&) { return {}; }
};
} // namespace amd
} // namespace fk
#endif
