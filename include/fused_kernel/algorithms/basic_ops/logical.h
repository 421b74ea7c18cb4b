// Equal<T>: host-side comparison of two values (all channels equal), the helper the reference's benchmarks and tests
// use to compare results they have downloaded; IsEven<I>: whether an integer (each channel of an integer vector) is
// even.  Interface counterpart: FK/algorithms/basic_ops/logical.h:23-35, 92-120.
// Max<I, P, O> / Min<I, P, O>: the larger / smaller of value and constant per channel, std::max / std::min of two values
// of one channel type (logical.h:37-88), and their two-input forms on a Tuple<I, P>.
#ifndef FK_AMD_LOGICAL_H
#define FK_AMD_LOGICAL_H
#include <fused_kernel/core/execution_model/operation_model/operation_model.h>
#include <fused_kernel/core/data/tuple.h>
#include <fused_kernel/algorithms/basic_ops/math.h>
namespace fk {
FK_AMD_VALUE_AND_CONSTANT(Max)
FK_AMD_VALUE_AND_CONSTANT(Min)
FK_AMD_TWO_INPUTS(Max)
FK_AMD_TWO_INPUTS(Min)
template <typename I1, typename I2 = I1> struct Equal : UnaryOperation<Tuple<I1, I2>, bool, Equal<I1, I2>> {
    using Parent = UnaryOperation<Tuple<I1, I2>, bool, Equal<I1, I2>>;
    FK_STATIC_STRUCT(Equal, Equal)
    static constexpr bool exec(const Tuple<I1, I2>& input) { return static_cast<bool>(get<0>(input) == get<1>(input)); }
};

template <typename I> struct IsEven : UnaryOperation<I, VectorType_t<bool, cn<I>>, IsEven<I>> {
    static_assert(std::is_integral_v<VBase<I>>, "IsEven works on integers and vectors of integers");
    using Parent = UnaryOperation<I, VectorType_t<bool, cn<I>>, IsEven<I>>;
    FK_STATIC_STRUCT(IsEven, IsEven)
};
namespace amd {
template <typename I> struct Lower<IsEven<I>> {
    static constexpr bool available = true;
    using type = fkd::IsEven<dev_t<I>>;
    static typename type::Params params(const OperationData<IsEven<I>>&) { return {}; }
};
} // namespace amd
} // namespace fk
#endif
