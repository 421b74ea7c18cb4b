// BwAnd, BwOr, BwXor (value op constant), BwNot, ShiftLeft, ShiftRight (value shifted by a constant), per channel, as
// Operations of a chain.  Interface counterpart: FK/algorithms/basic_ops/bitwise.h:23-157.  The results have the type
// the C++ operator yields on the channel types (int for anything narrower), converted to O's channel type.  BwAnd, BwOr
// and BwXor also have the two-input forms that take a Tuple<I1, I2>.
#ifndef FK_AMD_BITWISE_H
#define FK_AMD_BITWISE_H
#include <fused_kernel/algorithms/basic_ops/math.h>
namespace fk {
FK_AMD_VALUE_AND_CONSTANT(BwAnd)
FK_AMD_VALUE_AND_CONSTANT(BwOr)
FK_AMD_VALUE_AND_CONSTANT(BwXor)
FK_AMD_TWO_INPUTS(BwAnd)
FK_AMD_TWO_INPUTS(BwOr)
FK_AMD_TWO_INPUTS(BwXor)
template <typename I, typename O = I> struct BwNot : UnaryOperation<I, O, BwNot<I, O>> {
    using Parent = UnaryOperation<I, O, BwNot<I, O>>;
    FK_STATIC_STRUCT(BwNot, BwNot)
};
#define FK_AMD_SHIFT(Name)                                                                                       \
    template <typename I, typename P = I, typename O = I> struct Name : BinaryOperation<I, P, O, Name<I, P, O>> { \
        using Parent = BinaryOperation<I, P, O, Name<I, P, O>>;                                                  \
        FK_STATIC_STRUCT(Name, Name)                                                                             \
    };                                                                                                           \
    namespace amd {                                                                                              \
    template <typename I, typename P, typename O> struct Lower<Name<I, P, O>> {                                  \
        static constexpr bool available = true;                                                                  \
        using type = fkd::Map2<fkd::fn::Name, dev_t<I>, dev_t<P>, dev_t<O>>;                                     \
        static typename type::Params params(const OperationData<Name<I, P, O>>& d) { return typename type::Params{to_dev(d.params)}; } \
    };                                                                                                           \
    }
FK_AMD_SHIFT(ShiftLeft)
FK_AMD_SHIFT(ShiftRight)
#undef FK_AMD_SHIFT
namespace amd {
template <typename I, typename O> struct Lower<BwNot<I, O>> {
    static constexpr bool available = true;
    using type = fkd::Map1<fkd::fn::BwNot, dev_t<I>, dev_t<O>>;
    static typename type::Params params(const OperationData<BwNot<I, O>>&) { return {}; }
};
} // namespace amd
} // namespace fk
#endif
