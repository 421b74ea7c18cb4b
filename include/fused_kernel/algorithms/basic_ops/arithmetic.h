// Add / Sub / Mul / Div as Binary operations (value op parameter, channel-wise, a scalar parameter is broadcast) and in
// their two-input Unary forms (the value is a Tuple<I1, I2>, as DualSourceRead hands it over).
// Interface counterpart: FK/algorithms/basic_ops/arithmetic.h:26-124.
#ifndef FK_AMD_ARITHMETIC_H
#define FK_AMD_ARITHMETIC_H

#include <fused_kernel/core/execution_model/operation_model/operation_model.h>
#include <fused_kernel/core/data/tuple.h>

namespace fk {

// The two-input form of an Operation Name<I1, I2, O, IT> whose primary template is already declared: the value is a
// Tuple<I1, I2> and the body is the expression of fkd::fn::Name on its halves.  Shared with logical.h, bitwise.h, math.h.
#define FK_AMD_TWO_INPUTS(Name)                                                                                 \
    template <typename I1, typename I2, typename O>                                                             \
    struct Name<I1, I2, O, UnaryType> : UnaryOperation<Tuple<I1, I2>, O, Name<I1, I2, O, UnaryType>> {          \
        using Parent = UnaryOperation<Tuple<I1, I2>, O, Name<I1, I2, O, UnaryType>>;                            \
        FK_STATIC_STRUCT(Name, Name)                                                                            \
    };                                                                                                          \
    namespace amd {                                                                                             \
    template <typename I1, typename I2, typename O> struct Lower<Name<I1, I2, O, UnaryType>> {                  \
        static constexpr bool available = true;                                                                 \
        using type = fkd::Zip<fkd::fn::Name, dev_t<I1>, dev_t<I2>, dev_t<O>>;                                   \
        static typename type::Params params(const OperationData<Name<I1, I2, O, UnaryType>>&) { return {}; }    \
    };                                                                                                          \
    }

#define FK_AMD_ARITH(Name)                                                                                      \
    template <typename I1, typename I2 = I1, typename O = I1, typename IT = BinaryType> struct Name;            \
    template <typename I, typename P, typename O>                                                               \
    struct Name<I, P, O, BinaryType> : BinaryOperation<I, P, O, Name<I, P, O, BinaryType>> {                    \
        using Parent = BinaryOperation<I, P, O, Name<I, P, O, BinaryType>>;                                     \
        FK_STATIC_STRUCT(Name, Name)                                                                            \
    };                                                                                                          \
    namespace amd {                                                                                             \
    template <typename I, typename P, typename O> struct Lower<Name<I, P, O, BinaryType>> {                     \
        static constexpr bool available = true;                                                                 \
        using type = fkd::Name<dev_t<I>, dev_t<P>, dev_t<O>>;                                                   \
        static typename type::Params params(const OperationData<Name<I, P, O, BinaryType>>& d) {                \
            return typename type::Params{to_dev(d.params)};                                                     \
        }                                                                                                       \
    };                                                                                                          \
    }
FK_AMD_ARITH(Add)
FK_AMD_ARITH(Sub)
FK_AMD_ARITH(Mul)
#undef FK_AMD_ARITH
FK_AMD_TWO_INPUTS(Add)
FK_AMD_TWO_INPUTS(Sub)
FK_AMD_TWO_INPUTS(Mul)

// Div: the device parameter block also carries the correctly rounded reciprocal of the divisor (see fkd::Div).
template <typename I1, typename I2 = I1, typename O = I1, typename IT = BinaryType> struct Div;
template <typename I, typename P, typename O>
struct Div<I, P, O, BinaryType> : BinaryOperation<I, P, O, Div<I, P, O, BinaryType>> {
    using Parent = BinaryOperation<I, P, O, Div<I, P, O, BinaryType>>;
    FK_STATIC_STRUCT(Div, Div)
};
namespace amd {
template <typename I, typename P, typename O> struct Lower<Div<I, P, O, BinaryType>> {
    static constexpr bool available = true;
    using type = fkd::Div<dev_t<I>, dev_t<P>, dev_t<O>>;
    static typename type::Params params(const OperationData<Div<I, P, O, BinaryType>>& d) {
        return type::make(to_dev(d.params));
    }
};
}

FK_AMD_TWO_INPUTS(Div)

} // namespace fk
#endif
