// Abs, Sqr, Sqrt, Ln, Exp (one value in, per channel) and AbsDiff (|value - constant| per channel) as Operations of a
// chain.  Interface counterpart: FK/algorithms/basic_ops/math.h:59-170; the expressions themselves are in
// fkd::fn (include/fkd/ops.hpp).  As in the reference, O is the type the expression yields per channel (Sqr<uchar3>
// needs O = int3, Sqrt<uchar3> O = float3).  AbsDiff also has the two-input form that takes a Tuple<I1, I2>.
#ifndef FK_AMD_MATH_H
#define FK_AMD_MATH_H
#include <fused_kernel/algorithms/basic_ops/arithmetic.h>
namespace fk {
#define FK_AMD_MATH_UNARY(Name)                                                                                  \
    template <typename I, typename O = I> struct Name : UnaryOperation<I, O, Name<I, O>> {                       \
        using Parent = UnaryOperation<I, O, Name<I, O>>;                                                         \
        FK_STATIC_STRUCT(Name, Name)                                                                             \
    };                                                                                                           \
    namespace amd {                                                                                              \
    template <typename I, typename O> struct Lower<Name<I, O>> {                                                 \
        static constexpr bool available = true;                                                                  \
        using type = fkd::Map1<fkd::fn::Name, dev_t<I>, dev_t<O>>;                                               \
        static typename type::Params params(const OperationData<Name<I, O>>&) { return {}; }                     \
    };                                                                                                           \
    }
FK_AMD_MATH_UNARY(Abs)
FK_AMD_MATH_UNARY(Sqr)
FK_AMD_MATH_UNARY(Sqrt)
FK_AMD_MATH_UNARY(Ln)
FK_AMD_MATH_UNARY(Exp)
#undef FK_AMD_MATH_UNARY

// Binary Operations whose body is one expression on (value, constant): shared by math.h, logical.h and bitwise.h.
#define FK_AMD_VALUE_AND_CONSTANT(Name)                                                                          \
    template <typename I1, typename I2 = I1, typename O = I1, typename IT = BinaryType> struct Name;             \
    template <typename I, typename P, typename O>                                                                \
    struct Name<I, P, O, BinaryType> : BinaryOperation<I, P, O, Name<I, P, O, BinaryType>> {                     \
        using Parent = BinaryOperation<I, P, O, Name<I, P, O, BinaryType>>;                                      \
        FK_STATIC_STRUCT(Name, Name)                                                                             \
    };                                                                                                           \
    namespace amd {                                                                                              \
    template <typename I, typename P, typename O> struct Lower<Name<I, P, O, BinaryType>> {                      \
        static constexpr bool available = true;                                                                  \
        using type = fkd::Map2<fkd::fn::Name, dev_t<I>, dev_t<P>, dev_t<O>>;                                     \
        static typename type::Params params(const OperationData<Name<I, P, O, BinaryType>>& d) {                 \
            return typename type::Params{to_dev(d.params)};                                                      \
        }                                                                                                        \
    };                                                                                                           \
    }
FK_AMD_VALUE_AND_CONSTANT(AbsDiff)
FK_AMD_TWO_INPUTS(AbsDiff)
} // namespace fk
#endif
