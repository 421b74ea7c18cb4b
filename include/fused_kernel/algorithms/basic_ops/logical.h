// Equal<T>: host-side comparison of two values (all channels equal), the helper the reference's benchmarks and tests
// use to compare results they have downloaded.  Interface counterpart: FK/algorithms/basic_ops/logical.h:92-120.
// IsEven, Max and Min of that header have no MI355X kernel and are not provided.
#ifndef FK_AMD_LOGICAL_H
#define FK_AMD_LOGICAL_H
#include <fused_kernel/core/execution_model/operation_model/operation_model.h>
#include <fused_kernel/core/data/tuple.h>
namespace fk {
template <typename I1, typename I2 = I1> struct Equal : UnaryOperation<Tuple<I1, I2>, bool, Equal<I1, I2>> {
    using Parent = UnaryOperation<Tuple<I1, I2>, bool, Equal<I1, I2>>;
    FK_STATIC_STRUCT(Equal, Equal)
    static constexpr bool exec(const Tuple<I1, I2>& input) { return static_cast<bool>(get<0>(input) == get<1>(input)); }
};
} // namespace fk
#endif
