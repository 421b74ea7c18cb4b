// StaticLoop<Operation, ITERATIONS>: a Binary operation that applies Operation ITERATIONS times with the same
// parameters -- and once for ITERATIONS = 0, as the reference does (its first application is unconditional).
// Interface counterpart: FK/algorithms/basic_ops/static_loop.h:21-44.
#ifndef FK_AMD_STATIC_LOOP_H
#define FK_AMD_STATIC_LOOP_H

#include <fused_kernel/core/execution_model/operation_model/operation_model.h>

namespace fk {

template <typename Operation, int ITERATIONS>
struct StaticLoop : BinaryOperation<typename Operation::InputType, typename Operation::ParamsType, typename Operation::OutputType,
                                    StaticLoop<Operation, ITERATIONS>> {
    using Parent = BinaryOperation<typename Operation::InputType, typename Operation::ParamsType, typename Operation::OutputType,
                                   StaticLoop<Operation, ITERATIONS>>;
    FK_STATIC_STRUCT(StaticLoop, StaticLoop)
    static_assert(ITERATIONS >= 0, "StaticLoop cannot run a negative number of iterations");
    static_assert(std::is_same_v<typename Operation::InputType, typename Operation::OutputType>,
                  "the looped operation must map a type onto itself");
};

namespace amd {
template <typename Operation, int ITERATIONS> struct Lower<StaticLoop<Operation, ITERATIONS>> {
    static constexpr bool available = Lower<Operation>::available;
    using type = fkd::StaticLoop<typename Lower<Operation>::type, (ITERATIONS < 1 ? 1 : ITERATIONS)>;
    static typename type::Params params(const OperationData<StaticLoop<Operation, ITERATIONS>>& d) {
        return Lower<Operation>::params(OperationData<Operation>{d.params});
    }
};
} // namespace amd

} // namespace fk
#endif
