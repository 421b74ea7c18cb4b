// VectorReorder<T, i0, i1, i2, i3>: out[c] = in[i_c]; Discard<I, O>: the first cn<O> channels; AddLast<I, O>: one more
// channel holding the parameter.  Interface counterpart: FK/algorithms/basic_ops/vector_ops.h:22-56, 94-118.
#ifndef FK_AMD_VECTOR_OPS_H
#define FK_AMD_VECTOR_OPS_H
#include <fused_kernel/core/execution_model/operation_model/operation_model.h>
namespace fk {
template <typename T, int... Idx> struct VectorReorder : UnaryOperation<T, T, VectorReorder<T, Idx...>> {
    using Parent = UnaryOperation<T, T, VectorReorder<T, Idx...>>;
    FK_STATIC_STRUCT(VectorReorder, VectorReorder)
    static_assert(validCUDAVec<T>, "Non valid vector type: VectorReorder");
    static_assert(cn<T> >= 2, "Minimum number of channels to reorder: 2");
    static_assert(sizeof...(Idx) == cn<T>, "Wrong number of indexes for the vector type");
};
template <typename I, typename O> struct Discard : UnaryOperation<I, O, Discard<I, O>> {
    using Parent = UnaryOperation<I, O, Discard<I, O>>;
    FK_STATIC_STRUCT(Discard, Discard)
    static_assert(cn<I> > cn<O>, "Output type should at least have one channel less");
    static_assert(std::is_same_v<VBase<I>, VBase<O>>, "Base types should be the same");
};
template <typename I, typename O> struct AddLast : BinaryOperation<I, VBase<I>, O, AddLast<I, O>> {
    using Parent = BinaryOperation<I, VBase<I>, O, AddLast<I, O>>;
    FK_STATIC_STRUCT(AddLast, AddLast)
    static_assert(cn<I> == cn<O> - 1, "Output type should have one channel more");
    static_assert(std::is_same_v<VBase<I>, VBase<O>>, "Base types should be the same");
};
// The channels of the input folded left to right with a binary Operation on scalars: op(op(x, y), z).
template <typename T, typename Operation> struct VectorReduce : UnaryOperation<T, typename Operation::OutputType, VectorReduce<T, Operation>> {
    using Parent = UnaryOperation<T, typename Operation::OutputType, VectorReduce<T, Operation>>;
    FK_STATIC_STRUCT(VectorReduce, VectorReduce)
};
namespace amd {
template <typename T, typename Operation> struct Lower<VectorReduce<T, Operation>> {
    static constexpr bool available = Lower<Operation>::available;
    using type = fkd::VectorReduce<dev_t<T>, typename Lower<Operation>::type>;
    static typename type::Params params(const OperationData<VectorReduce<T, Operation>>&) { return {}; }
};
template <typename I, typename O> struct Lower<Discard<I, O>> {
    static constexpr bool available = true;
    using type = fkd::Discard<dev_t<I>, dev_t<O>>;
    static typename type::Params params(const OperationData<Discard<I, O>>&) { return {}; }
};
template <typename I, typename O> struct Lower<AddLast<I, O>> {
    static constexpr bool available = true;
    using type = fkd::AddLast<dev_t<I>>;
    static typename type::Params params(const OperationData<AddLast<I, O>>& d) { return typename type::Params{d.params}; }
};
template <typename T, int I0, int I1> struct Lower<VectorReorder<T, I0, I1>> {
    static constexpr bool available = true;
    using type = fkd::Reorder<dev_t<T>, I0, I1, 2, 3>;
    static typename type::Params params(const OperationData<VectorReorder<T, I0, I1>>&) { return {}; }
};
template <typename T, int I0, int I1, int I2> struct Lower<VectorReorder<T, I0, I1, I2>> {
    static constexpr bool available = true;
    using type = fkd::Reorder<dev_t<T>, I0, I1, I2, 3>;
    static typename type::Params params(const OperationData<VectorReorder<T, I0, I1, I2>>&) { return {}; }
};
template <typename T, int I0, int I1, int I2, int I3> struct Lower<VectorReorder<T, I0, I1, I2, I3>> {
    static constexpr bool available = true;
    using type = fkd::Reorder<dev_t<T>, I0, I1, I2, I3>;
    static typename type::Params params(const OperationData<VectorReorder<T, I0, I1, I2, I3>>&) { return {}; }
};
} // namespace amd
} // namespace fk
#endif
