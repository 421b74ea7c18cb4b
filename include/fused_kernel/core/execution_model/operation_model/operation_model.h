// The host-side operation model of the MI355X backend.
//
// A user lists "instantiable operations" (IOps): a static Operation type plus its run-time parameters.  This
// header provides the IOp wrappers (Read, ReadBack, IncompleteReadBack, Unary, Binary, Ternary, MidWrite,
// Write), the CRTP parents operations derive from, FusedOperation, BatchRead / BatchWrite, and the fusers
// (operator&, then(), fuse(), BackFuser::fuse_back) with the same names, template parameters and resulting
// types as the reference so existing chains compile unchanged:
//   FK/core/execution_model/operation_model/{operation_types,operation_data,instantiable_operations,
//   parent_operations,fused_operation,batch_operations,iop_fuser}.h
//
// What differs is what an Operation carries: no exec() body (host code never executes a pixel here).  Instead
// every Operation names its device counterpart through fk::amd::Lower<Operation>: the fkd:: type that implements
// it in the gfx950 kernels and the conversion of its parameters to that type's Params.  The executor turns a
// fused chain into fkd::Chain<...>, whose name() is the kernel signature and whose Params is the kernel argument.
#ifndef FK_AMD_OPERATION_MODEL_H
#define FK_AMD_OPERATION_MODEL_H

#include <array>
#include <cstring>
#include <tuple>
#include <type_traits>
#include <utility>

// The element-wise bodies of the device operations are compiled for the host as well: they are what
// Executor<TransformDPP<ParArch::CPU>> runs (core/execution_model/executors.h).
#ifndef FKD_HOST_EXEC
#define FKD_HOST_EXEC 1
#endif
#include <fkd/ops.hpp>

#include <fused_kernel/core/utils/utils.h>
#include <fused_kernel/core/utils/vector_utils.h>
#include <fused_kernel/core/data/array.h>
#include <fused_kernel/core/data/tuple.h>
#include <fused_kernel/core/data/point.h>
#include <fused_kernel/core/data/size.h>
#include <fused_kernel/core/data/rawptr.h>
#include <fused_kernel/core/data/ptr_nd.h>
#include <fused_kernel/core/execution_model/active_threads.h>
#include <fused_kernel/core/execution_model/thread_fusion.h>

namespace fk {

// ---- operation kinds (FK/core/execution_model/operation_model/operation_types.h:37-77) -------------------
struct ReadType {};
struct ReadBackType {};
struct IncompleteReadBackType {};
struct UnaryType {};
struct BinaryType {};
struct TernaryType {};
struct MidWriteType {};
struct WriteType {};
struct OpenType {};
struct ClosedType {};

struct NullType {};
template <typename... Ts> struct TypeList {
    static constexpr size_t size = sizeof...(Ts);
    template <size_t I> using at = std::tuple_element_t<I, std::tuple<Ts...>>;
};
// one_of_v<T, TypeList<...>>: T is one of the listed types.  EquivalentType_t<T, ListA, ListB>: the type of ListB at the
// position T has in ListA.  Interface counterpart: FK/core/utils/type_lists.h.
template <typename T, typename TL> struct one_of;
template <typename T, typename... Ts> struct one_of<T, TypeList<Ts...>> : std::bool_constant<(std::is_same_v<T, Ts> || ...)> {};
template <typename T, typename TL> constexpr bool one_of_v = one_of<T, TL>::value;
template <typename T, typename TL1, typename TL2> struct EquivalentType;
template <typename T, typename A, typename... As, typename B, typename... Bs> struct EquivalentType<T, TypeList<A, As...>, TypeList<B, Bs...>> {
    static_assert(sizeof...(As) == sizeof...(Bs), "the two lists must have the same length");
    using type = typename std::conditional_t<std::is_same_v<T, A>, std::type_identity<B>, EquivalentType<T, TypeList<As...>, TypeList<Bs...>>>::type;
};
template <typename T> struct EquivalentType<T, TypeList<>, TypeList<>> { using type = void; };
template <typename T, typename TL1, typename TL2> using EquivalentType_t = typename EquivalentType<T, TL1, TL2>::type;

namespace op_detail {
template <typename T, typename = void> struct has_instance : std::false_type {};
template <typename T> struct has_instance<T, std::void_t<typename T::InstanceType>> : std::true_type {};
template <typename T, typename = void> struct has_params : std::false_type {};
template <typename T> struct has_params<T, std::void_t<typename T::ParamsType>> : std::true_type {};
template <typename T, typename = void> struct has_back : std::false_type {};
template <typename T> struct has_back<T, std::void_t<typename T::BackIOp>> : std::true_type {};
template <typename T, typename = void> struct has_operation : std::false_type {};
template <typename T> struct has_operation<T, std::void_t<typename T::Operation>> : std::true_type {};
template <typename T, typename = void> struct has_batch : std::false_type {};
template <typename T> struct has_batch<T, std::void_t<decltype(T::BATCH)>> : std::true_type {};
template <typename T, typename = void> struct is_complete : std::true_type {};
template <typename T> struct is_complete<T, std::void_t<decltype(T::IS_COMPLETE)>> : std::bool_constant<T::IS_COMPLETE> {};

template <typename Tag, typename T, bool = has_instance<T>::value> struct op_is : std::false_type {};
template <typename Tag, typename T> struct op_is<Tag, T, true> : std::is_same<Tag, typename T::InstanceType> {};

template <typename T, bool = has_operation<T>::value> struct operation_of { using type = T; };
template <typename T> struct operation_of<T, true> { using type = typename T::Operation; };
} // namespace op_detail

// Works on Operations and on IOps alike.
template <typename Tag, typename T> constexpr bool opIs = op_detail::op_is<Tag, std::decay_t<T>>::value;
template <typename T> constexpr bool isOperation = op_detail::has_instance<std::decay_t<T>>::value;
// The class-template spellings of the same tests (FK/core/execution_model/operation_model/operation_types.h:79-91).
template <typename Tag, typename T, typename = void> struct OpIs : std::bool_constant<opIs<Tag, T>> {};
template <typename T, typename = void> struct HasInstanceType : std::bool_constant<isOperation<T>> {};
template <typename T> constexpr bool isAnyReadType = opIs<ReadType, T> || opIs<ReadBackType, T> || opIs<IncompleteReadBackType, T>;
template <typename T> constexpr bool isCompleteOperation =
    isOperation<T> && !opIs<IncompleteReadBackType, T> &&
    op_detail::is_complete<typename op_detail::operation_of<std::decay_t<T>>::type>::value;
template <typename T> constexpr bool isAnyCompleteReadType = (opIs<ReadType, T> || opIs<ReadBackType, T>) && isCompleteOperation<T>;
template <typename T> constexpr bool isComputeType = opIs<UnaryType, T> || opIs<BinaryType, T> || opIs<TernaryType, T>;
template <typename T> constexpr bool isBatchOperation =
    op_detail::has_batch<std::decay_t<T>>::value && op_detail::has_operation<std::decay_t<T>>::value;

// ---- parameter storage of an IOp (FK/core/execution_model/operation_model/operation_data.h) ----------------
template <typename Operation, typename Enabler = void> struct OperationData {};
template <typename Operation>
struct OperationData<Operation, std::enable_if_t<op_detail::has_params<Operation>::value && !op_detail::has_back<Operation>::value>> {
    typename Operation::ParamsType params;
};
template <typename Operation>
struct OperationData<Operation, std::enable_if_t<op_detail::has_params<Operation>::value && op_detail::has_back<Operation>::value>> {
    typename Operation::ParamsType params;
    typename Operation::BackIOp backIOp;
};

struct Fuser;

// ---- IOp wrappers (FK/core/execution_model/operation_model/instantiable_operations.h:66-325) ---------------
#define FK_AMD_IOP_COMMON(Tag)                                                                        \
    using Operation = Operation_t;                                                                    \
    using InstanceType = Tag;                                                                         \
    template <typename IT> static constexpr bool is{std::is_same_v<IT, InstanceType>};

#define FK_AMD_IOP_THEN                                                                               \
    template <typename ContinuationIOp, typename Fuser_t = Fuser>                                     \
    constexpr auto then(const ContinuationIOp& cIOp) const { return Fuser_t::fuse(*this, cIOp); }     \
    template <typename ContinuationIOp, typename... ContinuationIOps>                                 \
    constexpr auto then(const ContinuationIOp& cIOp, const ContinuationIOps&... cIOps) const {        \
        return then(cIOp).then(cIOps...);                                                             \
    }

template <typename Operation_t> struct ReadInstantiableOperation final : public OperationData<Operation_t> {
    FK_AMD_IOP_COMMON(ReadType)
    FK_AMD_IOP_THEN
    constexpr ActiveThreads getActiveThreads() const { return Operation::getActiveThreads(*this); }
};
template <typename Operation_t> struct ReadBackInstantiableOperation final : public OperationData<Operation_t> {
    FK_AMD_IOP_COMMON(ReadBackType)
    FK_AMD_IOP_THEN
    constexpr ActiveThreads getActiveThreads() const { return Operation::getActiveThreads(*this); }
};
template <typename Operation_t> struct IncompleteReadBackInstantiableOperation final : public OperationData<Operation_t> {
    FK_AMD_IOP_COMMON(IncompleteReadBackType)
    constexpr ActiveThreads getActiveThreads() const { return Operation::getActiveThreads(*this); }
};
template <typename Operation_t> struct UnaryInstantiableOperation {
    FK_AMD_IOP_COMMON(UnaryType)
    FK_AMD_IOP_THEN
};
template <typename Operation_t> struct BinaryInstantiableOperation final : public OperationData<Operation_t> {
    FK_AMD_IOP_COMMON(BinaryType)
    FK_AMD_IOP_THEN
};
template <typename Operation_t> struct TernaryInstantiableOperation final : public OperationData<Operation_t> {
    FK_AMD_IOP_COMMON(TernaryType)
    FK_AMD_IOP_THEN
};
template <typename Operation_t> struct MidWriteInstantiableOperation final : public OperationData<Operation_t> {
    FK_AMD_IOP_COMMON(MidWriteType)
    FK_AMD_IOP_THEN
};
template <typename Operation_t> struct WriteInstantiableOperation final : public OperationData<Operation_t> {
    FK_AMD_IOP_COMMON(WriteType)
};
#undef FK_AMD_IOP_COMMON
#undef FK_AMD_IOP_THEN

template <typename Operation> using Read = ReadInstantiableOperation<Operation>;
template <typename Operation> using ReadBack = ReadBackInstantiableOperation<Operation>;
template <typename Operation> using IncompleteReadBack = IncompleteReadBackInstantiableOperation<Operation>;
template <typename Operation> using Unary = UnaryInstantiableOperation<Operation>;
template <typename Operation> using Binary = BinaryInstantiableOperation<Operation>;
template <typename Operation> using Ternary = TernaryInstantiableOperation<Operation>;
template <typename Operation> using MidWrite = MidWriteInstantiableOperation<Operation>;
template <typename Operation> using Write = WriteInstantiableOperation<Operation>;

template <typename Operation, typename Enabler = void> struct InstantiableOperationType;
#define FK_AMD_INSTANTIABLE(Tag, Wrapper)                                                             \
    template <typename Operation>                                                                     \
    struct InstantiableOperationType<Operation, std::enable_if_t<opIs<Tag, Operation>>> { using type = Wrapper<Operation>; };
FK_AMD_INSTANTIABLE(ReadType, Read)
FK_AMD_INSTANTIABLE(ReadBackType, ReadBack)
FK_AMD_INSTANTIABLE(IncompleteReadBackType, IncompleteReadBack)
FK_AMD_INSTANTIABLE(UnaryType, Unary)
FK_AMD_INSTANTIABLE(BinaryType, Binary)
FK_AMD_INSTANTIABLE(TernaryType, Ternary)
FK_AMD_INSTANTIABLE(MidWriteType, MidWrite)
FK_AMD_INSTANTIABLE(WriteType, Write)
#undef FK_AMD_INSTANTIABLE
template <typename Operation> using Instantiable = typename InstantiableOperationType<Operation>::type;

// ---- device lowering ----------------------------------------------------------------------------------
namespace amd {

// fk element type -> fkd element type
template <typename T> struct DevType { using type = T; };
template <> struct DevType<bool> { using type = fkd::u8; };   // one byte holding 0 or 1
template <> struct DevType<unsigned char> { using type = fkd::u8; };
template <> struct DevType<signed char> { using type = fkd::i8; };
template <> struct DevType<char> { using type = fkd::i8; };
template <> struct DevType<unsigned short> { using type = fkd::u16; };
template <> struct DevType<short> { using type = fkd::i16; };
template <> struct DevType<unsigned int> { using type = fkd::u32; };
template <> struct DevType<int> { using type = fkd::i32; };
template <> struct DevType<float> { using type = fkd::f32; };
template <> struct DevType<double> { using type = fkd::f64; };
template <typename V> struct DevVec {
    using type = fkd::vec_t<typename DevType<VBase<V>>::type, cn<V>>;
};
template <typename V> using dev_t = typename DevVec<std::remove_cv_t<V>>::type;

template <typename V> dev_t<V> to_dev(const V& v) {
    dev_t<V> d{};
    static_assert(sizeof(VBase<V>) * cn<V> <= sizeof(dev_t<V>), "element layouts must agree");
    if constexpr (!isVector<V>) {
        d = static_cast<dev_t<V>>(v);
    } else {
        fkd::chan<0>(d) = v.x;
        if constexpr (cn<V> > 1) fkd::chan<1>(d) = v.y;
        if constexpr (cn<V> > 2) fkd::chan<2>(d) = v.z;
        if constexpr (cn<V> > 3) fkd::chan<3>(d) = v.w;
    }
    return d;
}

// ... and back: a device value as the host type V.
template <typename V> V from_dev(const dev_t<V>& d) {
    if constexpr (!isVector<V>) {
        return static_cast<V>(d);
    } else {
        V v{};
        v.x = static_cast<VBase<V>>(fkd::chan<0>(d));
        if constexpr (cn<V> > 1) v.y = static_cast<VBase<V>>(fkd::chan<1>(d));
        if constexpr (cn<V> > 2) v.z = static_cast<VBase<V>>(fkd::chan<2>(d));
        if constexpr (cn<V> > 3) v.w = static_cast<VBase<V>>(fkd::chan<3>(d));
        return v;
    }
}

template <typename T, typename Q = T> fkd::RawPtr2D<Q> to_dev(const RawPtr<ND::_2D, T>& p) {
    return fkd::RawPtr2D<Q>{reinterpret_cast<Q*>(p.data), p.dims.width, p.dims.height, p.dims.pitch};
}
template <typename T, typename Q = T> fkd::RawPtr3D<Q> to_dev3(const RawPtr<ND::_3D, T>& p) {
    return fkd::RawPtr3D<Q>{reinterpret_cast<Q*>(p.data), p.dims.width, p.dims.height, p.dims.planes,
                            p.dims.color_planes, p.dims.pitch, p.dims.plane_pitch};
}

template <typename T, typename Q = T> fkd::RawPtrT3D<Q> to_devT3(const RawPtr<ND::T3D, T>& p) {
    return fkd::RawPtrT3D<Q>{reinterpret_cast<Q*>(p.data), p.dims.width, p.dims.height, p.dims.planes,
                             p.dims.color_planes, p.dims.pitch, p.dims.plane_pitch, p.dims.color_planes_pitch};
}
// Colour plane 0 of a transposed tensor is an ordinary batch of planes (what PerThreadRead/Write<T3D> address).
template <typename T, typename Q = T> fkd::RawPtr3D<Q> first_color_plane(const RawPtr<ND::T3D, T>& p) {
    return fkd::RawPtr3D<Q>{reinterpret_cast<Q*>(p.data), p.dims.width, p.dims.height, p.dims.planes, 1u, p.dims.pitch, p.dims.plane_pitch};
}

// Primary: an Operation without a specialisation cannot run on this backend.
template <typename Operation, typename Enabler = void> struct Lower {
    static constexpr bool available = false;
};
template <typename Operation, typename = void> struct has_lowering : std::true_type {};
template <typename Operation> struct has_lowering<Operation, std::enable_if_t<!Lower<Operation>::available>> : std::false_type {};

template <typename Operation, bool = has_lowering<Operation>::value> struct DeviceOperationOf { using type = typename Lower<Operation>::type; };
template <typename Operation> struct DeviceOperationOf<Operation, false> {
    static_assert(has_lowering<Operation>::value,
                  "this Operation has no MI355X lowering: specialise fk::amd::Lower<Operation> (device type + parameter conversion)");
    using type = void;
};
template <typename IOp> using device_op_t = typename DeviceOperationOf<typename IOp::Operation>::type;
template <typename IOp> auto lower_iop(const IOp& iop) {
    using Op = typename IOp::Operation;
    static_assert(has_lowering<Op>::value,
                  "this Operation has no MI355X lowering: specialise fk::amd::Lower<Operation> (device type + parameter conversion)");
    if constexpr (std::is_base_of_v<OperationData<Op>, IOp>) return Lower<Op>::params(static_cast<const OperationData<Op>&>(iop));
    else return Lower<Op>::params(OperationData<Op>{});
}

} // namespace amd

// ---- CRTP parents (FK/core/execution_model/operation_model/parent_operations.h) --------------------------
struct BatchUtils;
template <typename... IOps> struct FusedOperation;

template <typename I, typename O, typename Child_, bool IS_FUSED = false> struct UnaryOperation {
    using Child = Child_;
    using InputType = I;
    using OutputType = O;
    using InstanceType = UnaryType;
    using InstantiableType = Unary<Child_>;
    static constexpr bool IS_FUSED_OP = IS_FUSED;
    static constexpr InstantiableType build() { return {}; }
    // The Operation applied to one value on the calling thread (the reference's Operations are host functions too): the
    // body is the device operation's own, compiled for the host.  An Operation that defines its own exec hides this one.
    template <typename C = Child_> static OutputType exec(const InputType& input) {
        using L = amd::Lower<C>;
        return amd::from_dev<OutputType>(L::type::exec(amd::to_dev(input), L::params(OperationData<C>{})));
    }
};

template <typename I, typename P, typename O, typename Child_, bool IS_FUSED = false> struct BinaryOperation {
    using Child = Child_;
    using InputType = I;
    using OutputType = O;
    using ParamsType = P;
    using InstanceType = BinaryType;
    using OperationDataType = OperationData<Child_>;
    using InstantiableType = Binary<Child_>;
    static constexpr bool IS_FUSED_OP = IS_FUSED;
    static constexpr InstantiableType build(const OperationDataType& opData) { return {opData}; }
    static constexpr InstantiableType build(const ParamsType& params) { return {{params}}; }
    // (see UnaryOperation::exec)
    template <typename C = Child_> static OutputType exec(const InputType& input, const ParamsType& params) {
        using L = amd::Lower<C>;
        return amd::from_dev<OutputType>(L::type::exec(amd::to_dev(input), L::params(OperationData<C>{params})));
    }
    template <typename C = Child_> static OutputType exec(const InputType& input, const OperationData<C>& opData) {
        return exec<C>(input, opData.params);
    }
};

template <typename I, typename P, typename BIOp, typename O, typename Child_, bool IS_FUSED = false> struct TernaryOperation {
    using Child = Child_;
    using InputType = I;
    using OutputType = O;
    using ParamsType = P;
    using BackIOp = BIOp;
    using InstanceType = TernaryType;
    using OperationDataType = OperationData<Child_>;
    using InstantiableType = Ternary<Child_>;
    static constexpr bool IS_FUSED_OP = IS_FUSED;
    static constexpr InstantiableType build(const OperationDataType& opData) { return {opData}; }
    static constexpr InstantiableType build(const ParamsType& params, const BackIOp& backIOp) { return {{params, backIOp}}; }
};


// Batch builders shared by Read / ReadBack / IncompleteReadBack parents (defined after BatchRead).
template <typename Child_> struct ReadBatchBuilders {
    template <size_t B, typename... ArrayTypes>
    static constexpr auto build_batch(const std::array<ArrayTypes, B>&... arrays);
    template <size_t B, typename... ArrayTypes>
    static constexpr auto build(const std::array<ArrayTypes, B>&... arrays);
    template <size_t B, typename DefaultValueType, typename... ArrayTypes>
    static constexpr auto build(const int& usedPlanes, const DefaultValueType& defaultValue, const std::array<ArrayTypes, B>&... arrays);
};

template <typename RT, typename P, typename O, TF TFE, typename Child_, bool IS_FUSED = false>
struct ReadOperation : ReadBatchBuilders<Child_> {
    using Child = Child_;
    using ParamsType = P;
    using ReadDataType = RT;
    using InstanceType = ReadType;
    static constexpr bool THREAD_FUSION{static_cast<bool>(TFE)};
    using OutputType = O;
    using OperationDataType = OperationData<Child_>;
    using InstantiableType = Read<Child_>;
    static constexpr bool IS_FUSED_OP = IS_FUSED;
    using ReadBatchBuilders<Child_>::build;
    static constexpr InstantiableType build(const OperationDataType& opData) { return {opData}; }
    static constexpr InstantiableType build(const ParamsType& params) { return {{params}}; }
};

template <typename RT, typename P, typename B, typename O, typename Child_, bool IS_FUSED = false>
struct ReadBackOperation : ReadBatchBuilders<Child_> {
    using Child = Child_;
    using ReadDataType = RT;
    using OutputType = O;
    using ParamsType = P;
    using BackIOp = B;
    using InstanceType = ReadBackType;
    using OperationDataType = OperationData<Child_>;
    using InstantiableType = ReadBack<Child_>;
    static constexpr bool IS_FUSED_OP = IS_FUSED;
    static constexpr bool THREAD_FUSION = false;
    using ReadBatchBuilders<Child_>::build;
    static constexpr InstantiableType build(const OperationDataType& opData) { return {opData}; }
    static constexpr InstantiableType build(const ParamsType& params, const BackIOp& backIOp) { return {{params, backIOp}}; }
};

template <typename RT, typename P, typename B, typename O, typename Child_, bool IS_FUSED = false>
struct IncompleteReadBackOperation : ReadBatchBuilders<Child_> {
    using Child = Child_;
    using ReadDataType = RT;
    using OutputType = O;
    using ParamsType = P;
    using BackIOp = B;
    using InstanceType = IncompleteReadBackType;
    using OperationDataType = OperationData<Child_>;
    using InstantiableType = IncompleteReadBack<Child_>;
    static constexpr bool IS_FUSED_OP = IS_FUSED;
    static constexpr bool THREAD_FUSION = false;
    static constexpr bool IS_COMPLETE = false;
    using ReadBatchBuilders<Child_>::build;
    static constexpr InstantiableType build(const OperationDataType& opData) { return {opData}; }
    static constexpr InstantiableType build(const ParamsType& params, const BackIOp& backIOp) { return {{params, backIOp}}; }
    static constexpr ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return {Child_::num_elems_x(Point{0, 0, 0}, opData), Child_::num_elems_y(Point{0, 0, 0}, opData),
                Child_::num_elems_z(Point{0, 0, 0}, opData)};
    }
};

template <typename Child_> struct WriteBatchBuilders {
    template <size_t BATCH_N, typename FirstType, typename... ArrayTypes>
    static constexpr auto build_batch(const std::array<FirstType, BATCH_N>& first, const ArrayTypes&... arrays);
    template <size_t BATCH_N, typename FirstType, typename... ArrayTypes>
    static constexpr auto build(const std::array<FirstType, BATCH_N>& first, const ArrayTypes&... arrays);
};

template <typename I, typename P, typename WT, TF TFE, typename Child_, bool IS_FUSED = false>
struct WriteOperation : WriteBatchBuilders<Child_> {
    using Child = Child_;
    using ParamsType = P;
    using InputType = I;
    using WriteDataType = WT;
    using InstanceType = WriteType;
    static constexpr bool THREAD_FUSION{static_cast<bool>(TFE)};
    using OperationDataType = OperationData<Child_>;
    using InstantiableType = Write<Child_>;
    static constexpr bool IS_FUSED_OP = IS_FUSED;
    using WriteBatchBuilders<Child_>::build;
    static constexpr InstantiableType build(const OperationDataType& opData) { return {opData}; }
    static constexpr InstantiableType build(const ParamsType& params) { return {{params}}; }
};

} // namespace fk

#include <fused_kernel/core/execution_model/operation_model/fused_operation.h>
#include <fused_kernel/core/execution_model/operation_model/batch_operations.h>
#include <fused_kernel/core/execution_model/operation_model/iop_fuser.h>

#endif
