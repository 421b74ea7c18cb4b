// Horizontal fusion on the host side: BatchRead<PlanePolicy, BATCH, Operation>, BatchWrite<BATCH, Operation>,
// BatchUtils, and the std::array build() overloads of the read / write parents.  One plane of the batch maps to
// one value of the launch grid's z index.  Interface counterpart:
// FK/core/execution_model/operation_model/batch_operations.h.
#ifndef FK_AMD_BATCH_OPERATIONS_H
#define FK_AMD_BATCH_OPERATIONS_H

#include <new>
#include <type_traits>

#ifndef FK_AMD_OPERATION_MODEL_H
#include <fused_kernel/core/execution_model/operation_model/operation_model.h>
#else

namespace fk {

enum class PlanePolicy { PROCESS_ALL = 0, CONDITIONAL_WITH_DEFAULT = 1 };

template <size_t BATCH, PlanePolicy PP, typename Operation, typename DefaultType = NullType> struct BatchReadParams;
template <size_t BATCH, typename Operation, typename DefaultType>
struct BatchReadParams<BATCH, PlanePolicy::CONDITIONAL_WITH_DEFAULT, Operation, DefaultType> {
    Array<OperationData<Operation>, BATCH> opData;
    int usedPlanes;
    DefaultType default_value;
    ActiveThreads activeThreads;
};
template <size_t BATCH, typename Operation>
struct BatchReadParams<BATCH, PlanePolicy::PROCESS_ALL, Operation, NullType> {
    Array<OperationData<Operation>, BATCH> opData;
    ActiveThreads activeThreads;
};

template <PlanePolicy PP = PlanePolicy::PROCESS_ALL, size_t BATCH = 1, typename Operation = TypeList<void>> struct BatchRead;

namespace batch_detail {
// slot = make(), with the value built where it lives: at run time the result of make() initialises the slot directly
// (an assignment builds it on the stack field by field and copies it over whole, which stalls once per plane of a batch).
template <typename T, typename F> constexpr void build_in(T& slot, F&& make) {
    if (std::is_constant_evaluated()) {
        slot = make();
    } else {
        static_assert(std::is_trivially_destructible_v<T>);
        ::new (static_cast<void*>(&slot)) T(make());
    }
}
// Members every concrete BatchRead flavour shares.
template <typename Self, typename Op, size_t B, PlanePolicy POLICY, typename Params, typename Out, bool COMPLETE>
struct ReadCommon {
    using Operation = Op;
    static constexpr size_t BATCH = B;
    static constexpr PlanePolicy PP = POLICY;
    using ParamsType = Params;
    using ReadDataType = typename Op::ReadDataType;
    using InstanceType = ReadType;
    using OutputType = Out;
    using OperationDataType = OperationData<Self>;
    using InstantiableType = Read<Self>;
    static constexpr bool IS_FUSED_OP = Op::IS_FUSED_OP;
    static constexpr bool THREAD_FUSION = POLICY == PlanePolicy::PROCESS_ALL ? Op::THREAD_FUSION : false;
    static constexpr bool IS_COMPLETE = COMPLETE;
    static constexpr uint num_elems_x(const Point thread, const OperationDataType& opData) {
        return Op::num_elems_x(thread, opData.params.opData[thread.z]);
    }
    static constexpr uint num_elems_y(const Point thread, const OperationDataType& opData) {
        return Op::num_elems_y(thread, opData.params.opData[thread.z]);
    }
    static constexpr uint num_elems_z(const Point, const OperationDataType&) { return uint(B); }
    static constexpr ActiveThreads getActiveThreads(const OperationDataType& opData) { return opData.params.activeThreads; }
    static constexpr InstantiableType build(const OperationDataType& opData) { return InstantiableType{opData}; }
    static constexpr InstantiableType build(const ParamsType& params) { return InstantiableType{{params}}; }
};
} // namespace batch_detail

template <size_t BATCH_, typename Op>
struct BatchRead<PlanePolicy::PROCESS_ALL, BATCH_, Op>
    : batch_detail::ReadCommon<BatchRead<PlanePolicy::PROCESS_ALL, BATCH_, Op>, Op, BATCH_, PlanePolicy::PROCESS_ALL,
                               BatchReadParams<BATCH_, PlanePolicy::PROCESS_ALL, Op>, typename Op::OutputType, true> {
    static_assert(isCompleteOperation<Op>, "The Operation passed as template parameter is not a complete operation");
};

template <size_t BATCH_, typename Op>
struct BatchRead<PlanePolicy::CONDITIONAL_WITH_DEFAULT, BATCH_, Op>
    : batch_detail::ReadCommon<BatchRead<PlanePolicy::CONDITIONAL_WITH_DEFAULT, BATCH_, Op>, Op, BATCH_,
                               PlanePolicy::CONDITIONAL_WITH_DEFAULT,
                               BatchReadParams<BATCH_, PlanePolicy::CONDITIONAL_WITH_DEFAULT, Op, typename Op::OutputType>,
                               typename Op::OutputType, true> {
    static_assert(isCompleteOperation<Op>, "The Operation passed as template parameter is not a complete operation");
};

// Batches of INCOMPLETE read-back operations (Crop<>, Resize<>): placeholders until fused with a source.
template <size_t BATCH_, typename Op>
struct BatchRead<PlanePolicy::PROCESS_ALL, BATCH_, TypeList<Op>>
    : batch_detail::ReadCommon<BatchRead<PlanePolicy::PROCESS_ALL, BATCH_, TypeList<Op>>, Op, BATCH_, PlanePolicy::PROCESS_ALL,
                               BatchReadParams<BATCH_, PlanePolicy::PROCESS_ALL, Op>, typename Op::OutputType, false> {};

template <size_t BATCH_, typename Op, typename DefType>
struct BatchRead<PlanePolicy::CONDITIONAL_WITH_DEFAULT, BATCH_, TypeList<Op, DefType>>
    : batch_detail::ReadCommon<BatchRead<PlanePolicy::CONDITIONAL_WITH_DEFAULT, BATCH_, TypeList<Op, DefType>>, Op, BATCH_,
                               PlanePolicy::CONDITIONAL_WITH_DEFAULT,
                               BatchReadParams<BATCH_, PlanePolicy::CONDITIONAL_WITH_DEFAULT, Op, DefType>, DefType, false> {};

// Builders: BatchRead<PlanePolicy::PROCESS_ALL>::build(std::array<IOp, N>) and the CONDITIONAL_WITH_DEFAULT form.
template <> struct BatchRead<PlanePolicy::PROCESS_ALL, 1, TypeList<void>> {
    template <typename IOp, size_t BATCH> static constexpr auto build(const std::array<IOp, BATCH>& iOps) {
        using NewOperation = typename IOp::Operation;
        uint max_width{0}, max_height{0};
        for (size_t i = 0; i < BATCH; ++i) {
            const uint w = NewOperation::num_elems_x(Point{0, 0, 0}, iOps[i]);
            const uint h = NewOperation::num_elems_y(Point{0, 0, 0}, iOps[i]);
            max_width = w > max_width ? w : max_width;
            max_height = h > max_height ? h : max_height;
        }
        using BatchReadType = std::conditional_t<isCompleteOperation<NewOperation>,
                                                 BatchRead<PlanePolicy::PROCESS_ALL, BATCH, NewOperation>,
                                                 BatchRead<PlanePolicy::PROCESS_ALL, BATCH, TypeList<NewOperation>>>;
        typename BatchReadType::ParamsType store{{}, ActiveThreads{max_width, max_height, uint(BATCH)}};
        for (size_t i = 0; i < BATCH; ++i) batch_detail::build_in(store.opData[i], [&]() -> std::remove_reference_t<decltype(store.opData[i])> { return iOps[i]; });
        return BatchReadType::build(store);
    }
};

template <> struct BatchRead<PlanePolicy::CONDITIONAL_WITH_DEFAULT, 1, TypeList<void>> {
    template <typename IOp, size_t BATCH, typename DefaultType>
    static constexpr auto build(const std::array<IOp, BATCH>& iOps, const int& usedPlanes, const DefaultType& defaultValue) {
        using NewOperation = typename IOp::Operation;
        uint max_width{0}, max_height{0};
        for (size_t i = 0; i < BATCH; ++i) {
            const uint w = NewOperation::num_elems_x(Point{0, 0, 0}, iOps[i]);
            const uint h = NewOperation::num_elems_y(Point{0, 0, 0}, iOps[i]);
            max_width = w > max_width ? w : max_width;
            max_height = h > max_height ? h : max_height;
        }
        using NewOutputType = std::conditional_t<std::is_same_v<typename NewOperation::OutputType, NullType>, DefaultType,
                                                 typename NewOperation::OutputType>;
        using BatchReadType = std::conditional_t<isCompleteOperation<NewOperation>,
                                                 BatchRead<PlanePolicy::CONDITIONAL_WITH_DEFAULT, BATCH, NewOperation>,
                                                 BatchRead<PlanePolicy::CONDITIONAL_WITH_DEFAULT, BATCH, TypeList<NewOperation, NewOutputType>>>;
        NewOutputType def{};
        if constexpr (std::is_same_v<NewOutputType, DefaultType>) def = defaultValue;
        else def = amd_cast_default<NewOutputType>(defaultValue);
        typename BatchReadType::ParamsType store{{}, usedPlanes, def, ActiveThreads{max_width, max_height, uint(BATCH)}};
        for (size_t i = 0; i < BATCH; ++i) batch_detail::build_in(store.opData[i], [&]() -> std::remove_reference_t<decltype(store.opData[i])> { return iOps[i]; });
        return BatchReadType::build(store);
    }
private:
    template <typename O, typename I> static constexpr O amd_cast_default(const I& v) {
        static_assert(cn<O> == cn<I>, "default value and operation output must have the same number of channels");
        if constexpr (!isVector<O>) return static_cast<O>(vectorAt<0>(v));
        else if constexpr (cn<O> == 1) return O{static_cast<VBase<O>>(vectorAt<0>(v))};
        else if constexpr (cn<O> == 2) return O{static_cast<VBase<O>>(v.x), static_cast<VBase<O>>(v.y)};
        else if constexpr (cn<O> == 3) return O{static_cast<VBase<O>>(v.x), static_cast<VBase<O>>(v.y), static_cast<VBase<O>>(v.z)};
        else return O{static_cast<VBase<O>>(v.x), static_cast<VBase<O>>(v.y), static_cast<VBase<O>>(v.z), static_cast<VBase<O>>(v.w)};
    }
};

struct BatchUtils {
    // Splits a batch IOp back into its per-plane IOps.
    template <typename InstantiableType> static constexpr auto toArray(const InstantiableType& batchIOp) {
        using IOpType = std::decay_t<InstantiableType>;
        static_assert(isBatchOperation<typename IOpType::Operation>, "The IOp passed as parameter is not a batch operation");
        using Operation = typename IOpType::Operation::Operation;
        constexpr size_t B = IOpType::Operation::BATCH;
        std::array<Instantiable<Operation>, B> result{};
        for (size_t i = 0; i < B; ++i) {
            if constexpr (IOpType::template is<ReadType>) batch_detail::build_in(result[i], [&] { return Operation::build(batchIOp.params.opData[i]); });
            else batch_detail::build_in(result[i], [&] { return Operation::build(OperationData<Operation>{batchIOp.params[i]}); });
        }
        return result;
    }

    // Element-wise Operation::build over N parallel arrays of arguments.
    template <typename Operation, size_t BATCH, typename ArrayType, typename... Arrays>
    static constexpr auto build_batch(const std::array<ArrayType, BATCH>& firstArray, const Arrays&... arrays) {
        using Built = decltype(Operation::build(std::declval<ArrayType>(), std::declval<Arrays>()[0]...));
        std::array<Built, BATCH> result{};
        for (size_t i = 0; i < BATCH; ++i) batch_detail::build_in(result[i], [&] { return Operation::build(firstArray[i], arrays[i]...); });
        return result;
    }
};

// std::array overloads of Operation::build for read-like operations.
template <typename Child_> template <size_t B, typename... ArrayTypes>
constexpr auto ReadBatchBuilders<Child_>::build_batch(const std::array<ArrayTypes, B>&... arrays) {
    return BatchUtils::template build_batch<Child_>(arrays...);
}
template <typename Child_> template <size_t B, typename... ArrayTypes>
constexpr auto ReadBatchBuilders<Child_>::build(const std::array<ArrayTypes, B>&... arrays) {
    return BatchRead<PlanePolicy::PROCESS_ALL>::build(build_batch(arrays...));
}
template <typename Child_> template <size_t B, typename DefaultValueType, typename... ArrayTypes>
constexpr auto ReadBatchBuilders<Child_>::build(const int& usedPlanes, const DefaultValueType& defaultValue,
                                                const std::array<ArrayTypes, B>&... arrays) {
    return BatchRead<PlanePolicy::CONDITIONAL_WITH_DEFAULT>::build(build_batch(arrays...), usedPlanes, defaultValue);
}

// ---- BatchWrite ------------------------------------------------------------------------------------------
template <size_t BATCH, typename Operation = void> struct BatchWrite {
    using Op = Operation;
    using Child = BatchWrite<BATCH, Operation>;
    using ParamsType = typename Operation::ParamsType[BATCH];
    using InputType = typename Operation::InputType;
    using WriteDataType = typename Operation::WriteDataType;
    using InstanceType = WriteType;
    using OperationDataType = OperationData<Child>;
    using InstantiableType = Write<Child>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool THREAD_FUSION = Operation::THREAD_FUSION;
    static constexpr size_t BATCH_SIZE = BATCH;
    static constexpr InstantiableType build(const std::array<Instantiable<Operation>, BATCH>& iOps) {
        InstantiableType iOp{};
        for (size_t i = 0; i < BATCH; ++i) iOp.params[i] = iOps[i].params;
        return iOp;
    }
};
template <size_t BATCH> struct BatchWrite<BATCH, void> {
    using InstaceType = WriteType;
    template <typename IOp> static constexpr auto build(const std::array<IOp, BATCH>& iOps) {
        return BatchWrite<BATCH, typename IOp::Operation>::build(iOps);
    }
};

template <typename Child_> template <size_t BATCH_N, typename FirstType, typename... ArrayTypes>
constexpr auto WriteBatchBuilders<Child_>::build_batch(const std::array<FirstType, BATCH_N>& first, const ArrayTypes&... arrays) {
    return BatchUtils::template build_batch<Child_>(first, arrays...);
}
template <typename Child_> template <size_t BATCH_N, typename FirstType, typename... ArrayTypes>
constexpr auto WriteBatchBuilders<Child_>::build(const std::array<FirstType, BATCH_N>& first, const ArrayTypes&... arrays) {
    return BatchWrite<BATCH_N>::build(build_batch(first, arrays...));
}

// ---- device lowering ---------------------------------------------------------------------------------------
namespace amd {
template <size_t B, typename Op>
struct Lower<BatchRead<PlanePolicy::PROCESS_ALL, B, Op>, std::enable_if_t<isCompleteOperation<Op>>> {
    static constexpr bool available = true;
    using Self = BatchRead<PlanePolicy::PROCESS_ALL, B, Op>;
    using type = fkd::BatchRead<int(B), typename Lower<Op>::type>;
    static typename type::Params params(const OperationData<Self>& d) {
        // each plane's parameters are built where they live (an assignment would build them on the stack in small
        // pieces and read them back whole, which stalls on every plane)
        typename type::Params p;
        using PlaneParams = std::remove_reference_t<decltype(p.plane[0])>;
        static_assert(std::is_trivially_destructible_v<PlaneParams>);
        for (size_t i = 0; i < B; ++i) ::new (static_cast<void*>(&p.plane[i])) PlaneParams(Lower<Op>::params(d.params.opData[i]));
        return p;
    }
};
template <size_t B, typename Op>
struct Lower<BatchRead<PlanePolicy::CONDITIONAL_WITH_DEFAULT, B, Op>, std::enable_if_t<isCompleteOperation<Op>>> {
    static constexpr bool available = true;
    using Self = BatchRead<PlanePolicy::CONDITIONAL_WITH_DEFAULT, B, Op>;
    using type = fkd::BatchReadDefault<int(B), typename Lower<Op>::type>;
    static typename type::Params params(const OperationData<Self>& d) {
        typename type::Params p{};
        for (size_t i = 0; i < B; ++i) p.plane[i] = Lower<Op>::params(d.params.opData[i]);
        p.used = d.params.usedPlanes;
        p.def = to_dev(d.params.default_value);
        return p;
    }
};
template <size_t B, typename Op> struct Lower<BatchWrite<B, Op>, std::enable_if_t<!std::is_void_v<Op>>> {
    static constexpr bool available = true;
    using type = fkd::BatchWrite<int(B), typename Lower<Op>::type>;
    static typename type::Params params(const OperationData<BatchWrite<B, Op>>& d) {
        typename type::Params p{};
        for (size_t i = 0; i < B; ++i) p.plane[i] = Lower<Op>::params(OperationData<Op>{d.params[i]});
        return p;
    }
};
} // namespace amd

} // namespace fk
#endif
#endif
