// CircularTensor: a Tensor of BATCH planes that always shows the last BATCH images handed to update(), newest first
// or oldest first, the temporal window of a video pipeline.  update() runs the caller's chain (read ... write) on the
// new image and shifts the others by one plane in ONE launch: a DivergentBatchTransformDPP of two sequences, the
// caller's chain with a store into a hidden circular copy put before its write, and a copy of the other BATCH - 1
// planes out of that hidden copy.
// Interface counterpart: FK/core/data/circular_tensor.h:24-168.  With ColorPlanes::Transposed the window is a TensorT
// (all first channel planes, then all second ones, ...) and the chain must end in Write<TensorTSplit<StoreT>>.
#ifndef FK_AMD_CIRCULAR_TENSOR_H
#define FK_AMD_CIRCULAR_TENSOR_H

#include <fused_kernel/core/data/ptr_nd.h>
#include <fused_kernel/core/data/tuple.h>
#include <fused_kernel/core/execution_model/executors.h>
#include <fused_kernel/algorithms/basic_ops/memory_operations.h>

#include <stdexcept>

namespace fk {

enum class CircularTensorOrder { NewestFirst, OldestFirst };

// Which sequence of update() a plane belongs to: 0 the caller's chain (the newest image), 1 the copy.
template <CircularTensorOrder CTO, int BATCH> struct SequenceSelectorType {
    static constexpr uint at(const uint& index) {
        if constexpr (CTO == CircularTensorOrder::NewestFirst) return index > 0 ? 1u : 0u;
        else return index != BATCH - 1 ? 1u : 0u;
    }
};

template <CircularTensorOrder CT_ORDER> struct CTReadDirection;
template <> struct CTReadDirection<CircularTensorOrder::NewestFirst> { static constexpr CircularDirection dir{CircularDirection::Descendent}; };
template <> struct CTReadDirection<CircularTensorOrder::OldestFirst> { static constexpr CircularDirection dir{CircularDirection::Ascendent}; };
template <CircularTensorOrder CT_ORDER> static constexpr CircularDirection CTReadDirection_v = CTReadDirection<CT_ORDER>::dir;

enum class ColorPlanes { Standard, Transposed };

template <typename T, ColorPlanes CP_MODE> struct CoreType;
template <typename T> struct CoreType<T, ColorPlanes::Standard> { using type = Tensor<T>; };
template <typename T> struct CoreType<T, ColorPlanes::Transposed> { using type = TensorT<T>; };
template <typename T, ColorPlanes CP_MODE> using CoreType_t = typename CoreType<T, CP_MODE>::type;

template <typename T, int COLOR_PLANES, typename Enabler = void> struct CircularTensorStoreType {};
template <typename T, int COLOR_PLANES> struct CircularTensorStoreType<T, COLOR_PLANES, std::enable_if_t<std::is_aggregate_v<T> && COLOR_PLANES == 1>> {
    using type = T;
};
template <typename T, int COLOR_PLANES> struct CircularTensorStoreType<T, COLOR_PLANES, std::enable_if_t<!std::is_aggregate_v<T> && (COLOR_PLANES > 1)>> {
    using type = VectorType_t<T, COLOR_PLANES>;
};

template <typename T, int COLOR_PLANES, int BATCH, CircularTensorOrder CT_ORDER, ColorPlanes CP_MODE> class CircularTensor : public CoreType_t<T, CP_MODE> {
    using ParentType = CoreType_t<T, CP_MODE>;
    using StoreT = typename CircularTensorStoreType<T, COLOR_PLANES>::type;
    using WriteInstantiableOperations = TypeList<Write<TensorWrite<StoreT>>, Write<TensorSplit<StoreT>>, Write<TensorTSplit<StoreT>>>;
    using ReadInstantiableOperations = TypeList<Read<CircularTensorRead<CTReadDirection_v<CT_ORDER>, TensorRead<StoreT>, BATCH>>,
                                                Read<CircularTensorRead<CTReadDirection_v<CT_ORDER>, TensorPack<StoreT>, BATCH>>,
                                                Read<CircularTensorRead<CTReadDirection_v<CT_ORDER>, TensorTPack<StoreT>, BATCH>>>;

public:
    CircularTensor() {}
    CircularTensor(const uint& width_, const uint& height_, const MemType& type_ = defaultMemType, const int& deviceID_ = 0)
        : ParentType(width_, height_, BATCH, COLOR_PLANES, type_, deviceID_), m_tempTensor(width_, height_, BATCH, COLOR_PLANES, type_, deviceID_) {}

    void Alloc(const uint& width_, const uint& height_, const MemType& type_ = defaultMemType, const int& deviceID_ = 0) {
        this->allocTensor(width_, height_, BATCH, COLOR_PLANES, type_, deviceID_);
        m_tempTensor.allocTensor(width_, height_, BATCH, COLOR_PLANES, type_, deviceID_);
    }

    // The IOps are a complete chain whose write is TensorWrite<StoreT> or TensorSplit<StoreT> on this tensor's ptr().
    template <ParArch PA, typename... IOpTypes> void update(Stream_<PA>& stream, const IOpTypes&... instantiableOperationInstances) {
        const auto writeInstantiableOperation = ppLast(instantiableOperationInstances...);
        using writeDFType = std::decay_t<decltype(writeInstantiableOperation)>;
        using writeOpType = typename writeDFType::Operation;
        if constexpr (CP_MODE == ColorPlanes::Transposed) {
            static_assert(std::is_same_v<writeDFType, Write<TensorTSplit<StoreT>>>,
                          "Need to use TensorTSplitWrite as write function because you are using a transposed CircularTensor (CP_MODE = Transposed)");
        } else {
            static_assert(one_of_v<writeDFType, TypeList<Write<TensorWrite<StoreT>>, Write<TensorSplit<StoreT>>>>,
                          "the chain given to CircularTensor::update must end in Write<TensorWrite<StoreT>> or Write<TensorSplit<StoreT>>");
        }
        using equivalentReadDFType = EquivalentType_t<writeDFType, WriteInstantiableOperations, ReadInstantiableOperations>;

        // The launch's planes are the planes of both sequences together: one for the new image, BATCH - 1 copied.
        constexpr uint COPY_PLANES = static_cast<uint>(BATCH) - 1u;

        MidWrite<CircularTensorWrite<CircularDirection::Ascendent, writeOpType, BATCH>> updateWriteToTemp;
        updateWriteToTemp.params.first = m_nextUpdateIdx;
        updateWriteToTemp.params.opData.params = m_tempTensor.ptr();
        const auto updateOps = buildOperationSequence_tup(insert_before_last(updateWriteToTemp, instantiableOperationInstances...));

        equivalentReadDFType nonUpdateRead;
        nonUpdateRead.params.first = m_nextUpdateIdx;
        nonUpdateRead.params.opData.params = m_tempTensor.ptr();
        nonUpdateRead.params.opData.params.dims.planes = COPY_PLANES;
        const auto copyOps = buildOperationSequence(nonUpdateRead, writeInstantiableOperation);

        if (PA == ParArch::GPU_AMD && !(this->getMemType() == MemType::Device || this->getMemType() == MemType::DeviceAndPinned)) {
            throw std::runtime_error("CircularTensor operations on Device memory only supported "
                                     "if the CircularTensor is MemType::Device or MemType::DeviceAndPinned");
        }
        Executor<DivergentBatchTransformDPP<PA, SequenceSelectorType<CT_ORDER, BATCH>>>::executeOperations(stream, updateOps, copyOps);
        m_nextUpdateIdx = (m_nextUpdateIdx + 1) % BATCH;
    }

private:
    CoreType_t<T, CP_MODE> m_tempTensor;
    int m_nextUpdateIdx{0};
};

} // namespace fk
#endif
