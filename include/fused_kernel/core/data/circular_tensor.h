// CircularTensor: a Tensor of BATCH planes that always shows the last BATCH images handed to update(), newest first
// or oldest first, the temporal window of a video pipeline.  update() runs the caller's chain (read ... write) on the
// new image and shifts the others by one plane in ONE launch: a DivergentBatchTransformDPP of two sequences, the
// caller's chain with a store into a hidden ring of BATCH planes put before its write, and a copy of the other
// BATCH - 1 planes out of that ring.
// Interface counterpart: FK/core/data/circular_tensor.h:24-168.  With ColorPlanes::Transposed the window is a TensorT
// (all first channel planes, then all second ones, ...) and the chain must end in Write<TensorTSplit<...>>.
#ifndef FK_AMD_CIRCULAR_TENSOR_H
#define FK_AMD_CIRCULAR_TENSOR_H

#include <fused_kernel/core/data/ptr_nd.h>
#include <fused_kernel/core/data/tuple.h>
#include <fused_kernel/core/execution_model/executors.h>
#include <fused_kernel/algorithms/basic_ops/memory_operations.h>

#include <stdexcept>
#include <type_traits>

namespace fk {

enum class CircularTensorOrder { NewestFirst, OldestFirst };
enum class ColorPlanes { Standard, Transposed };

namespace amd {

// The reader that fetches back, element for element, what a tensor writer stored.
template <typename Writer> struct StoredBy;
template <typename E> struct StoredBy<TensorWrite<E>> { using Reader = TensorRead<E>; };
template <typename E> struct StoredBy<TensorSplit<E>> { using Reader = TensorPack<E>; };
template <typename E> struct StoredBy<TensorTSplit<E>> { using Reader = TensorTPack<E>; };

template <typename T, int N> struct LazyVector { using type = VectorType_t<T, N>; };

// Everything the template arguments of a CircularTensor decide.
template <typename T, int CHANNELS, int BATCH, CircularTensorOrder ORDER, ColorPlanes LAYOUT> struct WindowTraits {
    // an element of the window: T itself when T already is a pixel in one plane, CHANNELS values of T otherwise
    static constexpr bool kPixelInOnePlane = std::is_aggregate_v<T> && CHANNELS == 1;
    static_assert(kPixelInOnePlane || (!std::is_aggregate_v<T> && CHANNELS > 1),
                  "CircularTensor<T, COLOR_PLANES, ...>: either a vector T in one plane or a scalar T in several");
    using Element = typename std::conditional_t<kPixelInOnePlane, std::type_identity<T>, LazyVector<T, CHANNELS>>::type;
    using Window = std::conditional_t<LAYOUT == ColorPlanes::Transposed, TensorT<T>, Tensor<T>>;

    static constexpr uint kNewestPlane = ORDER == CircularTensorOrder::NewestFirst ? 0u : uint(BATCH) - 1u;
    // the ring is filled upwards; showing the newest image first means walking it downwards
    static constexpr CircularDirection kWalk =
        ORDER == CircularTensorOrder::NewestFirst ? CircularDirection::Descendent : CircularDirection::Ascendent;
    // plane of the launch -> sequence: the caller's chain (0) for the plane that shows the newest image, the copy (1) elsewhere
    struct PlaneToSequence {
        static constexpr uint at(const uint& plane) { return plane == kNewestPlane ? 0u : 1u; }
    };
    template <typename WriteIOp> static constexpr bool accepts() {
        if constexpr (LAYOUT == ColorPlanes::Transposed) return std::is_same_v<WriteIOp, Write<TensorTSplit<Element>>>;
        else return std::is_same_v<WriteIOp, Write<TensorWrite<Element>>> || std::is_same_v<WriteIOp, Write<TensorSplit<Element>>>;
    }
};

} // namespace amd

template <typename T, int COLOR_PLANES, int BATCH, CircularTensorOrder CT_ORDER, ColorPlanes CP_MODE>
class CircularTensor : public amd::WindowTraits<T, COLOR_PLANES, BATCH, CT_ORDER, CP_MODE>::Window {
    using Traits = amd::WindowTraits<T, COLOR_PLANES, BATCH, CT_ORDER, CP_MODE>;
    using Window = typename Traits::Window;

public:
    CircularTensor() = default;
    CircularTensor(const uint& width, const uint& height, const MemType& mem = defaultMemType, const int& device = 0)
        : Window(width, height, BATCH, COLOR_PLANES, mem, device), ring_(width, height, BATCH, COLOR_PLANES, mem, device) {}

    void Alloc(const uint& width, const uint& height, const MemType& mem = defaultMemType, const int& device = 0) {
        this->allocTensor(width, height, BATCH, COLOR_PLANES, mem, device);
        ring_.allocTensor(width, height, BATCH, COLOR_PLANES, mem, device);
    }

    // `chain` is a complete chain (read ... write) whose write stores one image into this tensor's ptr().
    template <ParArch PA, typename... IOps> void update(Stream_<PA>& stream, const IOps&... chain) {
        using WriteIOp = std::decay_t<decltype(ppLast(chain...))>;
        static_assert(Traits::template accepts<WriteIOp>(),
                      "the chain given to CircularTensor::update must end in Write<TensorWrite<E>> or Write<TensorSplit<E>> "
                      "(ColorPlanes::Standard) or in Write<TensorTSplit<E>> (ColorPlanes::Transposed), E being the window's element");
        using Writer = typename WriteIOp::Operation;
        if (PA == ParArch::GPU_AMD && this->getMemType() != MemType::Device && this->getMemType() != MemType::DeviceAndPinned)
            throw std::runtime_error("CircularTensor::update on the GPU needs a window in MemType::Device or MemType::DeviceAndPinned");

        // sequence 0: the caller's chain; its result also goes into slot head_ of the ring, just before its own write
        MidWrite<CircularTensorWrite<CircularDirection::Ascendent, Writer, BATCH>> keep;
        keep.params.first = head_;
        keep.params.opData.params = ring_.ptr();
        // sequence 1: the other BATCH - 1 images, read back out of the ring in the window's order, through the same write
        Read<CircularTensorRead<Traits::kWalk, typename amd::StoredBy<Writer>::Reader, BATCH>> others;
        others.params.first = head_;
        others.params.opData.params = ring_.ptr();
        others.params.opData.params.dims.planes = uint(BATCH) - 1u;

        Executor<DivergentBatchTransformDPP<PA, typename Traits::PlaneToSequence>>::executeOperations(
            stream, buildOperationSequence_tup(insert_before_last(keep, chain...)), buildOperationSequence(others, ppLast(chain...)));
        head_ = (head_ + 1) % BATCH;
    }

private:
    Window ring_;     // every image ever stored, slot head_ next
    int head_{0};
};

} // namespace fk
#endif
