// Thread fusion: the switch of TransformDPP and the type arithmetic that goes with it.
// Interface counterpart: FK/core/execution_model/thread_fusion.h (TF :23, ThreadFusionInfo :82-139,
// isThreadFusionEnabled :141-146, isThreadDivisible :148-160).
//
// In the reference thread fusion widens what one thread reads and writes (two floats as a float2, four bytes as a
// uchar4) and never changes results.  This backend always moves four elements per lane where a chain reads rows, so
// TransformDPP<..., TF::ENABLED> and TF::DISABLED run the same kernel; the types below answer what the reference's
// answer would be, for user code and tests that ask.
#ifndef FK_AMD_THREAD_FUSION_H
#define FK_AMD_THREAD_FUSION_H

#include <tuple>
#include <type_traits>

#include <fused_kernel/core/data/point.h>
#include <fused_kernel/core/utils/vector_utils.h>

namespace fk {

enum class TF : bool { DISABLED = false, ENABLED = true };

namespace amd {
// How many elements of type T one fused access holds: as many as make up four channels of one byte, or two channels
// of two or four bytes; elements of three or four channels and channels of eight bytes stay alone.
template <typename T> constexpr int fused_elements() {
    constexpr int channels = cn<T>;
    constexpr size_t channel_bytes = sizeof(VBase<T>);
    if constexpr (channels > 2) return 1;
    else if constexpr (channel_bytes == 1) return 4 / channels;
    else if constexpr (channel_bytes <= 4) return channels == 1 ? 2 : 1;
    else return 1;
}
template <typename T> struct FusedAccess {
    static constexpr int elements = fused_elements<T>();
    // A lone one-channel element is spelled as its channel type (ulong1 -> ulong), everything else as the vector.
    using type = std::conditional_t<elements == 1, std::conditional_t<cn<T> == 1, VBase<T>, T>,
                                    VectorType_t<VBase<T>, cn<T> * elements>>;
};
} // namespace amd

template <typename SourceType> using TFBiggerType_t = typename amd::FusedAccess<SourceType>::type;

template <unsigned channelNumber> constexpr bool isValidChannelNumber = channelNumber >= 1 && channelNumber <= 4;

template <typename ReadType, typename WriteType, bool ENABLED_> struct ThreadFusionInfo {
    // Fusing is possible when the widened write still is a vector type: elements * channels of the write type <= 4.
    static constexpr bool ENABLED = ENABLED_ && isValidChannelNumber<unsigned(amd::FusedAccess<ReadType>::elements * cn<WriteType>)>;
    using BiggerReadType = std::conditional_t<ENABLED, TFBiggerType_t<ReadType>, ReadType>;
    static constexpr uint elems_per_thread{static_cast<uint>(cn<BiggerReadType> / cn<ReadType>)};
    using BiggerWriteType = VectorType_t<VBase<WriteType>, int(elems_per_thread) * cn<WriteType>>;

    // Element IDX of a fused read.
    template <int IDX> static constexpr ReadType get(const BiggerReadType& data) {
        static_assert(IDX >= 0 && IDX < int(elems_per_thread), "Index out of range for this ThreadFusionInfo");
        if constexpr (elems_per_thread == 1) return static_cast<ReadType>(data);
        else if constexpr (cn<ReadType> == 1) return make_<ReadType>(vectorAt<IDX>(data));
        else return make_<ReadType>(vectorAt<2 * IDX>(data), vectorAt<2 * IDX + 1>(data));      // two-channel elements
    }
    // The fused write made of elems_per_thread results.
    template <typename... OriginalTypes> static constexpr BiggerWriteType make(const OriginalTypes&... data) {
        static_assert((std::is_same_v<WriteType, OriginalTypes> && ...), "Not all types are the same when making the ThreadFusion BiggerType value");
        static_assert(sizeof...(OriginalTypes) == elems_per_thread, "one value per fused element");
        if constexpr (cn<WriteType> == 1) return make_<BiggerWriteType>(vectorAt<0>(data)...);
        else return join(data...);
    }

private:
    static constexpr BiggerWriteType join(const WriteType& only) { return only; }
    static constexpr BiggerWriteType join(const WriteType& first, const WriteType& second) {
        static_assert(cn<WriteType> == 2, "only two-channel elements fuse in pairs");
        return make_<BiggerWriteType>(first.x, first.y, second.x, second.y);
    }
};

// Whether a TransformDPP over these instantiable operations would fuse threads in the reference: the read and the write
// must both allow it (a back-reading read or a planar split does not).
template <bool THREAD_FUSION_ENABLED, typename... IOpTypes> constexpr bool isThreadFusionEnabled() {
    using ReadOperation = typename std::tuple_element_t<0, std::tuple<IOpTypes...>>::Operation;
    using WriteOperation = typename std::tuple_element_t<sizeof...(IOpTypes) - 1, std::tuple<IOpTypes...>>::Operation;
    return ReadOperation::THREAD_FUSION && WriteOperation::THREAD_FUSION && THREAD_FUSION_ENABLED;
}

// Whether both row lengths are whole numbers of fused accesses (otherwise the reference adds a scalar tail).
template <bool THREAD_FUSION_ENABLED, typename... IOpTypes>
inline bool isThreadDivisible(const uint& elems_per_thread, const IOpTypes&... iOps) {
    if constexpr (THREAD_FUSION_ENABLED) {
        const auto all = std::forward_as_tuple(iOps...);
        const auto& readOp = std::get<0>(all);
        const auto& writeOp = std::get<sizeof...(IOpTypes) - 1>(all);
        using ReadOperation = typename std::tuple_element_t<0, std::tuple<IOpTypes...>>::Operation;
        using WriteOperation = typename std::tuple_element_t<sizeof...(IOpTypes) - 1, std::tuple<IOpTypes...>>::Operation;
        const uint readRow = ReadOperation::num_elems_x(Point{0, 0, 0}, {readOp.params});
        const uint writeRow = WriteOperation::num_elems_x(Point{0, 0, 0}, {writeOp.params});
        return readRow % elems_per_thread == 0 && writeRow % elems_per_thread == 0;
    } else {
        return true;
    }
}

} // namespace fk
#endif
