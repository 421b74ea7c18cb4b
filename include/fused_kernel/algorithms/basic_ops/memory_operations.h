// Per-element memory operations: PerThreadRead / PerThreadWrite (pitched 1-D/2-D/3-D), TensorRead / TensorWrite,
// TensorSplit (planar writer) and TensorPack (its reader), and the circular-buffer views CircularTensorRead /
// CircularTensorWrite.  Interface counterpart: FK/algorithms/basic_ops/memory_operations.h:26-212, 243-290, 413-432,
// 505-587.  CircularBatchRead / CircularBatchWrite (434-503), the transposed-plane forms TensorTSplit / TensorTPack (214-241, 292-327)
// and SplitWrite (336-390: one image per channel) too.
#ifndef FK_AMD_MEMORY_OPERATIONS_H
#define FK_AMD_MEMORY_OPERATIONS_H

#include <vector>

#include <fused_kernel/core/execution_model/operation_model/operation_model.h>
#include <fused_kernel/core/data/tuple.h>

namespace fk {

template <ND D, typename T>
struct PerThreadRead : ReadOperation<T, RawPtr<D, T>, T, TF::ENABLED, PerThreadRead<D, T>> {
    using Parent = ReadOperation<T, RawPtr<D, T>, T, TF::ENABLED, PerThreadRead<D, T>>;
    using typename Parent::OperationDataType;
    FK_STATIC_STRUCT(PerThreadRead, PerThreadRead)
    static constexpr uint num_elems_x(const Point, const OperationDataType& opData) { return opData.params.dims.width; }
    static constexpr uint num_elems_y(const Point, const OperationDataType& opData) {
        if constexpr (D == ND::_1D) return 1; else return opData.params.dims.height;
    }
    static constexpr uint num_elems_z(const Point, const OperationDataType& opData) {
        if constexpr (D == ND::_1D || D == ND::_2D) return 1; else return opData.params.dims.planes;
    }
    static constexpr uint pitch(const Point, const OperationDataType& opData) { return opData.params.dims.pitch; }
    static constexpr ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return {num_elems_x(Point{0, 0, 0}, opData), num_elems_y(Point{0, 0, 0}, opData), num_elems_z(Point{0, 0, 0}, opData)};
    }
};

template <ND D, typename T>
struct PerThreadWrite : WriteOperation<T, RawPtr<D, T>, T, TF::ENABLED, PerThreadWrite<D, T>> {
    using Parent = WriteOperation<T, RawPtr<D, T>, T, TF::ENABLED, PerThreadWrite<D, T>>;
    using typename Parent::OperationDataType;
    using typename Parent::InstantiableType;
    FK_STATIC_STRUCT(PerThreadWrite, PerThreadWrite)
    using Parent::build;
    static InstantiableType build(const Ptr<D, T>& ptr) { return {{ptr.ptr()}}; }
    static constexpr uint num_elems_x(const Point, const OperationDataType& opData) { return opData.params.dims.width; }
    static constexpr uint pitch(const Point, const OperationDataType& opData) { return opData.params.dims.pitch; }
};

// SplitWrite<D, T>: channel c of every value goes to an image of its own (x, y, z, w), each with its own pitch.
// Interface counterpart: FK/algorithms/basic_ops/memory_operations.h:336-390.
template <ND D, typename T, typename Enabler = void> struct SplitWriteParams {};
template <ND D, typename T> struct SplitWriteParams<D, T, std::enable_if_t<cn<T> == 2>> {
    RawPtr<D, VBase<T>> x, y;
};
template <ND D, typename T> struct SplitWriteParams<D, T, std::enable_if_t<cn<T> == 3>> {
    RawPtr<D, VBase<T>> x, y, z;
};
template <ND D, typename T> struct SplitWriteParams<D, T, std::enable_if_t<cn<T> == 4>> {
    RawPtr<D, VBase<T>> x, y, z, w;
};
template <ND D, typename T>
struct SplitWrite : WriteOperation<T, SplitWriteParams<D, T>, VBase<T>, TF::DISABLED, SplitWrite<D, T>> {
    static_assert(cn<T> >= 2, "Split operations can only be used with types of 2, 3 or 4 channels.");
    using Parent = WriteOperation<T, SplitWriteParams<D, T>, VBase<T>, TF::DISABLED, SplitWrite<D, T>>;
    using typename Parent::OperationDataType;
    using typename Parent::InstantiableType;
    FK_STATIC_STRUCT(SplitWrite, SplitWrite)
    using Parent::build;
    // one image per channel, in channel order (at() throws when there are too few)
    static InstantiableType build(const std::vector<Ptr2D<VBase<T>>>& output) {
        if constexpr (cn<T> == 2) return {{{output.at(0).ptr(), output.at(1).ptr()}}};
        else if constexpr (cn<T> == 3) return {{{output.at(0).ptr(), output.at(1).ptr(), output.at(2).ptr()}}};
        else return {{{output.at(0).ptr(), output.at(1).ptr(), output.at(2).ptr(), output.at(3).ptr()}}};
    }
    static constexpr uint num_elems_x(const Point, const OperationDataType& opData) { return opData.params.x.dims.width; }
    static constexpr uint pitch(const Point, const OperationDataType& opData) { return opData.params.x.dims.pitch; }
};

// DualSourceRead<D, T>: the elements of two images at the same position as a Tuple<T, T>, for the two-input forms of the
// arithmetic, bitwise and comparison Operations (image-by-image work in one kernel).  The extent is the first image's.
// Interface counterpart: FK/algorithms/basic_ops/memory_operations.h:585-640.
template <ND D, typename T> struct DualSourceReadParams {
    RawPtr<D, T> src1;
    RawPtr<D, T> src2;
};
template <ND D, typename T>
struct DualSourceRead : ReadOperation<T, DualSourceReadParams<D, T>, Tuple<T, T>, TF::DISABLED, DualSourceRead<D, T>> {
    using Parent = ReadOperation<T, DualSourceReadParams<D, T>, Tuple<T, T>, TF::DISABLED, DualSourceRead<D, T>>;
    using typename Parent::OperationDataType;
    using typename Parent::InstantiableType;
    FK_STATIC_STRUCT(DualSourceRead, DualSourceRead)
    using Parent::build;
    static InstantiableType build(const Ptr<D, T>& src1, const Ptr<D, T>& src2) { return {{DualSourceReadParams<D, T>{src1.ptr(), src2.ptr()}}}; }
    static constexpr uint num_elems_x(const Point, const OperationDataType& opData) { return opData.params.src1.dims.width; }
    static constexpr uint num_elems_y(const Point, const OperationDataType& opData) {
        if constexpr (D == ND::_1D) return 1; else return opData.params.src1.dims.height;
    }
    static constexpr uint num_elems_z(const Point, const OperationDataType& opData) {
        if constexpr (D == ND::_1D || D == ND::_2D) return 1; else return opData.params.src1.dims.planes;
    }
    static constexpr uint pitch(const Point, const OperationDataType& opData) { return opData.params.src1.dims.pitch; }
    static constexpr ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return {num_elems_x(Point{0, 0, 0}, opData), num_elems_y(Point{0, 0, 0}, opData), num_elems_z(Point{0, 0, 0}, opData)};
    }
};

// Deduces dimension and element type from the pointer: ReadOp::build(ptr), WriteOp::build(ptr).
struct ReadOp {
    template <typename PtrType> static decltype(auto) build(PtrType&& ptr) {
        using P = std::decay_t<PtrType>;
        return PerThreadRead<P::nd, typename P::Type>::build(ptr.ptr());
    }
    template <typename PtrType, size_t N> static decltype(auto) build(const std::array<PtrType, N>& ptrs) {
        return PerThreadRead<PtrType::nd, typename PtrType::Type>::build(ptrs);
    }
};
struct WriteOp {
    template <typename PtrType> static decltype(auto) build(PtrType&& ptr) {
        using P = std::decay_t<PtrType>;
        return PerThreadWrite<P::nd, typename P::Type>::build(ptr.ptr());
    }
    template <typename PtrType, size_t N> static decltype(auto) build(const std::array<PtrType, N>& ptrs) {
        return PerThreadWrite<PtrType::nd, typename PtrType::Type>::build(ptrs);
    }
};

template <typename T> struct TensorRead : ReadOperation<T, RawPtr<ND::_3D, T>, T, TF::ENABLED, TensorRead<T>> {
    using Parent = ReadOperation<T, RawPtr<ND::_3D, T>, T, TF::ENABLED, TensorRead<T>>;
    using typename Parent::OperationDataType;
    FK_STATIC_STRUCT(TensorRead, TensorRead)
    static constexpr uint num_elems_x(const Point, const OperationDataType& opData) { return opData.params.dims.width; }
    static constexpr uint num_elems_y(const Point, const OperationDataType& opData) { return opData.params.dims.height; }
    static constexpr uint num_elems_z(const Point, const OperationDataType& opData) { return opData.params.dims.planes; }
    static constexpr uint pitch(const Point, const OperationDataType& opData) { return opData.params.dims.pitch; }
    static constexpr ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return {opData.params.dims.width, opData.params.dims.height, opData.params.dims.planes};
    }
};

template <typename T> struct TensorWrite : WriteOperation<T, RawPtr<ND::_3D, T>, T, TF::ENABLED, TensorWrite<T>> {
    using Parent = WriteOperation<T, RawPtr<ND::_3D, T>, T, TF::ENABLED, TensorWrite<T>>;
    using typename Parent::OperationDataType;
    FK_STATIC_STRUCT(TensorWrite, TensorWrite)
    static constexpr uint num_elems_x(const Point, const OperationDataType& opData) { return opData.params.dims.width; }
    static constexpr uint pitch(const Point, const OperationDataType& opData) { return opData.params.dims.pitch; }
};

// Planar writer: channel c of pixel (x, y, z) lands c * width * height base elements after the AoS position.
template <typename T> struct TensorSplit : WriteOperation<T, RawPtr<ND::_3D, VBase<T>>, VBase<T>, TF::DISABLED, TensorSplit<T>> {
    using Parent = WriteOperation<T, RawPtr<ND::_3D, VBase<T>>, VBase<T>, TF::DISABLED, TensorSplit<T>>;
    using typename Parent::OperationDataType;
    FK_STATIC_STRUCT(TensorSplit, TensorSplit)
    static_assert(cn<T> >= 2, "Wrong type for split tensor write. It must be one of <type>2, <type>3 or <type>4.");
    static constexpr uint num_elems_x(const Point, const OperationDataType& opData) { return opData.params.dims.width; }
    static constexpr uint pitch(const Point, const OperationDataType& opData) { return opData.params.dims.pitch; }
};

// Planar reader: the layout TensorSplit writes, read back as a vector.
template <typename T> struct TensorPack : ReadOperation<VBase<T>, RawPtr<ND::_3D, VBase<T>>, T, TF::DISABLED, TensorPack<T>> {
    using Parent = ReadOperation<VBase<T>, RawPtr<ND::_3D, VBase<T>>, T, TF::DISABLED, TensorPack<T>>;
    using typename Parent::OperationDataType;
    FK_STATIC_STRUCT(TensorPack, TensorPack)
    static_assert(cn<T> >= 2, "Wrong type for split tensor read. It must be one of <type>2, <type>3 or <type>4.");
    static constexpr uint num_elems_x(const Point, const OperationDataType& opData) { return opData.params.dims.width; }
    static constexpr uint num_elems_y(const Point, const OperationDataType& opData) { return opData.params.dims.height; }
    static constexpr uint num_elems_z(const Point, const OperationDataType& opData) { return opData.params.dims.planes; }
    static constexpr uint pitch(const Point, const OperationDataType& opData) { return opData.params.dims.pitch; }
    static constexpr ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return {opData.params.dims.width, opData.params.dims.height, opData.params.dims.planes};
    }
};

// Planar writer and reader of a transposed tensor (RawPtr<ND::T3D>): channel c of pixel (x, y, z) lies in colour plane c,
// c * color_planes_pitch bytes after channel 0.  Interface counterpart: FK/algorithms/basic_ops/memory_operations.h:214-241
// (TensorTSplit) and :292-327 (TensorTPack).
template <typename T> struct TensorTSplit : WriteOperation<T, RawPtr<ND::T3D, VBase<T>>, VBase<T>, TF::DISABLED, TensorTSplit<T>> {
    using Parent = WriteOperation<T, RawPtr<ND::T3D, VBase<T>>, VBase<T>, TF::DISABLED, TensorTSplit<T>>;
    using typename Parent::OperationDataType;
    FK_STATIC_STRUCT(TensorTSplit, TensorTSplit)
    static_assert(cn<T> >= 2, "Wrong type for split tensor write. It must be one of <type>2, <type>3 or <type>4.");
    static constexpr uint num_elems_x(const Point, const OperationDataType& opData) { return opData.params.dims.width; }
    static constexpr uint pitch(const Point, const OperationDataType& opData) { return opData.params.dims.pitch; }
};
template <typename T> struct TensorTPack : ReadOperation<T, RawPtr<ND::T3D, VBase<T>>, T, TF::DISABLED, TensorTPack<T>> {
    using Parent = ReadOperation<T, RawPtr<ND::T3D, VBase<T>>, T, TF::DISABLED, TensorTPack<T>>;
    using typename Parent::OperationDataType;
    FK_STATIC_STRUCT(TensorTPack, TensorTPack)
    static_assert(cn<T> >= 2, "Wrong type for split tensor read. It must be one of <type>2, <type>3 or <type>4.");
    static constexpr uint num_elems_x(const Point, const OperationDataType& opData) { return opData.params.dims.width; }
    static constexpr uint num_elems_y(const Point, const OperationDataType& opData) { return opData.params.dims.height; }
    static constexpr uint num_elems_z(const Point, const OperationDataType& opData) { return opData.params.dims.planes; }
    static constexpr uint pitch(const Point, const OperationDataType& opData) { return opData.params.dims.pitch; }
    static constexpr ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return {opData.params.dims.width, opData.params.dims.height, opData.params.dims.planes};
    }
};

// A tensor of BATCH planes used as a circular buffer: logical plane z lives at (first + z) mod BATCH (Ascendent) or
// (first - z) mod BATCH (Descendent).
enum class CircularDirection { Ascendent, Descendent };
template <typename OperationDataTypeArray> struct CircularMemoryParams {
    int first;
    OperationDataTypeArray opData;
};

// BATCH separate reads (or writes) used as a circular buffer: logical plane z is operation number (first +- z) mod BATCH.
template <CircularDirection direction, typename Operation, int BATCH>
struct CircularBatchRead : ReadOperation<typename Operation::ReadDataType, CircularMemoryParams<OperationData<Operation>[BATCH]>,
                                         typename Operation::OutputType, Operation::THREAD_FUSION ? TF::ENABLED : TF::DISABLED,
                                         CircularBatchRead<direction, Operation, BATCH>> {
    using Parent = ReadOperation<typename Operation::ReadDataType, CircularMemoryParams<OperationData<Operation>[BATCH]>,
                                 typename Operation::OutputType, Operation::THREAD_FUSION ? TF::ENABLED : TF::DISABLED,
                                 CircularBatchRead<direction, Operation, BATCH>>;
    using typename Parent::OperationDataType;
    FK_STATIC_STRUCT(CircularBatchRead, CircularBatchRead)
    static constexpr uint num_elems_x(const Point thread, const OperationDataType& opData) { return Operation::num_elems_x(thread, opData.params.opData[thread.z]); }
    static constexpr uint num_elems_y(const Point thread, const OperationDataType& opData) { return Operation::num_elems_y(thread, opData.params.opData[thread.z]); }
    static constexpr uint num_elems_z(const Point, const OperationDataType&) { return BATCH; }
    static constexpr uint pitch(const Point thread, const OperationDataType& opData) { return Operation::pitch(thread, opData.params.opData[thread.z]); }
    static constexpr ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return {num_elems_x(Point{0, 0, 0}, opData), num_elems_y(Point{0, 0, 0}, opData), uint(BATCH)};
    }
};
template <CircularDirection direction, typename Operation, int BATCH>
struct CircularBatchWrite : WriteOperation<typename Operation::InputType, CircularMemoryParams<OperationData<Operation>[BATCH]>,
                                           typename Operation::WriteDataType, Operation::THREAD_FUSION ? TF::ENABLED : TF::DISABLED,
                                           CircularBatchWrite<direction, Operation, BATCH>> {
    using Parent = WriteOperation<typename Operation::InputType, CircularMemoryParams<OperationData<Operation>[BATCH]>,
                                  typename Operation::WriteDataType, Operation::THREAD_FUSION ? TF::ENABLED : TF::DISABLED,
                                  CircularBatchWrite<direction, Operation, BATCH>>;
    using typename Parent::OperationDataType;
    FK_STATIC_STRUCT(CircularBatchWrite, CircularBatchWrite)
    static constexpr uint num_elems_x(const Point thread, const OperationDataType& opData) { return Operation::num_elems_x(thread, opData.params.opData[thread.z]); }
    static constexpr uint pitch(const Point thread, const OperationDataType& opData) { return Operation::pitch(thread, opData.params.opData[thread.z]); }
};

template <CircularDirection direction, typename Operation, int BATCH>
struct CircularTensorRead : ReadOperation<typename Operation::ReadDataType, CircularMemoryParams<OperationData<Operation>>,
                                          typename Operation::OutputType, Operation::THREAD_FUSION ? TF::ENABLED : TF::DISABLED,
                                          CircularTensorRead<direction, Operation, BATCH>> {
    using Parent = ReadOperation<typename Operation::ReadDataType, CircularMemoryParams<OperationData<Operation>>, typename Operation::OutputType,
                                 Operation::THREAD_FUSION ? TF::ENABLED : TF::DISABLED, CircularTensorRead<direction, Operation, BATCH>>;
    using typename Parent::OperationDataType;
    FK_STATIC_STRUCT(CircularTensorRead, CircularTensorRead)
    static constexpr uint num_elems_x(const Point thread, const OperationDataType& opData) { return Operation::num_elems_x(thread, opData.params.opData); }
    static constexpr uint num_elems_y(const Point thread, const OperationDataType& opData) { return Operation::num_elems_y(thread, opData.params.opData); }
    // the planes of the view this read was given, not BATCH (BATCH stays the modulus of the circular index)
    static constexpr uint num_elems_z(const Point thread, const OperationDataType& opData) { return Operation::num_elems_z(thread, opData.params.opData); }
    static constexpr uint pitch(const Point thread, const OperationDataType& opData) { return Operation::pitch(thread, opData.params.opData); }
    static constexpr ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return {num_elems_x(Point{0, 0, 0}, opData), num_elems_y(Point{0, 0, 0}, opData), num_elems_z(Point{0, 0, 0}, opData)};
    }
};

template <CircularDirection direction, typename Operation, int BATCH>
struct CircularTensorWrite : WriteOperation<typename Operation::InputType, CircularMemoryParams<OperationData<Operation>>,
                                            typename Operation::WriteDataType, Operation::THREAD_FUSION ? TF::ENABLED : TF::DISABLED,
                                            CircularTensorWrite<direction, Operation, BATCH>> {
    using Parent = WriteOperation<typename Operation::InputType, CircularMemoryParams<OperationData<Operation>>, typename Operation::WriteDataType,
                                  Operation::THREAD_FUSION ? TF::ENABLED : TF::DISABLED, CircularTensorWrite<direction, Operation, BATCH>>;
    using typename Parent::OperationDataType;
    FK_STATIC_STRUCT(CircularTensorWrite, CircularTensorWrite)
    static constexpr uint num_elems_x(const Point thread, const OperationDataType& opData) { return Operation::num_elems_x(thread, opData.params.opData); }
    static constexpr uint pitch(const Point thread, const OperationDataType& opData) { return Operation::pitch(thread, opData.params.opData); }
};

namespace amd {
template <typename T> struct Lower<TensorPack<T>> {
    static constexpr bool available = true;
    using type = fkd::TensorPack<dev_t<T>>;
    static typename type::Params params(const OperationData<TensorPack<T>>& d) {
        return to_dev3<VBase<T>, const typename DevType<VBase<T>>::type>(d.params);
    }
};
template <typename T> struct Lower<TensorTPack<T>> {
    static constexpr bool available = true;
    using type = fkd::TensorTPack<dev_t<T>>;
    static typename type::Params params(const OperationData<TensorTPack<T>>& d) {
        return to_devT3<VBase<T>, const typename DevType<VBase<T>>::type>(d.params);
    }
};
template <CircularDirection direction, typename Operation, int BATCH> struct Lower<CircularBatchRead<direction, Operation, BATCH>> {
    static constexpr bool available = true;
    using type = fkd::CircularBatchRead<int(direction), BATCH, typename Lower<Operation>::type>;
    static typename type::Params params(const OperationData<CircularBatchRead<direction, Operation, BATCH>>& d) {
        typename type::Params p{};
        p.first = d.params.first;
        for (int i = 0; i < BATCH; ++i) p.plane[i] = Lower<Operation>::params(d.params.opData[i]);
        return p;
    }
};
template <CircularDirection direction, typename Operation, int BATCH> struct Lower<CircularBatchWrite<direction, Operation, BATCH>> {
    static constexpr bool available = true;
    using type = fkd::CircularBatchWrite<int(direction), BATCH, typename Lower<Operation>::type>;
    static typename type::Params params(const OperationData<CircularBatchWrite<direction, Operation, BATCH>>& d) {
        typename type::Params p{};
        p.first = d.params.first;
        for (int i = 0; i < BATCH; ++i) p.plane[i] = Lower<Operation>::params(d.params.opData[i]);
        return p;
    }
};
template <CircularDirection direction, typename Operation, int BATCH> struct Lower<CircularTensorRead<direction, Operation, BATCH>> {
    static constexpr bool available = true;
    using type = fkd::CircularRead<int(direction), BATCH, typename Lower<Operation>::type>;
    static typename type::Params params(const OperationData<CircularTensorRead<direction, Operation, BATCH>>& d) {
        return typename type::Params{d.params.first, Lower<Operation>::params(d.params.opData)};
    }
};
template <CircularDirection direction, typename Operation, int BATCH> struct Lower<CircularTensorWrite<direction, Operation, BATCH>> {
    static constexpr bool available = true;
    using type = fkd::CircularWrite<int(direction), BATCH, typename Lower<Operation>::type>;
    static typename type::Params params(const OperationData<CircularTensorWrite<direction, Operation, BATCH>>& d) {
        return typename type::Params{d.params.first, Lower<Operation>::params(d.params.opData)};
    }
};
template <typename T> struct Lower<PerThreadRead<ND::_2D, T>> {
    static constexpr bool available = true;
    using type = fkd::Read2D<dev_t<T>>;
    static typename type::Params params(const OperationData<PerThreadRead<ND::_2D, T>>& d) { return to_dev<T, const dev_t<T>>(d.params); }
};
template <typename T> struct Lower<DualSourceRead<ND::_2D, T>> {
    static constexpr bool available = true;
    using type = fkd::DualRead2D<dev_t<T>>;
    static typename type::Params params(const OperationData<DualSourceRead<ND::_2D, T>>& d) {
        return typename type::Params{to_dev<T, const dev_t<T>>(d.params.src1), to_dev<T, const dev_t<T>>(d.params.src2)};
    }
};
template <typename T> struct Lower<PerThreadRead<ND::_1D, T>> {
    static constexpr bool available = true;
    using type = fkd::Read2D<dev_t<T>>;   // a 1-D array is a one-row image
    static typename type::Params params(const OperationData<PerThreadRead<ND::_1D, T>>& d) {
        return typename type::Params{reinterpret_cast<const dev_t<T>*>(d.params.data), d.params.dims.width, 1u, d.params.dims.pitch};
    }
};
template <typename T> struct Lower<PerThreadRead<ND::_3D, T>> {
    static constexpr bool available = true;
    using type = fkd::Read3D<dev_t<T>>;
    static typename type::Params params(const OperationData<PerThreadRead<ND::_3D, T>>& d) { return to_dev3<T, const dev_t<T>>(d.params); }
};
template <typename T> struct Lower<TensorRead<T>> {
    static constexpr bool available = true;
    using type = fkd::Read3D<dev_t<T>>;
    static typename type::Params params(const OperationData<TensorRead<T>>& d) { return to_dev3<T, const dev_t<T>>(d.params); }
};
template <typename T> struct Lower<PerThreadWrite<ND::_2D, T>> {
    static constexpr bool available = true;
    using type = fkd::Write2D<dev_t<T>>;
    static typename type::Params params(const OperationData<PerThreadWrite<ND::_2D, T>>& d) { return to_dev<T, dev_t<T>>(d.params); }
};
template <typename T> struct Lower<SplitWrite<ND::_2D, T>> {
    static constexpr bool available = true;
    using B = typename DevType<VBase<T>>::type;
    using type = fkd::SplitWrite2D<dev_t<T>>;
    static typename type::Params params(const OperationData<SplitWrite<ND::_2D, T>>& d) {
        typename type::Params p{};
        p.c[0] = to_dev<VBase<T>, B>(d.params.x);
        p.c[1] = to_dev<VBase<T>, B>(d.params.y);
        if constexpr (cn<T> > 2) p.c[2] = to_dev<VBase<T>, B>(d.params.z);
        if constexpr (cn<T> > 3) p.c[3] = to_dev<VBase<T>, B>(d.params.w);
        return p;
    }
};
template <typename T> struct Lower<PerThreadWrite<ND::_1D, T>> {
    static constexpr bool available = true;
    using type = fkd::Write2D<dev_t<T>>;
    static typename type::Params params(const OperationData<PerThreadWrite<ND::_1D, T>>& d) {
        return typename type::Params{reinterpret_cast<dev_t<T>*>(d.params.data), d.params.dims.width, 1u, d.params.dims.pitch};
    }
};
template <typename T> struct Lower<PerThreadWrite<ND::_3D, T>> {
    static constexpr bool available = true;
    using type = fkd::TensorWrite<dev_t<T>>;
    static typename type::Params params(const OperationData<PerThreadWrite<ND::_3D, T>>& d) { return to_dev3<T, dev_t<T>>(d.params); }
};
template <typename T> struct Lower<TensorWrite<T>> {
    static constexpr bool available = true;
    using type = fkd::TensorWrite<dev_t<T>>;
    static typename type::Params params(const OperationData<TensorWrite<T>>& d) { return to_dev3<T, dev_t<T>>(d.params); }
};
template <typename T> struct Lower<TensorSplit<T>> {
    static constexpr bool available = true;
    using type = fkd::TensorSplit<dev_t<T>>;
    static typename type::Params params(const OperationData<TensorSplit<T>>& d) {
        return to_dev3<VBase<T>, typename DevType<VBase<T>>::type>(d.params);
    }
};
template <typename T> struct Lower<TensorTSplit<T>> {
    static constexpr bool available = true;
    using type = fkd::TensorTSplit<dev_t<T>>;
    static typename type::Params params(const OperationData<TensorTSplit<T>>& d) {
        return to_devT3<VBase<T>, typename DevType<VBase<T>>::type>(d.params);
    }
};
// PerThreadRead / PerThreadWrite on a transposed tensor address colour plane 0 only (the accessor's default), as in the
// reference (FK/core/data/rawptr.h:229-240).
template <typename T> struct Lower<PerThreadRead<ND::T3D, T>> {
    static constexpr bool available = true;
    using type = fkd::Read3D<dev_t<T>>;
    static typename type::Params params(const OperationData<PerThreadRead<ND::T3D, T>>& d) { return first_color_plane<T, const dev_t<T>>(d.params); }
};
template <typename T> struct Lower<PerThreadWrite<ND::T3D, T>> {
    static constexpr bool available = true;
    using type = fkd::TensorWrite<dev_t<T>>;
    static typename type::Params params(const OperationData<PerThreadWrite<ND::T3D, T>>& d) { return first_color_plane<T, dev_t<T>>(d.params); }
};
} // namespace amd

} // namespace fk
#endif
