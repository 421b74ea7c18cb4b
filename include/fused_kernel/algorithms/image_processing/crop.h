// Crop: a read-back operation that shifts the coordinates it forwards to the operation behind it by the origin of
// a rectangle and reports the rectangle's extent as its size.  Crop<> (no back operation yet) is the
// incomplete form users write; fusing it after a read gives Crop<BackIOp>.
// Interface counterpart: FK/algorithms/image_processing/crop.h.
#ifndef FK_AMD_CROP_H
#define FK_AMD_CROP_H

#include <fused_kernel/core/execution_model/operation_model/operation_model.h>
#include <fused_kernel/core/data/rect.h>

namespace fk {

template <typename BackIOp_ = NullType>
struct Crop : ReadBackOperation<typename BackIOp_::Operation::OutputType, Rect, BackIOp_,
                                typename BackIOp_::Operation::OutputType, Crop<BackIOp_>> {
    static_assert(isAnyCompleteReadType<BackIOp_>, "The BackIOp_ must be a complete Read type");
    using Parent = ReadBackOperation<typename BackIOp_::Operation::OutputType, Rect, BackIOp_,
                                     typename BackIOp_::Operation::OutputType, Crop<BackIOp_>>;
    using typename Parent::OperationDataType;
    using typename Parent::InstantiableType;
    using typename Parent::BackIOp;
    FK_STATIC_STRUCT(Crop, Crop)
    static constexpr uint num_elems_x(const Point, const OperationDataType& opData) { return opData.params.width; }
    static constexpr uint num_elems_y(const Point, const OperationDataType& opData) { return opData.params.height; }
    static constexpr uint num_elems_z(const Point, const OperationDataType&) { return 1; }
    static constexpr ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return {uint(opData.params.width), uint(opData.params.height), 1u};
    }
    using Parent::build;
    static constexpr InstantiableType build(const BackIOp& backIOp, const Rect& rect) { return InstantiableType{{rect, backIOp}}; }
};

template <> struct Crop<NullType> : IncompleteReadBackOperation<NullType, Rect, NullType, NullType, Crop<NullType>> {
    using Parent = IncompleteReadBackOperation<NullType, Rect, NullType, NullType, Crop<NullType>>;
    FK_STATIC_STRUCT(Crop, Crop)
    static constexpr uint num_elems_x(const Point, const OperationDataType& opData) { return opData.params.width; }
    static constexpr uint num_elems_y(const Point, const OperationDataType& opData) { return opData.params.height; }
    static constexpr uint num_elems_z(const Point, const OperationDataType&) { return 1; }
    using Parent::build;
    static constexpr auto build(const Rect& rectCrop) { return InstantiableType{{rectCrop, NullType{}}}; }
    template <typename BackIOp, std::enable_if_t<isOperation<BackIOp>, int> = 0>
    static constexpr auto build(const BackIOp& bIOp, const InstantiableType& iOp) { return Crop<BackIOp>::build(bIOp, iOp.params); }
};

namespace amd {
template <typename BackIOp> struct Lower<Crop<BackIOp>, std::enable_if_t<!std::is_same_v<BackIOp, NullType>>> {
    static constexpr bool available = true;
    using type = fkd::Crop<device_op_t<BackIOp>>;
    static typename type::Params params(const OperationData<Crop<BackIOp>>& d) {
        return typename type::Params{int(d.params.x), int(d.params.y), int(d.params.width), int(d.params.height), lower_iop(d.backIOp)};
    }
};
} // namespace amd

} // namespace fk
#endif
