// Warping<Affine|Perspective>: a read-back operation that maps every destination pixel through a transform matrix
// into the source and reads it there with bilinear interpolation; destinations that map outside the source are 0.
// Interface counterpart: FK/algorithms/image_processing/warping.h:25-146.
#ifndef FK_AMD_WARPING_H
#define FK_AMD_WARPING_H

#include <fused_kernel/algorithms/image_processing/interpolation.h>
#include <fused_kernel/core/data/rawptr.h>
#include <fused_kernel/core/data/size.h>
#include <fused_kernel/core/execution_model/operation_model/operation_model.h>
#include <fused_kernel/core/utils/vector_utils.h>

namespace fk {

enum class WarpType { Affine = 0, Perspective = 1 };

template <WarpType WType> struct WarpingParameters;
template <> struct WarpingParameters<WarpType::Affine> {
    StaticRawPtr<StaticPtrDims2D<3, 2>, float> transformMatrix;
    Size dstSize;
};
template <> struct WarpingParameters<WarpType::Perspective> {
    StaticRawPtr<StaticPtrDims2D<3, 3>, float> transformMatrix;
    Size dstSize;
};

// The coordinate part alone, as a Binary operation on a Point (kept for interface compatibility; Warping computes it
// on the device as part of the read).
template <WarpType WT> struct WarpingCoords : BinaryOperation<Point, WarpingParameters<WT>, float2, WarpingCoords<WT>> {
    using Parent = BinaryOperation<Point, WarpingParameters<WT>, float2, WarpingCoords<WT>>;
    FK_STATIC_STRUCT(WarpingCoords, WarpingCoords)
};

template <WarpType WT, typename BackIOp_ = NullType>
struct Warping : ReadBackOperation<typename BackIOp_::Operation::ReadDataType, WarpingParameters<WT>, BackIOp_,
                                   float_<cn<typename BackIOp_::Operation::ReadDataType>>, Warping<WT, BackIOp_>> {
    static_assert(isAnyCompleteReadType<BackIOp_>, "BackIOp must be a complete type for this specialization");
    using Parent = ReadBackOperation<typename BackIOp_::Operation::ReadDataType, WarpingParameters<WT>, BackIOp_,
                                     float_<cn<typename BackIOp_::Operation::ReadDataType>>, Warping<WT, BackIOp_>>;
    using typename Parent::OperationDataType;
    FK_STATIC_STRUCT(Warping, Warping)
    static constexpr uint num_elems_x(const Point, const OperationDataType& opData) { return opData.params.dstSize.width; }
    static constexpr uint num_elems_y(const Point, const OperationDataType& opData) { return opData.params.dstSize.height; }
    static constexpr uint num_elems_z(const Point, const OperationDataType&) { return 1; }
    static constexpr ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return {uint(opData.params.dstSize.width), uint(opData.params.dstSize.height), 1u};
    }
    using Parent::build;
};

template <WarpType WT>
struct Warping<WT, NullType> : IncompleteReadBackOperation<NullType, WarpingParameters<WT>, NullType, NullType, Warping<WT, NullType>> {
    using Parent = IncompleteReadBackOperation<NullType, WarpingParameters<WT>, NullType, NullType, Warping<WT, NullType>>;
    using typename Parent::OperationDataType;
    using typename Parent::InstantiableType;
    using typename Parent::ParamsType;
    FK_STATIC_STRUCT(Warping, Warping)
    static constexpr uint num_elems_x(const Point, const OperationDataType& opData) { return opData.params.dstSize.width; }
    static constexpr uint num_elems_y(const Point, const OperationDataType& opData) { return opData.params.dstSize.height; }
    static constexpr uint num_elems_z(const Point, const OperationDataType&) { return 1; }
    using Parent::build;
    static constexpr auto build(const ParamsType& params) { return InstantiableType{{params, {}}}; }
    template <typename BackIOp, std::enable_if_t<isOperation<BackIOp>, int> = 0>
    static constexpr auto build(const BackIOp& backIOp, const InstantiableType& iOp) {
        return ReadBack<Warping<WT, BackIOp>>{{iOp.params, backIOp}};
    }
};

namespace amd {
template <WarpType WT, typename BackIOp> struct Lower<Warping<WT, BackIOp>, std::enable_if_t<!std::is_same_v<BackIOp, NullType>>> {
    static constexpr bool available = true;
    using type = fkd::Warp<int(WT), device_op_t<BackIOp>>;
    static typename type::Params params(const OperationData<Warping<WT, BackIOp>>& d) {
        typename type::Params p{};
        constexpr int rows = WT == WarpType::Affine ? 2 : 3;
        for (int r = 0; r < rows; ++r)
            for (int c = 0; c < 3; ++c) p.m[r * 3 + c] = d.params.transformMatrix.data[r][c];
        p.dst_w = d.params.dstSize.width;
        p.dst_h = d.params.dstSize.height;
        p.back = lower_iop(d.backIOp);
        return p;
    }
};
} // namespace amd

} // namespace fk
#endif
