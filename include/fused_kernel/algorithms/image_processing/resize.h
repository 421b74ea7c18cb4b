// Resize: bilinear resampling of whatever read sits behind it to a destination size, optionally preserving the
// aspect ratio by letterboxing onto a background value.  Resize<IType, AR, DefaultType> is the incomplete form
// users write; fused after a read it becomes ResizeComplete<AR, Ternary<InterpolateComplete<IType, BackIOp>>>.
// Interface counterpart: FK/algorithms/image_processing/resize.h.
//
// The per-plane geometry is computed HERE, on the host, exactly as the reference does it (resize.h:164-233,
// 266-278): scale factors in double narrowed once to float, letterbox size through round-half-away-from-zero in
// float.  The kernels only consume the resulting numbers.
#ifndef FK_AMD_RESIZE_H
#define FK_AMD_RESIZE_H

#include <cmath>

#include <fused_kernel/algorithms/image_processing/interpolation.h>
#include <fused_kernel/algorithms/image_processing/saturate.h>
#include <fused_kernel/algorithms/basic_ops/memory_operations.h>

namespace fk {

enum class AspectRatio { PRESERVE_AR = 0, IGNORE_AR = 1, PRESERVE_AR_RN_EVEN = 2, PRESERVE_AR_LEFT = 3 };

template <AspectRatio AR = AspectRatio::IGNORE_AR, typename T = NullType> struct ResizeParams {
    static_assert(!std::is_same_v<T, NullType>, "DefaultType must be different than NullType");
    Size dstSize;
    float2 src_conv_factors;
    int x1, y1;   // top left of the resized image inside the destination
    int x2, y2;   // bottom right (inclusive)
    T defaultValue;
};
template <typename T> struct ResizeParams<AspectRatio::IGNORE_AR, T> {
    Size dstSize;
    float2 src_conv_factors;
};

template <AspectRatio AR, typename T = NullType> struct IncompleteResizeParams {
    Size dstSize;
    T defaultValue;
};
template <typename T> struct IncompleteResizeParams<AspectRatio::IGNORE_AR, T> {
    Size dstSize;
};

struct NumElems {
    template <typename IOp> static constexpr Size size(const Point thread, const IOp& iOp) {
        return Size(int(IOp::Operation::num_elems_x(thread, iOp)), int(IOp::Operation::num_elems_y(thread, iOp)));
    }
};

template <AspectRatio AR, typename BackIOp_>
struct ResizeComplete : ReadBackOperation<typename BackIOp_::Operation::OutputType,
                                          ResizeParams<AR, float_<cn<typename BackIOp_::Operation::OutputType>>>, BackIOp_,
                                          float_<cn<typename BackIOp_::Operation::OutputType>>, ResizeComplete<AR, BackIOp_>> {
    static_assert(opIs<TernaryType, BackIOp_>, "BackIOp must be a ternary type for this specialization");
    using DefaultType = float_<cn<typename BackIOp_::Operation::OutputType>>;
    using Parent = ReadBackOperation<typename BackIOp_::Operation::OutputType, ResizeParams<AR, DefaultType>, BackIOp_,
                                     DefaultType, ResizeComplete<AR, BackIOp_>>;
    using typename Parent::OperationDataType;
    FK_STATIC_STRUCT(ResizeComplete, ResizeComplete)
    static constexpr uint num_elems_x(const Point, const OperationDataType& opData) { return opData.params.dstSize.width; }
    static constexpr uint num_elems_y(const Point, const OperationDataType& opData) { return opData.params.dstSize.height; }
    static constexpr uint num_elems_z(const Point, const OperationDataType&) { return 1; }
    static constexpr ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return {uint(opData.params.dstSize.width), uint(opData.params.dstSize.height), 1u};
    }
};

namespace resize_detail {
// cxp::round of the reference is std::round (half away from zero); written out so that build() stays constexpr.
// The operands here are letterbox sizes: non-negative and far below 2^23.
constexpr int round_to_int(float v) {
    const float a = v < 0.f ? -v : v;
    const int t = static_cast<int>(a);
    const int r = (a - static_cast<float>(t)) >= 0.5f ? t + 1 : t;
    return v < 0.f ? -r : r;
}

template <AspectRatio AR> constexpr Size target_size(const Size& srcSize, const Size& dstSize) {
    const float scaleFactor = dstSize.height / (float)srcSize.height;
    const int targetHeight = dstSize.height;
    const int targetWidth = round_to_int(scaleFactor * srcSize.width);
    if constexpr (AR == AspectRatio::PRESERVE_AR_RN_EVEN) {
        const int evenWidth = targetWidth - (targetWidth % 2);
        if (evenWidth > dstSize.width) {
            const float scaleW = dstSize.width / (float)srcSize.width;
            const int h = round_to_int(scaleW * srcSize.height);
            return Size(dstSize.width, h - (h % 2));
        }
        return Size(evenWidth, targetHeight);
    } else {
        if (targetWidth > dstSize.width) {
            const float scaleW = dstSize.width / (float)srcSize.width;
            return Size(dstSize.width, round_to_int(scaleW * srcSize.height));
        }
        return Size(targetWidth, targetHeight);
    }
}
} // namespace resize_detail

template <InterpolationType IType = InterpolationType::INTER_LINEAR, AspectRatio AR = AspectRatio::IGNORE_AR, typename DefaultType = NullType>
struct Resize : IncompleteReadBackOperation<NullType, IncompleteResizeParams<AR, DefaultType>, NullType, NullType, Resize<IType, AR, DefaultType>> {
    using Parent = IncompleteReadBackOperation<NullType, IncompleteResizeParams<AR, DefaultType>, NullType, NullType, Resize<IType, AR, DefaultType>>;
    using typename Parent::OperationDataType;
    using typename Parent::InstantiableType;
    FK_STATIC_STRUCT(Resize, Resize)
    template <typename BackIOp_> using NewInstantiableType = ResizeComplete<AR, Ternary<InterpolateComplete<IType, BackIOp_>>>;

    static constexpr uint num_elems_x(const Point, const OperationDataType& opData) { return opData.params.dstSize.width; }
    static constexpr uint num_elems_y(const Point, const OperationDataType& opData) { return opData.params.dstSize.height; }
    static constexpr uint num_elems_z(const Point, const OperationDataType&) { return 1; }

    using Parent::build;

    // Resize<..., AR>::build(dstSize, background): the incomplete IOp users write.
    template <typename DefaultType_, std::enable_if_t<!isOperation<DefaultType_>, int> = 0>
    static constexpr auto build(const Size& dstSize, const DefaultType_& backgroundValue) {
        return Resize<IType, AR, DefaultType_>::build(IncompleteResizeParams<AR, DefaultType_>{dstSize, backgroundValue}, NullType{});
    }

    // Completion against the read behind it.
    template <typename NewBackIOp, std::enable_if_t<isOperation<NewBackIOp>, int> = 0>
    static constexpr auto build(const NewBackIOp& backIOp, const InstantiableType& iOp) {
        static_assert(isCompleteOperation<NewBackIOp>, "NewBackIOp must be a complete IOp");
        using NewDefaultType = float_<cn<typename NewBackIOp::Operation::OutputType>>;
        static_assert(std::is_same_v<NewDefaultType, DefaultType>, "Default value type and Op::OutputType must be the same.");
        return build(backIOp, iOp.params.dstSize, iOp.params.defaultValue);
    }

    template <typename NewBackIOp, std::enable_if_t<isOperation<NewBackIOp>, int> = 0>
    static constexpr auto build(const NewBackIOp& backIOp, const Size& dstSize,
                                const VectorType_t<float, cn<typename NewBackIOp::Operation::OutputType>>& backgroundValue) {
        static_assert(isCompleteOperation<NewBackIOp>, "NewBackIOp must be a complete IOp");
        const Size srcSize = NumElems::size(Point{0, 0, 0}, backIOp);
        const Size targetSize = resize_detail::target_size<AR>(srcSize, dstSize);
        const double cfx = static_cast<double>(targetSize.width) / srcSize.width;
        const double cfy = static_cast<double>(targetSize.height) / srcSize.height;
        using NewOutputType = float_<cn<typename NewBackIOp::Operation::OutputType>>;
        const int x1 = AR == AspectRatio::PRESERVE_AR_LEFT ? 0 : static_cast<int>((dstSize.width - targetSize.width) / 2);
        const int y1 = static_cast<int>((dstSize.height - targetSize.height) / 2);
        const ResizeParams<AR, NewOutputType> resizeParams{dstSize,
                                                           {static_cast<float>(1.0 / cfx), static_cast<float>(1.0 / cfy)},
                                                           x1, y1, x1 + targetSize.width - 1, y1 + targetSize.height - 1,
                                                           backgroundValue};
        return NewInstantiableType<NewBackIOp>::build(resizeParams, Interpolate<IType>::build(backIOp));
    }
};

template <> struct Resize<InterpolationType::INTER_LINEAR, AspectRatio::IGNORE_AR, NullType>
    : IncompleteReadBackOperation<NullType, IncompleteResizeParams<AspectRatio::IGNORE_AR>, NullType, NullType,
                                  Resize<InterpolationType::INTER_LINEAR, AspectRatio::IGNORE_AR, NullType>> {
    using Parent = IncompleteReadBackOperation<NullType, IncompleteResizeParams<AspectRatio::IGNORE_AR>, NullType, NullType,
                                               Resize<InterpolationType::INTER_LINEAR, AspectRatio::IGNORE_AR, NullType>>;
    static constexpr InterpolationType IType{InterpolationType::INTER_LINEAR};
    FK_STATIC_STRUCT(Resize, Resize)
    template <typename NewBackIOp>
    using NewInstantiableType = ResizeComplete<AspectRatio::IGNORE_AR, Ternary<InterpolateComplete<InterpolationType::INTER_LINEAR, NewBackIOp>>>;

    static constexpr uint num_elems_x(const Point, const OperationDataType& opData) { return opData.params.dstSize.width; }
    static constexpr uint num_elems_y(const Point, const OperationDataType& opData) { return opData.params.dstSize.height; }
    static constexpr uint num_elems_z(const Point, const OperationDataType&) { return 1; }

    using Parent::build;
    static constexpr auto build(const Size& dstSize) { return InstantiableType{{ParamsType{dstSize}, BackIOp{}}}; }

    template <typename NewBackIOp, std::enable_if_t<isOperation<NewBackIOp>, int> = 0>
    static constexpr auto build(const NewBackIOp& backIOp, const Size& dstSize) {
        static_assert(isCompleteOperation<NewBackIOp>, "NewBackIOp must be a complete IOp");
        const Size srcSize = NumElems::size(Point{0, 0, 0}, backIOp);
        const double cfx = static_cast<double>(dstSize.width) / static_cast<double>(srcSize.width);
        const double cfy = static_cast<double>(dstSize.height) / static_cast<double>(srcSize.height);
        const typename NewInstantiableType<NewBackIOp>::ParamsType resizeParams{
            dstSize, {static_cast<float>(1.0 / cfx), static_cast<float>(1.0 / cfy)}};
        return NewInstantiableType<NewBackIOp>::build(resizeParams, Interpolate<IType>::build(backIOp));
    }

    template <typename NewBackIOp, std::enable_if_t<isOperation<NewBackIOp>, int> = 0>
    static constexpr auto build(const NewBackIOp& backIOp, const InstantiableType& selfIOp) {
        return build(backIOp, selfIOp.params.dstSize);
    }

    // Resize straight from a pointer: destination size, or scale factors when the size is empty.
    template <typename T>
    static auto build(const RawPtr<ND::_2D, T>& input, const Size& dSize, const double& fx, const double& fy) {
        const auto readIOp = PerThreadRead<ND::_2D, T>::build(input);
        if (dSize.width != 0 && dSize.height != 0) return build(readIOp, dSize);
        const Size computed{static_cast<int>(std::nearbyint(input.dims.width * fx)), static_cast<int>(std::nearbyint(input.dims.height * fy))};
        return build(readIOp, computed);
    }
};

namespace amd {
template <AspectRatio AR, InterpolationType IT, typename BackIOp>
struct Lower<ResizeComplete<AR, Ternary<InterpolateComplete<IT, BackIOp>>>> {
    static_assert(IT == InterpolationType::INTER_LINEAR);
    static constexpr bool available = true;
    using Self = ResizeComplete<AR, Ternary<InterpolateComplete<IT, BackIOp>>>;
    using type = fkd::ResizeLinear<(AR == AspectRatio::IGNORE_AR ? fkd::IGNORE_AR : fkd::PRESERVE_AR), device_op_t<BackIOp>>;
    static typename type::Params params(const OperationData<Self>& d) {
        // (one aggregate initialisation, the back operation's parameters built in place: this runs once per plane of a batch)
        const int dw = d.params.dstSize.width, dh = d.params.dstSize.height;
        const float fx = d.params.src_conv_factors.x, fy = d.params.src_conv_factors.y;
        if constexpr (AR == AspectRatio::IGNORE_AR) {
            return typename type::Params{dw, dh, fx, fy, 0, 0, dw - 1, dh - 1, typename type::Out{}, type::whole_factors(dw, dh, fx, fy),
                                         lower_iop(d.backIOp.backIOp)};
        } else {
            return typename type::Params{dw, dh, fx, fy, d.params.x1, d.params.y1, d.params.x2, d.params.y2, to_dev(d.params.defaultValue),
                                         type::whole_factors(dw, dh, fx, fy), lower_iop(d.backIOp.backIOp)};
        }
    }
};
} // namespace amd

} // namespace fk
#endif
