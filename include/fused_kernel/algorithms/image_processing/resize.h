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

// Size of the resized image on a canvas when the aspect ratio is kept: the source is fitted to the canvas height, and to
// the canvas width instead if that comes out wider than the canvas.  Scale factors and products are single precision, the
// rounding is half away from zero; PRESERVE_AR_RN_EVEN then takes the even number at or below the rounded side.
template <AspectRatio AR> constexpr Size target_size(const Size& source, const Size& canvas) {
    constexpr bool kEven = AR == AspectRatio::PRESERVE_AR_RN_EVEN;
    auto even_floor = [](int v) { return kEven ? v - (v % 2) : v; };
    // the free side of an image scaled so that `fitted` source pixels become `to` output pixels
    auto free_side = [](int to, int fitted, int other) { return round_to_int((to / static_cast<float>(fitted)) * other); };
    const int width_by_height = even_floor(free_side(canvas.height, source.height, source.width));
    if (width_by_height <= canvas.width) return Size(width_by_height, canvas.height);
    return Size(canvas.width, even_floor(free_side(canvas.width, source.width, source.height)));
}

// How far the source advances per output pixel along one axis: the single-precision value of 1 / (outputs / inputs),
// both divisions in double, which is the rounding the device's coordinates are checked against.
constexpr float source_step(int outputs, int inputs) {
    const double enlargement = static_cast<double>(outputs) / static_cast<double>(inputs);
    return static_cast<float>(1.0 / enlargement);
}

// Where the resized image sits on the output canvas: its size under the aspect-ratio mode and its first column and row
// (centred, halves truncated; PRESERVE_AR_LEFT pins it to column 0).
struct Letterbox {
    Size image;
    int left, top;
    constexpr int right() const { return left + image.width - 1; }
    constexpr int bottom() const { return top + image.height - 1; }
};
template <AspectRatio AR> constexpr Letterbox place_on_canvas(const Size& source, const Size& canvas) {
    const Size image = target_size<AR>(source, canvas);
    const int left = AR == AspectRatio::PRESERVE_AR_LEFT ? 0 : (canvas.width - image.width) / 2;
    return Letterbox{image, left, (canvas.height - image.height) / 2};
}

// The extent of whatever a complete read IOp delivers.
template <typename ReadIOp> constexpr Size extent_of(const ReadIOp& read) {
    static_assert(isCompleteOperation<ReadIOp>, "a Resize can only be completed against a complete read IOp (one that knows its source)");
    return NumElems::size(Point{0, 0, 0}, read);
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

    // Completion of the incomplete IOp against the read it was fused onto.
    template <typename SourceIOp, std::enable_if_t<isOperation<SourceIOp>, int> = 0>
    static constexpr auto build(const SourceIOp& source, const InstantiableType& pending) {
        static_assert(std::is_same_v<float_<cn<typename SourceIOp::Operation::OutputType>>, DefaultType>,
                      "the background value of a letterboxing Resize must be the float vector with the channel count of the pixels it reads");
        return build(source, pending.params.dstSize, pending.params.defaultValue);
    }

    // Complete in one call: the letterbox is placed on the canvas, the band around it takes the background value.
    template <typename SourceIOp, std::enable_if_t<isOperation<SourceIOp>, int> = 0>
    static constexpr auto build(const SourceIOp& source, const Size& canvas,
                                const VectorType_t<float, cn<typename SourceIOp::Operation::OutputType>>& background) {
        using Pixel = float_<cn<typename SourceIOp::Operation::OutputType>>;
        const Size from = resize_detail::extent_of(source);
        const resize_detail::Letterbox box = resize_detail::place_on_canvas<AR>(from, canvas);
        return NewInstantiableType<SourceIOp>::build(
            ResizeParams<AR, Pixel>{canvas,
                                    {resize_detail::source_step(box.image.width, from.width), resize_detail::source_step(box.image.height, from.height)},
                                    box.left, box.top, box.right(), box.bottom(), background},
            Interpolate<IType>::build(source));
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

    // The whole source stretched over the whole output.
    template <typename SourceIOp, std::enable_if_t<isOperation<SourceIOp>, int> = 0>
    static constexpr auto build(const SourceIOp& source, const Size& outputSize) {
        const Size from = resize_detail::extent_of(source);
        using Completed = NewInstantiableType<SourceIOp>;
        return Completed::build(
            typename Completed::ParamsType{outputSize, {resize_detail::source_step(outputSize.width, from.width),
                                                        resize_detail::source_step(outputSize.height, from.height)}},
            Interpolate<IType>::build(source));
    }

    template <typename SourceIOp, std::enable_if_t<isOperation<SourceIOp>, int> = 0>
    static constexpr auto build(const SourceIOp& source, const InstantiableType& pending) {
        return build(source, pending.params.dstSize);
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
