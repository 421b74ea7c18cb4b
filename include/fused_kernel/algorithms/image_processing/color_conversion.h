// Colour operations of the fused path: channel swaps (ColorConversion<COLOR_BGR2RGB, ...> and friends), the NV12
// reader ReadYUV<PixelFormat::NV12> and ConvertYUVToRGB<p8bit, Full, bt709>.
// Interface counterpart: FK/algorithms/image_processing/color_conversion.h:150-174, 206-238, 408-505.
// Conversions outside that set (alpha insertion/removal, gray, other pixel formats / ranges / primaries) have no
// gfx950 kernel yet and fail at compile time with a message that says so.
#ifndef FK_AMD_COLOR_CONVERSION_H
#define FK_AMD_COLOR_CONVERSION_H

#include <fused_kernel/core/execution_model/operation_model/operation_model.h>
#include <fused_kernel/algorithms/basic_ops/vector_ops.h>
#include <fused_kernel/algorithms/image_processing/raw_image.h>
#include <fused_kernel/algorithms/image_processing/saturate.h>

namespace fk {

template <PixelFormat PF> class Image;

template <ColorDepth CD, ColorRange CR, ColorPrimitives CP>
struct ConvertYUVToRGB : UnaryOperation<ColorDepthPixelType<CD>, float3, ConvertYUVToRGB<CD, CR, CP>> {
    using Parent = UnaryOperation<ColorDepthPixelType<CD>, float3, ConvertYUVToRGB<CD, CR, CP>>;
    FK_STATIC_STRUCT(ConvertYUVToRGB, ConvertYUVToRGB)
};

// Direct chroma replication, no chroma interpolation.
template <PixelFormat PF>
struct ReadYUV : ReadOperation<ColorDepthPixelBaseType<PixelFormatTraits<PF>::depth>, RawImage<PF>,
                               ColorDepthPixelType<PixelFormatTraits<PF>::depth>, TF::DISABLED, ReadYUV<PF>> {
    using PixelBaseType = ColorDepthPixelBaseType<PixelFormatTraits<PF>::depth>;
    using Parent = ReadOperation<PixelBaseType, RawImage<PF>, ColorDepthPixelType<PixelFormatTraits<PF>::depth>, TF::DISABLED, ReadYUV<PF>>;
    using typename Parent::OperationDataType;
    using typename Parent::InstantiableType;
    FK_STATIC_STRUCT(ReadYUV, ReadYUV)
    static constexpr uint num_elems_x(const Point, const OperationDataType& opData) { return opData.params.width; }
    static constexpr uint num_elems_y(const Point, const OperationDataType& opData) { return opData.params.height; }
    static constexpr uint num_elems_z(const Point, const OperationDataType&) { return 1; }
    static constexpr uint pitch(const Point, const OperationDataType& opData) { return opData.params.data.dims.pitch; }
    static constexpr ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return {opData.params.width, opData.params.height, 1u};
    }
    using Parent::build;
    static InstantiableType build(const Image<PF>& data) { return {{data.ptr()}}; }
};

enum class ColorConversionCodes {
    COLOR_BGR2BGRA = 0, COLOR_RGB2RGBA = 0,
    COLOR_BGRA2BGR = 1, COLOR_RGBA2RGB = 1,
    COLOR_BGR2RGBA = 2, COLOR_RGB2BGRA = 2,
    COLOR_RGBA2BGR = 3, COLOR_BGRA2RGB = 3,
    COLOR_BGR2RGB = 4, COLOR_RGB2BGR = 4,
    COLOR_BGRA2RGBA = 5, COLOR_RGBA2BGRA = 5,
    COLOR_BGR2GRAY = 6, COLOR_RGB2GRAY = 7,
    COLOR_BGRA2GRAY = 10, COLOR_RGBA2GRAY = 11
};

template <ColorConversionCodes CODE, typename I, typename O, ColorDepth CD = ColorDepth::p8bit> struct ColorConversionType {
    static_assert(CODE == ColorConversionCodes::COLOR_BGR2RGB || CODE == ColorConversionCodes::COLOR_BGRA2RGBA,
                  "this colour conversion code has no MI355X kernel yet: only the channel swaps BGR<->RGB and BGRA<->RGBA are built");
};
template <typename I, typename O, ColorDepth CD> struct ColorConversionType<ColorConversionCodes::COLOR_BGR2RGB, I, O, CD> {
    using type = VectorReorder<I, 2, 1, 0>;
};
template <typename I, typename O, ColorDepth CD> struct ColorConversionType<ColorConversionCodes::COLOR_BGRA2RGBA, I, O, CD> {
    using type = VectorReorder<I, 2, 1, 0, 3>;
};
template <ColorConversionCodes code, typename I, typename O, ColorDepth CD = ColorDepth::p8bit>
using ColorConversion = typename ColorConversionType<code, I, O, CD>::type;

namespace amd {
template <> struct Lower<ReadYUV<PixelFormat::NV12>> {
    static constexpr bool available = true;
    using type = fkd::ReadNV12;
    static type::Params params(const OperationData<ReadYUV<PixelFormat::NV12>>& d) {
        return fkd::RawNV12{d.params.data.data, d.params.width, d.params.height, d.params.data.dims.pitch};
    }
};
template <> struct Lower<ConvertYUVToRGB<ColorDepth::p8bit, ColorRange::Full, ColorPrimitives::bt709>> {
    static constexpr bool available = true;
    using type = fkd::YUV2RGB709Full8;
    static type::Params params(const OperationData<ConvertYUVToRGB<ColorDepth::p8bit, ColorRange::Full, ColorPrimitives::bt709>>&) { return {}; }
};
} // namespace amd

} // namespace fk
#endif
