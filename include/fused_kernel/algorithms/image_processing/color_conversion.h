// Colour operations of the fused path: channel swaps, alpha insertion/removal and gray (ColorConversion<code, ...>),
// the pixel-format readers and writers ReadYUV<PF> / WriteYUV<PF>, the YCbCr<->RGB conversions for every depth, range
// and set of primaries, NormalizePixel, SaturateDepth, DenormalizePixel and SaturateDenormalizePixel.
// Interface counterpart: FK/algorithms/image_processing/color_conversion.h:28-201, 206-389, 391-505.
// Pixel formats the reference declares but gives no reader/writer (YV12, P016, P216, Y216), or whose reader does not
// compile there (Y416: four values into a three-channel pixel), fail at compile time here with a message that says so.
#ifndef FK_AMD_COLOR_CONVERSION_H
#define FK_AMD_COLOR_CONVERSION_H

#include <fused_kernel/core/execution_model/operation_model/operation_model.h>
#include <fused_kernel/algorithms/basic_ops/vector_ops.h>
#include <fused_kernel/algorithms/image_processing/raw_image.h>
#include <fused_kernel/algorithms/image_processing/saturate.h>

namespace fk {

template <PixelFormat PF> class Image;

template <typename I> using VOneMore = VectorType_t<VBase<I>, (cn<I> + 1)>;

// input + one more channel holding the compile-time value `alpha`.
template <typename I, VBase<I> alpha> struct StaticAddAlpha : UnaryOperation<I, VOneMore<I>, StaticAddAlpha<I, alpha>> {
    using Parent = UnaryOperation<I, VOneMore<I>, StaticAddAlpha<I, alpha>>;
    FK_STATIC_STRUCT(StaticAddAlpha, StaticAddAlpha)
};

enum class GrayFormula { CCIR_601 };

// 0.299*R + 0.587*G + 0.114*B rounded to the nearest integer, ties to even (float outputs too, as in the reference).
// A fourth input channel is ignored.
template <typename I, typename O = VBase<I>, GrayFormula GF = GrayFormula::CCIR_601>
struct RGB2Gray : UnaryOperation<I, O, RGB2Gray<I, O, GF>> {
    using Parent = UnaryOperation<I, O, RGB2Gray<I, O, GF>>;
    FK_STATIC_STRUCT(RGB2Gray, RGB2Gray)
};

// input + one more channel holding the largest value of the depth.
template <typename I, ColorDepth CD> struct AddOpaqueAlpha : UnaryOperation<I, VOneMore<I>, AddOpaqueAlpha<I, CD>> {
    using Parent = UnaryOperation<I, VOneMore<I>, AddOpaqueAlpha<I, CD>>;
    FK_STATIC_STRUCT(AddOpaqueAlpha, AddOpaqueAlpha)
};

// input / largest value of the depth, per channel, as float.
template <typename I, ColorDepth CD> struct NormalizePixel : UnaryOperation<I, VectorType_t<float, cn<I>>, NormalizePixel<I, CD>> {
    using Parent = UnaryOperation<I, VectorType_t<float, cn<I>>, NormalizePixel<I, CD>>;
    FK_STATIC_STRUCT(NormalizePixel, NormalizePixel)
};

// Every channel clamped to [0, largest value of the depth].  The reference spells this for T = float only (its body calls
// Saturate<float>); vectors of float work the same way here.
template <typename T, ColorDepth CD> struct SaturateDepth : UnaryOperation<T, T, SaturateDepth<T, CD>> {
    using Parent = UnaryOperation<T, T, SaturateDepth<T, CD>>;
    FK_STATIC_STRUCT(SaturateDepth, SaturateDepth)
    static_assert(std::is_same_v<VBase<T>, float>, "SaturateDepth works on float channels");
};

// float channels * largest value of the depth, converted to O's channel type like a C cast (towards zero).
template <typename O, ColorDepth CD> struct DenormalizePixel : UnaryOperation<VectorType_t<float, cn<O>>, O, DenormalizePixel<O, CD>> {
    using Parent = UnaryOperation<VectorType_t<float, cn<O>>, O, DenormalizePixel<O, CD>>;
    FK_STATIC_STRUCT(DenormalizePixel, DenormalizePixel)
};

// SaturateFloat (clamp to [0, 1], NaN -> 1), then DenormalizePixel.
template <typename I, typename O, ColorDepth CD> struct SaturateDenormalizePixel : UnaryOperation<I, O, SaturateDenormalizePixel<I, O, CD>> {
    using Parent = UnaryOperation<I, O, SaturateDenormalizePixel<I, O, CD>>;
    FK_STATIC_STRUCT(SaturateDenormalizePixel, SaturateDenormalizePixel)
    static_assert(std::is_same_v<VBase<I>, float>, "SaturateDenormalizePixel only works with float base types.");
};

// (Y, Cb, Cr) -> float3 (R, G, B); no clamp.
template <ColorDepth CD, ColorRange CR, ColorPrimitives CP>
struct ConvertYUVToRGB : UnaryOperation<ColorDepthPixelType<CD>, float3, ConvertYUVToRGB<CD, CR, CP>> {
    using Parent = UnaryOperation<ColorDepthPixelType<CD>, float3, ConvertYUVToRGB<CD, CR, CP>>;
    FK_STATIC_STRUCT(ConvertYUVToRGB, ConvertYUVToRGB)
};

// (R, G, B) -> float3 (Y, Cb, Cr); no rounding, no clamp.
template <ColorDepth CD, ColorRange CR, ColorPrimitives CP>
struct ConvertRGBToYUV : UnaryOperation<ColorDepthPixelType<CD>, float3, ConvertRGBToYUV<CD, CR, CP>> {
    using Parent = UnaryOperation<ColorDepthPixelType<CD>, float3, ConvertRGBToYUV<CD, CR, CP>>;
    FK_STATIC_STRUCT(ConvertRGBToYUV, ConvertRGBToYUV)
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

// Takes (Y, U, V); chroma is stored from one pixel of each chroma block, with no averaging.
template <PixelFormat PF>
struct WriteYUV : WriteOperation<ColorDepthPixelType<PixelFormatTraits<PF>::depth>, RawImage<PF>,
                                 ColorDepthPixelBaseType<PixelFormatTraits<PF>::depth>, TF::DISABLED, WriteYUV<PF>> {
    using PixelBaseType = ColorDepthPixelBaseType<PixelFormatTraits<PF>::depth>;
    using Parent = WriteOperation<ColorDepthPixelType<PixelFormatTraits<PF>::depth>, RawImage<PF>, PixelBaseType, TF::DISABLED, WriteYUV<PF>>;
    using typename Parent::OperationDataType;
    using typename Parent::InstantiableType;
    FK_STATIC_STRUCT(WriteYUV, WriteYUV)
    static constexpr uint num_elems_x(const Point, const OperationDataType& opData) { return opData.params.width; }
    static constexpr uint num_elems_y(const Point, const OperationDataType& opData) { return opData.params.height; }
    static constexpr uint num_elems_z(const Point, const OperationDataType&) { return 1; }
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
    static_assert(sizeof(I) == 0, "Color conversion code not supported");
};
template <typename I, typename O, ColorDepth CD> struct ColorConversionType<ColorConversionCodes::COLOR_BGR2BGRA, I, O, CD> {
    using type = AddOpaqueAlpha<I, CD>;
};
template <typename I, typename O, ColorDepth CD> struct ColorConversionType<ColorConversionCodes::COLOR_BGRA2BGR, I, O, CD> {
    using type = Discard<I, VectorType_t<VBase<I>, 3>>;
};
template <typename I, typename O, ColorDepth CD> struct ColorConversionType<ColorConversionCodes::COLOR_BGR2RGBA, I, O, CD> {
    using type = FusedOperation<Unary<VectorReorder<I, 2, 1, 0>>, Unary<AddOpaqueAlpha<I, CD>>>;
};
template <typename I, typename O, ColorDepth CD> struct ColorConversionType<ColorConversionCodes::COLOR_BGRA2RGB, I, O, CD> {
    using type = FusedOperation<Unary<VectorReorder<I, 2, 1, 0, 3>>, Unary<Discard<I, VectorType_t<VBase<I>, 3>>>>;
};
template <typename I, typename O, ColorDepth CD> struct ColorConversionType<ColorConversionCodes::COLOR_BGR2RGB, I, O, CD> {
    using type = VectorReorder<I, 2, 1, 0>;
};
template <typename I, typename O, ColorDepth CD> struct ColorConversionType<ColorConversionCodes::COLOR_BGRA2RGBA, I, O, CD> {
    using type = VectorReorder<I, 2, 1, 0, 3>;
};
template <typename I, typename O, ColorDepth CD> struct ColorConversionType<ColorConversionCodes::COLOR_RGB2GRAY, I, O, CD> {
    using type = RGB2Gray<I, O>;
};
template <typename I, typename O, ColorDepth CD> struct ColorConversionType<ColorConversionCodes::COLOR_BGR2GRAY, I, O, CD> {
    using type = FusedOperation<Unary<VectorReorder<I, 2, 1, 0>>, Unary<RGB2Gray<I, O>>>;
};
template <typename I, typename O, ColorDepth CD> struct ColorConversionType<ColorConversionCodes::COLOR_RGBA2GRAY, I, O, CD> {
    using type = RGB2Gray<I, O>;
};
template <typename I, typename O, ColorDepth CD> struct ColorConversionType<ColorConversionCodes::COLOR_BGRA2GRAY, I, O, CD> {
    using type = FusedOperation<Unary<VectorReorder<I, 2, 1, 0, 3>>, Unary<RGB2Gray<I, O>>>;
};
template <ColorConversionCodes code, typename I, typename O, ColorDepth CD = ColorDepth::p8bit>
using ColorConversion = typename ColorConversionType<code, I, O, CD>::type;

namespace amd {
template <PixelFormat PF> constexpr bool nv_format = PF == PixelFormat::NV12 || PF == PixelFormat::NV21;
template <PixelFormat PF> constexpr bool read_write_format = nv_format<PF> || PF == PixelFormat::P010 || PF == PixelFormat::P210 ||
                                                             PF == PixelFormat::Y210 || PF == PixelFormat::UYVY;
// NV12 and NV21 have their own reader (it also feeds the bilinear gather kernel); the other formats share one.
template <PixelFormat PF> struct Lower<ReadYUV<PF>> {
    static_assert(read_write_format<PF>, "ReadYUV: the reference has no (working) reader for this pixel format, and neither has this library");
    static constexpr bool available = true;
    using type = std::conditional_t<nv_format<PF>, fkd::ReadNV<PF == PixelFormat::NV21>, fkd::ReadYUV<int(PF)>>;
    static typename type::Params params(const OperationData<ReadYUV<PF>>& d) {
        return fkd::RawYUV{reinterpret_cast<const fkd::u8*>(d.params.data.data), d.params.width, d.params.height, d.params.data.dims.pitch};
    }
};
template <PixelFormat PF> struct Lower<WriteYUV<PF>> {
    static_assert(read_write_format<PF>, "WriteYUV: the reference has no (working) writer for this pixel format, and neither has this library");
    static constexpr bool available = true;
    using type = fkd::WriteYUV<int(PF)>;
    static typename type::Params params(const OperationData<WriteYUV<PF>>& d) {
        return fkd::RawYUVOut{reinterpret_cast<fkd::u8*>(d.params.data.data), d.params.width, d.params.height, d.params.data.dims.pitch};
    }
};
template <ColorDepth CD, ColorRange CR, ColorPrimitives CP> struct Lower<ConvertYUVToRGB<CD, CR, CP>> {
    static constexpr bool available = true;
    using type = fkd::YUV2RGB<int(CD), int(CR), int(CP)>;
    static typename type::Params params(const OperationData<ConvertYUVToRGB<CD, CR, CP>>&) { return {}; }
};
template <ColorDepth CD, ColorRange CR, ColorPrimitives CP> struct Lower<ConvertRGBToYUV<CD, CR, CP>> {
    static constexpr bool available = true;
    using type = fkd::RGB2YUV<int(CD), int(CR), int(CP)>;
    static typename type::Params params(const OperationData<ConvertRGBToYUV<CD, CR, CP>>&) { return {}; }
};
template <typename I, typename O, GrayFormula GF> struct Lower<RGB2Gray<I, O, GF>> {
    static constexpr bool available = true;
    using type = fkd::RGB2Gray<dev_t<I>, dev_t<O>>;
    static typename type::Params params(const OperationData<RGB2Gray<I, O, GF>>&) { return {}; }
};
template <typename I, ColorDepth CD> struct Lower<AddOpaqueAlpha<I, CD>> {
    static constexpr bool available = true;
    using type = fkd::AddLast<dev_t<I>>;
    static typename type::Params params(const OperationData<AddOpaqueAlpha<I, CD>>&) {
        return typename type::Params{static_cast<dev_t<VBase<I>>>(maxDepthValue<CD>)};
    }
};
template <typename I, VBase<I> alpha> struct Lower<StaticAddAlpha<I, alpha>> {
    static constexpr bool available = true;
    using type = fkd::AddLast<dev_t<I>>;
    static typename type::Params params(const OperationData<StaticAddAlpha<I, alpha>>&) { return typename type::Params{alpha}; }
};
// input / float(max) is the per-channel IEEE division the Div operation performs.
template <typename I, ColorDepth CD> struct Lower<NormalizePixel<I, CD>> {
    static constexpr bool available = true;
    using type = fkd::Div<dev_t<I>, fkd::f32, dev_t<VectorType_t<float, cn<I>>>>;
    static typename type::Params params(const OperationData<NormalizePixel<I, CD>>&) { return type::make(static_cast<float>(maxDepthValue<CD>)); }
};
template <typename T, ColorDepth CD> struct Lower<SaturateDepth<T, CD>> {
    static constexpr bool available = true;
    using type = fkd::Saturate<dev_t<T>>;
    static typename type::Params params(const OperationData<SaturateDepth<T, CD>>&) {
        return typename type::Params{0.f, static_cast<float>(maxDepthValue<CD>)};
    }
};
template <typename O, ColorDepth CD> struct Lower<DenormalizePixel<O, CD>> {
    static constexpr bool available = true;
    using type = fkd::DenormalizePixel<dev_t<O>, int(CD)>;
    static typename type::Params params(const OperationData<DenormalizePixel<O, CD>>&) { return {}; }
};
template <typename I, typename O, ColorDepth CD> struct Lower<SaturateDenormalizePixel<I, O, CD>> {
    static constexpr bool available = true;
    using type = fkd::SaturateDenormalizePixel<dev_t<I>, dev_t<O>, int(CD)>;
    static typename type::Params params(const OperationData<SaturateDenormalizePixel<I, O, CD>>&) { return {}; }
};
} // namespace amd

} // namespace fk
#endif
