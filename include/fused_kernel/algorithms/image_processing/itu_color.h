// Colour-format vocabulary: colour spaces, ranges, primaries, depths and pixel formats, with the per-format traits
// and per-depth constants.  Interface counterpart: FK/algorithms/image_processing/itu_color.h:21-183.
// The YCbCr<->RGB matrices themselves are evaluated at compile time inside the device code (fkd::color_matrix), in
// binary32 and in the reference's expression order (itu_color.h:185-265).
#ifndef FK_AMD_ITU_COLOR_H
#define FK_AMD_ITU_COLOR_H

#include <fused_kernel/core/utils/vector_utils.h>
#include <fused_kernel/core/utils/type_lists.h>
#include <fused_kernel/core/utils/template_operations.h>
#include <fused_kernel/core/data/static_matrix.h>
#include <fkd/ops.hpp>

namespace fk {

enum class ColorSpace { YUV420, YUV422, YUV444, RGB, RGBA };
enum class ColorRange { Limited, Full };
enum class ColorPrimitives { bt601, bt709, bt2020 };
enum class ColorDepth { p8bit, p10bit, p12bit, fn8bit, fn10bit, fn12bit };
enum class PixelFormat { NV12, NV21, YV12, P010, P016, P216, P210, Y216, Y210, Y416, UYVY };

template <ColorDepth CD> struct CD_t { ColorDepth value{CD}; };   // a depth as a type, for type lists
template <ColorDepth CD> struct ColorDepthTraits;
template <> struct ColorDepthTraits<ColorDepth::p8bit> { using base = uchar; using pixel = uchar3; };
template <> struct ColorDepthTraits<ColorDepth::p10bit> { using base = ushort; using pixel = ushort3; };
template <> struct ColorDepthTraits<ColorDepth::p12bit> { using base = ushort; using pixel = ushort3; };
template <> struct ColorDepthTraits<ColorDepth::fn8bit> { using base = float; using pixel = float3; };
template <> struct ColorDepthTraits<ColorDepth::fn10bit> { using base = float; using pixel = float3; };
template <> struct ColorDepthTraits<ColorDepth::fn12bit> { using base = float; using pixel = float3; };
template <ColorDepth CD> using ColorDepthPixelBaseType = typename ColorDepthTraits<CD>::base;
template <ColorDepth CD> using ColorDepthPixelType = typename ColorDepthTraits<CD>::pixel;

// Number of base-type elements per image column / row of the backing buffer.
struct ResolutionFactors { float width_f; float height_f; };

template <PixelFormat PF> struct PixelFormatTraits;
template <> struct PixelFormatTraits<PixelFormat::NV12> {
    static constexpr ColorSpace space = ColorSpace::YUV420;
    static constexpr ColorDepth depth = ColorDepth::p8bit;
    static constexpr size_t cn = 3;
    static constexpr ResolutionFactors rf{1.f, 1.5f};
};
template <> struct PixelFormatTraits<PixelFormat::NV21> {
    static constexpr ColorSpace space = ColorSpace::YUV420;
    static constexpr ColorDepth depth = ColorDepth::p8bit;
    static constexpr size_t cn = 3;
    static constexpr ResolutionFactors rf{1.f, 1.5f};
};
template <> struct PixelFormatTraits<PixelFormat::YV12> {
    static constexpr ColorSpace space = ColorSpace::YUV420;
    static constexpr ColorDepth depth = ColorDepth::p8bit;
    static constexpr size_t cn = 3;
    static constexpr ResolutionFactors rf{1.f, 1.5f};
};
template <> struct PixelFormatTraits<PixelFormat::P010> {
    static constexpr ColorSpace space = ColorSpace::YUV420;
    static constexpr ColorDepth depth = ColorDepth::p10bit;
    static constexpr size_t cn = 3;
    static constexpr ResolutionFactors rf{1.f, 1.5f};
};
template <> struct PixelFormatTraits<PixelFormat::P210> {
    static constexpr ColorSpace space = ColorSpace::YUV422;
    static constexpr ColorDepth depth = ColorDepth::p10bit;
    static constexpr size_t cn = 3;
    static constexpr ResolutionFactors rf{1.f, 2.f};
};
template <> struct PixelFormatTraits<PixelFormat::Y210> {
    static constexpr ColorSpace space = ColorSpace::YUV422;
    static constexpr ColorDepth depth = ColorDepth::p10bit;
    static constexpr size_t cn = 3;
    static constexpr ResolutionFactors rf{2.f, 1.f};
};
template <> struct PixelFormatTraits<PixelFormat::Y416> {
    static constexpr ColorSpace space = ColorSpace::YUV444;
    static constexpr ColorDepth depth = ColorDepth::p12bit;
    static constexpr size_t cn = 4;
    static constexpr ResolutionFactors rf{4.f, 1.f};
};
template <> struct PixelFormatTraits<PixelFormat::UYVY> {
    static constexpr ColorSpace space = ColorSpace::YUV422;
    static constexpr ColorDepth depth = ColorDepth::p8bit;
    static constexpr size_t cn = 3;
    static constexpr ResolutionFactors rf{2.f, 1.f};
};

// Largest sample value of a depth (1.f for the normalised-float depths).
template <ColorDepth CD> constexpr ColorDepthPixelBaseType<CD> maxDepthValue{};
template <> inline constexpr uchar maxDepthValue<ColorDepth::p8bit>{255u};
template <> inline constexpr ushort maxDepthValue<ColorDepth::p10bit>{1023u};
template <> inline constexpr ushort maxDepthValue<ColorDepth::p12bit>{4095u};
template <> inline constexpr float maxDepthValue<ColorDepth::fn8bit>{1.f};
template <> inline constexpr float maxDepthValue<ColorDepth::fn10bit>{1.f};
template <> inline constexpr float maxDepthValue<ColorDepth::fn12bit>{1.f};

// The constants of the conversions, as the device code holds them (fkd::DepthConsts, fkd::luma_weight_*): what is
// subtracted from luma and chroma samples, the ITU luma weights of the primaries, the limited-range spans.
// FK/algorithms/image_processing/itu_color.h:103-183.
struct SubCoefficients { float luma; float chroma; };
template <ColorDepth CD> constexpr SubCoefficients subCoefficients{fkd::DepthConsts<int(CD)>::luma, fkd::DepthConsts<int(CD)>::chroma};
struct ITUWeights { float Kr{0.f}; float Kb{0.f}; };
template <ColorPrimitives CP> constexpr ITUWeights iTUWeights{fkd::luma_weight_red(int(CP)), fkd::luma_weight_blue(int(CP))};
struct RangeLimits { float limitY; float limitC; };
template <ColorDepth CD> constexpr RangeLimits rangeLimits{fkd::DepthConsts<int(CD)>::limit_y, fkd::DepthConsts<int(CD)>::limit_c};

enum class ColorConversionDir { YCbCr2RGB, RGB2YCbCr };

// The coefficients the device code multiplies by, as a host-visible constant (FK/.../itu_color.h:185-272): the same
// compile-time evaluation, fkd::color_matrix, so host and device cannot disagree.
template <ColorRange CR, ColorPrimitives CP, ColorConversionDir CCD, ColorDepth CD>
constexpr M3x3Float computeMatrix() {
    constexpr fkd::ColorMatrix c = fkd::color_matrix<int(CD), int(CR), int(CP), CCD == ColorConversionDir::YCbCr2RGB>();
    return M3x3Float{{c.m[0], c.m[1], c.m[2]}, {c.m[3], c.m[4], c.m[5]}, {c.m[6], c.m[7], c.m[8]}};
}
template <ColorRange CR, ColorPrimitives CP, ColorConversionDir CCD, ColorDepth CD>
constexpr M3x3Float ccMatrix = computeMatrix<CR, CP, CCD, CD>();

} // namespace fk
#endif
