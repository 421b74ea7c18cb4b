// Host-side use of Operations and of the array helpers, the way the reference's unit tests use them: Operation::exec on
// one value on the calling thread, ArrayVector / toArray / transformArray, and the colour constants.  Compiled and run
// by tests/test_host_values.py; every check is a closed form or a value the standards fix.  No device involved.
#include <cstdio>
#include <fused_kernel/fused_kernel.h>
#include <fused_kernel/algorithms/basic_ops/arithmetic.h>
#include <fused_kernel/algorithms/basic_ops/cast.h>
#include <fused_kernel/algorithms/basic_ops/logical.h>
#include <fused_kernel/algorithms/image_processing/color_conversion.h>
#include <fused_kernel/algorithms/image_processing/saturate.h>

static int failures = 0;
#define CHECK(cond) do { if (!(cond)) { std::printf("FAILED line %d: %s\n", __LINE__, #cond); ++failures; } } while (0)

static bool near(float a, float b, float tol) { return std::fabs(a - b) <= tol; }

int main() {
    using namespace fk;
    // ---- array helpers ----
    constexpr auto a3 = toArray(float3{1.f, 2.f, 3.f});
    static_assert(a3.size == 3 && a3.at[0] == 1.f && a3[2] == 3.f && a3(1) == 2.f);
    static_assert(std::is_same_v<std::decay_t<decltype(a3)>, ArrayVector<float, 3>>);
    static_assert(toArray(7u).size == 1 && toArray(7u).at[0] == 7u, "a scalar is a one-channel value");
    constexpr float3 back = toVector(a3);
    static_assert(back.x == 1.f && back.y == 2.f && back.z == 3.f);
    static_assert(ArrayVector<int, 4>(5)[3] == 5 && ArrayVector<int, 2>(1, 2).at[1] == 2);
    constexpr auto idx = makeIndexArray<4>();
    static_assert(idx[0] == 0 && idx[3] == 3);
    constexpr auto doubled = transformArray(idx, [](const size_t& i) { return int(2 * i); });
    static_assert(std::is_same_v<std::decay_t<decltype(doubled)>, ArrayVector<int, 4>> && doubled[3] == 6);
    constexpr std::array<int, 3> in{1, 2, 3};
    constexpr auto squares = transformArray(in, [](const int& v) { return float(v * v); });
    static_assert(std::is_same_v<std::decay_t<decltype(squares)>, std::array<float, 3>> && squares[2] == 9.f);
    static_assert(allValuesAre(true, ArrayVector<bool, 3>(true, true, true)) && !allValuesAre(true, ArrayVector<bool, 3>(true, false, true)));
    static_assert(arraySize<std::array<int, 5>> == 5 && arraySize<ArrayVector<float, 2>> == 2);
    static_assert(and_v<true, true> && !and_v<true, false> && or_v<false, true> && !or_v<false, false>);
    static_assert(Find<int, 3>::in(std::integer_sequence<int, 5, 3, 1>{}) == 1 && !Find<int, 4>::one_of(std::integer_sequence<int, 5, 3, 1>{}));
    static_assert(OpIs<UnaryType, Cast<uchar, float>>::value && !OpIs<BinaryType, Cast<uchar, float>>::value);

    // ---- colour constants: BT.709 as the recommendation prints it, limited range spans, offsets ----
    static_assert(iTUWeights<ColorPrimitives::bt709>.Kr == 0.2126f && iTUWeights<ColorPrimitives::bt709>.Kb == 0.0722f);
    static_assert(iTUWeights<ColorPrimitives::bt601>.Kr == 0.299f && iTUWeights<ColorPrimitives::bt2020>.Kb == 0.0593f);
    static_assert(rangeLimits<ColorDepth::p8bit>.limitY == 219.f && rangeLimits<ColorDepth::p10bit>.limitC == 896.f);
    static_assert(subCoefficients<ColorDepth::p8bit>.luma == 16.f && subCoefficients<ColorDepth::p12bit>.chroma == 2048.f);
    constexpr M3x3Float to_rgb = ccMatrix<ColorRange::Full, ColorPrimitives::bt709, ColorConversionDir::YCbCr2RGB, ColorDepth::p8bit>;
    static_assert(to_rgb.x.x == 1.f && to_rgb.x.y == 0.f && to_rgb.z.z == 0.f);
    CHECK(near(to_rgb.x.z, 1.5748f, 1e-6f) && near(to_rgb.z.y, 1.8556f, 1e-6f));         // 2(1-Kr), 2(1-Kb)
    CHECK(near(to_rgb.y.y, -0.187324f, 1e-6f) && near(to_rgb.y.z, -0.468124f, 1e-6f));
    constexpr M3x3Float twice = to_rgb * 2.f;
    static_assert(twice.x.z == to_rgb.x.z * 2.f && (to_rgb * to_rgb).y.y == to_rgb.y.y * to_rgb.y.y, "products are element by element");

    // ---- Operation::exec on the calling thread ----
    CHECK(Add<float>::exec(1.f, 2.f) == 3.f);
    CHECK((Mul<float3, float3, float3>::exec(float3{1.f, 2.f, 3.f}, float3{2.f, 2.f, 2.f}).z == 6.f));
    const float3 f = Cast<uchar3, float3>::exec(uchar3{1, 2, 250});
    CHECK(f.x == 1.f && f.y == 2.f && f.z == 250.f);
    CHECK(IsEven<uint>::exec(2u) == true && IsEven<uint>::exec(3u) == false);
    const auto even2 = IsEven<int2>::exec(int2{4, -3});
    CHECK(even2.x == true && even2.y == false);
    CHECK((SaturateCast<float, uchar>::exec(300.f) == 255 && SaturateCast<float, uchar>::exec(-3.f) == 0 && SaturateCast<float, uchar>::exec(2.5f) == 2));
    // pure red, BT.601 full range, 8 bit: Y = 0.299 * 255, Cb = (B - Y) / (2 (1 - Kb)) + 128, Cr = (R - Y) / (2 (1 - Kr)) + 128
    const float3 yuv = ConvertRGBToYUV<ColorDepth::p8bit, ColorRange::Full, ColorPrimitives::bt601>::exec(uchar3{255, 0, 0});
    CHECK(near(yuv.x, 76.245f, 1e-3f) && near(yuv.y, 128.f - 76.245f / 1.772f, 1e-3f) && near(yuv.z, 255.5f, 1e-3f));
    const float3 rgb = ConvertYUVToRGB<ColorDepth::p8bit, ColorRange::Full, ColorPrimitives::bt601>::exec(uchar3{76, 85, 255});
    CHECK(near(rgb.x, 254.f, 1.f) && near(rgb.y, 0.f, 1.f) && near(rgb.z, 0.f, 1.f));
    CHECK((RGB2Gray<uchar3, uchar>::exec(uchar3{255, 0, 0}) == 76));
    const uchar4 with_alpha = AddOpaqueAlpha<uchar3, ColorDepth::p8bit>::exec(uchar3{1, 2, 3});
    CHECK(with_alpha.x == 1 && with_alpha.w == 255);
    const uchar3 denorm = SaturateDenormalizePixel<float3, uchar3, ColorDepth::p8bit>::exec(float3{-0.5f, 0.5f, 1.5f});
    CHECK(denorm.x == 0 && denorm.y == 127 && denorm.z == 255);
    // ---- BorderReader's index folding: the division-free form used within one image size of the image gives what the
    // reference's formulas give (FK/algorithms/image_processing/border_reader.h:177-327), for every extent up to 70 and every
    // index from four extents below the image to five above (the formulas as written take over beyond one extent) ----
    {
        using fkd::Border; using fkd::Read2D; using fkd::u8;
        int differing = 0;
        for (int n = 1; n <= 70; ++n)
            for (int i = -4 * n - 5; i <= 5 * n + 5; ++i) {
                differing += Border<1, Read2D<u8>>::fold(i, n) != Border<1, Read2D<u8>>::fold_as_written(i, n);
                differing += Border<2, Read2D<u8>>::fold(i, n) != Border<2, Read2D<u8>>::fold_as_written(i, n);
                differing += Border<3, Read2D<u8>>::fold(i, n) != Border<3, Read2D<u8>>::fold_as_written(i, n);
                differing += Border<4, Read2D<u8>>::fold(i, n) != Border<4, Read2D<u8>>::fold_as_written(i, n);
            }
        CHECK(differing == 0);
        // and the patterns themselves on a 4-wide axis: aaa|abcd|ddd, cba|abcd|dcb, bcd|abcd|abc, dcb|abcd|cba
        CHECK((Border<1, Read2D<u8>>::fold(-2, 4) == 0 && Border<1, Read2D<u8>>::fold(5, 4) == 3));
        CHECK((Border<2, Read2D<u8>>::fold(-1, 4) == 0 && Border<2, Read2D<u8>>::fold(-3, 4) == 2 && Border<2, Read2D<u8>>::fold(4, 4) == 3 && Border<2, Read2D<u8>>::fold(6, 4) == 1));
        CHECK((Border<3, Read2D<u8>>::fold(-1, 4) == 3 && Border<3, Read2D<u8>>::fold(-3, 4) == 1 && Border<3, Read2D<u8>>::fold(4, 4) == 0 && Border<3, Read2D<u8>>::fold(6, 4) == 2));
        CHECK((Border<4, Read2D<u8>>::fold(-1, 4) == 1 && Border<4, Read2D<u8>>::fold(-3, 4) == 3 && Border<4, Read2D<u8>>::fold(4, 4) == 2 && Border<4, Read2D<u8>>::fold(6, 4) == 0));
    }
    std::printf(failures ? "host values: %d check(s) failed\n" : "host values: all checks passed\n", failures);
    return failures ? 1 : 0;
}
