// color_chains.h -- chains over pixel formats and colour conversions, spelled ONCE with the public C++ API of the
// fused-kernel library (names, template arguments and argument order of the reference).
//
// This text is compiled twice: by tests/cases/fkl_cases.cpp against this repository's headers (the chains then run
// as gfx950 kernels on device memory), and by oracle/ref_chains.cpp against the reference library's own headers (the
// chains then run on its CPU backend on host memory).  Nothing in here names either implementation: DPP is the
// data-parallel pattern (TransformDPP<> / TransformDPP<ParArch::CPU>), StreamT the matching stream type and `mem` the
// kind of memory the caller's pointers refer to.
//
// Every entry returns 0 on success and 2 when the requested combination is not in its list.
#pragma once

#include <cstdint>

namespace color_chains {

using namespace fk;

constexpr int key(PixelFormat pf, ColorRange cr, ColorPrimitives cp) { return int(pf) * 100 + int(cr) * 10 + int(cp); }
constexpr int key(ColorDepth cd, ColorRange cr, ColorPrimitives cp) { return int(cd) * 100 + int(cr) * 10 + int(cp); }

template <class DPP, class StreamT> struct Chains {
    template <class T> static Ptr2D<T> wrap(const void* data, int w, int h, int pitch, MemType mem) {
        return Ptr2D<T>(reinterpret_cast<T*>(const_cast<void*>(data)), uint(w), uint(h), uint(pitch), mem, 0);
    }
    // A caller-owned frame of w x h pixels in pixel format PF: the backing array is w*rf.width_f x h*rf.height_f samples.
    template <PixelFormat PF> static Image<PF> image(const void* data, int w, int h, int pitch, MemType mem) {
        using B = typename Image<PF>::BaseType;
        const uint dw = uint(float(w) * PixelFormatTraits<PF>::rf.width_f), dh = uint(float(h) * PixelFormatTraits<PF>::rf.height_f);
        return Image<PF>(wrap<B>(data, int(dw), int(dh), pitch, mem), uint(w), uint(h));
    }

    // ---- ReadYUV<PF> -> ConvertYUVToRGB<depth of PF, CR, CP> -> float3 image --------------------------------
    template <PixelFormat PF, ColorRange CR, ColorPrimitives CP>
    static void yuv_to_rgb_one(StreamT& s, MemType mem, const void* src, int w, int h, int pitch, float* out, int out_pitch) {
        constexpr ColorDepth CD = PixelFormatTraits<PF>::depth;
        const auto img = image<PF>(src, w, h, pitch, mem);
        const auto o = wrap<float3>(out, w, h, out_pitch, mem);
        executeOperations<DPP>(s, ReadYUV<PF>::build(img.ptr()), ConvertYUVToRGB<CD, CR, CP>::build(),
                               PerThreadWrite<ND::_2D, float3>::build(o.ptr()));
    }
#define COLOR_CHAINS_YUV2RGB(X)                                                                                  \
    X(NV12, Limited, bt601) X(NV12, Full, bt601) X(NV12, Limited, bt709) X(NV12, Limited, bt2020) X(NV12, Full, bt2020) \
    X(NV21, Full, bt709) X(NV21, Limited, bt601) X(P010, Limited, bt2020) X(P210, Full, bt709)                    \
    X(Y210, Limited, bt709) X(UYVY, Limited, bt601) X(UYVY, Full, bt709)
    static int yuv_to_rgb(StreamT& s, MemType mem, int pf, int cr, int cp, const void* src, int w, int h, int pitch, float* out,
                          int out_pitch) {
        switch (pf * 100 + cr * 10 + cp) {
#define X(PF, CR, CP)                                                                                            \
    case key(PixelFormat::PF, ColorRange::CR, ColorPrimitives::CP):                                              \
        yuv_to_rgb_one<PixelFormat::PF, ColorRange::CR, ColorPrimitives::CP>(s, mem, src, w, h, pitch, out, out_pitch); \
        return 0;
            COLOR_CHAINS_YUV2RGB(X)
#undef X
        default: return 2;
        }
    }

    // ---- RGB image -> ConvertRGBToYUV -> SaturateCast -> WriteYUV<PF> ----------------------------------------
    template <PixelFormat PF, ColorRange CR, ColorPrimitives CP>
    static void rgb_to_yuv_one(StreamT& s, MemType mem, const void* src, int w, int h, int pitch, void* out, int out_pitch) {
        constexpr ColorDepth CD = PixelFormatTraits<PF>::depth;
        using Pixel = ColorDepthPixelType<CD>;
        const auto in = wrap<Pixel>(src, w, h, pitch, mem);
        const auto img = image<PF>(out, w, h, out_pitch, mem);
        executeOperations<DPP>(s, PerThreadRead<ND::_2D, Pixel>::build(in.ptr()), ConvertRGBToYUV<CD, CR, CP>::build(),
                               SaturateCast<float3, Pixel>::build(), WriteYUV<PF>::build(img.ptr()));
    }
#define COLOR_CHAINS_RGB2YUV(X)                                                                                  \
    X(NV12, Limited, bt709) X(NV21, Full, bt601) X(P010, Limited, bt2020) X(P210, Full, bt709) X(Y210, Limited, bt601) \
    X(UYVY, Full, bt2020)
    static int rgb_to_yuv(StreamT& s, MemType mem, int pf, int cr, int cp, const void* src, int w, int h, int pitch, void* out,
                          int out_pitch) {
        switch (pf * 100 + cr * 10 + cp) {
#define X(PF, CR, CP)                                                                                            \
    case key(PixelFormat::PF, ColorRange::CR, ColorPrimitives::CP):                                              \
        rgb_to_yuv_one<PixelFormat::PF, ColorRange::CR, ColorPrimitives::CP>(s, mem, src, w, h, pitch, out, out_pitch); \
        return 0;
            COLOR_CHAINS_RGB2YUV(X)
#undef X
        default: return 2;
        }
    }

    // ---- ReadYUV<PF> -> ConvertYUVToRGB -> bilinear resize -> Mul -> float3 image ------------------------------
    template <PixelFormat PF, ColorRange CR, ColorPrimitives CP>
    static void yuv_resize_one(StreamT& s, MemType mem, const void* src, int w, int h, int pitch, int dw, int dh, float scale,
                               float* out, int out_pitch) {
        constexpr ColorDepth CD = PixelFormatTraits<PF>::depth;
        const auto img = image<PF>(src, w, h, pitch, mem);
        const auto o = wrap<float3>(out, dw, dh, out_pitch, mem);
        executeOperations<DPP>(s, ReadYUV<PF>::build(img.ptr()), ConvertYUVToRGB<CD, CR, CP>::build(),
                               Resize<InterpolationType::INTER_LINEAR>::build(Size(dw, dh)), Mul<float3, float>::build(scale),
                               PerThreadWrite<ND::_2D, float3>::build(o.ptr()));
    }
    static int yuv_resize(StreamT& s, MemType mem, int pf, const void* src, int w, int h, int pitch, int dw, int dh, float scale,
                          float* out, int out_pitch) {
        switch (PixelFormat(pf)) {
        case PixelFormat::NV21:
            yuv_resize_one<PixelFormat::NV21, ColorRange::Full, ColorPrimitives::bt601>(s, mem, src, w, h, pitch, dw, dh, scale, out, out_pitch);
            return 0;
        case PixelFormat::UYVY:
            yuv_resize_one<PixelFormat::UYVY, ColorRange::Limited, ColorPrimitives::bt709>(s, mem, src, w, h, pitch, dw, dh, scale, out, out_pitch);
            return 0;
        case PixelFormat::P010:
            yuv_resize_one<PixelFormat::P010, ColorRange::Limited, ColorPrimitives::bt2020>(s, mem, src, w, h, pitch, dw, dh, scale, out, out_pitch);
            return 0;
        default: return 2;
        }
    }

    // ---- pixel image -> ConvertYUVToRGB / ConvertRGBToYUV<CD, CR, CP> -> float3 image (any depth) ----------------
    template <ColorDepth CD, ColorRange CR, ColorPrimitives CP, bool TO_RGB>
    static void convert_depth_one(StreamT& s, MemType mem, const void* src, int w, int h, int pitch, float* out, int out_pitch) {
        using Pixel = ColorDepthPixelType<CD>;
        const auto in = wrap<Pixel>(src, w, h, pitch, mem);
        const auto o = wrap<float3>(out, w, h, out_pitch, mem);
        if constexpr (TO_RGB)
            executeOperations<DPP>(s, PerThreadRead<ND::_2D, Pixel>::build(in.ptr()), ConvertYUVToRGB<CD, CR, CP>::build(),
                                   PerThreadWrite<ND::_2D, float3>::build(o.ptr()));
        else
            executeOperations<DPP>(s, PerThreadRead<ND::_2D, Pixel>::build(in.ptr()), ConvertRGBToYUV<CD, CR, CP>::build(),
                                   PerThreadWrite<ND::_2D, float3>::build(o.ptr()));
    }
#define COLOR_CHAINS_DEPTHS(X)                                                                                   \
    X(p8bit, Limited, bt2020) X(p12bit, Limited, bt601) X(p12bit, Full, bt709) X(fn8bit, Limited, bt709)          \
    X(fn10bit, Full, bt601) X(fn12bit, Limited, bt2020)
    static int convert_depth(StreamT& s, MemType mem, int cd, int cr, int cp, int to_rgb, const void* src, int w, int h, int pitch,
                             float* out, int out_pitch) {
        switch (cd * 100 + cr * 10 + cp) {
#define X(CD, CR, CP)                                                                                            \
    case key(ColorDepth::CD, ColorRange::CR, ColorPrimitives::CP):                                               \
        if (to_rgb) convert_depth_one<ColorDepth::CD, ColorRange::CR, ColorPrimitives::CP, true>(s, mem, src, w, h, pitch, out, out_pitch); \
        else convert_depth_one<ColorDepth::CD, ColorRange::CR, ColorPrimitives::CP, false>(s, mem, src, w, h, pitch, out, out_pitch); \
        return 0;
            COLOR_CHAINS_DEPTHS(X)
#undef X
        default: return 2;
        }
    }

    // ---- image of I -> ColorConversion<CODE, I, O, CD> -> image of O ---------------------------------------------
    template <ColorConversionCodes CODE, class I, class O, ColorDepth CD = ColorDepth::p8bit>
    static void convert_code_one(StreamT& s, MemType mem, const void* src, int w, int h, int pitch, void* out, int out_pitch) {
        const auto in = wrap<I>(src, w, h, pitch, mem);
        const auto o = wrap<O>(out, w, h, out_pitch, mem);
        executeOperations<DPP>(s, PerThreadRead<ND::_2D, I>::build(in.ptr()), ColorConversion<CODE, I, O, CD>::build(),
                               PerThreadWrite<ND::_2D, O>::build(o.ptr()));
    }
    // `which` numbers the list below.
    static int convert_code(StreamT& s, MemType mem, int which, const void* src, int w, int h, int pitch, void* out, int out_pitch) {
        using C = ColorConversionCodes;
        switch (which) {
        case 0: convert_code_one<C::COLOR_BGR2BGRA, uchar3, uchar4>(s, mem, src, w, h, pitch, out, out_pitch); return 0;
        case 1: convert_code_one<C::COLOR_BGRA2BGR, uchar4, uchar3>(s, mem, src, w, h, pitch, out, out_pitch); return 0;
        case 2: convert_code_one<C::COLOR_BGR2RGBA, uchar3, uchar4>(s, mem, src, w, h, pitch, out, out_pitch); return 0;
        case 3: convert_code_one<C::COLOR_BGRA2RGB, uchar4, uchar3>(s, mem, src, w, h, pitch, out, out_pitch); return 0;
        case 4: convert_code_one<C::COLOR_BGRA2RGBA, uchar4, uchar4>(s, mem, src, w, h, pitch, out, out_pitch); return 0;
        case 5: convert_code_one<C::COLOR_RGB2GRAY, uchar3, uchar>(s, mem, src, w, h, pitch, out, out_pitch); return 0;
        case 6: convert_code_one<C::COLOR_BGR2GRAY, uchar3, uchar>(s, mem, src, w, h, pitch, out, out_pitch); return 0;
        case 7: convert_code_one<C::COLOR_RGBA2GRAY, uchar4, uchar>(s, mem, src, w, h, pitch, out, out_pitch); return 0;
        case 8: convert_code_one<C::COLOR_BGRA2GRAY, uchar4, uchar>(s, mem, src, w, h, pitch, out, out_pitch); return 0;
        case 9: convert_code_one<C::COLOR_RGB2GRAY, float3, float>(s, mem, src, w, h, pitch, out, out_pitch); return 0;
        case 10: convert_code_one<C::COLOR_BGR2BGRA, ushort3, ushort4, ColorDepth::p10bit>(s, mem, src, w, h, pitch, out, out_pitch); return 0;
        default: return 2;
        }
    }

    // ---- image of I -> NormalizePixel<I, CD> -> float image -------------------------------------------------------
    static int normalize(StreamT& s, MemType mem, int which, const void* src, int w, int h, int pitch, float* out, int out_pitch) {
        if (which == 0) {
            const auto in = wrap<uchar3>(src, w, h, pitch, mem);
            const auto o = wrap<float3>(out, w, h, out_pitch, mem);
            executeOperations<DPP>(s, PerThreadRead<ND::_2D, uchar3>::build(in.ptr()), NormalizePixel<uchar3, ColorDepth::p8bit>::build(),
                                   PerThreadWrite<ND::_2D, float3>::build(o.ptr()));
            return 0;
        }
        if (which == 1) {
            const auto in = wrap<ushort3>(src, w, h, pitch, mem);
            const auto o = wrap<float3>(out, w, h, out_pitch, mem);
            executeOperations<DPP>(s, PerThreadRead<ND::_2D, ushort3>::build(in.ptr()), NormalizePixel<ushort3, ColorDepth::p10bit>::build(),
                                   PerThreadWrite<ND::_2D, float3>::build(o.ptr()));
            return 0;
        }
        return 2;
    }

    // ---- float image -> SaturateDepth / DenormalizePixel / SaturateDenormalizePixel / Saturate / SaturateFloat -> image ----
    template <class I, class O, class IOp>
    static void depth_one(StreamT& s, MemType mem, const IOp& iop, const void* src, int w, int h, int pitch, void* out, int out_pitch) {
        const auto in = wrap<I>(src, w, h, pitch, mem);
        const auto o = wrap<O>(out, w, h, out_pitch, mem);
        executeOperations<DPP>(s, PerThreadRead<ND::_2D, I>::build(in.ptr()), iop, PerThreadWrite<ND::_2D, O>::build(o.ptr()));
    }
    // which: 0 SaturateDepth<float, p8bit>, 1 SaturateDepth<float, p10bit>, 2 DenormalizePixel<uchar3, p8bit>,
    // 3 DenormalizePixel<float3, p8bit>, 4 SaturateDenormalizePixel<float3, uchar3, p8bit>,
    // 5 SaturateDenormalizePixel<float3, ushort3, p10bit>, 6 SaturateFloat<float4>, 7 Saturate<float3>{lo, hi},
    // 8 DenormalizePixel<ushort3, p12bit>, 9 SaturateDenormalizePixel<float4, uchar4, p8bit>
    static int depth_ops(StreamT& s, MemType mem, int which, const void* src, int w, int h, int pitch, void* out, int out_pitch, float lo, float hi) {
        constexpr auto p8 = ColorDepth::p8bit, p10 = ColorDepth::p10bit, p12 = ColorDepth::p12bit;
        switch (which) {
        case 0: depth_one<float, float>(s, mem, SaturateDepth<float, p8>::build(), src, w, h, pitch, out, out_pitch); return 0;
        case 1: depth_one<float, float>(s, mem, SaturateDepth<float, p10>::build(), src, w, h, pitch, out, out_pitch); return 0;
        case 2: depth_one<float3, uchar3>(s, mem, DenormalizePixel<uchar3, p8>::build(), src, w, h, pitch, out, out_pitch); return 0;
        case 3: depth_one<float3, float3>(s, mem, DenormalizePixel<float3, p8>::build(), src, w, h, pitch, out, out_pitch); return 0;
        case 4: depth_one<float3, uchar3>(s, mem, SaturateDenormalizePixel<float3, uchar3, p8>::build(), src, w, h, pitch, out, out_pitch); return 0;
        case 5: depth_one<float3, ushort3>(s, mem, SaturateDenormalizePixel<float3, ushort3, p10>::build(), src, w, h, pitch, out, out_pitch); return 0;
        case 6: depth_one<float4, float4>(s, mem, SaturateFloat<float4>::build(), src, w, h, pitch, out, out_pitch); return 0;
        case 7: depth_one<float3, float3>(s, mem, Saturate<float3>::build(make_<float2>(lo, hi)), src, w, h, pitch, out, out_pitch); return 0;
        case 8: depth_one<float3, ushort3>(s, mem, DenormalizePixel<ushort3, p12>::build(), src, w, h, pitch, out, out_pitch); return 0;
        case 9: depth_one<float4, uchar4>(s, mem, SaturateDenormalizePixel<float4, uchar4, p8>::build(), src, w, h, pitch, out, out_pitch); return 0;
        default: return 2;
        }
    }
};

} // namespace color_chains
