// ref_chains.cpp -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.
//
// (Compiled a second time with -DFKL_HARNESS_PUBLIC_API_ONLY against THIS repository's headers -- oracle/Makefile,
// target hostexec -- the same chain text runs on this repository's own TransformDPP<ParArch::CPU> executor; tests then
// hold that executor against the oracle.  The few probes of reference internals are left out of that build.)
//
// A thin C-ABI harness around the REFERENCE library's own CPU backend.  It is compiled against the
// reference's headers where they lie on disk (see oracle/Makefile: -I$(FKL_REFERENCE)), never copied,
// and the resulting shared object goes to oracle/_ref/ (git-ignored).  Each entry point spells one fused
// chain with the reference's public API, runs it with TransformDPP<ParArch::CPU> on caller-owned host
// buffers and returns.  Tests use it to validate the plain-C restatement in fkl_oracle.c and the HIP
// kernels; bench.py may time it as the CPU baseline.
//
// Build flags: -std=c++20 -O2 -ffp-contract=off (contraction off makes the floats compiler independent).
#include <fused_kernel/algorithms/basic_ops/memory_operations.h>
#include <fused_kernel/algorithms/basic_ops/arithmetic.h>
#include <fused_kernel/algorithms/basic_ops/cast.h>
#include <fused_kernel/algorithms/basic_ops/math.h>
#include <fused_kernel/algorithms/basic_ops/logical.h>
#include <fused_kernel/algorithms/basic_ops/bitwise.h>
#include <fused_kernel/algorithms/basic_ops/algebraic.h>
#include <fused_kernel/algorithms/image_processing/crop.h>
#include <fused_kernel/algorithms/image_processing/color_conversion.h>
#include <fused_kernel/algorithms/image_processing/resize.h>
#include <fused_kernel/algorithms/image_processing/warping.h>
#include <fused_kernel/algorithms/image_processing/deinterlace.h>
#include <fused_kernel/algorithms/image_processing/border_reader.h>
#include <fused_kernel/algorithms/image_processing/saturate.h>
#include <fused_kernel/algorithms/image_processing/image.h>
#include <fused_kernel/fused_kernel.h>
#include <fused_kernel/core/data/circular_tensor.h>
#include <fused_kernel/core/data/ptr_utils.h>

#include <array>
#include <cstdint>
#include <utility>

// Pixel-format and colour-conversion chains: the same text the GPU case drivers compile against this repository's
// headers, compiled here against the reference's.
#include "../tests/cases/color_chains.h"
#include "../tests/cases/border_chains.h"
#include "../tests/cases/circular_chains.h"
#include "../tests/cases/pointwise_chains.h"

using namespace fk;
using CpuDPP = TransformDPP<ParArch::CPU>;
using CpuDPPTF = TransformDPP<ParArch::CPU, TF::ENABLED>;
using CpuStream = Stream_<ParArch::CPU>;

namespace {

template <typename T>
Ptr2D<T> wrap2d(const void* data, int w, int h, int pitch) {
    return Ptr2D<T>(reinterpret_cast<T*>(const_cast<void*>(data)), uint(w), uint(h), uint(pitch), MemType::Host, 0);
}

template <size_t B>
std::array<Rect, B> rects_from(const int32_t* r) {
    std::array<Rect, B> a{};
    for (size_t i = 0; i < B; ++i) a[i] = Rect(r[4 * i + 0], r[4 * i + 1], r[4 * i + 2], r[4 * i + 3]);
    return a;
}

// README chain (benchmark configuration 1): uchar3 source, B crops, bilinear resize with PRESERVE_AR and a
// background, Mul, Sub, SaturateCast, TensorWrite<uchar3>.
template <size_t B>
int crop_resize_par_u8(const uint8_t* src, int w, int h, int pitch, const int32_t* rects, int dw, int dh,
                       const float* bg, const float* mul, const float* sub, uint8_t* out) {
    CpuStream stream;
    const auto in = wrap2d<uchar3>(src, w, h, pitch);
    Tensor<uchar3> o(reinterpret_cast<uchar3*>(out), uint(dw), uint(dh), uint(B), 1, MemType::Host, 0);
    const auto crops = rects_from<B>(rects);
    executeOperations<CpuDPP>(stream,
        PerThreadRead<ND::_2D, uchar3>::build(in.ptr()),
        Crop<>::build(crops),
        Resize<InterpolationType::INTER_LINEAR, AspectRatio::PRESERVE_AR>::build(Size(dw, dh), float3{bg[0], bg[1], bg[2]}),
        Mul<float3>::build(make_<float3>(mul[0], mul[1], mul[2])),
        Sub<float3>::build(make_<float3>(sub[0], sub[1], sub[2])),
        SaturateCast<float3, uchar3>::build(),
        TensorWrite<uchar3>::build(o.ptr()));
    stream.sync();
    return 0;
}

// Benchmark configuration 3: BGR uchar3 source, B crops, bilinear resize IGNORE_AR, BGR->RGB, Sub, Div,
// TensorSplit to planar float B x 3 x dh x dw.
template <size_t B>
int crop_resize_norm_split(const uint8_t* src, int w, int h, int pitch, const int32_t* rects, int dw, int dh,
                           const float* sub, const float* div, float* out) {
    CpuStream stream;
    const auto in = wrap2d<uchar3>(src, w, h, pitch);
    Tensor<float> o(out, uint(dw), uint(dh), uint(B), 3, MemType::Host, 0);
    const auto crops = rects_from<B>(rects);
    executeOperations<CpuDPP>(stream,
        PerThreadRead<ND::_2D, uchar3>::build(in.ptr()),
        Crop<>::build(crops),
        Resize<InterpolationType::INTER_LINEAR>::build(Size(dw, dh)),
        ColorConversion<ColorConversionCodes::COLOR_BGR2RGB, float3, float3>::build(),
        Sub<float3>::build(make_<float3>(sub[0], sub[1], sub[2])),
        Div<float3>::build(make_<float3>(div[0], div[1], div[2])),
        TensorSplit<float3>::build(o.ptr()));
    stream.sync();
    return 0;
}

// Horizontal fusion with fewer live planes than the compiled batch (BatchRead<CONDITIONAL_WITH_DEFAULT>): planes
// >= used_planes produce default_value instead of reading.  Same chain as configuration 3 otherwise.
template <size_t B>
int crop_resize_default_norm_split(const uint8_t* src, int w, int h, int pitch, const int32_t* rects, int dw, int dh,
                                   int used_planes, const float* def, const float* sub, const float* div, float* out) {
    CpuStream stream;
    const auto in = wrap2d<uchar3>(src, w, h, pitch);
    Tensor<float> o(out, uint(dw), uint(dh), uint(B), 3, MemType::Host, 0);
    const auto crops = rects_from<B>(rects);
    std::array<Size, B> sizes{};
    for (auto& s : sizes) s = Size(dw, dh);
    executeOperations<CpuDPP>(stream,
        PerThreadRead<ND::_2D, uchar3>::build(in.ptr())
            .then(Crop<>::build(crops))
            .then(Resize<InterpolationType::INTER_LINEAR>::build(used_planes, make_<float3>(def[0], def[1], def[2]), sizes)),
        ColorConversion<ColorConversionCodes::COLOR_BGR2RGB, float3, float3>::build(),
        Sub<float3>::build(make_<float3>(sub[0], sub[1], sub[2])),
        Div<float3>::build(make_<float3>(div[0], div[1], div[2])),
        TensorSplit<float3>::build(o.ptr()));
    stream.sync();
    return 0;
}

// The executor overload for an array of images with active batch and default value:
// executeOperations(std::array<Ptr2D<I>,B>, activeBatch, defaultValue, Tensor<O>, stream, ops...).
template <size_t B>
int batch_default_cast_mul(const uint8_t* const* srcs, int w, int h, int pitch, int active, const uint8_t* def,
                           const float* mul, float* out) {
    CpuStream stream;
    std::array<Ptr2D<uchar3>, B> ins{};
    for (size_t i = 0; i < B; ++i) ins[i] = wrap2d<uchar3>(srcs[i], w, h, pitch);
    Tensor<float3> o(reinterpret_cast<float3*>(out), uint(w), uint(h), uint(B), 1, MemType::Host, 0);
    executeOperations<CpuDPP>(ins, active, uchar3{def[0], def[1], def[2]}, o, stream,
        Cast<uchar3, float3>::build(),
        Mul<float3>::build(make_<float3>(mul[0], mul[1], mul[2])));
    stream.sync();
    return 0;
}

// Warping<Affine|Perspective> of a uchar3 image into a float3 image (matrix row-major, 6 or 9 values).
template <WarpType WT>
int warp_u8x3(const uint8_t* src, int w, int h, int pitch, const float* m, int dw, int dh, float* out) {
    CpuStream stream;
    const auto in = wrap2d<uchar3>(src, w, h, pitch);
    Ptr2D<float3> o(reinterpret_cast<float3*>(out), uint(dw), uint(dh), uint(dw) * uint(sizeof(float3)), MemType::Host, 0);
    WarpingParameters<WT> params{};
    constexpr int rows = WT == WarpType::Affine ? 2 : 3;
    for (int r = 0; r < rows; ++r)
        for (int c = 0; c < 3; ++c) params.transformMatrix.data[r][c] = m[r * 3 + c];
    params.dstSize = Size(dw, dh);
    executeOperations<CpuDPP>(stream, PerThreadRead<ND::_2D, uchar3>::build(in.ptr()).then(Warping<WT>::build(params)),
                              PerThreadWrite<ND::_2D, float3>::build(o.ptr()));
    stream.sync();
    return 0;
}

template <WarpType WT, class T, class O>
int warp_any(const void* src, int w, int h, int pitch, const float* m, int dw, int dh, float* out) {
    CpuStream stream;
    const auto in = wrap2d<T>(src, w, h, pitch);
    Ptr2D<O> o(reinterpret_cast<O*>(out), uint(dw), uint(dh), uint(dw) * uint(sizeof(O)), MemType::Host, 0);
    WarpingParameters<WT> params{};
    constexpr int rows = WT == WarpType::Affine ? 2 : 3;
    for (int r = 0; r < rows; ++r)
        for (int c = 0; c < 3; ++c) params.transformMatrix.data[r][c] = m[r * 3 + c];
    params.dstSize = Size(dw, dh);
    executeOperations<CpuDPP>(stream, PerThreadRead<ND::_2D, T>::build(in.ptr()).then(Warping<WT>::build(params)),
                              PerThreadWrite<ND::_2D, O>::build(o.ptr()));
    stream.sync();
    return 0;
}

// Benchmark configuration 4: B independent uchar3 images, per-image Mul and Add fused into each plane's
// read, SaturateCast, B separate outputs in one launch.
template <size_t B>
int batch_muladd_sat(const uint8_t* const* srcs, int w, int h, int pitch, const float* mul, const float* add,
                     uint8_t* const* outs, int out_pitch) {
    CpuStream stream;
    using PlaneIOp = decltype(PerThreadRead<ND::_2D, uchar3>::build(std::declval<RawPtr<ND::_2D, uchar3>>())
                                  .then(Mul<uchar3, float3, float3>::build(float3{}))
                                  .then(Add<float3>::build(float3{})));
    std::array<PlaneIOp, B> planes{};
    std::array<Ptr2D<uchar3>, B> outPtrs{};
    for (size_t i = 0; i < B; ++i) {
        const auto in = wrap2d<uchar3>(srcs[i], w, h, pitch);
        planes[i] = PerThreadRead<ND::_2D, uchar3>::build(in.ptr())
                        .then(Mul<uchar3, float3, float3>::build(make_<float3>(mul[3 * i], mul[3 * i + 1], mul[3 * i + 2])))
                        .then(Add<float3>::build(make_<float3>(add[3 * i], add[3 * i + 1], add[3 * i + 2])));
        outPtrs[i] = wrap2d<uchar3>(outs[i], w, h, out_pitch);
    }
    executeOperations<CpuDPP>(stream,
        BatchRead<PlanePolicy::PROCESS_ALL>::build(planes),
        SaturateCast<float3, uchar3>::build(),
        PerThreadWrite<ND::_2D, uchar3>::build(outPtrs));
    stream.sync();
    return 0;
}

// Benchmark configuration 2: N alternating Add(0.5f)/Mul(1.0001f) on a float image, starting with Add.
template <typename DPP, size_t... Is>
void add_mul_chain(CpuStream& stream, const Ptr2D<float>& in, const Ptr2D<float>& out, float addv, float mulv,
                   std::index_sequence<Is...>) {
    const auto pick = [&](auto idx) {
        if constexpr (decltype(idx)::value % 2 == 0) return Add<float>::build(addv);
        else return Mul<float>::build(mulv);
    };
    executeOperations<DPP>(stream, PerThreadRead<ND::_2D, float>::build(in.ptr()),
                           pick(std::integral_constant<size_t, Is>{})...,
                           PerThreadWrite<ND::_2D, float>::build(out.ptr()));
}

template <size_t N>
int add_mul_n(const float* in, int w, int h, int pitch, float addv, float mulv, float* out, int out_pitch, int tf) {
    CpuStream stream;
    const auto i = wrap2d<float>(in, w, h, pitch);
    const auto o = wrap2d<float>(out, w, h, out_pitch);
    if (tf) add_mul_chain<CpuDPPTF>(stream, i, o, addv, mulv, std::make_index_sequence<N>{});
    else add_mul_chain<CpuDPP>(stream, i, o, addv, mulv, std::make_index_sequence<N>{});
    stream.sync();
    return 0;
}

// Integer-only chain: uchar3 source, B crops of one size, BGR->RGB on uchar3, TensorWrite<uchar3>.
template <size_t B>
int crop_swap_u8(const uint8_t* src, int w, int h, int pitch, const int32_t* rects, uint8_t* out) {
    CpuStream stream;
    const auto in = wrap2d<uchar3>(src, w, h, pitch);
    Tensor<uchar3> o(reinterpret_cast<uchar3*>(out), uint(rects[2]), uint(rects[3]), uint(B), 1, MemType::Host, 0);
    const auto crops = rects_from<B>(rects);
    // A batched Crop is only fused backwards by executeOperations when a Resize follows it, so this chain
    // fuses the read explicitly with then().
    executeOperations<CpuDPP>(stream,
        PerThreadRead<ND::_2D, uchar3>::build(in.ptr()).then(Crop<>::build(crops)),
        ColorConversion<ColorConversionCodes::COLOR_BGR2RGB, uchar3, uchar3>::build(),
        TensorWrite<uchar3>::build(o.ptr()));
    stream.sync();
    return 0;
}

} // namespace

extern "C" {

int fklref_crop_resize_par_u8_b5(const uint8_t* src, int w, int h, int pitch, const int32_t* rects, int dw, int dh,
                                 const float* bg, const float* mul, const float* sub, uint8_t* out) {
    return crop_resize_par_u8<5>(src, w, h, pitch, rects, dw, dh, bg, mul, sub, out);
}

int fklref_crop_resize_norm_split_b8(const uint8_t* src, int w, int h, int pitch, const int32_t* rects, int dw,
                                     int dh, const float* sub, const float* div, float* out) {
    return crop_resize_norm_split<8>(src, w, h, pitch, rects, dw, dh, sub, div, out);
}
int fklref_crop_resize_norm_split_b64(const uint8_t* src, int w, int h, int pitch, const int32_t* rects, int dw,
                                      int dh, const float* sub, const float* div, float* out) {
    return crop_resize_norm_split<64>(src, w, h, pitch, rects, dw, dh, sub, div, out);
}

int fklref_crop_resize_default_norm_split_b8(const uint8_t* src, int w, int h, int pitch, const int32_t* rects, int dw, int dh,
                                             int used_planes, const float* def, const float* sub, const float* div, float* out) {
    return crop_resize_default_norm_split<8>(src, w, h, pitch, rects, dw, dh, used_planes, def, sub, div, out);
}
int fklref_batch_default_cast_mul_b4(const uint8_t* const* srcs, int w, int h, int pitch, int active, const uint8_t* def,
                                     const float* mul, float* out) {
    return batch_default_cast_mul<4>(srcs, w, h, pitch, active, def, mul, out);
}

int fklref_warp_u8x3(const uint8_t* src, int w, int h, int pitch, const float* m, int perspective, int dw, int dh, float* out) {
    return perspective ? warp_u8x3<WarpType::Perspective>(src, w, h, pitch, m, dw, dh, out)
                       : warp_u8x3<WarpType::Affine>(src, w, h, pitch, m, dw, dh, out);
}
// The same for other pixel types: kind 2 uchar4 -> float4, 3 ushort3 -> float3, 4 uchar -> float (tight float output).
int fklref_warp_kind(int kind, const void* src, int w, int h, int pitch, const float* m, int perspective, int dw, int dh, float* out) {
    auto run = [&](auto in_tag, auto out_tag) {
        using T = decltype(in_tag); using O = decltype(out_tag);
        return perspective ? warp_any<WarpType::Perspective, T, O>(src, w, h, pitch, m, dw, dh, out)
                           : warp_any<WarpType::Affine, T, O>(src, w, h, pitch, m, dw, dh, out);
    };
    if (kind == 2) return run(uchar4{}, float4{});
    if (kind == 3) return run(ushort3{}, float3{});
    if (kind == 4) return run(uchar{}, float{});
    return 2;
}

// Deinterlace of a uchar3 image into a float3 image: mode 1 BLEND, 2 INTER_LINEAR keeping even lines, 3 keeping odd.
int fklref_deinterlace_u8x3(const uint8_t* src, int w, int h, int pitch, int mode, float* out) {
    CpuStream stream;
    const auto in = wrap2d<uchar3>(src, w, h, pitch);
    Ptr2D<float3> o(reinterpret_cast<float3*>(out), uint(w), uint(h), uint(w) * uint(sizeof(float3)), MemType::Host, 0);
    const auto read = PerThreadRead<ND::_2D, uchar3>::build(in.ptr());
    const auto write = PerThreadWrite<ND::_2D, float3>::build(o.ptr());
    if (mode == 1) executeOperations<CpuDPP>(stream, read.then(Deinterlace<DeinterlaceType::BLEND>::build()), write);
    else executeOperations<CpuDPP>(stream, read.then(Deinterlace<DeinterlaceType::INTER_LINEAR>::build(
                                               DeinterlaceParameters<DeinterlaceType::INTER_LINEAR>{mode == 2})), write);
    stream.sync();
    return 0;
}

int fklref_batch_muladd_sat_b4(const uint8_t* const* srcs, int w, int h, int pitch, const float* mul,
                               const float* add, uint8_t* const* outs, int out_pitch) {
    return batch_muladd_sat<4>(srcs, w, h, pitch, mul, add, outs, out_pitch);
}
int fklref_batch_muladd_sat_b100(const uint8_t* const* srcs, int w, int h, int pitch, const float* mul,
                                 const float* add, uint8_t* const* outs, int out_pitch) {
    return batch_muladd_sat<100>(srcs, w, h, pitch, mul, add, outs, out_pitch);
}

int fklref_add_mul_chain(const float* in, int w, int h, int pitch, int n_ops, float addv, float mulv, float* out,
                         int out_pitch, int tf) {
    switch (n_ops) {
    case 1: return add_mul_n<1>(in, w, h, pitch, addv, mulv, out, out_pitch, tf);
    case 2: return add_mul_n<2>(in, w, h, pitch, addv, mulv, out, out_pitch, tf);
    case 3: return add_mul_n<3>(in, w, h, pitch, addv, mulv, out, out_pitch, tf);
    case 10: return add_mul_n<10>(in, w, h, pitch, addv, mulv, out, out_pitch, tf);
    case 20: return add_mul_n<20>(in, w, h, pitch, addv, mulv, out, out_pitch, tf);
    case 30: return add_mul_n<30>(in, w, h, pitch, addv, mulv, out, out_pitch, tf);
    case 40: return add_mul_n<40>(in, w, h, pitch, addv, mulv, out, out_pitch, tf);
    case 50: return add_mul_n<50>(in, w, h, pitch, addv, mulv, out, out_pitch, tf);
    case 100: return add_mul_n<100>(in, w, h, pitch, addv, mulv, out, out_pitch, tf);
    default: return 1;
    }
}

// Benchmark configuration 5: NV12 frame -> RGB (BT.709 full range) -> bilinear resize -> Mul by a scalar ->
// TensorSplit to planar float 3 x dh x dw.  `nv12` is w x (h*3/2) bytes with row pitch `pitch`.
int fklref_nv12_rgb_resize_split(const uint8_t* nv12, int w, int h, int pitch, int dw, int dh, float scale,
                                 float* out) {
    CpuStream stream;
    const Ptr2D<uchar> data(const_cast<uchar*>(nv12), uint(w), uint(h + h / 2), uint(pitch), MemType::Host, 0);
    const Image<PixelFormat::NV12> img(data, uint(w), uint(h));
    Tensor<float> o(out, uint(dw), uint(dh), 1, 3, MemType::Host, 0);
    executeOperations<CpuDPP>(stream,
        ReadYUV<PixelFormat::NV12>::build(img.ptr()),
        ConvertYUVToRGB<ColorDepth::p8bit, ColorRange::Full, ColorPrimitives::bt709>::build(),
        Resize<InterpolationType::INTER_LINEAR>::build(Size(dw, dh)),
        Mul<float3, float>::build(scale),
        TensorSplit<float3>::build(o.ptr()));
    stream.sync();
    return 0;
}

int fklref_crop_swap_u8_b4(const uint8_t* src, int w, int h, int pitch, const int32_t* rects, uint8_t* out) {
    return crop_swap_u8<4>(src, w, h, pitch, rects, out);
}

#ifndef FKL_HARNESS_PUBLIC_API_ONLY   // probes of reference internals (static exec, the constexpr matrix)
// SaturateCast<float, uchar> over an array, one element at a time.
int fklref_saturate_cast_u8(const float* in, int n, uint8_t* out) {
    for (int i = 0; i < n; ++i) out[i] = SaturateCast<float, uchar>::exec(in[i]);
    return 0;
}

// The constexpr BT.709 full-range YCbCr->RGB matrix the reference computes, row major.
int fklref_yuv2rgb_709_full_matrix(float* m9) {
    constexpr M3x3Float m = ccMatrix<ColorRange::Full, ColorPrimitives::bt709, ColorConversionDir::YCbCr2RGB, ColorDepth::p8bit>;
    m9[0] = m.x.x; m9[1] = m.x.y; m9[2] = m.x.z;
    m9[3] = m.y.x; m9[4] = m.y.y; m9[5] = m.y.z;
    m9[6] = m.z.x; m9[7] = m.z.y; m9[8] = m.z.z;
    return 0;
}

#endif

// The same for any aspect-ratio mode (0 PRESERVE_AR, 2 PRESERVE_AR_RN_EVEN, 3 PRESERVE_AR_LEFT).
extern "C++" template <AspectRatio AR> void resize_params_of(int sw, int sh, int dw, int dh, int32_t* out4, float* f2) {
    constexpr RawPtr<ND::_2D, uchar3> dummy{nullptr, {1u << 14, 1u << 14, 3u << 14}};
    const auto back = PerThreadRead<ND::_2D, uchar3>::build(dummy).then(Crop<>::build(Rect(0, 0, sw, sh)));
    const auto r = back.then(Resize<InterpolationType::INTER_LINEAR, AR>::build(Size(dw, dh), float3{0.f, 0.f, 0.f}));
    out4[0] = r.params.x1; out4[1] = r.params.y1; out4[2] = r.params.x2; out4[3] = r.params.y2;
    f2[0] = r.params.src_conv_factors.x; f2[1] = r.params.src_conv_factors.y;
}
int fklref_resize_params_ar(int ar, int sw, int sh, int dw, int dh, int32_t* out4, float* f2) {
    switch (ar) {
    case 0: resize_params_of<AspectRatio::PRESERVE_AR>(sw, sh, dw, dh, out4, f2); return 0;
    case 2: resize_params_of<AspectRatio::PRESERVE_AR_RN_EVEN>(sw, sh, dw, dh, out4, f2); return 0;
    case 3: resize_params_of<AspectRatio::PRESERVE_AR_LEFT>(sw, sh, dw, dh, out4, f2); return 0;
    default: return 2;
    }
}

// Letterbox geometry and factors the reference computes for one crop size (PRESERVE_AR), read back from the
// built IOp: out = {x1, y1, x2, y2}, f = {fx, fy}.
int fklref_resize_params_par(int sw, int sh, int dw, int dh, int32_t* out4, float* f2) {
    constexpr RawPtr<ND::_2D, uchar3> dummy{nullptr, {1u << 14, 1u << 14, 3u << 14}};
    const auto back = PerThreadRead<ND::_2D, uchar3>::build(dummy).then(Crop<>::build(Rect(0, 0, sw, sh)));
    const auto r = back.then(Resize<InterpolationType::INTER_LINEAR, AspectRatio::PRESERVE_AR>::build(Size(dw, dh), float3{0.f, 0.f, 0.f}));
    out4[0] = r.params.x1; out4[1] = r.params.y1; out4[2] = r.params.x2; out4[3] = r.params.y2;
    f2[0] = r.params.src_conv_factors.x; f2[1] = r.params.src_conv_factors.y;
    return 0;
}

} // extern "C"

// ---- pixel formats and colour conversions (tests/cases/color_chains.h on the reference's CPU backend) ----------
namespace {
using RefColor = color_chains::Chains<CpuDPP, CpuStream>;
#ifndef FKL_HARNESS_PUBLIC_API_ONLY
template <int CD, int CR, int CP, int DIR> void color_matrix_of(float* m9) {
    constexpr M3x3Float m = ccMatrix<ColorRange(CR), ColorPrimitives(CP), ColorConversionDir(DIR), ColorDepth(CD)>;
    m9[0] = m.x.x; m9[1] = m.x.y; m9[2] = m.x.z;
    m9[3] = m.y.x; m9[4] = m.y.y; m9[5] = m.y.z;
    m9[6] = m.z.x; m9[7] = m.z.y; m9[8] = m.z.z;
}
using MatrixFn = void (*)(float*);
template <size_t... I> MatrixFn matrix_fn(size_t i, std::index_sequence<I...>) {
    static constexpr MatrixFn table[] = {&color_matrix_of<int(I / 12), int((I / 6) % 2), int((I / 2) % 3), int(I % 2)>...};
    return table[i];
}
#endif
} // namespace

extern "C" {

int fklref_yuv_to_rgb(int pf, int cr, int cp, const void* src, int w, int h, int pitch, float* out, int out_pitch) {
    CpuStream s;
    const int rc = RefColor::yuv_to_rgb(s, MemType::Host, pf, cr, cp, src, w, h, pitch, out, out_pitch);
    s.sync();
    return rc;
}
int fklref_rgb_to_yuv(int pf, int cr, int cp, const void* src, int w, int h, int pitch, void* out, int out_pitch) {
    CpuStream s;
    const int rc = RefColor::rgb_to_yuv(s, MemType::Host, pf, cr, cp, src, w, h, pitch, out, out_pitch);
    s.sync();
    return rc;
}
int fklref_yuv_resize(int pf, const void* src, int w, int h, int pitch, int dw, int dh, float scale, float* out, int out_pitch) {
    CpuStream s;
    const int rc = RefColor::yuv_resize(s, MemType::Host, pf, src, w, h, pitch, dw, dh, scale, out, out_pitch);
    s.sync();
    return rc;
}
int fklref_convert_depth(int cd, int cr, int cp, int to_rgb, const void* src, int w, int h, int pitch, float* out, int out_pitch) {
    CpuStream s;
    const int rc = RefColor::convert_depth(s, MemType::Host, cd, cr, cp, to_rgb, src, w, h, pitch, out, out_pitch);
    s.sync();
    return rc;
}
int fklref_convert_code(int which, const void* src, int w, int h, int pitch, void* out, int out_pitch) {
    CpuStream s;
    const int rc = RefColor::convert_code(s, MemType::Host, which, src, w, h, pitch, out, out_pitch);
    s.sync();
    return rc;
}
int fklref_normalize(int which, const void* src, int w, int h, int pitch, float* out, int out_pitch) {
    CpuStream s;
    const int rc = RefColor::normalize(s, MemType::Host, which, src, w, h, pitch, out, out_pitch);
    s.sync();
    return rc;
}
int fklref_depth_ops(int which, const void* src, int w, int h, int pitch, void* out, int out_pitch, float lo, float hi) {
    CpuStream s;
    const int rc = RefColor::depth_ops(s, MemType::Host, which, src, w, h, pitch, out, out_pitch, lo, hi);
    s.sync();
    return rc;
}
// Operation number `which` of tests/cases/pointwise_chains.h on the CPU backend.
int fklref_pointwise(int which, const void* src, int w, int h, int pitch, void* out, int out_pitch, const float* c, const float* m) {
    CpuStream s;
    const int rc = pointwise_chains::Chains<CpuDPP, CpuStream>::run(s, MemType::Host, which, src, w, h, pitch, out, out_pitch, c, m);
    s.sync();
    return rc;
}
// SplitWrite chain number `which` of tests/cases/pointwise_chains.h on the CPU backend.
int fklref_split_write(int which, const void* src, int w, int h, int pitch, int dw, int dh, void* const* outs, const int* out_pitch,
                       const float* c) {
    CpuStream s;
    const int rc = pointwise_chains::Chains<CpuDPP, CpuStream>::split_write(s, MemType::Host, which, src, w, h, pitch, dw, dh, outs, out_pitch, c);
    s.sync();
    return rc;
}
// Two-image chain number `which` of tests/cases/pointwise_chains.h on the CPU backend.
int fklref_dual(int which, const void* a, const void* b, int w, int h, int pitch_a, int pitch_b, void* out, int out_pitch) {
    CpuStream s;
    const int rc = pointwise_chains::Chains<CpuDPP, CpuStream>::dual(s, MemType::Host, which, a, b, w, h, pitch_a, pitch_b, out, out_pitch);
    s.sync();
    return rc;
}
#ifndef FKL_HARNESS_PUBLIC_API_ONLY
// ccMatrix<range, primaries, direction, depth> as the reference computes it at compile time, row major.
// to_rgb = 1 selects YCbCr2RGB.
int fklref_color_matrix(int cd, int cr, int cp, int to_rgb, float* m9) {
    if (cd < 0 || cd > 5 || cr < 0 || cr > 1 || cp < 0 || cp > 2) return 1;
    const size_t dir = to_rgb ? size_t(ColorConversionDir::YCbCr2RGB) : size_t(ColorConversionDir::RGB2YCbCr);
    matrix_fn(((size_t(cd) * 2 + size_t(cr)) * 3 + size_t(cp)) * 2 + dir, std::make_index_sequence<72>{})(m9);
    return 0;
}
#endif

} // extern "C"

// ---- padding through BorderReader (tests/cases/border_chains.h on the reference's CPU backend) ------------------
extern "C" int fklref_pad(int elem, int border_type, const void* src, int w, int h, int pitch, int left, int top, int out_w, int out_h,
                          const float* value, void* out, int out_pitch) {
    CpuStream s;
    const int rc = border_chains::Chains<CpuDPP, CpuStream>::pad(s, MemType::Host, elem, border_type, src, w, h, pitch, left, top, out_w,
                                                                  out_h, value, out, out_pitch);
    s.sync();
    return rc;
}

// ---- divergent launches and the CircularTensor window (tests/cases/circular_chains.h on the reference's CPU backend) ----
extern "C" {
int fklref_divergent_two(const uint32_t* a, const uint32_t* b, int w, int h, int pitch, uint32_t add, uint32_t* out) {
    CpuStream s;
    circular_chains::Chains<ParArch::CPU>::divergent_two(s, MemType::Host, a, b, w, h, pitch, add, out);
    s.sync();
    return 0;
}
int fklref_divergent_mixed(const float* tensor4, int w, int h, float mul, const uint8_t* img, int iw, int ih, int ipitch, float* out) {
    CpuStream s;
    circular_chains::Chains<ParArch::CPU>::divergent_mixed(s, MemType::Host, tensor4, w, h, mul, img, iw, ih, ipitch, out);
    s.sync();
    return 0;
}
int fklref_transposed_round_trip(const uint8_t* const* images, int planes, int w, int h, int pitch, float mul, float* tensor_t, float mul2,
                                 float* packed) {
    CpuStream s;
    circular_chains::Chains<ParArch::CPU>::transposed_round_trip(s, MemType::Host, images, planes, w, h, pitch, mul, tensor_t, mul2, packed);
    s.sync();
    return 0;
}
int fklref_circular_transposed(int batch, int oldest_first, const uint8_t* const* images, int iters, int w, int h, int pitch, float fill,
                               float* states) {
    CpuStream s;
    return circular_chains::Chains<ParArch::CPU>::circular_transposed(s, batch, oldest_first, images, iters, w, h, pitch, MemType::Host, fill, states);
}
int fklref_circular(int batch, int oldest_first, const uint8_t* const* images, int iters, int w, int h, int pitch, float fill, float* states) {
    CpuStream s;
    return circular_chains::Chains<ParArch::CPU>::circular(s, batch, oldest_first, images, iters, w, h, pitch, MemType::Host, fill, states);
}
} // extern "C"
