// fkl_cases.cpp -- the benchmark chains spelled with the library's C++ host API, exactly as a user of the
// reference library writes them (same names, same argument order), behind extern "C" drivers so pytest and
// bench.py can hand in device pointers.  Everything here runs through executeOperations<TransformDPP<>> ->
// host-side fusion -> fklhip_launch_handle -> gfx950 kernel; nothing computes on the CPU.
//
// Compiled by g++ (no HIP headers): g++ -std=c++20 -I include tests/cases/fkl_cases.cpp -L... -lfklhip
#include <fused_kernel/algorithms/basic_ops/memory_operations.h>
#include <fused_kernel/algorithms/basic_ops/arithmetic.h>
#include <fused_kernel/algorithms/basic_ops/cast.h>
#include <fused_kernel/algorithms/basic_ops/static_loop.h>
#include <fused_kernel/algorithms/basic_ops/math.h>
#include <fused_kernel/algorithms/basic_ops/logical.h>
#include <fused_kernel/algorithms/basic_ops/bitwise.h>
#include <fused_kernel/algorithms/basic_ops/algebraic.h>
#include <fused_kernel/core/data/ptr_utils.h>
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

#include <array>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <exception>
#include <utility>

#include "color_chains.h"   // pixel-format and colour-conversion chains, shared with the reference-backend harness
#include "border_chains.h"  // padding chains, shared the same way
#include "circular_chains.h"  // divergent launches and the CircularTensor window, shared the same way
#include "pointwise_chains.h" // one per-channel Operation of math.h / logical.h / bitwise.h / algebraic.h, shared the same way

#include <time.h>

using namespace fk;

namespace {

thread_local char g_error[2048] = "";
thread_local int g_reps = 1;   // how many times the next chain is enqueued (benchmarks time the whole run)

// Timing of the next driver call (benchmarks): one event recorded on `stream` right before the call's first launch and one
// right after its last, so the bracket holds the `reps` launches and nothing of the caller's own preparations.
struct Timing { void* stream = nullptr; void* first = nullptr; void* last = nullptr; bool armed = false; long long start_ns = 0; };
thread_local Timing g_timing;
long long monotonic_ns() {
    timespec ts{};
    clock_gettime(CLOCK_MONOTONIC, &ts);
    return (long long)ts.tv_sec * 1000000000ll + ts.tv_nsec;
}

template <typename F> int guarded(F body) {
    const bool timed = g_timing.armed;
    g_timing.armed = false;
    try {
        if (timed) { g_timing.start_ns = monotonic_ns(); gpuErrchk(fklhip_event_record(g_timing.first, g_timing.stream)); }
        body();
        if (timed) gpuErrchk(fklhip_event_record(g_timing.last, g_timing.stream));
        g_reps = 1;
        return 0;
    } catch (const std::exception& e) {
        g_reps = 1;
        std::snprintf(g_error, sizeof(g_error), "%s", e.what());
        return 1;
    }
}

template <typename T> Ptr2D<T> dev2d(const void* data, int w, int h, int pitch) {
    return Ptr2D<T>(reinterpret_cast<T*>(const_cast<void*>(data)), uint(w), uint(h), uint(pitch), MemType::Device, 0);
}

template <size_t B> std::array<Rect, B> rects_from(const int32_t* r) {
    std::array<Rect, B> a{};
    for (size_t i = 0; i < B; ++i) a[i] = Rect(r[4 * i + 0], r[4 * i + 1], r[4 * i + 2], r[4 * i + 3]);
    return a;
}

// Configuration 1 (README chain).
template <size_t B>
void crop_resize_par_u8(void* stream_, const uint8_t* src, int w, int h, int pitch, const int32_t* rects, int dw, int dh,
                        const float* bg, const float* mul, const float* sub, uint8_t* out) {
    Stream stream(stream_);
    const auto in = dev2d<uchar3>(src, w, h, pitch);
    Tensor<uchar3> o(reinterpret_cast<uchar3*>(out), uint(dw), uint(dh), uint(B), 1, MemType::Device, 0);
    const auto crops = rects_from<B>(rects);
    for (int rep = 0; rep < g_reps; ++rep) executeOperations<TransformDPP<>>(stream,
        PerThreadRead<ND::_2D, uchar3>::build(in.ptr()),
        Crop<>::build(crops),
        Resize<InterpolationType::INTER_LINEAR, AspectRatio::PRESERVE_AR>::build(Size(dw, dh), float3{bg[0], bg[1], bg[2]}),
        Mul<float3>::build(make_<float3>(mul[0], mul[1], mul[2])),
        Sub<float3>::build(make_<float3>(sub[0], sub[1], sub[2])),
        SaturateCast<float3, uchar3>::build(),
        TensorWrite<uchar3>::build(o.ptr()));
}

// Configuration 3.
template <size_t B>
void crop_resize_norm_split(void* stream_, const uint8_t* src, int w, int h, int pitch, const int32_t* rects, int dw, int dh,
                            const float* sub, const float* div, float* out) {
    Stream stream(stream_);
    const auto in = dev2d<uchar3>(src, w, h, pitch);
    Tensor<float> o(out, uint(dw), uint(dh), uint(B), 3, MemType::Device, 0);
    const auto crops = rects_from<B>(rects);
    for (int rep = 0; rep < g_reps; ++rep) executeOperations<TransformDPP<>>(stream,
        PerThreadRead<ND::_2D, uchar3>::build(in.ptr()),
        Crop<>::build(crops),
        Resize<InterpolationType::INTER_LINEAR>::build(Size(dw, dh)),
        ColorConversion<ColorConversionCodes::COLOR_BGR2RGB, float3, float3>::build(),
        Sub<float3>::build(make_<float3>(sub[0], sub[1], sub[2])),
        Div<float3>::build(make_<float3>(div[0], div[1], div[2])),
        TensorSplit<float3>::build(o.ptr()));
}

// Configuration 4.
template <size_t B>
void batch_muladd_sat(void* stream_, const uint8_t* const* srcs, int w, int h, int pitch, const float* mul, const float* add,
                      uint8_t* const* outs, int out_pitch) {
    Stream stream(stream_);
    using PlaneIOp = decltype(PerThreadRead<ND::_2D, uchar3>::build(std::declval<RawPtr<ND::_2D, uchar3>>())
                                  .then(Mul<uchar3, float3, float3>::build(float3{}))
                                  .then(Add<float3>::build(float3{})));
    std::array<PlaneIOp, B> planes{};
    std::array<Ptr2D<uchar3>, B> outPtrs{};
    for (size_t i = 0; i < B; ++i) {
        const auto in = dev2d<uchar3>(srcs[i], w, h, pitch);
        planes[i] = PerThreadRead<ND::_2D, uchar3>::build(in.ptr())
                        .then(Mul<uchar3, float3, float3>::build(make_<float3>(mul[3 * i], mul[3 * i + 1], mul[3 * i + 2])))
                        .then(Add<float3>::build(make_<float3>(add[3 * i], add[3 * i + 1], add[3 * i + 2])));
        outPtrs[i] = dev2d<uchar3>(outs[i], w, h, out_pitch);
    }
    for (int rep = 0; rep < g_reps; ++rep) executeOperations<TransformDPP<>>(stream,
        BatchRead<PlanePolicy::PROCESS_ALL>::build(planes),
        SaturateCast<float3, uchar3>::build(),
        PerThreadWrite<ND::_2D, uchar3>::build(outPtrs));
}

// Configuration 2.
template <typename DPP, size_t... Is>
void add_mul_chain(Stream& stream, const Ptr2D<float>& in, const Ptr2D<float>& out, float addv, float mulv,
                   std::index_sequence<Is...>) {
    const auto pick = [&](auto idx) {
        if constexpr (decltype(idx)::value % 2 == 0) return Add<float>::build(addv);
        else return Mul<float>::build(mulv);
    };
    for (int rep = 0; rep < g_reps; ++rep) executeOperations<DPP>(stream, PerThreadRead<ND::_2D, float>::build(in.ptr()),
                           pick(std::integral_constant<size_t, Is>{})...,
                           PerThreadWrite<ND::_2D, float>::build(out.ptr()));
}

template <size_t N>
void add_mul_n(void* stream_, const float* in, int w, int h, int pitch, float addv, float mulv, float* out, int out_pitch, int tf) {
    Stream stream(stream_);
    const auto i = dev2d<float>(in, w, h, pitch);
    const auto o = dev2d<float>(out, w, h, out_pitch);
    if (tf) add_mul_chain<TransformDPP<ParArch::GPU_AMD, TF::ENABLED>>(stream, i, o, addv, mulv, std::make_index_sequence<N>{});
    else add_mul_chain<TransformDPP<>>(stream, i, o, addv, mulv, std::make_index_sequence<N>{});
}

// Integer-only chain.
template <size_t B>
void crop_swap_u8(void* stream_, const uint8_t* src, int w, int h, int pitch, const int32_t* rects, uint8_t* out) {
    Stream stream(stream_);
    const auto in = dev2d<uchar3>(src, w, h, pitch);
    Tensor<uchar3> o(reinterpret_cast<uchar3*>(out), uint(rects[2]), uint(rects[3]), uint(B), 1, MemType::Device, 0);
    const auto crops = rects_from<B>(rects);
    for (int rep = 0; rep < g_reps; ++rep) executeOperations<TransformDPP<>>(stream,
        PerThreadRead<ND::_2D, uchar3>::build(in.ptr()).then(Crop<>::build(crops)),
        ColorConversion<ColorConversionCodes::COLOR_BGR2RGB, uchar3, uchar3>::build(),
        TensorWrite<uchar3>::build(o.ptr()));
}

} // namespace

// setTo + StaticLoop, spelled like the reference's instruction-count benchmark
// (benchmarks/numinstructions/benchmark_numinstructions_x_operation.h:40-75): library-owned 1-D device arrays are
// filled with setTo, run through StaticLoop<Add<float>, N> and downloaded into `host_out`.
template <int N> void set_and_loop(Stream& stream, int n, float init, float add, float* host_out) {
    Ptr1D<float> in(uint(n), 0, MemType::DeviceAndPinned), out(uint(n), 0, MemType::DeviceAndPinned);
    setTo(init, in, stream);
    setTo(0.f, out, stream);
    constexpr auto singleOp = Add<float>::build(1.f);
    const auto loop = StaticLoop<typename decltype(singleOp)::Operation, N>::build(add);
    executeOperations<TransformDPP<>>(stream, PerThreadRead<ND::_1D, float>::build(in), loop, PerThreadWrite<ND::_1D, float>::build(out));
    out.download(stream);
    stream.sync();
    std::memcpy(host_out, out.ptrPinned().data, size_t(n) * sizeof(float));
}

// Warping<Affine|Perspective> of an image of T into a float image with the same channel count (row-major matrix).
template <WarpType WT, typename T, typename O>
void warp_image(void* stream_, const void* src, int w, int h, int pitch, const float* m, int dw, int dh, void* out, int out_pitch) {
    Stream stream(stream_);
    const auto in = dev2d<T>(src, w, h, pitch);
    const auto o = dev2d<O>(out, dw, dh, out_pitch);
    WarpingParameters<WT> params{};
    constexpr int rows = WT == WarpType::Affine ? 2 : 3;
    for (int r = 0; r < rows; ++r)
        for (int c = 0; c < 3; ++c) params.transformMatrix.data[r][c] = m[r * 3 + c];
    params.dstSize = Size(dw, dh);
    for (int rep = 0; rep < g_reps; ++rep)
        executeOperations<TransformDPP<>>(stream, PerThreadRead<ND::_2D, T>::build(in.ptr()).then(Warping<WT>::build(params)),
                                          PerThreadWrite<ND::_2D, O>::build(o.ptr()));
}

// Deinterlace: mode 1 BLEND, 2 INTER_LINEAR keeping even lines, 3 keeping odd lines.
template <typename T, typename O> void deinterlace_image(void* stream_, const void* src, int w, int h, int pitch, int mode, void* out, int out_pitch) {
    Stream stream(stream_);
    const auto in = dev2d<T>(src, w, h, pitch);
    const auto o = dev2d<O>(out, w, h, out_pitch);
    const auto read = PerThreadRead<ND::_2D, T>::build(in.ptr());
    const auto write = PerThreadWrite<ND::_2D, O>::build(o.ptr());
    for (int rep = 0; rep < g_reps; ++rep) {
        if (mode == 1) executeOperations<TransformDPP<>>(stream, read.then(Deinterlace<DeinterlaceType::BLEND>::build()), write);
        else executeOperations<TransformDPP<>>(stream, read.then(Deinterlace<DeinterlaceType::INTER_LINEAR>::build(
                                                          DeinterlaceParameters<DeinterlaceType::INTER_LINEAR>{mode == 2})), write);
    }
}

extern "C" {

const char* fklcase_last_error(void) { return g_error; }
// The next driver call on this thread enqueues its chain `reps` times back to back (through the full host API
// each time); resets to 1 afterwards.
void fklcase_set_reps(int reps) { g_reps = reps > 0 ? reps : 1; }
// The next driver call on this thread records `first` on `stream` before its first launch and `last` after its last one.
void fklcase_time_next(void* stream, void* first, void* last) { g_timing = Timing{stream, first, last, true, 0}; }
// CLOCK_MONOTONIC at the start of the last timed driver call, in nanoseconds.
long long fklcase_timed_start_ns(void) { return g_timing.start_ns; }

int fklcase_crop_resize_par_u8_b5(void* stream, const uint8_t* src, int w, int h, int pitch, const int32_t* rects, int dw,
                                  int dh, const float* bg, const float* mul, const float* sub, uint8_t* out) {
    return guarded([&] { crop_resize_par_u8<5>(stream, src, w, h, pitch, rects, dw, dh, bg, mul, sub, out); });
}
int fklcase_crop_resize_norm_split_b8(void* stream, const uint8_t* src, int w, int h, int pitch, const int32_t* rects,
                                      int dw, int dh, const float* sub, const float* div, float* out) {
    return guarded([&] { crop_resize_norm_split<8>(stream, src, w, h, pitch, rects, dw, dh, sub, div, out); });
}
int fklcase_crop_resize_norm_split_b64(void* stream, const uint8_t* src, int w, int h, int pitch, const int32_t* rects,
                                       int dw, int dh, const float* sub, const float* div, float* out) {
    return guarded([&] { crop_resize_norm_split<64>(stream, src, w, h, pitch, rects, dw, dh, sub, div, out); });
}
int fklcase_batch_muladd_sat_b4(void* stream, const uint8_t* const* srcs, int w, int h, int pitch, const float* mul,
                                const float* add, uint8_t* const* outs, int out_pitch) {
    return guarded([&] { batch_muladd_sat<4>(stream, srcs, w, h, pitch, mul, add, outs, out_pitch); });
}
int fklcase_batch_muladd_sat_b100(void* stream, const uint8_t* const* srcs, int w, int h, int pitch, const float* mul,
                                  const float* add, uint8_t* const* outs, int out_pitch) {
    return guarded([&] { batch_muladd_sat<100>(stream, srcs, w, h, pitch, mul, add, outs, out_pitch); });
}
int fklcase_add_mul_chain(void* stream, const float* in, int w, int h, int pitch, int n_ops, float addv, float mulv,
                          float* out, int out_pitch, int tf) {
    return guarded([&] {
        switch (n_ops) {
        case 1: add_mul_n<1>(stream, in, w, h, pitch, addv, mulv, out, out_pitch, tf); break;
        case 2: add_mul_n<2>(stream, in, w, h, pitch, addv, mulv, out, out_pitch, tf); break;
        case 3: add_mul_n<3>(stream, in, w, h, pitch, addv, mulv, out, out_pitch, tf); break;
        case 10: add_mul_n<10>(stream, in, w, h, pitch, addv, mulv, out, out_pitch, tf); break;
        case 20: add_mul_n<20>(stream, in, w, h, pitch, addv, mulv, out, out_pitch, tf); break;
        case 30: add_mul_n<30>(stream, in, w, h, pitch, addv, mulv, out, out_pitch, tf); break;
        case 40: add_mul_n<40>(stream, in, w, h, pitch, addv, mulv, out, out_pitch, tf); break;
        case 50: add_mul_n<50>(stream, in, w, h, pitch, addv, mulv, out, out_pitch, tf); break;
        case 100: add_mul_n<100>(stream, in, w, h, pitch, addv, mulv, out, out_pitch, tf); break;
        default: throw std::runtime_error("add_mul_chain: unsupported operation count");
        }
    });
}
// Configuration 5.
int fklcase_nv12_rgb_resize_split(void* stream_, const uint8_t* nv12, int w, int h, int pitch, int dw, int dh, float scale,
                                  float* out) {
    return guarded([&] {
        Stream stream(stream_);
        const Ptr2D<uchar> data(const_cast<uchar*>(nv12), uint(w), uint(h + h / 2), uint(pitch), MemType::Device, 0);
        const Image<PixelFormat::NV12> img(data, uint(w), uint(h));
        Tensor<float> o(out, uint(dw), uint(dh), 1, 3, MemType::Device, 0);
        for (int rep = 0; rep < g_reps; ++rep) executeOperations<TransformDPP<>>(stream,
            ReadYUV<PixelFormat::NV12>::build(img.ptr()),
            ConvertYUVToRGB<ColorDepth::p8bit, ColorRange::Full, ColorPrimitives::bt709>::build(),
            Resize<InterpolationType::INTER_LINEAR>::build(Size(dw, dh)),
            Mul<float3, float>::build(scale),
            TensorSplit<float3>::build(o.ptr()));
    });
}
// Plain pitched copy of a float image: read, no compute operation, write.
int fklcase_copy_f32(void* stream_, const float* in, int w, int h, int pitch, float* out, int out_pitch) {
    return guarded([&] {
        Stream stream(stream_);
        const auto i = dev2d<float>(in, w, h, pitch);
        const auto o = dev2d<float>(out, w, h, out_pitch);
        for (int rep = 0; rep < g_reps; ++rep) executeOperations<TransformDPP<>>(i, o, stream);
    });
}
// Horizontal fusion with fewer live planes than the compiled batch (BatchRead<CONDITIONAL_WITH_DEFAULT>).
int fklcase_crop_resize_default_norm_split_b8(void* stream_, const uint8_t* src, int w, int h, int pitch, const int32_t* rects,
                                              int dw, int dh, int used_planes, const float* def, const float* sub,
                                              const float* div, float* out) {
    return guarded([&] {
        constexpr size_t B = 8;
        Stream stream(stream_);
        const auto in = dev2d<uchar3>(src, w, h, pitch);
        Tensor<float> o(out, uint(dw), uint(dh), uint(B), 3, MemType::Device, 0);
        const auto crops = rects_from<B>(rects);
        std::array<Size, B> sizes{};
        for (auto& s : sizes) s = Size(dw, dh);
        for (int rep = 0; rep < g_reps; ++rep) executeOperations<TransformDPP<>>(stream,
            PerThreadRead<ND::_2D, uchar3>::build(in.ptr())
                .then(Crop<>::build(crops))
                .then(Resize<InterpolationType::INTER_LINEAR>::build(used_planes, make_<float3>(def[0], def[1], def[2]), sizes)),
            ColorConversion<ColorConversionCodes::COLOR_BGR2RGB, float3, float3>::build(),
            Sub<float3>::build(make_<float3>(sub[0], sub[1], sub[2])),
            Div<float3>::build(make_<float3>(div[0], div[1], div[2])),
            TensorSplit<float3>::build(o.ptr()));
    });
}
// executeOperations(std::array<Ptr2D<I>,B>, activeBatch, defaultValue, Tensor<O>, stream, ops...)
int fklcase_batch_default_cast_mul_b4(void* stream_, const uint8_t* const* srcs, int w, int h, int pitch, int active,
                                      const uint8_t* def, const float* mul, float* out) {
    return guarded([&] {
        constexpr size_t B = 4;
        Stream stream(stream_);
        std::array<Ptr2D<uchar3>, B> ins{};
        for (size_t i = 0; i < B; ++i) ins[i] = dev2d<uchar3>(srcs[i], w, h, pitch);
        Tensor<float3> o(reinterpret_cast<float3*>(out), uint(w), uint(h), uint(B), 1, MemType::Device, 0);
        executeOperations<TransformDPP<>>(ins, active, uchar3{def[0], def[1], def[2]}, o, stream,
            Cast<uchar3, float3>::build(),
            Mul<float3>::build(make_<float3>(mul[0], mul[1], mul[2])));
    });
}

int fklcase_set_and_loop_f32(void* stream_, int n, float init, float add, int iterations, float* host_out) {
    return guarded([&] {
        Stream stream(stream_);
        switch (iterations) {
        case 1: set_and_loop<1>(stream, n, init, add, host_out); break;
        case 6: set_and_loop<6>(stream, n, init, add, host_out); break;
        case 50: set_and_loop<50>(stream, n, init, add, host_out); break;
        default: throw std::runtime_error("fklcase_set_and_loop_f32: iterations must be 1, 6 or 50");
        }
    });
}
// setTo on a pitched 2-D uchar3 image and on a float tensor; results downloaded into host buffers.
int fklcase_set_to_shapes(void* stream_, int w, int h, int planes, const uint8_t* v3, float vf, uint8_t* host_img, int* host_pitch,
                          float* host_tensor) {
    return guarded([&] {
        Stream stream(stream_);
        Ptr2D<uchar3> img(uint(w), uint(h), 0, MemType::DeviceAndPinned);
        Tensor<float> t(uint(w), uint(h), uint(planes), 1, MemType::DeviceAndPinned);
        setTo(uchar3{v3[0], v3[1], v3[2]}, img, stream);
        setTo(vf, t, stream);
        img.download(stream);
        t.download(stream);
        stream.sync();
        const auto mirror = img.ptrPinned();    // tightly packed, unlike the pitched device image
        *host_pitch = int(mirror.dims.pitch);
        std::memcpy(host_img, mirror.data, size_t(mirror.dims.pitch) * size_t(h));
        std::memcpy(host_tensor, t.ptrPinned().data, size_t(w) * size_t(h) * size_t(planes) * sizeof(float));
    });
}

// setTo on a transposed tensor (ND::T3D) of `planes` images with `color_planes` channel planes each, filled with a
// sentinel first: host_tensor receives color_planes * planes * h * w floats, as they lie in memory.
int fklcase_set_to_transposed(void* stream_, int w, int h, int planes, int color_planes, float sentinel, float value, float* host_tensor) {
    return guarded([&] {
        Stream stream(stream_);
        TensorT<float> t(uint(w), uint(h), uint(planes), uint(color_planes), MemType::DeviceAndPinned);
        const size_t n = size_t(w) * size_t(h) * size_t(planes) * size_t(color_planes);
        float* mirror = t.ptrPinned().data;
        for (size_t i = 0; i < n; ++i) mirror[i] = sentinel;
        t.upload(stream);
        stream.sync();
        setTo(value, t, stream);
        for (size_t i = 0; i < n; ++i) mirror[i] = sentinel;      // setTo filled the mirror too: only the device copy is checked
        t.download(stream);
        stream.sync();
        std::memcpy(host_tensor, t.ptrPinned().data, n * sizeof(float));
    });
}

// Chains that are NOT in the ahead-of-time list: the library compiles them when it first sees them.
int fklcase_uncompiled_pointwise_f32(void* stream_, const float* in, int w, int h, int pitch, float* out, int out_pitch) {
    return guarded([&] {
        Stream stream(stream_);
        const auto i = dev2d<float>(in, w, h, pitch);
        const auto o = dev2d<float>(out, w, h, out_pitch);
        executeOperations<TransformDPP<>>(stream, PerThreadRead<ND::_2D, float>::build(i.ptr()), Mul<float>::build(1.5f),
                                          Sub<float>::build(0.25f), Div<float>::build(3.f), Add<float>::build(7.f),
                                          PerThreadWrite<ND::_2D, float>::build(o.ptr()));
    });
}
// one-channel uchar image -> crop -> bilinear resize -> Mul -> float image
int fklcase_uncompiled_gray_resize(void* stream_, const uint8_t* in, int w, int h, int pitch, const int32_t* rect, int dw, int dh,
                                   float mul, float* out, int out_pitch) {
    return guarded([&] {
        Stream stream(stream_);
        const auto i = dev2d<uchar>(in, w, h, pitch);
        const auto o = dev2d<float>(out, dw, dh, out_pitch);
        executeOperations<TransformDPP<>>(stream, PerThreadRead<ND::_2D, uchar>::build(i.ptr()),
                                          Crop<>::build(Rect(rect[0], rect[1], rect[2], rect[3])),
                                          Resize<InterpolationType::INTER_LINEAR>::build(Size(dw, dh)), Mul<float>::build(mul),
                                          PerThreadWrite<ND::_2D, float>::build(o.ptr()));
    });
}
// three crops of a uchar3 image -> letterboxed bilinear resize -> Mul -> planar float tensor (a bilinear chain with narrow
// planar output that is not compiled ahead of time: the strip form of the kernel, through the run-time compiler)
int fklcase_uncompiled_letterbox_split_b3(void* stream_, const uint8_t* src, int w, int h, int pitch, const int32_t* rects, int dw, int dh,
                                          const float* bg, const float* mul, float* out) {
    return guarded([&] {
        Stream stream(stream_);
        const auto in = dev2d<uchar3>(src, w, h, pitch);
        Tensor<float> o(out, uint(dw), uint(dh), 3u, 3, MemType::Device, 0);
        const auto crops = rects_from<3>(rects);
        for (int rep = 0; rep < g_reps; ++rep) executeOperations<TransformDPP<>>(stream,
            PerThreadRead<ND::_2D, uchar3>::build(in.ptr()),
            Crop<>::build(crops),
            Resize<InterpolationType::INTER_LINEAR, AspectRatio::PRESERVE_AR>::build(Size(dw, dh), float3{bg[0], bg[1], bg[2]}),
            Mul<float3>::build(make_<float3>(mul[0], mul[1], mul[2])),
            TensorSplit<float3>::build(o.ptr()));
    });
}
// crop of an image of 2-, 4- or 6-byte pixels (uchar2, uchar4, ushort3) -> bilinear resize -> Mul by a scalar -> planar float
// tensor: narrow planar outputs of pixel types other than uchar3 (the strip form's other ways of handling a clamped tap pair)
extern "C++" {
template <typename Px, typename Fx>
void resize_split_of(void* stream_, const void* src, int w, int h, int pitch, const int32_t* rect, int dw, int dh, float mul, float* out) {
    Stream stream(stream_);
    const auto in = dev2d<Px>(src, w, h, pitch);
    Tensor<float> o(out, uint(dw), uint(dh), 1u, cn<Px>, MemType::Device, 0);
    executeOperations<TransformDPP<>>(stream, PerThreadRead<ND::_2D, Px>::build(in.ptr()),
                                      Crop<>::build(Rect(rect[0], rect[1], rect[2], rect[3])),
                                      Resize<InterpolationType::INTER_LINEAR>::build(Size(dw, dh)), Mul<Fx, float, Fx>::build(mul),
                                      TensorSplit<Fx>::build(o.ptr()));
}
}   // extern "C++"
int fklcase_uncompiled_resize_split(void* stream_, int kind, const void* src, int w, int h, int pitch, const int32_t* rect, int dw, int dh,
                                    float mul, float* out) {
    return guarded([&] {
        switch (kind) {
        case 0: resize_split_of<uchar2, float2>(stream_, src, w, h, pitch, rect, dw, dh, mul, out); break;
        case 1: resize_split_of<uchar4, float4>(stream_, src, w, h, pitch, rect, dw, dh, mul, out); break;
        case 2: resize_split_of<ushort3, float3>(stream_, src, w, h, pitch, rect, dw, dh, mul, out); break;
        default: throw std::runtime_error("fklcase_uncompiled_resize_split: kind must be 0 (uchar2), 1 (uchar4) or 2 (ushort3)");
        }
    });
}
// uchar3 image -> crop -> letterboxed bilinear resize in one of the aspect-ratio modes -> float3 image
// (0 PRESERVE_AR, 2 PRESERVE_AR_RN_EVEN, 3 PRESERVE_AR_LEFT: one kernel, the geometry is made on the host)
extern "C++" template <AspectRatio AR>
void letterbox_of(void* stream_, const uint8_t* src, int w, int h, int pitch, const int32_t* rect, int dw, int dh, const float* bg, float* out, int out_pitch) {
    Stream stream(stream_);
    const auto i = dev2d<uchar3>(src, w, h, pitch);
    const auto o = dev2d<float3>(out, dw, dh, out_pitch);
    executeOperations<TransformDPP<>>(stream, PerThreadRead<ND::_2D, uchar3>::build(i.ptr()), Crop<>::build(Rect(rect[0], rect[1], rect[2], rect[3])),
                                      Resize<InterpolationType::INTER_LINEAR, AR>::build(Size(dw, dh), make_<float3>(bg[0], bg[1], bg[2])),
                                      PerThreadWrite<ND::_2D, float3>::build(o.ptr()));
}
int fklcase_letterbox_ar(void* stream_, int ar, const uint8_t* src, int w, int h, int pitch, const int32_t* rect, int dw, int dh,
                         const float* bg, float* out, int out_pitch) {
    return guarded([&] {
        switch (ar) {
        case 0: letterbox_of<AspectRatio::PRESERVE_AR>(stream_, src, w, h, pitch, rect, dw, dh, bg, out, out_pitch); break;
        case 2: letterbox_of<AspectRatio::PRESERVE_AR_RN_EVEN>(stream_, src, w, h, pitch, rect, dw, dh, bg, out, out_pitch); break;
        case 3: letterbox_of<AspectRatio::PRESERVE_AR_LEFT>(stream_, src, w, h, pitch, rect, dw, dh, bg, out, out_pitch); break;
        default: throw std::runtime_error("fklcase_letterbox_ar: ar must be 0, 2 or 3");
        }
    });
}
// float4 image -> bilinear resize -> float4 image (16-byte elements: one access per tap)
int fklcase_uncompiled_float4_resize(void* stream_, const float* in, int w, int h, int pitch, int dw, int dh, float* out, int out_pitch) {
    return guarded([&] {
        Stream stream(stream_);
        const auto i = dev2d<float4>(in, w, h, pitch);
        const auto o = dev2d<float4>(out, dw, dh, out_pitch);
        executeOperations<TransformDPP<>>(stream, PerThreadRead<ND::_2D, float4>::build(i.ptr()),
                                          Resize<InterpolationType::INTER_LINEAR>::build(Size(dw, dh)),
                                          PerThreadWrite<ND::_2D, float4>::build(o.ptr()));
    });
}

int fklcase_warp_u8x3(void* stream, const uint8_t* src, int w, int h, int pitch, const float* m, int perspective, int dw, int dh,
                      float* out, int out_pitch) {
    return guarded([&] {
        if (perspective) warp_image<WarpType::Perspective, uchar3, float3>(stream, src, w, h, pitch, m, dw, dh, out, out_pitch);
        else warp_image<WarpType::Affine, uchar3, float3>(stream, src, w, h, pitch, m, dw, dh, out, out_pitch);
    });
}
int fklcase_warp_f32(void* stream, const float* src, int w, int h, int pitch, const float* m, int perspective, int dw, int dh,
                     float* out, int out_pitch) {
    return guarded([&] {
        if (perspective) warp_image<WarpType::Perspective, float, float>(stream, src, w, h, pitch, m, dw, dh, out, out_pitch);
        else warp_image<WarpType::Affine, float, float>(stream, src, w, h, pitch, m, dw, dh, out, out_pitch);
    });
}

// Other pixel types (compiled on first use): kind 2 uchar4 -> float4, 3 ushort3 -> float3, 4 uchar -> float.
int fklcase_warp_kind(void* stream, int kind, const void* src, int w, int h, int pitch, const float* m, int perspective, int dw, int dh,
                      float* out, int out_pitch) {
    int rc = 0;
    const int g = guarded([&] {
        auto run = [&](auto in_tag, auto out_tag) {
            using T = decltype(in_tag); using O = decltype(out_tag);
            if (perspective) warp_image<WarpType::Perspective, T, O>(stream, src, w, h, pitch, m, dw, dh, out, out_pitch);
            else warp_image<WarpType::Affine, T, O>(stream, src, w, h, pitch, m, dw, dh, out, out_pitch);
        };
        if (kind == 2) run(uchar4{}, float4{});
        else if (kind == 3) run(ushort3{}, float3{});
        else if (kind == 4) run(uchar{}, float{});
        else rc = 2;
    });
    return g ? g : rc;
}

int fklcase_deinterlace_u8x3(void* stream, const uint8_t* src, int w, int h, int pitch, int mode, float* out, int out_pitch) {
    return guarded([&] { deinterlace_image<uchar3, float3>(stream, src, w, h, pitch, mode, out, out_pitch); });
}
int fklcase_deinterlace_f32(void* stream, const float* src, int w, int h, int pitch, int mode, float* out, int out_pitch) {
    return guarded([&] { deinterlace_image<float, float>(stream, src, w, h, pitch, mode, out, out_pitch); });
}

// Single-operation chains for the exhaustive numeric tests.
int fklcase_div_f32(void* stream_, const float* in, int w, int h, int pitch, float d, float* out, int out_pitch) {
    return guarded([&] {
        Stream stream(stream_);
        const auto i = dev2d<float>(in, w, h, pitch);
        const auto o = dev2d<float>(out, w, h, out_pitch);
        executeOperations<TransformDPP<>>(stream, PerThreadRead<ND::_2D, float>::build(i.ptr()), Div<float>::build(d),
                                          PerThreadWrite<ND::_2D, float>::build(o.ptr()));
    });
}
// The division mode word (fkd::Div::Params::fast) that the chain-level pass leaves for "(x - sub) / div" behind three
// kinds of read: 0 a bilinear resize of uchar3 pixels (values bounded by construction), 1 a float image (anything
// may arrive), 2 a letterboxed resize (the background colour is a run-time value).
int fklcase_normalise_mode(int kind, const float* sub, const float* div) {
    using namespace fkd;
    using F3 = Vec<f32, 3>;
    using SubOp = fkd::Sub<F3, F3, F3>;
    using DivOp = fkd::Div<F3, F3, F3>;
    auto run = [&](auto chain_tag) {
        using C = typename decltype(chain_tag)::type;
        typename C::Params p{};
        constexpr int k = int(sizeof(p.ops) > sizeof(Tup<SubOp::Params, DivOp::Params>));   // a Reorder in front or not
        tup_get<k>(p.ops).v = F3{sub[0], sub[1], sub[2]};
        tup_get<k + 1>(p.ops) = DivOp::make(F3{div[0], div[1], div[2]});
        C::finalize(p);
        return int(tup_get<k + 1>(p.ops).fast);
    };
    using Px = Vec<u8, 3>;
    switch (kind) {
    case 0: return run(std::type_identity<Chain<ResizeLinear<1, fkd::Crop<Read2D<Px>>>, OpList<Reorder<F3, 2, 1, 0, 3>, SubOp, DivOp>, fkd::TensorSplit<F3>>>{});
    case 1: return run(std::type_identity<Chain<Read2D<F3>, OpList<SubOp, DivOp>, Write2D<F3>>>{});
    case 2: return run(std::type_identity<Chain<ResizeLinear<0, fkd::Crop<Read2D<Px>>>, OpList<SubOp, DivOp>, fkd::TensorSplit<F3>>>{});
    default: return -1;
    }
}
// How the host would divide by d on the device: 0 generic division, 1 five-instruction sequence, 2 two-instruction
// sequence proven exact for this divisor (fkd::Div).
int fklcase_div_mode(float d) { return fkd::Div<float, float, float>::make(d).fast; }
// The same one-operation chain with the sequence chosen by the caller instead of by the host's proof, through the C
// ABI with a hand-built parameter block: lets a test compare the proof's verdict with what the device really computes.
int fklcase_div_f32_forced(void* stream_, const float* in, int w, int h, int pitch, float d, int mode, float* out, int out_pitch) {
    using DivOp = fkd::Div<float, float, float>;
    using Chain = fkd::Chain<fkd::Read2D<float>, fkd::OpList<DivOp>, fkd::Write2D<float>>;
    Chain::Params p{};
    p.active_w = unsigned(w); p.active_h = unsigned(h); p.active_z = 1;
    p.read = {in, unsigned(w), unsigned(h), unsigned(pitch)};
    p.ops.head = DivOp::make(d);
    if (p.ops.head.fast == 0 && mode != 0) return -2;          // the reciprocals were not computed for this divisor
    p.ops.head.fast = mode;
    p.write = {out, unsigned(w), unsigned(h), unsigned(out_pitch)};
    return fklhip_launch(Chain::name().c_str(), &p, sizeof(p), stream_);
}
int fklcase_div_f32x3(void* stream_, const float* in, int w, int h, int pitch, const float* d, float* out, int out_pitch) {
    return guarded([&] {
        Stream stream(stream_);
        const auto i = dev2d<float3>(in, w, h, pitch);
        const auto o = dev2d<float3>(out, w, h, out_pitch);
        executeOperations<TransformDPP<>>(stream, PerThreadRead<ND::_2D, float3>::build(i.ptr()),
                                          Div<float3>::build(make_<float3>(d[0], d[1], d[2])),
                                          PerThreadWrite<ND::_2D, float3>::build(o.ptr()));
    });
}
int fklcase_saturate_f32_u8(void* stream_, const float* in, int w, int h, int pitch, uint8_t* out, int out_pitch) {
    return guarded([&] {
        Stream stream(stream_);
        const auto i = dev2d<float>(in, w, h, pitch);
        const auto o = dev2d<uchar>(out, w, h, out_pitch);
        executeOperations<TransformDPP<>>(stream, PerThreadRead<ND::_2D, float>::build(i.ptr()), SaturateCast<float, uchar>::build(),
                                          PerThreadWrite<ND::_2D, uchar>::build(o.ptr()));
    });
}
int fklcase_crop_swap_u8_b4(void* stream, const uint8_t* src, int w, int h, int pitch, const int32_t* rects, uint8_t* out) {
    return guarded([&] { crop_swap_u8<4>(stream, src, w, h, pitch, rects, out); });
}

} // extern "C"

// ---- pixel formats and colour conversions (color_chains.h on the GPU) --------------------------------------------
namespace {
using GpuColor = color_chains::Chains<TransformDPP<>, Stream>;
// body() runs once per repetition asked for with fklcase_set_reps (benchmarks time the whole run)
template <typename F> int guarded_rc(F body) {
    int rc = 0;
    const int g = guarded([&] { for (int rep = 0; rep < g_reps && rc == 0; ++rep) rc = body(); });
    return g ? g : rc;
}
} // namespace

extern "C" {

int fklcase_yuv_to_rgb(void* stream_, int pf, int cr, int cp, const void* src, int w, int h, int pitch, float* out, int out_pitch) {
    return guarded_rc([&] { Stream s(stream_); return GpuColor::yuv_to_rgb(s, MemType::Device, pf, cr, cp, src, w, h, pitch, out, out_pitch); });
}
int fklcase_rgb_to_yuv(void* stream_, int pf, int cr, int cp, const void* src, int w, int h, int pitch, void* out, int out_pitch) {
    return guarded_rc([&] { Stream s(stream_); return GpuColor::rgb_to_yuv(s, MemType::Device, pf, cr, cp, src, w, h, pitch, out, out_pitch); });
}
int fklcase_yuv_resize(void* stream_, int pf, const void* src, int w, int h, int pitch, int dw, int dh, float scale, float* out,
                       int out_pitch) {
    return guarded_rc([&] { Stream s(stream_); return GpuColor::yuv_resize(s, MemType::Device, pf, src, w, h, pitch, dw, dh, scale, out, out_pitch); });
}
int fklcase_convert_depth(void* stream_, int cd, int cr, int cp, int to_rgb, const void* src, int w, int h, int pitch, float* out,
                          int out_pitch) {
    return guarded_rc([&] { Stream s(stream_); return GpuColor::convert_depth(s, MemType::Device, cd, cr, cp, to_rgb, src, w, h, pitch, out, out_pitch); });
}
int fklcase_convert_code(void* stream_, int which, const void* src, int w, int h, int pitch, void* out, int out_pitch) {
    return guarded_rc([&] { Stream s(stream_); return GpuColor::convert_code(s, MemType::Device, which, src, w, h, pitch, out, out_pitch); });
}
int fklcase_normalize(void* stream_, int which, const void* src, int w, int h, int pitch, float* out, int out_pitch) {
    return guarded_rc([&] { Stream s(stream_); return GpuColor::normalize(s, MemType::Device, which, src, w, h, pitch, out, out_pitch); });
}
int fklcase_depth_ops(void* stream_, int which, const void* src, int w, int h, int pitch, void* out, int out_pitch, float lo, float hi) {
    return guarded_rc([&] { Stream s(stream_); return GpuColor::depth_ops(s, MemType::Device, which, src, w, h, pitch, out, out_pitch, lo, hi); });
}

} // extern "C"

// ---- per-channel Operations (pointwise_chains.h on the GPU) --------------------------------------------------------
extern "C" int fklcase_pointwise(void* stream_, int which, const void* src, int w, int h, int pitch, void* out, int out_pitch,
                                 const float* c, const float* m) {
    return guarded_rc([&] {
        Stream s(stream_);
        return pointwise_chains::Chains<TransformDPP<>, Stream>::run(s, MemType::Device, which, src, w, h, pitch, out, out_pitch, c, m);
    });
}

extern "C" int fklcase_split_write(void* stream_, int which, const void* src, int w, int h, int pitch, int dw, int dh, void* const* outs,
                                   const int* out_pitch, const float* c) {
    return guarded_rc([&] {
        Stream s(stream_);
        return pointwise_chains::Chains<TransformDPP<>, Stream>::split_write(s, MemType::Device, which, src, w, h, pitch, dw, dh, outs, out_pitch, c);
    });
}

extern "C" int fklcase_dual(void* stream_, int which, const void* a, const void* b, int w, int h, int pitch_a, int pitch_b, void* out,
                            int out_pitch) {
    return guarded_rc([&] {
        Stream s(stream_);
        return pointwise_chains::Chains<TransformDPP<>, Stream>::dual(s, MemType::Device, which, a, b, w, h, pitch_a, pitch_b, out, out_pitch);
    });
}

// ---- padding through BorderReader (border_chains.h on the GPU) ----------------------------------------------------
extern "C" int fklcase_pad(void* stream_, int elem, int border_type, const void* src, int w, int h, int pitch, int left, int top,
                           int out_w, int out_h, const float* value, void* out, int out_pitch) {
    return guarded_rc([&] {
        Stream s(stream_);
        return border_chains::Chains<TransformDPP<>, Stream>::pad(s, MemType::Device, elem, border_type, src, w, h, pitch, left, top, out_w,
                                                                  out_h, value, out, out_pitch);
    });
}

// ---- divergent launches and the CircularTensor window (circular_chains.h on the GPU) -------------------------------
extern "C" {
int fklcase_divergent_two(void* stream_, const uint32_t* a, const uint32_t* b, int w, int h, int pitch, uint32_t add, uint32_t* out) {
    return guarded_rc([&] { Stream s(stream_); circular_chains::Chains<ParArch::GPU_AMD>::divergent_two(s, MemType::Device, a, b, w, h, pitch, add, out); return 0; });
}
int fklcase_divergent_mixed(void* stream_, const float* tensor4, int w, int h, float mul, const uint8_t* img, int iw, int ih, int ipitch, float* out) {
    return guarded_rc([&] { Stream s(stream_); circular_chains::Chains<ParArch::GPU_AMD>::divergent_mixed(s, MemType::Device, tensor4, w, h, mul, img, iw, ih, ipitch, out); return 0; });
}
// images: `iters` device pointers to uchar3 images; states: host memory, iters x batch x 3 x h x w floats
int fklcase_circular(void* stream_, int batch, int oldest_first, const uint8_t* const* images, int iters, int w, int h, int pitch, float fill,
                     float* states) {
    int rc = 0;
    const int g = guarded([&] {
        Stream s(stream_);
        rc = circular_chains::Chains<ParArch::GPU_AMD>::circular(s, batch, oldest_first, images, iters, w, h, pitch, MemType::Device, fill, states);
    });
    return g ? g : rc;
}
// images: `planes` device pointers to uchar3 images; tensor_t (planes x 3 channel planes, transposed) and packed
// (planes x h x w float3) are device memory
int fklcase_transposed_round_trip(void* stream_, const uint8_t* const* images, int planes, int w, int h, int pitch, float mul, float* tensor_t,
                                  float mul2, float* packed) {
    return guarded([&] {
        Stream s(stream_);
        circular_chains::Chains<ParArch::GPU_AMD>::transposed_round_trip(s, MemType::Device, images, planes, w, h, pitch, mul, tensor_t, mul2, packed);
    });
}
int fklcase_circular_transposed(void* stream_, int batch, int oldest_first, const uint8_t* const* images, int iters, int w, int h, int pitch,
                                float fill, float* states) {
    int rc = 0;
    const int g = guarded([&] {
        Stream s(stream_);
        rc = circular_chains::Chains<ParArch::GPU_AMD>::circular_transposed(s, batch, oldest_first, images, iters, w, h, pitch, MemType::Device, fill, states);
    });
    return g ? g : rc;
}
// Benchmark form of the window: an 8-plane float window (NewestFirst, planar), one update per repetition asked for with
// fklcase_set_reps, cycling through the given uchar3 images; nothing is downloaded.  The window lives until `release`.
int fklcase_circular_update_b8(void* stream_, const uint8_t* const* images, int n_images, int w, int h, int pitch, int release) {
    using Window = CircularTensor<float, 3, 8, CircularTensorOrder::NewestFirst, ColorPlanes::Standard>;
    static Window* window = nullptr;
    static int next = 0;
    return guarded([&] {
        if (release) { delete window; window = nullptr; next = 0; return; }
        Stream s(stream_);
        if (!window) { const uint uw = uint(w), uh = uint(h); window = new Window(uw, uh); setTo(0.f, *window, s); }
        for (int rep = 0; rep < g_reps; ++rep) {
            const auto in = dev2d<uchar3>(images[next % n_images], w, h, pitch);
            window->update(s, Read<PerThreadRead<ND::_2D, uchar3>>{in.ptr()}, Unary<SaturateCast<uchar3, float3>>{},
                           Write<TensorSplit<float3>>{window->ptr()});
            ++next;
        }
    });
}
} // extern "C"
