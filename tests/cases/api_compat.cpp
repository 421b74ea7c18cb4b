// api_compat.cpp -- compile-only check that code written against the reference library's public API builds against
// this backend's headers with a plain host compiler, and that host-side fusion produces the same TYPES the
// reference documents (README "Sample code" walk-through; type expectations as in
// utests/core/execution_model/utest_executors.h:36-89 and tests/algorithm/test_crop.h:23-46).
#include <fused_kernel/core/execution_model/memory_operations.h>
#include <fused_kernel/algorithms/basic_ops/arithmetic.h>
#include <fused_kernel/algorithms/basic_ops/cast.h>
#include <fused_kernel/algorithms/basic_ops/set.h>
#include <fused_kernel/algorithms/image_processing/crop.h>
#include <fused_kernel/algorithms/image_processing/color_conversion.h>
#include <fused_kernel/algorithms/image_processing/resize.h>
#include <fused_kernel/algorithms/image_processing/saturate.h>
#include <fused_kernel/algorithms/image_processing/image.h>
#include <fused_kernel/fused_kernel.h>
#include <fused_kernel/core/execution_model/execution_model.h>
#include <fused_kernel/algorithms/algorithms.h>
#include <fused_kernel/core/data/circular_tensor.h>

#include <type_traits>

using namespace fk;

// ---- fusion types -------------------------------------------------------------------------------------------
constexpr RawPtr<ND::_2D, uchar3> input{nullptr, {128, 128, 0}};
constexpr auto readOp = PerThreadRead<ND::_2D, uchar3>::build({input});
constexpr auto cropOp = Crop<>::build(Rect(0, 0, 16, 16));
constexpr auto resizeOp = Resize<InterpolationType::INTER_LINEAR>::build(Size(1024, 1024));
constexpr auto castU3F3 = Cast<uchar3, float3>::build();
constexpr auto mulOpU3 = Mul<uchar3>::build(uchar3{2, 2, 2});
constexpr auto mulOpF3 = Mul<float3>::build(float3{2, 2, 2});
constexpr RawPtr<ND::_2D, float3> outputF3{nullptr, {1024, 1024, 0}};
constexpr auto writeF3 = PerThreadWrite<ND::_2D, float3>::build({outputF3});

static_assert(std::is_same_v<std::decay_t<decltype(readOp)>, Read<PerThreadRead<ND::_2D, uchar3>>>);
static_assert(std::is_same_v<std::decay_t<decltype(cropOp)>, IncompleteReadBack<Crop<>>>);
static_assert(std::is_same_v<std::decay_t<decltype(mulOpF3)>, Binary<Mul<float3, float3, float3, BinaryType>>>);
static_assert(std::is_same_v<std::decay_t<decltype(castU3F3)>, Unary<Cast<uchar3, float3>>>);

// read & crop -> ReadBack<Crop<Read<...>>>
static_assert(std::is_same_v<std::decay_t<decltype(readOp.then(cropOp))>, ReadBack<Crop<std::decay_t<decltype(readOp)>>>>);
static_assert(std::is_same_v<std::decay_t<decltype(readOp & cropOp)>, std::decay_t<decltype(fuse(readOp, cropOp))>>);

void fusion_types() {
    // no read-back in the list: nothing is fused
    const auto t1 = BackFuser::fuse_back(readOp, castU3F3, mulOpF3, writeF3);
    static_assert(std::is_same_v<std::decay_t<decltype(get<0>(t1))>, std::decay_t<decltype(readOp)>>);
    // read, crop, compute, write: the crop is pulled into the read
    const auto t2 = BackFuser::fuse_back(readOp, cropOp, castU3F3, writeF3);
    static_assert(std::is_same_v<std::decay_t<decltype(get<0>(t2))>, ReadBack<Crop<std::decay_t<decltype(readOp)>>>>);
    static_assert(std::tuple_size_v<std::decay_t<decltype(t2)>> == 3);
    // read, crop, compute, resize, ...: everything up to the resize becomes the resize's source
    const auto t3 = BackFuser::fuse_back(readOp, cropOp, mulOpU3, resizeOp, mulOpF3, writeF3);
    using Fused3 = std::decay_t<decltype(get<0>(t3))>;
    using Expected3 = ReadBack<ResizeComplete<AspectRatio::IGNORE_AR, Ternary<InterpolateComplete<InterpolationType::INTER_LINEAR,
        Read<FusedOperation<ReadBack<Crop<Read<PerThreadRead<ND::_2D, uchar3>>>>, Binary<Mul<uchar3>>>>>>>>;
    static_assert(std::is_same_v<Fused3, Expected3>);
    static_assert(Fused3::Operation::BackIOp::Operation::BackIOp::Operation::IS_FUSED_OP);
    (void)t1; (void)t2; (void)t3;
}

void batch_types() {
    constexpr std::array<Rect, 2> crops{Rect(0, 0, 34, 25), Rect(10, 10, 70, 15)};
    const auto batchCrop = Crop<>::build(crops);
    static_assert(std::is_same_v<std::decay_t<decltype(batchCrop)>, Read<BatchRead<PlanePolicy::PROCESS_ALL, 2, TypeList<Crop<>>>>>);
    const auto fused = readOp.then(batchCrop).then(Resize<InterpolationType::INTER_LINEAR>::build(Size(100, 100)));
    using F = std::decay_t<decltype(fused)>;
    static_assert(isBatchOperation<F::Operation> && F::Operation::BATCH == 2);
    const ActiveThreads at = fused.getActiveThreads();   // 100 x 100 x 2, as tests/algorithm/test_crop.h expects
    (void)at;
    static_assert(std::is_same_v<F, Read<BatchRead<PlanePolicy::PROCESS_ALL, 2,
        ResizeComplete<AspectRatio::IGNORE_AR, Ternary<InterpolateComplete<InterpolationType::INTER_LINEAR,
            ReadBack<Crop<Read<PerThreadRead<ND::_2D, uchar3>>>>>>>>>>);
}

// ---- the README program, as written there ------------------------------------------------------------------
void readme_program() {
    Stream stream;
    constexpr Size outputSize(60, 60);
    constexpr int BATCH = 5;
    Ptr2D<uchar3> inputImage(3840, 2160);
    Tensor<float3> output(outputSize.width, outputSize.height, BATCH);
    constexpr std::array<Rect, BATCH> crops{Rect(0, 0, 34, 25), Rect(10, 10, 70, 15), Rect(20, 20, 60, 59),
                                            Rect(30, 30, 20, 23), Rect(40, 40, 12, 11)};
    constexpr float3 backgroundColor{0.f, 0.f, 0.f};
    constexpr float3 mulValue = make_set<float3>(1.4f);
    constexpr float3 subValue = make_set<float3>(0.5f);
    constexpr float3 divValue = make_set<float3>(255.f);
    const auto mySender = PerThreadRead<ND::_2D, uchar3>::build(inputImage)
                              .then(Crop<>::build(crops))
                              .then(Resize<InterpolationType::INTER_LINEAR, AspectRatio::PRESERVE_AR>::build(outputSize, backgroundColor))
                              .then(Mul<float3>::build(mulValue))
                              .then(Sub<float3>::build(subValue))
                              .then(Div<float3>::build(divValue))
                              .then(ColorConversion<ColorConversionCodes::COLOR_RGB2BGR, float3, float3>::build());
    const auto myReceiver = TensorWrite<float3>::build(output);
    executeOperations<fk::TransformDPP<>>(stream, mySender, myReceiver);
    stream.sync();
}

// ---- the compiler-explorer example: executeOperations(input, stream, ops...) --------------------------------
void lts_example() {
    Ptr2D<uchar4> in(1920, 1080);
    std::array<Rect, 5> crops{Rect(0, 0, 120, 40), Rect(100, 200, 60, 40), Rect(400, 20, 30, 50), Rect(1000, 800, 30, 30), Rect(40, 40, 40, 40)};
    Tensor<uchar4> output(64, 64, 5);
    Stream stream;
    executeOperations<TransformDPP<>>(in, stream, Crop<>::build(crops), Resize<InterpolationType::INTER_LINEAR>::build(Size(64, 64)),
                                      Mul<float4>::build(make_set<float4>(1.f / 255.f)), Mul<float4>::build(make_set<float4>(0.33f)),
                                      Add<float4>::build(make_set<float4>(0.5f)), Mul<float4>::build(make_set<float4>(255.f)),
                                      SaturateCast<float4, uchar4>::build(), TensorWrite<uchar4>::build(output));
    stream.sync();
}

// ---- two spellings of read -> crop -> resize -> mul, and the (input, output, stream, ops...) overload --------
void two_spellings() {
    Stream stream;
    Ptr2D<float2> in(1920, 1080), out1(16, 16), out2(16, 16);
    in.at(3, 4) = make_<float2>(3.f, 4.f);
    in.upload(stream);
    const auto r = PerThreadRead<ND::_2D, float2>::build(in);
    const auto c = Crop<>::build(Rect(128, 256, 64, 64));
    const auto z = Resize<InterpolationType::INTER_LINEAR>::build(Size(16, 16));
    const auto m = Mul<float2>::build(make_<float2>(3.f, 5.f));
    Executor<TransformDPP<>>::executeOperations(stream, r, c, z, m, PerThreadWrite<ND::_2D, float2>::build(out1));
    Executor<TransformDPP<>>::executeOperations(stream, r.then(c).then(z), m, PerThreadWrite<ND::_2D, float2>::build(out2));
    out1.download(stream);
    stream.sync();
    Ptr2D<float> a(64, 64), b(64, 64);
    executeOperations<TransformDPP<ParArch::GPU_AMD, TF::ENABLED>>(a, b, stream, Add<float>::build(0.5f), Mul<float>::build(2.f));
    const bool same = out1.at(0, 0) == out2.at(0, 0);
    (void)same;
}

// ---- horizontal fusion over separate images, NV12 --------------------------------------------------------------
void batch_and_video() {
    Stream stream;
    std::array<Ptr2D<uchar3>, 3> ins{Ptr2D<uchar3>(64, 32), Ptr2D<uchar3>(64, 32), Ptr2D<uchar3>(64, 32)};
    std::array<Ptr2D<uchar3>, 3> outs{Ptr2D<uchar3>(64, 32), Ptr2D<uchar3>(64, 32), Ptr2D<uchar3>(64, 32)};
    executeOperations<TransformDPP<>>(ins, stream, Cast<uchar3, float3>::build(), Mul<float3>::build(make_set<float3>(2.f)),
                                      SaturateCast<float3, uchar3>::build(), PerThreadWrite<ND::_2D, uchar3>::build(outs));
    Tensor<float3> t(64, 32, 3);
    executeOperations<TransformDPP<>>(ins, t, stream, Cast<uchar3, float3>::build());
    Image<PixelFormat::NV12> frame(256, 128);
    Tensor<float> planar(128, 64, 1, 3);
    executeOperations<TransformDPP<>>(stream, ReadYUV<PixelFormat::NV12>::build(frame),
                                      ConvertYUVToRGB<ColorDepth::p8bit, ColorRange::Full, ColorPrimitives::bt709>::build(),
                                      Resize<InterpolationType::INTER_LINEAR>::build(Size(128, 64)), Mul<float3, float>::build(1.f / 255.f),
                                      TensorSplit<float3>::build(planar));
    stream.sync();
}

// ---- setTo, StaticLoop and the activeBatch/defaultValue overloads, as the reference's benchmarks spell them ------
// (benchmarks/numinstructions/benchmark_numinstructions_x_operation.h:40-75, executors.h:80-100)
#include <fused_kernel/algorithms/basic_ops/static_loop.h>
#include <fused_kernel/core/data/ptr_utils.h>
constexpr auto singleOp = fk::Add<float>::build(1.f);
constexpr auto allInstr = fk::StaticLoop<typename decltype(singleOp)::Operation, 50>::build(1.f);
static_assert(std::is_same_v<std::decay_t<decltype(allInstr)>, fk::Binary<fk::StaticLoop<fk::Add<float>, 50>>>);
void set_loop_and_conditional_batch() {
    using namespace fk;
    Stream stream;
    Ptr1D<float> in(1024), out(1024);
    setTo(1.f, in, stream);
    setTo(0.f, out, stream);
    executeOperations<TransformDPP<>>(stream, PerThreadRead<ND::_1D, float>::build(in), allInstr,
                                      PerThreadWrite<ND::_1D, float>::build(out));
    Ptr2D<uchar> img(60, 120);
    setTo(uchar(10), img, stream);
    std::array<Ptr2D<uchar3>, 4> ins{Ptr2D<uchar3>(64, 32), Ptr2D<uchar3>(64, 32), Ptr2D<uchar3>(64, 32), Ptr2D<uchar3>(64, 32)};
    Tensor<float3> t(64, 32, 4);
    executeOperations<TransformDPP<>>(ins, 2, uchar3{1, 2, 3}, t, stream, Cast<uchar3, float3>::build());
    stream.sync();
}

// ---- Warping, as the reference's own test spells it (tests/algorithm/test_warp.h:20-33) -------------------------
#include <fused_kernel/algorithms/image_processing/warping.h>
constexpr auto warpReadIOp = fk::PerThreadRead<fk::ND::_2D, uchar3>::build(
    fk::RawPtr<fk::ND::_2D, uchar3>{nullptr, {128, 128, 128 * sizeof(uchar3)}});
constexpr auto warpIOp = fk::Warping<fk::WarpType::Perspective>::build(fk::WarpingParameters<fk::WarpType::Perspective>{});
constexpr auto warpFusedIOp = warpReadIOp.then(warpIOp);
static_assert(std::is_same_v<std::decay_t<decltype(warpFusedIOp)>,
                             fk::ReadBack<fk::Warping<fk::WarpType::Perspective, fk::Read<fk::PerThreadRead<fk::ND::_2D, uchar3>>>>>,
              "Unexpected type for fusedIOp");

// ---- BorderReader, as the reference's own test spells it (tests/algorithm/test_border_reader.h:16-24), plus the
// forms that complete later (.then) ---------------------------------------------------------------------------
#include <fused_kernel/algorithms/image_processing/border_reader.h>
constexpr auto borderReadIOp = fk::PerThreadRead<fk::ND::_2D, uchar3>::build(
    fk::RawPtr<fk::ND::_2D, uchar3>{nullptr, {128, 128, 128 * sizeof(uchar3)}});
constexpr auto borderIOp = fk::BorderReader<fk::BorderType::CONSTANT>::build(borderReadIOp, fk::make_set<uchar3>(0));
static_assert(std::is_same_v<std::decay_t<decltype(borderIOp)>,
                             fk::ReadBack<fk::BorderReader<fk::BorderType::CONSTANT, fk::BorderReaderParameters<fk::BorderType::CONSTANT, uchar3>,
                                                           fk::Read<fk::PerThreadRead<fk::ND::_2D, uchar3>>>>>,
              "Unexpected type for borderIOp");
constexpr auto reflectLater = borderReadIOp.then(fk::BorderReader<fk::BorderType::REFLECT_101>::build());
static_assert(std::is_same_v<std::decay_t<decltype(reflectLater)>,
                             fk::ReadBack<fk::BorderReader<fk::BorderType::REFLECT_101, fk::BorderReaderParameters<fk::BorderType::REFLECT_101>,
                                                           fk::Read<fk::PerThreadRead<fk::ND::_2D, uchar3>>>>>);
constexpr auto constantLater = borderReadIOp.then(fk::BorderReader<fk::BorderType::CONSTANT>::build(fk::make_set<float3>(1.f)));
static_assert(std::is_same_v<std::decay_t<decltype(constantLater)>, std::decay_t<decltype(borderIOp)>>,
              "a border value of another type is converted to the pixels' type");

// ---- Colour vocabulary: every conversion code names a type, every built pixel format has a reader and a writer ----
static_assert(std::is_same_v<fk::ColorConversion<fk::ColorConversionCodes::COLOR_RGB2GRAY, uchar3, uchar>, fk::RGB2Gray<uchar3, uchar>>);
static_assert(std::is_same_v<fk::ColorConversion<fk::ColorConversionCodes::COLOR_BGR2BGRA, uchar3, uchar4>, fk::AddOpaqueAlpha<uchar3, fk::ColorDepth::p8bit>>);
static_assert(std::is_same_v<decltype(fk::ReadYUV<fk::PixelFormat::UYVY>::build(fk::RawImage<fk::PixelFormat::UYVY>{})),
                             fk::Read<fk::ReadYUV<fk::PixelFormat::UYVY>>>);
static_assert(std::is_same_v<decltype(fk::WriteYUV<fk::PixelFormat::P010>::build(fk::RawImage<fk::PixelFormat::P010>{})),
                             fk::Write<fk::WriteYUV<fk::PixelFormat::P010>>>);
static_assert(fk::maxDepthValue<fk::ColorDepth::p10bit> == 1023 && fk::maxDepthValue<fk::ColorDepth::fn12bit> == 1.f);

// ---- A user-defined Operation, declared the way the reference documents it (Parent + DECLARE_*_PARENT + exec):
// it builds, fuses and type-checks on the host; launching it needs fk::amd::Lower<> (checked by tests/test_abi.py, which
// compiles this file a second time with FK_API_COMPAT_LAUNCH_USER_OP and expects the explanatory static_assert) --------
#include <fused_kernel/core/execution_model/operation_model/parent_operations.h>
#include <fused_kernel/core/execution_model/thread_fusion.h>
#include <fused_kernel/core/utils/vlimits.h>
namespace user_ops {
template <typename I, typename O> struct Twice {
private:
    using SelfType = Twice<I, O>;
public:
    FK_STATIC_STRUCT(Twice, SelfType)
    using Parent = fk::UnaryOperation<I, O, Twice<I, O>>;
    DECLARE_UNARY_PARENT
    FK_HOST_DEVICE_FUSE OutputType exec(const InputType& input) { return static_cast<O>(input * 2); }
};
template <typename I, typename P = I, typename O = I> struct AddThrice {
private:
    using SelfType = AddThrice<I, P, O>;
public:
    FK_STATIC_STRUCT(AddThrice, SelfType)
    using Parent = fk::BinaryOperation<I, P, O, AddThrice<I, P, O>>;
    DECLARE_BINARY_PARENT
    FK_HOST_DEVICE_FUSE OutputType exec(const InputType& input, const ParamsType& params) { return input + params * 3; }
};
} // namespace user_ops
static_assert(user_ops::Twice<int, float>::exec(4) == 8.f);
constexpr auto userBinary = user_ops::AddThrice<float>::build(2.f);
static_assert(user_ops::AddThrice<float>::exec(1.f, userBinary) == 7.f);
static_assert(fk::opIs<fk::UnaryType, decltype(user_ops::Twice<int, float>::build())> && fk::opIs<fk::BinaryType, decltype(userBinary)>);
constexpr auto userFused = fk::PerThreadRead<fk::ND::_2D, float>::build(fk::RawPtr<fk::ND::_2D, float>{nullptr, {8, 8, 32}}).then(userBinary);
static_assert(fk::opIs<fk::ReadType, decltype(userFused)>, "a user-defined Operation fuses onto a read like any other");
#ifdef FK_API_COMPAT_LAUNCH_USER_OP
inline void launch_user_op(fk::Stream& s, const fk::Ptr2D<float>& a, const fk::Ptr2D<float>& b) {
    fk::executeOperations<fk::TransformDPP<>>(s, fk::PerThreadRead<fk::ND::_2D, float>::build(a), userBinary,
                                              fk::PerThreadWrite<fk::ND::_2D, float>::build(b));
}
#endif

// ---- Thread-fusion type arithmetic and numeric limits, the reference's answers --------------------------------------
static_assert(fk::ThreadFusionInfo<uchar, uchar, true>::elems_per_thread == 4 && fk::ThreadFusionInfo<float, float, true>::elems_per_thread == 2);
static_assert(fk::ThreadFusionInfo<uchar3, uchar3, true>::elems_per_thread == 1 && fk::ThreadFusionInfo<double, double, true>::elems_per_thread == 1);
static_assert(std::is_same_v<fk::ThreadFusionInfo<float, float, true>::BiggerReadType, float2> &&
              std::is_same_v<fk::ThreadFusionInfo<uchar2, uchar2, true>::BiggerWriteType, uchar4>);
static_assert(!fk::ThreadFusionInfo<uchar, float3, true>::ENABLED && fk::ThreadFusionInfo<uchar, float3, true>::elems_per_thread == 1,
              "four fused reads times three channels is no vector type: fusion is off");
static_assert(fk::isThreadFusionEnabled<true, fk::Read<fk::PerThreadRead<fk::ND::_2D, float>>, fk::Write<fk::PerThreadWrite<fk::ND::_2D, float>>>());
static_assert(!fk::isThreadFusionEnabled<true, fk::Read<fk::PerThreadRead<fk::ND::_2D, float3>>, fk::Write<fk::TensorSplit<float3>>>(),
              "a planar split never fuses threads");
static_assert(fk::maxValue<uchar> == 255 && fk::minValue<float3>.y == -3.402823466e+38f);

// ---- Depth operations and transposed tensors: the reference's types ---------------------------------------------------
static_assert(std::is_same_v<fk::DenormalizePixel<uchar3, fk::ColorDepth::p8bit>::InputType, float3> &&
              std::is_same_v<fk::DenormalizePixel<uchar3, fk::ColorDepth::p8bit>::OutputType, uchar3>);
static_assert(std::is_same_v<fk::SaturateDenormalizePixel<float4, ushort4, fk::ColorDepth::p10bit>::OutputType, ushort4>);
static_assert(std::is_same_v<fk::Saturate<float3>::ParamsType, float2> && fk::opIs<fk::BinaryType, decltype(fk::Saturate<float>::build(float2{0.f, 1.f}))>);
static_assert(fk::opIs<fk::UnaryType, decltype(fk::SaturateDepth<float, fk::ColorDepth::p12bit>::build())>);
static_assert(std::is_same_v<fk::TensorTSplit<float3>::ParamsType, fk::RawPtr<fk::ND::T3D, float>> &&
              std::is_same_v<fk::TensorTPack<float3>::OutputType, float3> && !fk::TensorTSplit<float3>::THREAD_FUSION);
static_assert(std::is_base_of_v<fk::TensorT<float>, fk::CircularTensor<float, 3, 4, fk::CircularTensorOrder::NewestFirst, fk::ColorPlanes::Transposed>> &&
              std::is_base_of_v<fk::Tensor<float>, fk::CircularTensor<float, 3, 4, fk::CircularTensorOrder::NewestFirst, fk::ColorPlanes::Standard>>);

// ---- Two-image chains, SplitWrite and the per-channel Operations: the reference's types -------------------------------
#include <fused_kernel/algorithms/basic_ops/basic_ops.h>
static_assert(std::is_same_v<fk::DualSourceRead<fk::ND::_2D, uchar3>::OutputType, fk::Tuple<uchar3, uchar3>> &&
              fk::opIs<fk::ReadType, fk::DualSourceRead<fk::ND::_2D, uchar3>> && !fk::DualSourceRead<fk::ND::_2D, uchar3>::THREAD_FUSION);
static_assert(std::is_same_v<fk::Add<uchar3, uchar3, int3, fk::UnaryType>::InputType, fk::Tuple<uchar3, uchar3>> &&
              fk::opIs<fk::UnaryType, fk::Add<uchar3, uchar3, int3, fk::UnaryType>> && fk::opIs<fk::BinaryType, fk::Add<float>>);
static_assert(fk::opIs<fk::UnaryType, fk::AbsDiff<float, float, float, fk::UnaryType>> && fk::opIs<fk::BinaryType, fk::AbsDiff<float>> &&
              fk::opIs<fk::UnaryType, fk::BwNot<uint>> && fk::opIs<fk::BinaryType, fk::ShiftLeft<uint>> && fk::opIs<fk::BinaryType, fk::Max<float3>>);
static_assert(std::is_same_v<fk::SplitWrite<fk::ND::_2D, float3>::InputType, float3> && fk::opIs<fk::WriteType, fk::SplitWrite<fk::ND::_2D, float3>> &&
              std::is_same_v<decltype(fk::SplitWriteParams<fk::ND::_2D, uchar4>::w), fk::RawPtr<fk::ND::_2D, uchar>>);
static_assert(std::is_same_v<fk::MxVFloat3<>::ParamsType, fk::M3x3Float> && std::is_same_v<fk::Sqrt<uchar3, float3>::OutputType, float3>);
constexpr auto twoImages = fk::DualSourceRead<fk::ND::_2D, float>::build(fk::DualSourceReadParams<fk::ND::_2D, float>{
    fk::RawPtr<fk::ND::_2D, float>{nullptr, {8, 8, 32}}, fk::RawPtr<fk::ND::_2D, float>{nullptr, {8, 8, 32}}});
constexpr auto summed = twoImages.then(fk::Add<float, float, float, fk::UnaryType>::build()).then(fk::Mul<float>::build(0.5f));
static_assert(fk::opIs<fk::ReadType, decltype(summed)>, "the two-input form fuses onto the read of two images");

// ---- A batch whose parameters would not fit the by-value kernel arguments: tests/test_abi.py compiles this file once more
// with FK_API_COMPAT_HUGE_BATCH and expects the static_assert that names FKLHIP_MAX_BLOB_BYTES (reference: every plane of a
// BatchRead carries its own parameters, FK/core/execution_model/operation_model/batch_operations.h:164-219) ----------
#ifdef FK_API_COMPAT_HUGE_BATCH
inline void launch_huge_batch(fk::Stream& s, const std::array<fk::Ptr2D<uchar3>, 45000>& in, const std::array<fk::Ptr2D<uchar3>, 45000>& out) {
    fk::executeOperations<fk::TransformDPP<>>(s, fk::PerThreadRead<fk::ND::_2D, uchar3>::build(in), fk::PerThreadWrite<fk::ND::_2D, uchar3>::build(out));
}
#endif
