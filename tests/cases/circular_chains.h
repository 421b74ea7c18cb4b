// circular_chains.h -- a DivergentBatchTransformDPP launch and the CircularTensor temporal window, spelled once with
// the public C++ API of the fused-kernel library and compiled twice, like color_chains.h: against this repository's
// headers for the GPU and against the reference's headers for its CPU backend.
#pragma once

#include <array>
#include <cstdint>
#include <cstring>

namespace circular_chains {

using namespace fk;

// Plane z runs sequence z (the selector of the reference's own test, tests/data_parallel_patterns/test_divergent_batch.h).
struct OneToOne {
    FK_HOST_DEVICE_FUSE uint at(const uint& zIdx) { return zIdx; }
};
// Planes 0 and 3 run sequence 0, planes 1 and 2 sequence 1.
struct OuterInner {
    FK_HOST_DEVICE_FUSE uint at(const uint& zIdx) { return (zIdx == 0 || zIdx == 3) ? 0u : 1u; }
};

template <ParArch PA> struct Chains {
    using StreamT = Stream_<PA>;
    template <class T> static Ptr2D<T> wrap(const void* data, int w, int h, int pitch, MemType mem) {
        return Ptr2D<T>(reinterpret_cast<T*>(const_cast<void*>(data)), uint(w), uint(h), uint(pitch), mem, 0);
    }

    // Two images into a two-plane tensor: plane 0 = a + add, plane 1 = b (the reference's divergent-batch test).
    static void divergent_two(StreamT& s, MemType mem, const uint32_t* a, const uint32_t* b, int w, int h, int pitch, uint32_t add, uint32_t* out) {
        const auto ia = wrap<uint>(a, w, h, pitch, mem), ib = wrap<uint>(b, w, h, pitch, mem);
        Tensor<uint> o(reinterpret_cast<uint*>(out), uint(w), uint(h), 2, 1, mem, 0);
        auto opSeq1 = buildOperationSequence(Read<PerThreadRead<ND::_2D, uint>>{ia.ptr()}, Binary<Add<uint>>{add},
                                             Write<PerThreadWrite<ND::_3D, uint>>{o.ptr()});
        auto opSeq2 = buildOperationSequence(Read<PerThreadRead<ND::_2D, uint>>{ib.ptr()}, Write<PerThreadWrite<ND::_3D, uint>>{o.ptr()});
        executeOperations<DivergentBatchTransformDPP<PA, OneToOne>>(s, opSeq1, opSeq2);
    }

    // Sequences of different element types, shapes and plane counts in one launch: a float tensor of two planes scaled
    // into planes 0 and 3 of the output, a smaller uchar3 image resized into planes 1 and 2 (each sequence sees the
    // launch's plane index, so its own reads must make sense of it: the tensor read below is given four planes).
    static void divergent_mixed(StreamT& s, MemType mem, const float* tensor4, int w, int h, float mul, const uint8_t* img, int iw, int ih,
                                int ipitch, float* out) {
        Tensor<float3> t(reinterpret_cast<float3*>(const_cast<float*>(tensor4)), uint(w), uint(h), 4, 1, mem, 0);
        auto view = t.ptr();
        view.dims.planes = 2;      // this sequence declares two of the launch's four planes
        Tensor<float3> o(reinterpret_cast<float3*>(out), uint(w), uint(h), 4, 1, mem, 0);
        const auto im = wrap<uchar3>(img, iw, ih, ipitch, mem);
        auto seqA = buildOperationSequence(Read<TensorRead<float3>>{view}, Binary<Mul<float3, float>>{mul}, Write<TensorWrite<float3>>{o.ptr()});
        auto view2 = im.ptr();
        auto seqB = buildOperationSequence(PerThreadRead<ND::_2D, uchar3>::build(view2), Resize<InterpolationType::INTER_LINEAR>::build(Size(w, h)),
                                           Write<TensorWrite<float3>>{o.ptr()});
        // seqB declares one plane (a 2-D read); a second 2-D sequence brings the launch to four planes
        executeOperations<DivergentBatchTransformDPP<PA, OuterInner>>(s, seqA, seqB, seqB);
    }

    // The reference's CircularTensor test scenario on caller-supplied images: the tensor starts at `fill`, then every
    // image goes through update(read -> SaturateCast<uchar3, float3> -> TensorSplit); after each update the whole
    // tensor is copied to `states` (iters x BATCH x 3 x h x w floats, host memory).
    // A transposed tensor over caller-owned memory: planes * 3 channel planes of w x h floats, tightly packed, all first
    // channel planes first.
    static PtrT3D<float> wrap_t(const float* data, int w, int h, int planes, MemType mem) {
        PtrDims<ND::T3D> d(uint(w), uint(h), uint(planes), 3);
        d.pitch = uint(w) * uint(sizeof(float));
        d.plane_pitch = d.pitch * uint(h);
        d.color_planes_pitch = d.plane_pitch * uint(planes);
        return PtrT3D<float>(const_cast<float*>(data), d, mem, 0);
    }
    // uchar3 images -> Cast -> Mul -> TensorTSplit<float3>: image z into plane z of a transposed tensor of `planes` planes
    // (one launch per image, each through a view of one plane), then the tensor back as float3 pixels * mul2 through
    // TensorTPack<float3> into an ordinary tensor.
    static void transposed_round_trip(StreamT& s, MemType mem, const uint8_t* const* images, int planes, int w, int h, int pitch, float mul,
                                      float* tensor_t, float mul2, float* packed) {
        const auto t = wrap_t(tensor_t, w, h, planes, mem);
        for (int z = 0; z < planes; ++z) {
            const auto in = wrap<uchar3>(images[z], w, h, pitch, mem);
            auto view = t.ptr();
            view.data = PtrAccessor<ND::T3D>::point(Point{0, 0, z}, t.ptr());    // plane z; the channel planes keep their distance
            executeOperations<TransformDPP<PA>>(s, PerThreadRead<ND::_2D, uchar3>::build(in.ptr()), Cast<uchar3, float3>::build(),
                                                Binary<Mul<float3, float>>{mul}, Write<TensorTSplit<float3>>{view});
        }
        Tensor<float3> o(reinterpret_cast<float3*>(packed), uint(w), uint(h), uint(planes), 1, mem, 0);
        executeOperations<TransformDPP<PA>>(s, Read<TensorTPack<float3>>{t.ptr()}, Binary<Mul<float3, float>>{mul2}, Write<TensorWrite<float3>>{o.ptr()});
    }

    // circular_one with ColorPlanes::Transposed: update(read -> SaturateCast -> TensorTSplit); `states` has the layout of
    // circular_one's (iters x BATCH x 3 x h x w), gathered from the transposed window.  Only colour plane 0 is filled
    // before the first update (the reference's setTo reaches no other plane of a transposed tensor).
    template <int BATCH, CircularTensorOrder ORDER>
    static void circular_transposed_one(StreamT& s, const uint8_t* const* images, int iters, int w, int h, int pitch, MemType mem, float fill, float* states) {
        const uint width = uint(w), height = uint(h);
        CircularTensor<float, 3, BATCH, ORDER, ColorPlanes::Transposed> window(width, height, mem == MemType::Host ? MemType::Host : defaultMemType);
        setTo(fill, window, s);
        const size_t plane = size_t(w) * size_t(h) * 3;
        for (int i = 0; i < iters; ++i) {
            const auto in = wrap<uchar3>(images[i], w, h, pitch, mem);
            window.update(s, Read<PerThreadRead<ND::_2D, uchar3>>{in.ptr()}, Unary<SaturateCast<uchar3, float3>>{},
                          Write<TensorTSplit<float3>>{window.ptr()});
            window.download(s);
            s.sync();
            const RawPtr<ND::T3D, float> host = mem == MemType::Host ? window.ptr() : window.ptrPinned();
            for (int z = 0; z < BATCH; ++z)
                for (int c = 0; c < 3; ++c)
                    for (int y = 0; y < h; ++y)
                        std::memcpy(states + (size_t(i) * BATCH + z) * plane + (size_t(c) * h + y) * w,
                                    PtrAccessor<ND::T3D>::cr_point(Point{0, y, z}, host, uint(c)), size_t(w) * sizeof(float));
        }
    }
    static int circular_transposed(StreamT& s, int batch, int oldest_first, const uint8_t* const* images, int iters, int w, int h, int pitch,
                                   MemType mem, float fill, float* states) {
        constexpr auto NF = CircularTensorOrder::NewestFirst, OF = CircularTensorOrder::OldestFirst;
#define CIRCULAR_CASE(B) case B: if (oldest_first) circular_transposed_one<B, OF>(s, images, iters, w, h, pitch, mem, fill, states); \
                                 else circular_transposed_one<B, NF>(s, images, iters, w, h, pitch, mem, fill, states); return 0;
        switch (batch) {
            CIRCULAR_CASE(2) CIRCULAR_CASE(3) CIRCULAR_CASE(5)
        default: return 2;
        }
#undef CIRCULAR_CASE
    }

    template <int BATCH, CircularTensorOrder ORDER>
    static void circular_one(StreamT& s, const uint8_t* const* images, int iters, int w, int h, int pitch, MemType mem, float fill, float* states) {
        const uint width = uint(w), height = uint(h);
        // the window lives where the caller's images do (a host build of the reference has no other memory anyway)
        CircularTensor<float, 3, BATCH, ORDER, ColorPlanes::Standard> window(width, height, mem == MemType::Host ? MemType::Host : defaultMemType);
        setTo(fill, window, s);
        const size_t plane = size_t(w) * size_t(h) * 3;
        for (int i = 0; i < iters; ++i) {
            const auto in = wrap<uchar3>(images[i], w, h, pitch, mem);
            window.update(s, Read<PerThreadRead<ND::_2D, uchar3>>{in.ptr()}, Unary<SaturateCast<uchar3, float3>>{},
                          Write<TensorSplit<float3>>{window.ptr()});
            window.download(s);
            s.sync();
            for (int z = 0; z < BATCH; ++z)
                for (int c = 0; c < 3; ++c)
                    for (int y = 0; y < h; ++y) {
                        const RawPtr<ND::_3D, float> host = mem == MemType::Host ? window.ptr() : window.ptrPinned();
                        const char* row = reinterpret_cast<const char*>(host.data) + size_t(host.dims.plane_pitch) * host.dims.color_planes * z +
                                          size_t(host.dims.pitch) * (size_t(c) * h + y);
                        std::memcpy(states + (size_t(i) * BATCH + z) * plane + (size_t(c) * h + y) * w, row, size_t(w) * sizeof(float));
                    }
        }
    }
    static int circular(StreamT& s, int batch, int oldest_first, const uint8_t* const* images, int iters, int w, int h, int pitch, MemType mem,
                        float fill, float* states) {
        constexpr auto NF = CircularTensorOrder::NewestFirst, OF = CircularTensorOrder::OldestFirst;
#define CIRCULAR_CASE(B) case B: if (oldest_first) circular_one<B, OF>(s, images, iters, w, h, pitch, mem, fill, states); \
                                 else circular_one<B, NF>(s, images, iters, w, h, pitch, mem, fill, states); return 0;
        switch (batch) {
            CIRCULAR_CASE(2) CIRCULAR_CASE(3) CIRCULAR_CASE(4) CIRCULAR_CASE(15)
        default: return 2;
        }
#undef CIRCULAR_CASE
    }
};

} // namespace circular_chains
