// border_chains.h -- padding chains (read -> BorderReader -> Crop with a rectangle that leaves the image -> write),
// spelled once with the public C++ API of the fused-kernel library and compiled twice, like color_chains.h: against
// this repository's headers for the GPU and against the reference's headers for its CPU backend.
#pragma once

#include <cstdint>
#include <type_traits>

namespace border_chains {

using namespace fk;

template <class DPP, class StreamT> struct Chains {
    template <class T> static Ptr2D<T> wrap(const void* data, int w, int h, int pitch, MemType mem) {
        return Ptr2D<T>(reinterpret_cast<T*>(const_cast<void*>(data)), uint(w), uint(h), uint(pitch), mem, 0);
    }
    // The image grows by `left`/`top` pixels before its origin and to out_w x out_h in all.
    template <BorderType BT, class T>
    static void pad_one(StreamT& s, MemType mem, const void* src, int w, int h, int pitch, int left, int top, int out_w, int out_h,
                        const T& value, void* out, int out_pitch) {
        const auto in = wrap<T>(src, w, h, pitch, mem);
        const auto o = wrap<T>(out, out_w, out_h, out_pitch, mem);
        const auto readIOp = PerThreadRead<ND::_2D, T>::build(in.ptr());
        const Rect rect(uint(-left), uint(-top), out_w, out_h);
        if constexpr (BT == BorderType::CONSTANT) {
            const auto bordered = BorderReader<BT>::build(readIOp, value);
            const auto cropped = Crop<std::decay_t<decltype(bordered)>>::build(bordered, rect);
            executeOperations<DPP>(s, cropped, PerThreadWrite<ND::_2D, T>::build(o.ptr()));
        } else {
            const auto bordered = BorderReader<BT>::build(readIOp);
            const auto cropped = Crop<std::decay_t<decltype(bordered)>>::build(bordered, rect);
            executeOperations<DPP>(s, cropped, PerThreadWrite<ND::_2D, T>::build(o.ptr()));
        }
    }
    template <class T>
    static int pad_t(StreamT& s, MemType mem, int border_type, const void* src, int w, int h, int pitch, int left, int top, int out_w,
                     int out_h, const T& value, void* out, int out_pitch) {
        switch (BorderType(border_type)) {
        case BorderType::CONSTANT: pad_one<BorderType::CONSTANT, T>(s, mem, src, w, h, pitch, left, top, out_w, out_h, value, out, out_pitch); return 0;
        case BorderType::REPLICATE: pad_one<BorderType::REPLICATE, T>(s, mem, src, w, h, pitch, left, top, out_w, out_h, value, out, out_pitch); return 0;
        case BorderType::REFLECT: pad_one<BorderType::REFLECT, T>(s, mem, src, w, h, pitch, left, top, out_w, out_h, value, out, out_pitch); return 0;
        case BorderType::WRAP: pad_one<BorderType::WRAP, T>(s, mem, src, w, h, pitch, left, top, out_w, out_h, value, out, out_pitch); return 0;
        case BorderType::REFLECT_101: pad_one<BorderType::REFLECT_101, T>(s, mem, src, w, h, pitch, left, top, out_w, out_h, value, out, out_pitch); return 0;
        default: return 2;
        }
    }
    // elem: 0 uchar3 images (value = 3 bytes), 1 float images (value = 1 float), 2 uchar4, 3 ushort3, 4 uchar, 5 float3
    static int pad(StreamT& s, MemType mem, int elem, int border_type, const void* src, int w, int h, int pitch, int left, int top,
                   int out_w, int out_h, const float* value, void* out, int out_pitch) {
        if (elem == 0) return pad_t<uchar3>(s, mem, border_type, src, w, h, pitch, left, top, out_w, out_h,
                                            make_<uchar3>(uchar(value[0]), uchar(value[1]), uchar(value[2])), out, out_pitch);
        if (elem == 1) return pad_t<float>(s, mem, border_type, src, w, h, pitch, left, top, out_w, out_h, value[0], out, out_pitch);
        if (elem == 2) return pad_t<uchar4>(s, mem, border_type, src, w, h, pitch, left, top, out_w, out_h,
                                            make_<uchar4>(uchar(value[0]), uchar(value[1]), uchar(value[2]), uchar(value[3])), out, out_pitch);
        if (elem == 3) return pad_t<ushort3>(s, mem, border_type, src, w, h, pitch, left, top, out_w, out_h,
                                             make_<ushort3>(ushort(value[0]), ushort(value[1]), ushort(value[2])), out, out_pitch);
        if (elem == 4) return pad_t<uchar>(s, mem, border_type, src, w, h, pitch, left, top, out_w, out_h, uchar(value[0]), out, out_pitch);
        if (elem == 5) return pad_t<float3>(s, mem, border_type, src, w, h, pitch, left, top, out_w, out_h,
                                            make_<float3>(value[0], value[1], value[2]), out, out_pitch);
        return 2;
    }
};

} // namespace border_chains
