// fkd/types.hpp -- value types shared by the host lowering layer and the gfx950 device code.
//
// Everything here is plain C++17 with standard-layout types only, so a parameter block assembled by the host
// compiler (g++/clang++) has byte-for-byte the layout the device compiler (hipcc) expects.  Device-only code is
// fenced by FKD_DEVICE_CODE (defined by the HIP translation units); host-only naming helpers by FKD_HOST_NAMES.
#pragma once

#if defined(__HIPCC_RTC__)
// Run-time compilation has no C library headers: name the fixed-width types through the compiler's own macros.
typedef __UINT8_TYPE__ uint8_t;
typedef __INT8_TYPE__ int8_t;
typedef __UINT16_TYPE__ uint16_t;
typedef __INT16_TYPE__ int16_t;
typedef __UINT32_TYPE__ uint32_t;
typedef __INT32_TYPE__ int32_t;
typedef __UINTPTR_TYPE__ uintptr_t;
typedef __PTRDIFF_TYPE__ ptrdiff_t;
typedef __SIZE_TYPE__ size_t;
#else
#include <stddef.h>
#include <stdint.h>
#endif

#if defined(FKD_DEVICE_CODE)
#define FKD_DEV __device__ __forceinline__
#define FKD_HD __host__ __device__ __forceinline__
#else
#define FKD_DEV inline
#define FKD_HD inline
#endif

#if !defined(FKD_NO_NAMES)
#include <string>
#define FKD_HOST_NAMES 1
#endif

namespace fkd {

using u8 = uint8_t;
using i8 = int8_t;
using u16 = uint16_t;
using i16 = int16_t;
using u32 = uint32_t;
using i32 = int32_t;
using f32 = float;
using f64 = double;

// N-channel element.  One-channel elements are the bare scalar type.
template <class T, int N> struct Vec;
template <class T> struct Vec<T, 2> { T x, y; };
template <class T> struct Vec<T, 3> { T x, y, z; };
template <class T> struct Vec<T, 4> { T x, y, z, w; };

template <class T, int N> struct VecOf { using type = Vec<T, N>; };
template <class T> struct VecOf<T, 1> { using type = T; };
template <class T, int N> using vec_t = typename VecOf<T, N>::type;

template <class V> struct Traits { using base = V; static constexpr int cn = 1; };
template <class T, int N> struct Traits<Vec<T, N>> { using base = T; static constexpr int cn = N; };
template <class V> using base_t = typename Traits<V>::base;
template <class V> constexpr int cn_v = Traits<V>::cn;

template <int I, class V> FKD_HD auto& chan(V& v) {
    if constexpr (cn_v<V> == 1) { static_assert(I == 0); return v; }
    else if constexpr (I == 0) return v.x;
    else if constexpr (I == 1) return v.y;
    else if constexpr (I == 2) return v.z;
    else return v.w;
}
template <int I, class V> FKD_HD const auto& chan(const V& v) {
    if constexpr (cn_v<V> == 1) { static_assert(I == 0); return v; }
    else if constexpr (I == 0) return v.x;
    else if constexpr (I == 1) return v.y;
    else if constexpr (I == 2) return v.z;
    else return v.w;
}

// out[c] = f(a[c])  /  out[c] = f(a[c], b[c]) with b either a scalar (broadcast) or a vector of equal width.
template <class O, class A, class F> FKD_HD O map1(const A& a, F f) {
    O o;
    chan<0>(o) = f(chan<0>(a));
    if constexpr (cn_v<O> > 1) chan<1>(o) = f(chan<1>(a));
    if constexpr (cn_v<O> > 2) chan<2>(o) = f(chan<2>(a));
    if constexpr (cn_v<O> > 3) chan<3>(o) = f(chan<3>(a));
    return o;
}
template <int I, class B> FKD_HD const auto& chan_or_scalar(const B& b) {
    if constexpr (cn_v<B> == 1) return b; else return chan<I>(b);
}
template <class O, class A, class B, class F> FKD_HD O map2(const A& a, const B& b, F f) {
    O o;
    chan<0>(o) = f(chan_or_scalar<0>(a), chan_or_scalar<0>(b));
    if constexpr (cn_v<O> > 1) chan<1>(o) = f(chan_or_scalar<1>(a), chan_or_scalar<1>(b));
    if constexpr (cn_v<O> > 2) chan<2>(o) = f(chan_or_scalar<2>(a), chan_or_scalar<2>(b));
    if constexpr (cn_v<O> > 3) chan<3>(o) = f(chan_or_scalar<3>(a), chan_or_scalar<3>(b));
    return o;
}

struct Empty {};

// Two values travelling through a chain side by side (what a read of two sources hands to a two-input operation).
// Each half starts on a dword when its size is not a multiple of four (uchar3 ...), like an element of a per-thread array
// (fkd::Slot): halves packed at byte offsets make the optimiser build 24-bit vectors that only scratch memory can hold.
template <class A, class B> struct Two {
    alignas(sizeof(A) % 4 != 0 ? 4 : alignof(A)) A a;
    alignas(sizeof(B) % 4 != 0 ? 4 : alignof(B)) B b;
};

// Heterogeneous parameter pack with a layout both compilers agree on (plain nested aggregates).
template <class... Ts> struct Tup;
template <> struct Tup<> {};
template <class T, class... Rest> struct Tup<T, Rest...> { T head; Tup<Rest...> tail; };

template <int I, class T, class... Rest> FKD_HD const auto& tup_get(const Tup<T, Rest...>& t) {
    if constexpr (I == 0) return t.head; else return tup_get<I - 1>(t.tail);
}
template <int I, class T, class... Rest> FKD_HD auto& tup_get(Tup<T, Rest...>& t) {
    if constexpr (I == 0) return t.head; else return tup_get<I - 1>(t.tail);
}

// Pitched 2-D view: element (x, y) lives at data + y*pitch + x*sizeof(T).
template <class T> struct RawPtr2D {
    T* data;
    u32 width, height, pitch;
};
// Batched 3-D view: plane z starts at data + z*plane_pitch*color_planes, plane_pitch = pitch*height.
template <class T> struct RawPtr3D {
    T* data;
    u32 width, height, planes, color_planes, pitch, plane_pitch;
};
// Batched 3-D view with the channel planes outermost ("transposed": all R planes, then all G planes, ...): channel
// plane c of image z starts at data + c*color_planes_pitch + z*plane_pitch, plane_pitch = pitch*height,
// color_planes_pitch = plane_pitch*planes.
template <class T> struct RawPtrT3D {
    T* data;
    u32 width, height, planes, color_planes, pitch, plane_pitch, color_planes_pitch;
};
// NV12 frame: luma rows 0..height-1, then height/2 rows of interleaved (U,V) pairs, all with one pitch.
struct RawNV12 {
    const u8* data;
    u32 width, height, pitch;
};
// Any other pixel-format frame (semi-planar 16-bit, packed 4:2:2): same fields, width and height in pixels.
using RawYUV = RawNV12;
struct RawYUVOut {
    u8* data;
    u32 width, height, pitch;
};

#if defined(FKD_HOST_NAMES)
template <class T> struct TypeName;
#define FKD_TN(T, S) template <> struct TypeName<T> { static std::string get() { return S; } };
FKD_TN(u8, "u8") FKD_TN(i8, "i8") FKD_TN(u16, "u16") FKD_TN(i16, "i16") FKD_TN(u32, "u32") FKD_TN(i32, "i32")
FKD_TN(f32, "f32") FKD_TN(f64, "f64")
#undef FKD_TN
template <class T, int N> struct TypeName<Vec<T, N>> {
    static std::string get() { return "Vec<" + TypeName<T>::get() + "," + std::to_string(N) + ">"; }
};
template <class A, class B> struct TypeName<Two<A, B>> {
    static std::string get() { return "Two<" + TypeName<A>::get() + "," + TypeName<B>::get() + ">"; }
};
template <class T> std::string type_name() { return TypeName<T>::get(); }
#endif

} // namespace fkd
