// pointwise_chains.h -- chains of one per-channel Operation of the basic_ops headers (math.h, logical.h, bitwise.h,
// algebraic.h) between a read and a write, and chains that end in SplitWrite, spelled ONCE with the public C++ API of the
// fused-kernel library.
//
// This text is compiled twice: by tests/cases/fkl_cases.cpp against this repository's headers (the chains then run as
// gfx950 kernels on device memory), and by oracle/ref_chains.cpp against the reference library's own headers (the
// chains then run on its CPU backend on host memory).  DPP is the data-parallel pattern, StreamT the matching stream
// type and `mem` the kind of memory the caller's pointers refer to.
//
// Every entry returns 0 on success and 2 when `which` is not in the list.
#pragma once

#include <cstdint>
#include <vector>

namespace pointwise_chains {

using namespace fk;

template <class DPP, class StreamT> struct Chains {
    template <class T> static Ptr2D<T> wrap(const void* data, int w, int h, int pitch, MemType mem) {
        return Ptr2D<T>(reinterpret_cast<T*>(const_cast<void*>(data)), uint(w), uint(h), uint(pitch), mem, 0);
    }
    template <class I, class O, class IOp>
    static void one(StreamT& s, MemType mem, const IOp& iop, const void* src, int w, int h, int pitch, void* out, int out_pitch) {
        const auto in = wrap<I>(src, w, h, pitch, mem);
        const auto o = wrap<O>(out, w, h, out_pitch, mem);
        executeOperations<DPP>(s, PerThreadRead<ND::_2D, I>::build(in.ptr()), iop, PerThreadWrite<ND::_2D, O>::build(o.ptr()));
    }
    // `c` holds the constant(s) of the Operation as four floats (converted to the constant's type); `m` a 3x3 matrix.
    //  0 Abs<float3>            1 Abs<int>                 2 Abs<char3 -> char3>       3 Sqr<float3>
    //  4 Sqr<uchar3, int3>      5 Sqrt<float3>             6 Sqrt<uchar3, float3>      7 Ln<float>
    //  8 Exp<float3>            9 AbsDiff<float3>{c}      10 AbsDiff<int, int, int>{c} 11 Max<float3>{c}
    // 12 Min<float3>{c}        13 Max<uchar>{c}           14 Min<int3>{c}             15 BwAnd<uint>{c}
    // 16 BwOr<int3>{c}         17 BwXor<uint>{c}          18 BwNot<uint>              19 ShiftLeft<uint>{c}
    // 20 ShiftRight<int>{c}    21 MxVFloat3<BinaryType>{m} 22 Exp<uchar, float>       23 Abs<short2>
    static int run(StreamT& s, MemType mem, int which, const void* src, int w, int h, int pitch, void* out, int out_pitch,
                   const float* c, const float* m) {
        const float3 cf3 = make_<float3>(c[0], c[1], c[2]);
        const int3 ci3 = make_<int3>(int(c[0]), int(c[1]), int(c[2]));
        const M3x3Float mat{{m[0], m[1], m[2]}, {m[3], m[4], m[5]}, {m[6], m[7], m[8]}};
        switch (which) {
        case 0: one<float3, float3>(s, mem, Abs<float3>::build(), src, w, h, pitch, out, out_pitch); return 0;
        case 1: one<int, int>(s, mem, Abs<int>::build(), src, w, h, pitch, out, out_pitch); return 0;
        case 2: one<char3, char3>(s, mem, Abs<char3>::build(), src, w, h, pitch, out, out_pitch); return 0;
        case 3: one<float3, float3>(s, mem, Sqr<float3>::build(), src, w, h, pitch, out, out_pitch); return 0;
        case 4: one<uchar3, int3>(s, mem, Sqr<uchar3, int3>::build(), src, w, h, pitch, out, out_pitch); return 0;
        case 5: one<float3, float3>(s, mem, Sqrt<float3>::build(), src, w, h, pitch, out, out_pitch); return 0;
        case 6: one<uchar3, float3>(s, mem, Sqrt<uchar3, float3>::build(), src, w, h, pitch, out, out_pitch); return 0;
        case 7: one<float, float>(s, mem, Ln<float>::build(), src, w, h, pitch, out, out_pitch); return 0;
        case 8: one<float3, float3>(s, mem, Exp<float3>::build(), src, w, h, pitch, out, out_pitch); return 0;
        case 9: one<float3, float3>(s, mem, AbsDiff<float3>::build(cf3), src, w, h, pitch, out, out_pitch); return 0;
        case 10: one<int, int>(s, mem, AbsDiff<int, int, int>::build(int(c[0])), src, w, h, pitch, out, out_pitch); return 0;
        case 11: one<float3, float3>(s, mem, Max<float3>::build(cf3), src, w, h, pitch, out, out_pitch); return 0;
        case 12: one<float3, float3>(s, mem, Min<float3>::build(cf3), src, w, h, pitch, out, out_pitch); return 0;
        case 13: one<uchar, uchar>(s, mem, Max<uchar>::build(uchar(c[0])), src, w, h, pitch, out, out_pitch); return 0;
        case 14: one<int3, int3>(s, mem, Min<int3>::build(ci3), src, w, h, pitch, out, out_pitch); return 0;
        case 15: one<uint, uint>(s, mem, BwAnd<uint>::build(uint(c[0])), src, w, h, pitch, out, out_pitch); return 0;
        case 16: one<int3, int3>(s, mem, BwOr<int3>::build(ci3), src, w, h, pitch, out, out_pitch); return 0;
        case 17: one<uint, uint>(s, mem, BwXor<uint>::build(uint(c[0])), src, w, h, pitch, out, out_pitch); return 0;
        case 18: one<uint, uint>(s, mem, BwNot<uint>::build(), src, w, h, pitch, out, out_pitch); return 0;
        case 19: one<uint, uint>(s, mem, ShiftLeft<uint>::build(uint(c[0])), src, w, h, pitch, out, out_pitch); return 0;
        case 20: one<int, int>(s, mem, ShiftRight<int>::build(int(c[0])), src, w, h, pitch, out, out_pitch); return 0;
        case 21: one<float3, float3>(s, mem, MxVFloat3<BinaryType>::build(mat), src, w, h, pitch, out, out_pitch); return 0;
        case 22: one<uchar, float>(s, mem, Exp<uchar, float>::build(), src, w, h, pitch, out, out_pitch); return 0;
        case 23: one<short2, short2>(s, mem, Abs<short2>::build(), src, w, h, pitch, out, out_pitch); return 0;
        default: return 2;
        }
    }

    // ---- SplitWrite<_2D, T>: one output image per channel, each with its own pitch --------------------------------
    template <class O> static std::vector<Ptr2D<VBase<O>>> planes_of(void* const* outs, const int* out_pitch, int w, int h, MemType mem) {
        std::vector<Ptr2D<VBase<O>>> v;
        for (int c = 0; c < cn<O>; ++c) v.push_back(wrap<VBase<O>>(outs[c], w, h, out_pitch[c], mem));
        return v;
    }
    // 0 uchar3 image -> its three planes              1 uchar3 -> Cast -> Mul{c} -> three float planes
    // 2 float4 image -> its four planes               3 uchar3 -> Crop(8, 4, w - 16, h - 8) -> Resize(dw x dh) -> three float planes
    // 4 float2 image -> its two planes
    static int split_write(StreamT& s, MemType mem, int which, const void* src, int w, int h, int pitch, int dw, int dh,
                           void* const* outs, const int* out_pitch, const float* c) {
        switch (which) {
        case 0: {
            const auto in = wrap<uchar3>(src, w, h, pitch, mem);
            executeOperations<DPP>(s, PerThreadRead<ND::_2D, uchar3>::build(in.ptr()),
                                   SplitWrite<ND::_2D, uchar3>::build(planes_of<uchar3>(outs, out_pitch, w, h, mem)));
            return 0;
        }
        case 1: {
            const auto in = wrap<uchar3>(src, w, h, pitch, mem);
            executeOperations<DPP>(s, PerThreadRead<ND::_2D, uchar3>::build(in.ptr()), Cast<uchar3, float3>::build(),
                                   Mul<float3>::build(make_<float3>(c[0], c[1], c[2])),
                                   SplitWrite<ND::_2D, float3>::build(planes_of<float3>(outs, out_pitch, w, h, mem)));
            return 0;
        }
        case 2: {
            const auto in = wrap<float4>(src, w, h, pitch, mem);
            executeOperations<DPP>(s, PerThreadRead<ND::_2D, float4>::build(in.ptr()),
                                   SplitWrite<ND::_2D, float4>::build(planes_of<float4>(outs, out_pitch, w, h, mem)));
            return 0;
        }
        case 3: {
            const auto in = wrap<uchar3>(src, w, h, pitch, mem);
            executeOperations<DPP>(s, PerThreadRead<ND::_2D, uchar3>::build(in.ptr()), Crop<>::build(Rect(8, 4, w - 16, h - 8)),
                                   Resize<InterpolationType::INTER_LINEAR>::build(Size(dw, dh)),
                                   SplitWrite<ND::_2D, float3>::build(planes_of<float3>(outs, out_pitch, dw, dh, mem)));
            return 0;
        }
        case 4: {
            const auto in = wrap<float2>(src, w, h, pitch, mem);
            executeOperations<DPP>(s, PerThreadRead<ND::_2D, float2>::build(in.ptr()),
                                   SplitWrite<ND::_2D, float2>::build(planes_of<float2>(outs, out_pitch, w, h, mem)));
            return 0;
        }
        default: return 2;
        }
    }

    // ---- DualSourceRead<_2D, T> -> the two-input form of an Operation -> write ------------------------------------
    template <class T, class O, class... IOps>
    static void two(StreamT& s, MemType mem, const void* a, const void* b, int w, int h, int pitch_a, int pitch_b, void* out, int out_pitch,
                    const IOps&... iops) {
        const auto pa = wrap<T>(a, w, h, pitch_a, mem);
        const auto pb = wrap<T>(b, w, h, pitch_b, mem);
        const auto o = wrap<O>(out, w, h, out_pitch, mem);
        executeOperations<DPP>(s, DualSourceRead<ND::_2D, T>::build(pa, pb), iops..., PerThreadWrite<ND::_2D, O>::build(o.ptr()));
    }
    // 0 Add<float3>            1 AbsDiff<uchar3 -> int3>   2 Mul<float>              3 Div<float3>
    // 4 Sub<float3>            5 BwXor<uint>               6 Max<float3>             7 Min<int>
    // 8 the mean of two uchar3 images: Add<uchar3 -> int3> -> Cast<int3, float3> -> Mul{0.5} -> SaturateCast<float3, uchar3>
    // 9 BwAnd<uint>           10 BwOr<uint>
    static int dual(StreamT& s, MemType mem, int which, const void* a, const void* b, int w, int h, int pitch_a, int pitch_b,
                    void* out, int out_pitch) {
        switch (which) {
        case 0: two<float3, float3>(s, mem, a, b, w, h, pitch_a, pitch_b, out, out_pitch, Add<float3, float3, float3, UnaryType>::build()); return 0;
        case 1: two<uchar3, int3>(s, mem, a, b, w, h, pitch_a, pitch_b, out, out_pitch, AbsDiff<uchar3, uchar3, int3, UnaryType>::build()); return 0;
        case 2: two<float, float>(s, mem, a, b, w, h, pitch_a, pitch_b, out, out_pitch, Mul<float, float, float, UnaryType>::build()); return 0;
        case 3: two<float3, float3>(s, mem, a, b, w, h, pitch_a, pitch_b, out, out_pitch, Div<float3, float3, float3, UnaryType>::build()); return 0;
        case 4: two<float3, float3>(s, mem, a, b, w, h, pitch_a, pitch_b, out, out_pitch, Sub<float3, float3, float3, UnaryType>::build()); return 0;
        case 5: two<uint, uint>(s, mem, a, b, w, h, pitch_a, pitch_b, out, out_pitch, BwXor<uint, uint, uint, UnaryType>::build()); return 0;
        case 6: two<float3, float3>(s, mem, a, b, w, h, pitch_a, pitch_b, out, out_pitch, Max<float3, float3, float3, UnaryType>::build()); return 0;
        case 7: two<int, int>(s, mem, a, b, w, h, pitch_a, pitch_b, out, out_pitch, Min<int, int, int, UnaryType>::build()); return 0;
        case 8: two<uchar3, uchar3>(s, mem, a, b, w, h, pitch_a, pitch_b, out, out_pitch, Add<uchar3, uchar3, int3, UnaryType>::build(),
                                    Cast<int3, float3>::build(), Mul<float3>::build(make_set<float3>(0.5f)), SaturateCast<float3, uchar3>::build()); return 0;
        case 9: two<uint, uint>(s, mem, a, b, w, h, pitch_a, pitch_b, out, out_pitch, BwAnd<uint, uint, uint, UnaryType>::build()); return 0;
        case 10: two<uint, uint>(s, mem, a, b, w, h, pitch_a, pitch_b, out, out_pitch, BwOr<uint, uint, uint, UnaryType>::build()); return 0;
        default: return 2;
        }
    }
};

} // namespace pointwise_chains
