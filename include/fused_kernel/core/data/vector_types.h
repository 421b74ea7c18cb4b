// 1..4 channel element types (uchar3, float4, ...) with the alignment the GPU element layouts use, and their
// global aliases.  Interface counterpart: FK/core/data/vector_types.h:68-312.
#ifndef FK_AMD_VECTOR_TYPES_H
#define FK_AMD_VECTOR_TYPES_H

#include <fused_kernel/core/utils/utils.h>

namespace fk {

#define FK_AMD_VEC_FAMILY(Name, T, A2, A4)                          \
    struct Name##1 { T x; };                                        \
    struct alignas(A2) Name##2 { T x, y; };                         \
    struct Name##3 { T x, y, z; };                                  \
    struct alignas(A4) Name##4 { T x, y, z, w; };

// Results of channel-wise comparisons; in a boolean context a BoolN is true when every channel is.
struct Bool1 { bool x; constexpr operator bool() const { return x; } };
struct alignas(2) Bool2 { bool x, y; constexpr operator bool() const { return x && y; } };
struct Bool3 { bool x, y, z; constexpr operator bool() const { return x && y && z; } };
struct alignas(4) Bool4 { bool x, y, z, w; constexpr operator bool() const { return x && y && z && w; } };
struct Bool {
    static constexpr bool vAnd(const Bool1& b) { return b.x; }
    static constexpr bool vAnd(const Bool2& b) { return b.x && b.y; }
    static constexpr bool vAnd(const Bool3& b) { return b.x && b.y && b.z; }
    static constexpr bool vAnd(const Bool4& b) { return b.x && b.y && b.z && b.w; }
    static constexpr bool vOr(const Bool1& b) { return b.x; }
    static constexpr bool vOr(const Bool2& b) { return b.x || b.y; }
    static constexpr bool vOr(const Bool3& b) { return b.x || b.y || b.z; }
    static constexpr bool vOr(const Bool4& b) { return b.x || b.y || b.z || b.w; }
};
FK_AMD_VEC_FAMILY(Char, signed char, 2, 4)
FK_AMD_VEC_FAMILY(Uchar, unsigned char, 2, 4)
FK_AMD_VEC_FAMILY(Short, short, 4, 8)
FK_AMD_VEC_FAMILY(Ushort, unsigned short, 4, 8)
FK_AMD_VEC_FAMILY(Int, int, 8, 16)
FK_AMD_VEC_FAMILY(Uint, unsigned int, 8, 16)
FK_AMD_VEC_FAMILY(Long, long, 16, 16)
FK_AMD_VEC_FAMILY(Ulong, unsigned long, 16, 16)
FK_AMD_VEC_FAMILY(Longlong, long long, 16, 16)
FK_AMD_VEC_FAMILY(Ulonglong, unsigned long long, 16, 16)
FK_AMD_VEC_FAMILY(Float, float, 8, 16)
FK_AMD_VEC_FAMILY(Double, double, 16, 16)
#undef FK_AMD_VEC_FAMILY

} // namespace fk

#define FK_AMD_VEC_ALIASES(lower, Upper)   \
    using lower##1 = fk::Upper##1;         \
    using lower##2 = fk::Upper##2;         \
    using lower##3 = fk::Upper##3;         \
    using lower##4 = fk::Upper##4;
FK_AMD_VEC_ALIASES(bool, Bool)
FK_AMD_VEC_ALIASES(char, Char)
FK_AMD_VEC_ALIASES(uchar, Uchar)
FK_AMD_VEC_ALIASES(short, Short)
FK_AMD_VEC_ALIASES(ushort, Ushort)
FK_AMD_VEC_ALIASES(int, Int)
FK_AMD_VEC_ALIASES(uint, Uint)
FK_AMD_VEC_ALIASES(long, Long)
FK_AMD_VEC_ALIASES(ulong, Ulong)
FK_AMD_VEC_ALIASES(longlong, Longlong)
FK_AMD_VEC_ALIASES(ulonglong, Ulonglong)
FK_AMD_VEC_ALIASES(float, Float)
FK_AMD_VEC_ALIASES(double, Double)
#undef FK_AMD_VEC_ALIASES

#endif
