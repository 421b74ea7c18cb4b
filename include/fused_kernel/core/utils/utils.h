// Host-side utilities of the MI355X backend: function qualifiers, the error convention, integer aliases.
//
// This backend keeps host code and device code in separate compilers: everything under include/fused_kernel/
// is plain C++20 for g++/clang++ and never includes a HIP header.  The qualifier macros therefore carry no
// device attributes.  Interface counterpart: FK/core/utils/utils.h:34-74 (qualifiers), :98-153 (gpuErrchk).
#ifndef FK_AMD_UTILS_H
#define FK_AMD_UTILS_H

#include <cstddef>
#include <cstdint>
#include <iostream>
#include <stdexcept>
#include <string>

#include <fklhip.h>

#define FK_HOST_FUSE static constexpr inline
#define FK_HOST_CNST constexpr inline
#define FK_HOST_STATIC static inline
#define FK_HOST_INLINE inline
#define FK_HOST_DEVICE_FUSE static constexpr inline
#define FK_HOST_DEVICE_CNST constexpr inline
#define FK_HOST_DEVICE_STATIC static inline
#define FK_DEVICE_FUSE static constexpr inline
#define FK_DEVICE_CNST constexpr inline
#define FK_RESTRICT __restrict__

// A struct that only carries static members and type aliases.
#define FK_STATIC_STRUCT(StructName, SelfAlias)  \
    StructName() = delete;                       \
    StructName(const SelfAlias&) = delete;       \
    SelfAlias& operator=(const SelfAlias&) = delete;

using uchar = unsigned char;
using schar = signed char;
using ushort = unsigned short;
using uint = unsigned int;
using ulong = unsigned long;
using longlong = long long;
using ulonglong = unsigned long long;

namespace fk {

// Turns a non-zero code of the C ABI into the exception the CUDA backend throws for a failed runtime call:
// std::runtime_error("GPU Error: <text> File: <file> Line:<line>\n").
inline void gpuAssert(int code, const char* file, int line) {
    if (code != FKLHIP_OK) {
        throw std::runtime_error(std::string("GPU Error: ") + fklhip_error_string(code) + " File: " + file +
                                 " Line:" + std::to_string(line) + "\n");
    }
}

} // namespace fk

#define gpuErrchk(expr) ::fk::gpuAssert(static_cast<int>(expr), __FILE__, __LINE__)

#endif
