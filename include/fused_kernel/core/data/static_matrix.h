// A 3x3 float matrix as three rows, for the colour-conversion coefficients.  Interface counterpart:
// FK/core/data/static_matrix.h:20-42 (the product of two matrices is element by element there, and here).
#ifndef FK_AMD_STATIC_MATRIX_H
#define FK_AMD_STATIC_MATRIX_H
#include <fused_kernel/core/utils/vector_utils.h>
namespace fk {
struct M3x3Float {
    const float3 x;
    const float3 y;
    const float3 z;
};
} // namespace fk
constexpr fk::M3x3Float operator*(const fk::M3x3Float& m, float s) { return {m.x * s, m.y * s, m.z * s}; }
constexpr fk::M3x3Float operator*(float s, const fk::M3x3Float& m) { return m * s; }
constexpr fk::M3x3Float operator*(const fk::M3x3Float& a, const fk::M3x3Float& b) { return {a.x * b.x, a.y * b.y, a.z * b.z}; }
#endif
