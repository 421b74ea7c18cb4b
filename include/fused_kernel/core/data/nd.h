#ifndef FK_AMD_ND_H
#define FK_AMD_ND_H
namespace fk {
// Dimensionality of a pointer: FK/core/data/nd.h:20.
enum class ND { _1D = 1, _2D = 2, _3D = 3, T3D = 4 };
} // namespace fk
#endif
