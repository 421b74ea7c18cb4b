// MxVFloat3<BinaryType>: a float3 value times a 3x3 matrix given as the Operation's parameter (row r of the result is
// (v.x * m[r].x + v.y * m[r].y) + v.z * m[r].z).  Interface counterpart: FK/algorithms/basic_ops/algebraic.h:22-40; the
// form that takes value and matrix in a Tuple is not provided.
#ifndef FK_AMD_ALGEBRAIC_H
#define FK_AMD_ALGEBRAIC_H
#include <fused_kernel/core/execution_model/operation_model/operation_model.h>
#include <fused_kernel/core/data/static_matrix.h>
namespace fk {
template <typename OpInstanceType = BinaryType> struct MxVFloat3;
template <> struct MxVFloat3<BinaryType> : BinaryOperation<float3, M3x3Float, float3, MxVFloat3<BinaryType>> {
    using Parent = BinaryOperation<float3, M3x3Float, float3, MxVFloat3<BinaryType>>;
    FK_STATIC_STRUCT(MxVFloat3, MxVFloat3)
};
namespace amd {
template <> struct Lower<MxVFloat3<BinaryType>> {
    static constexpr bool available = true;
    using type = fkd::MxV3;
    static type::Params params(const OperationData<MxVFloat3<BinaryType>>& d) {
        const M3x3Float& m = d.params;
        return type::Params{{m.x.x, m.x.y, m.x.z, m.y.x, m.y.y, m.y.z, m.z.x, m.z.y, m.z.z}};
    }
};
} // namespace amd
} // namespace fk
#endif
