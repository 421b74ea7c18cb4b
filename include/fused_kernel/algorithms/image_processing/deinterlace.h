// Deinterlace<BLEND|INTER_LINEAR>: a read-back operation that rebuilds progressive lines from an interlaced frame:
// BLEND averages every line with the one above it, INTER_LINEAR keeps the lines of one field and replaces the
// others by the average of their vertical neighbours.  Output is float_<channels>.
// Interface counterpart: FK/algorithms/image_processing/deinterlace.h:24-182.
#ifndef FK_AMD_DEINTERLACE_H
#define FK_AMD_DEINTERLACE_H

#include <fused_kernel/algorithms/basic_ops/memory_operations.h>
#include <fused_kernel/core/data/size.h>
#include <fused_kernel/core/execution_model/operation_model/operation_model.h>

namespace fk {

enum class DeinterlaceType { BLEND, INTER_LINEAR };

template <DeinterlaceType DType> struct DeinterlaceParameters {};
template <> struct DeinterlaceParameters<DeinterlaceType::BLEND> {};
template <> struct DeinterlaceParameters<DeinterlaceType::INTER_LINEAR> {
    bool useEvenLines{true};
};

enum class DeinterlaceLinear : bool { USE_EVEN = true, USE_ODD = false };

template <DeinterlaceType DType, typename BackIOp_ = NullType>
struct Deinterlace : ReadBackOperation<typename BackIOp_::Operation::OutputType, DeinterlaceParameters<DType>, BackIOp_,
                                       float_<cn<typename BackIOp_::Operation::OutputType>>, Deinterlace<DType, BackIOp_>> {
    static_assert(isAnyCompleteReadType<BackIOp_>, "BackIOp must be a complete type for this specialization");
    using Parent = ReadBackOperation<typename BackIOp_::Operation::OutputType, DeinterlaceParameters<DType>, BackIOp_,
                                     float_<cn<typename BackIOp_::Operation::OutputType>>, Deinterlace<DType, BackIOp_>>;
    using typename Parent::OperationDataType;
    using typename Parent::BackIOp;
    FK_STATIC_STRUCT(Deinterlace, Deinterlace)
    static constexpr uint num_elems_x(const Point thread, const OperationDataType& opData) {
        return BackIOp::Operation::num_elems_x(thread, opData.backIOp);
    }
    static constexpr uint num_elems_y(const Point thread, const OperationDataType& opData) {
        return BackIOp::Operation::num_elems_y(thread, opData.backIOp);
    }
    static constexpr uint num_elems_z(const Point, const OperationDataType&) { return 1; }
    static constexpr ActiveThreads getActiveThreads(const OperationDataType& opData) {
        return {num_elems_x(Point{0, 0, 0}, opData), num_elems_y(Point{0, 0, 0}, opData), 1u};
    }
    using Parent::build;
};

template <DeinterlaceType DType>
struct Deinterlace<DType, NullType>
    : IncompleteReadBackOperation<NullType, DeinterlaceParameters<DType>, NullType, NullType, Deinterlace<DType, NullType>> {
    using Parent = IncompleteReadBackOperation<NullType, DeinterlaceParameters<DType>, NullType, NullType, Deinterlace<DType, NullType>>;
    using typename Parent::OperationDataType;
    using typename Parent::InstantiableType;
    using typename Parent::ParamsType;
    template <typename BackIOp_> using NewInstantiableType = ReadBack<Deinterlace<DType, BackIOp_>>;
    FK_STATIC_STRUCT(Deinterlace, Deinterlace)
    static constexpr uint num_elems_x(const Point, const OperationDataType&) { return 1; }
    static constexpr uint num_elems_y(const Point, const OperationDataType&) { return 1; }
    static constexpr uint num_elems_z(const Point, const OperationDataType&) { return 1; }
    using Parent::build;
    static constexpr InstantiableType build(const ParamsType& params) { return {{params, {}}}; }
    template <DeinterlaceType DT = DType>
    static constexpr auto build(const DeinterlaceType& type) -> std::enable_if_t<DT == DeinterlaceType::INTER_LINEAR, InstantiableType> {
        return {{ParamsType{static_cast<bool>(type)}, {}}};   // as in the reference: the enumerator's value becomes useEvenLines
    }
    template <DeinterlaceType DT = DType>
    static constexpr auto build() -> std::enable_if_t<DT == DeinterlaceType::BLEND, InstantiableType> {
        return InstantiableType{{ParamsType{}, {}}};
    }
    template <typename BackIOp_, std::enable_if_t<isOperation<BackIOp_>, int> = 0>
    static constexpr auto build(const BackIOp_& backIOp, const InstantiableType& iOp) {
        return NewInstantiableType<BackIOp_>{{iOp.params, backIOp}};
    }
    template <typename BIOp, DeinterlaceType DT = DType, std::enable_if_t<isOperation<BIOp>, int> = 0>
    static constexpr auto build(const BIOp& backIOp) -> std::enable_if_t<DT == DeinterlaceType::BLEND, NewInstantiableType<BIOp>> {
        return NewInstantiableType<BIOp>{{ParamsType{}, backIOp}};
    }
    template <typename BIOp, DeinterlaceType DT = DType>
    static constexpr auto build(const DeinterlaceLinear& lin, const BIOp& backIOp)
        -> std::enable_if_t<DT == DeinterlaceType::INTER_LINEAR, NewInstantiableType<BIOp>> {
        return NewInstantiableType<BIOp>{{DeinterlaceParameters<DeinterlaceType::INTER_LINEAR>{static_cast<bool>(lin)}, backIOp}};
    }
};

namespace amd {
template <DeinterlaceType DT, typename BackIOp>
struct Lower<Deinterlace<DT, BackIOp>, std::enable_if_t<!std::is_same_v<BackIOp, NullType>>> {
    static constexpr bool available = true;
    using type = fkd::Deinterlace<int(DT), device_op_t<BackIOp>>;
    static typename type::Params params(const OperationData<Deinterlace<DT, BackIOp>>& d) {
        typename type::Params p{};
        if constexpr (DT == DeinterlaceType::INTER_LINEAR) p.use_even = d.params.useEvenLines ? 1 : 0;
        p.back = lower_iop(d.backIOp);
        return p;
    }
};
} // namespace amd

} // namespace fk
#endif
