// Bilinear interpolation as a Ternary operation over a back operation (the pixel source it samples).
// Interface counterpart: FK/algorithms/image_processing/interpolation.h.  On this backend the arithmetic lives
// in fkd::ResizeLinear (taps, weights, summation order); the host types only carry the source along.
#ifndef FK_AMD_INTERPOLATION_H
#define FK_AMD_INTERPOLATION_H

#include <fused_kernel/core/execution_model/operation_model/operation_model.h>

namespace fk {

template <typename T> struct Slice2x2 { T _0x0; T _1x0; T _0x1; T _1x1; };

enum class InterpolationType { INTER_LINEAR = 1, NONE = 17 };

template <InterpolationType INTER_T> struct InterpolationParameters;
template <> struct InterpolationParameters<InterpolationType::INTER_LINEAR> {};

template <InterpolationType IType, typename BackIOp_> struct InterpolateComplete;

template <typename BackIOp_>
struct InterpolateComplete<InterpolationType::INTER_LINEAR, BackIOp_>
    : TernaryOperation<float2, InterpolationParameters<InterpolationType::INTER_LINEAR>, BackIOp_,
                       float_<cn<typename BackIOp_::Operation::OutputType>>,
                       InterpolateComplete<InterpolationType::INTER_LINEAR, BackIOp_>> {
    static_assert(isCompleteOperation<BackIOp_>, "NewBackIOp must be a complete operation.");
    using Parent = TernaryOperation<float2, InterpolationParameters<InterpolationType::INTER_LINEAR>, BackIOp_,
                                    float_<cn<typename BackIOp_::Operation::OutputType>>,
                                    InterpolateComplete<InterpolationType::INTER_LINEAR, BackIOp_>>;
    using typename Parent::OperationDataType;
    FK_STATIC_STRUCT(InterpolateComplete, InterpolateComplete)
    static constexpr uint num_elems_x(const Point thread, const OperationDataType& opData) {
        return BackIOp_::Operation::num_elems_x(thread, opData.backIOp);
    }
    static constexpr uint num_elems_y(const Point thread, const OperationDataType& opData) {
        return BackIOp_::Operation::num_elems_y(thread, opData.backIOp);
    }
    static constexpr uint num_elems_z(const Point, const OperationDataType&) { return 1; }
};

template <InterpolationType IT> struct Interpolate;
template <> struct Interpolate<InterpolationType::INTER_LINEAR> {
    FK_STATIC_STRUCT(Interpolate, Interpolate)
    using InputType = float2;
    using OutputType = NullType;
    using ParamsType = InterpolationParameters<InterpolationType::INTER_LINEAR>;
    using BackIOp = NullType;
    using InstanceType = TernaryType;
    using OperationDataType = OperationData<Interpolate<InterpolationType::INTER_LINEAR>>;
    using InstantiableType = Ternary<Interpolate<InterpolationType::INTER_LINEAR>>;
    static constexpr bool IS_FUSED_OP = false;
    static constexpr bool IS_COMPLETE = false;
    static constexpr auto build(const OperationDataType& opData) { return InstantiableType{opData}; }
    static constexpr auto build(const ParamsType& params, const BackIOp& backIOp) { return InstantiableType{{params, backIOp}}; }
    static constexpr auto build() { return InstantiableType{}; }
    template <typename NewBackIOp, std::enable_if_t<isOperation<NewBackIOp>, int> = 0>
    static constexpr auto build(const NewBackIOp& newBackIOp) {
        return InterpolateComplete<InterpolationType::INTER_LINEAR, NewBackIOp>::build(ParamsType{}, newBackIOp);
    }
};

} // namespace fk
#endif
