// SaturateCast<I,O>: OpenCV-style saturating conversion (float -> integer: NaN -> 0, round half to even, clamp).
// Saturate<T>: every channel clamped to [params.x, params.y].  SaturateFloat<T>: float channels clamped to [0, 1].
// Interface counterpart: FK/algorithms/image_processing/saturate.h:25-64.
#ifndef FK_AMD_SATURATE_H
#define FK_AMD_SATURATE_H
#include <fused_kernel/core/execution_model/operation_model/operation_model.h>
namespace fk {
template <typename I, typename O> struct SaturateCast : UnaryOperation<I, O, SaturateCast<I, O>> {
    using Parent = UnaryOperation<I, O, SaturateCast<I, O>>;
    FK_STATIC_STRUCT(SaturateCast, SaturateCast)
    static_assert(cn<I> == cn<O>, "SaturateCast needs the same number of channels on both sides");
};
// (v < lo) ? lo : ((hi < v) ? hi : v) per channel: a NaN channel stays NaN.
template <typename T> struct Saturate : BinaryOperation<T, VectorType_t<VBase<T>, 2>, T, Saturate<T>> {
    using Parent = BinaryOperation<T, VectorType_t<VBase<T>, 2>, T, Saturate<T>>;
    FK_STATIC_STRUCT(Saturate, Saturate)
};
// fmaxf(0, fminf(s, 1)) per channel as the reference's CPU backend computes it: NaN -> 1, -0 stays -0.
template <typename T> struct SaturateFloat : UnaryOperation<T, T, SaturateFloat<T>> {
    using Parent = UnaryOperation<T, T, SaturateFloat<T>>;
    FK_STATIC_STRUCT(SaturateFloat, SaturateFloat)
    static_assert(std::is_same_v<VBase<T>, float>, "Saturate float only works with float base types.");
};
namespace amd {
template <typename T> struct Lower<Saturate<T>> {
    static constexpr bool available = true;
    using type = fkd::Saturate<dev_t<T>>;
    static typename type::Params params(const OperationData<Saturate<T>>& d) { return typename type::Params{d.params.x, d.params.y}; }
};
template <typename T> struct Lower<SaturateFloat<T>> {
    static constexpr bool available = true;
    using type = fkd::SaturateFloat<dev_t<T>>;
    static typename type::Params params(const OperationData<SaturateFloat<T>>&) { return {}; }
};
template <typename I, typename O> struct Lower<SaturateCast<I, O>> {
    static constexpr bool available = true;
    using type = fkd::SaturateCast<dev_t<I>, dev_t<O>>;
    static typename type::Params params(const OperationData<SaturateCast<I, O>>&) { return {}; }
};
} // namespace amd
} // namespace fk
#endif
